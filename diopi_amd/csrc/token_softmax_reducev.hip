// diopiTokenSoftmaxReduceVInference for gfx950: softmax over each sequence's logits, then the
// probability-weighted sum of the cached V rows.
//
// Semantics: impl/torch/functions/functions_lightllm.cpp:82-107 of the reference (Python statement
// customized_test.py:715-733).  For sequence i with length L_i and query head h:
//   P      = softmax(logics[h, b_start_loc[i] : b_start_loc[i] + L_i])       (fp32 inside)
//   slots  = b_loc[i, max_input_len - L_i : max_input_len]
//   out[i, h, :] = sum_t P[t] * v[slots[t], h / G, :]                         (fp32 accumulate)
// other_kv_index is ignored, as in the reference.
//
// Kernel shape (16-bit types, D == 128): a split-K ("flash decoding") pass followed by a small
// merge.  A work-group owns (token range, sequence, group of HB kv heads).  It walks its range in
// sub-tiles of 128 tokens:
//   1. each wave takes query heads of the group in turn, reads the sub-tile's logits as one
//      coalesced row segment, updates the running maximum / denominator of that head and leaves
//      the un-normalised probabilities exp(x - max) in LDS together with the rescale factor;
//   2. 16 lanes own one V row segment (one kv head of one token, 256 bytes, one 16-byte load per
//      lane); the 16 such lane groups of the work-group cover HB heads x 16/HB tokens per step.
//      Each lane multiplies its 8 V elements by the probabilities of the G query heads sharing
//      that kv head and accumulates in fp32 registers.  V bytes are read exactly once.
// At the end the lane groups that worked on the same head are summed through LDS and the range's
// (max, denominator, accumulator) triple is written to context-owned scratch; a merge kernel
// combines the ranges of a sequence.  A sequence that fits one range is finished in place and
// skips the scratch round trip.  Nothing on the host depends on the sequence lengths.
#include <cmath>

#include "common.hpp"
#include "decode.hpp"
#include "device.hpp"

namespace rocm {
namespace {

constexpr int kRvThreads = 256;
constexpr int kRvWaves = kRvThreads / kWave;
constexpr int kSub = 128;          // tokens per sub-tile
constexpr int kLaneGroups = 16;    // 16-lane groups per work-group
constexpr int kMaxHeadsQ = 64;     // query heads per work-group (HB * G) the LDS tile is sized for
constexpr int kD = 128;

// c + a.lo*b.lo + a.hi*b.hi on packed 16-bit pairs, accumulated in fp32 (v_dot2_f32_f16 / v_dot2_f32_bf16).
// The last argument only selects the element type.
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c, half_t*) {
    union {
        uint32_t u;
        f16x2 v;
    } ua, ub;
    ua.u = a;
    ub.u = b;
    return __builtin_amdgcn_fdot2(ua.v, ub.v, c, false);
}
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c, bf16_t*) {
    union {
        uint32_t u;
        bf16x2 v;
    } ua, ub;
    ua.u = a;
    ub.u = b;
    return __builtin_amdgcn_fdot2_f32_bf16(ua.v, ub.v, c, false);
}

struct SplitArgs {
    float* partAcc;  // [batch, splits, H, D]
    float* partMl;   // [batch, splits, H, 2]  (running max, denominator)
    int splits;      // ranges per sequence the scratch is sized for
    int TT;          // tokens per range (multiple of kSub)
    int HB;          // kv heads per work-group: 1, 2, 4, 8 or 16
};

template <typename T, int G>
__global__ __launch_bounds__(kRvThreads) void softmaxReduceVSplit(T* __restrict__ out, const T* __restrict__ logits, const T* __restrict__ v, DecodeArgs a,
                                                                  SplitArgs sp) {
    // un-normalised probabilities of the sub-tile; after the sweep the same storage holds the
    // [query head][dim] sums over the token phases
    __shared__ float sP[kMaxHeadsQ][kSub];
    __shared__ float sAlpha[kMaxHeadsQ];        // rescale factor of the accumulators for this sub-tile
    __shared__ float sM[kMaxHeadsQ];            // running maximum per query head
    __shared__ float sL[kMaxHeadsQ];            // running denominator per query head
    __shared__ int64_t sSlot[kSub];             // element offset of each token's cache row

    const int i = blockIdx.y;
    int64_t L = loadIndex(a.bSeqLen, i, a.len64);
    if (L > a.maxInputLen) L = a.maxInputLen;
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * sp.TT;
    if (t0 >= L) return;
    const int64_t tEnd = (t0 + sp.TT < L) ? t0 + sp.TT : L;
    const int64_t start = loadIndex(a.bStartLoc, i, a.start64);
    const int64_t locBase = static_cast<int64_t>(i) * a.bLocStride + (a.maxInputLen - L);
    const int tid = threadIdx.x;
    const int lane = tid % kWave;
    const int wave = tid / kWave;
    const int HB = sp.HB;
    const int hkBegin = blockIdx.z * HB;
    const int headsQ = HB * G;  // query heads handled here (some may lie beyond H when Hkv % HB != 0)

    // lane group -> (kv head inside the group, token phase)
    const int lg = tid / 16;
    const int c = tid % 16;  // 16-byte packet of the 256-byte row segment
    const int hl = lg % HB;  // local kv head
    const int tp = lg / HB;  // token phase
    const int TP = kLaneGroups / HB;
    const int hk = hkBegin + hl;
    const bool headValid = hk < a.Hkv;
    const int64_t rowStride = static_cast<int64_t>(a.Hkv) * kD;

    float acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
    }
    for (int h = tid; h < headsQ; h += kRvThreads) {
        sM[h] = -INFINITY;
        sL[h] = 0.f;
    }
    __syncthreads();

    for (int64_t ts = t0; ts < tEnd; ts += kSub) {
        const int nTok = static_cast<int>((tEnd - ts < kSub) ? tEnd - ts : kSub);
        // ---- phase 1: slots and probabilities of the sub-tile ----
        for (int t = tid; t < kSub; t += kRvThreads) {
            // tokens past the end alias the last valid one (their probability is zero)
            int64_t slot = loadIndex(a.bLoc, locBase + ts + (t < nTok ? t : nTok - 1), a.loc64);
            slot = slot < 0 ? 0 : (slot >= a.numSlots ? a.numSlots - 1 : slot);
            sSlot[t] = slot * rowStride;
        }
        for (int h = wave; h < headsQ; h += kRvWaves) {
            const int qh = hkBegin * G + h;
            float x[kSub / kWave];
            float mloc = -INFINITY;
#pragma unroll
            for (int j = 0; j < kSub / kWave; ++j) {
                const int t = j * kWave + lane;
                const int64_t col = start + ts + t;
                x[j] = -INFINITY;
                if (t < nTok && qh < a.H && col >= 0 && col < a.logitCols) x[j] = static_cast<float>(logits[static_cast<int64_t>(qh) * a.logitCols + col]);
                mloc = fmaxf(mloc, x[j]);
            }
            mloc = waveMax(mloc);
            const float mOld = sM[h];
            const float mNew = fmaxf(mOld, mloc);
            float lsum = 0.f;
#pragma unroll
            for (int j = 0; j < kSub / kWave; ++j) {
                const int t = j * kWave + lane;
                // a row of -inf logits keeps p = 0 instead of exp(nan)
                const float p = (x[j] == -INFINITY) ? 0.f : __expf(x[j] - mNew);
                if constexpr (G == 1) {
                    sP[h][t] = p;
                } else {
                    // grouped heads: probabilities rounded to the element type and stored as token pairs,
                    // [token pair][query head] -> one dword per (pair, head), the operand layout of the dot2 path
                    reinterpret_cast<T*>(&sP[0][0])[((t >> 1) * kMaxHeadsQ + h) * 2 + (t & 1)] = static_cast<T>(p);
                }
                lsum += p;
            }
            lsum = waveSum(lsum);
            if (lane == 0) {
                const float alpha = (mOld == -INFINITY) ? 0.f : __expf(mOld - mNew);
                sAlpha[h] = alpha;
                sM[h] = mNew;
                sL[h] = sL[h] * alpha + lsum;
            }
        }
        __syncthreads();
        // ---- phase 2: accumulate V rows ----
        if (headValid) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const float alpha = sAlpha[hl * G + g];
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[g][e] *= alpha;
            }
            const T* vHead = v + hk * kD + c * 8;
            constexpr int U = 8;  // rows in flight per lane
            if constexpr (G > 1) {
                // Two tokens at a time: the rows of tokens (t, t+1) are interleaved element-wise with byte permutes
                // and multiplied against the packed probability pairs with v_dot2 (fp32 accumulate): half the VALU
                // work of convert + fma per element, which is what bounds this kernel once G query heads share a row.
                const uint32_t* sPairs = reinterpret_cast<const uint32_t*>(&sP[0][0]);
                const int nPairs = (nTok + 1) / 2;
                constexpr int UP = U / 2;
                for (int pb = tp; pb < nPairs; pb += TP * UP) {
                    u32x4 v0[UP], v1[UP];
#pragma unroll
                    for (int u = 0; u < UP; ++u) {
                        const int pr = pb + u * TP;
                        if (pr < nPairs) {
                            v0[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vHead + sSlot[2 * pr]));
                            v1[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vHead + sSlot[2 * pr + 1]));
                        }
                    }
#pragma unroll
                    for (int u = 0; u < UP; ++u) {
                        const int pr = pb + u * TP;
                        if (pr < nPairs) {
                            uint32_t pp[G];
#pragma unroll
                            for (int g = 0; g < G; ++g) pp[g] = sPairs[pr * kMaxHeadsQ + hl * G + g];
#pragma unroll
                            for (int kk = 0; kk < 4; ++kk) {
                                // (row t elem 2kk, row t+1 elem 2kk) and (row t elem 2kk+1, row t+1 elem 2kk+1)
                                const uint32_t lo = __builtin_amdgcn_perm(v1[u][kk], v0[u][kk], 0x05040100u);
                                const uint32_t hi = __builtin_amdgcn_perm(v1[u][kk], v0[u][kk], 0x07060302u);
#pragma unroll
                                for (int g = 0; g < G; ++g) {
                                    acc[g][2 * kk] = dot2(lo, pp[g], acc[g][2 * kk], static_cast<T*>(nullptr));
                                    acc[g][2 * kk + 1] = dot2(hi, pp[g], acc[g][2 * kk + 1], static_cast<T*>(nullptr));
                                }
                            }
                        }
                    }
                }
            } else
            for (int tb = tp; tb < nTok; tb += TP * U) {
                Pack16<T> vv[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int t = tb + u * TP;
                    if (t < nTok) vv[u] = loadPackStream(vHead + sSlot[t]);
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int t = tb + u * TP;
                    if (t < nTok) {
                        float vf[8];
#pragma unroll
                        for (int e = 0; e < 8; ++e) vf[e] = static_cast<float>(vv[u].e[e]);
#pragma unroll
                        for (int g = 0; g < G; ++g) {
                            const float p = sP[hl * G + g][t];
#pragma unroll
                            for (int e = 0; e < 8; ++e) acc[g][e] += p * vf[e];
                        }
                    }
                }
            }
        }
        __syncthreads();
    }

    // ---- fold the token phases (kSub == kD, so sP doubles as a [query head][dim] buffer) ----
    static_assert(kSub == kD, "the probability tile is reused as the fold buffer");
    for (int p = 0; p < TP; ++p) {
        if (tp == p && headValid) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float* dst = &sP[hl * G + g][c * 8 + e];
                    *dst = (p == 0) ? acc[g][e] : *dst + acc[g][e];
                }
            }
        }
        __syncthreads();
    }
    const bool single = L <= sp.TT;  // the whole sequence lives in this range
    const int64_t split = blockIdx.x;
    for (int idx = tid; idx < headsQ * kD; idx += kRvThreads) {
        const int h = idx / kD;   // local query head = hl * G + g
        const int d = idx % kD;
        const int hlq = h / G, g = h % G;
        const int qh = hkBegin * G + h;
        if (hkBegin + hlq >= a.Hkv || qh >= a.H) continue;
        (void)g;
        const float s = sP[h][d];
        if (single) {
            out[(static_cast<int64_t>(i) * a.H + qh) * kD + d] = static_cast<T>(s / sL[h]);
        } else {
            sp.partAcc[((static_cast<int64_t>(i) * sp.splits + split) * a.H + qh) * kD + d] = s;
        }
    }
    if (!single) {
        for (int h = tid; h < headsQ; h += kRvThreads) {
            const int qh = hkBegin * G + h;
            if (hkBegin + h / G >= a.Hkv || qh >= a.H) continue;
            float* ml = sp.partMl + ((static_cast<int64_t>(i) * sp.splits + split) * a.H + qh) * 2;
            ml[0] = sM[h];
            ml[1] = sL[h];
        }
    }
}

// Grouped-head variant (G query heads share one kv head, 2 <= G <= 16): the weighted sum becomes a small matrix
// product per kv head,  out^T[d, g] += V^T[d, t] . P^T[t, g],  on v_mfma_f32_16x16x32 (16 dims x 16 heads x 32 tokens),
// so the per-byte VALU cost no longer grows with G.
//   * a wave owns one kv head of one token range; it reads each V row segment (256 bytes) with 16 adjacent lanes, eight
//     16-byte loads per lane in flight, and parks the [32 tokens x 128 dims] block in a wave-private LDS tile;
//   * the A operand (8 tokens of one dim per lane) is gathered from the tile with 16-bit reads; the tile columns are
//     XOR-swizzled by (token / 8) in units of 16 dims so that the four k blocks of a wave hit disjoint LDS banks;
//   * the B operand (8 consecutive tokens of one query head per lane) is read straight from the logits tensor, which is
//     head-major, and exponentiated in registers: the softmax statistics of head g live in the lanes with l % 16 == g
//     and the running maximum / denominator / rescale never leave registers (two cross-lane exchanges per 32 tokens);
//   * every wave writes its own (max, denominator, accumulator) partial; softmaxReduceVMerge combines them.
constexpr int kVTileTokens = 32;
constexpr int kVTilePitch = kD + 8;  // elements; 272 bytes

template <typename T>
__global__ __launch_bounds__(kRvThreads) void softmaxReduceVMfma(T* __restrict__ out, const T* __restrict__ logits, const T* __restrict__ v, DecodeArgs a,
                                                                 SplitArgs sp, int HS) {
    using Ops = Mfma16<T>;
    using Frag = typename Ops::Frag;
    __shared__ __attribute__((aligned(16))) T tile[kRvWaves][kVTileTokens * kVTilePitch];
    const int i = blockIdx.y;
    int64_t L = loadIndex(a.bSeqLen, i, a.len64);
    if (L > a.maxInputLen) L = a.maxInputLen;
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int TPH = kRvWaves / HS;      // token ranges handled by this work-group
    const int hs = wave % HS;
    const int tph = wave / HS;
    const int hk = blockIdx.z * HS + hs;
    const int64_t split = static_cast<int64_t>(blockIdx.x) * TPH + tph;
    const int64_t t0 = split * sp.TT;
    if (hk >= a.Hkv || t0 >= L) return;  // no work-group barrier below: waves are independent
    const int64_t tEnd = (t0 + sp.TT < L) ? t0 + sp.TT : L;
    const int64_t start = loadIndex(a.bStartLoc, i, a.start64);
    const int64_t locBase = static_cast<int64_t>(i) * a.bLocStride + (a.maxInputLen - L);
    const int64_t rowStride = static_cast<int64_t>(a.Hkv) * kD;
    const int n = lane % 16;   // A: dim inside a 16-dim block; B and C: query head inside the group
    const int kq = lane / 16;  // k block: tokens 8*kq .. 8*kq+7 of the tile; loads: token inside a quad
    const int G = a.G;
    const bool headOk = n < G;
    const int qh = hk * G + n;
    const T* logitRow = logits + static_cast<int64_t>(headOk ? qh : hk * G) * a.logitCols;
    T* myTile = tile[wave];
    const T* vHead = v + hk * kD + n * 8;  // loads: lane n covers packet n of the 256-byte row segment

    f32x4 acc[kD / 16];
#pragma unroll
    for (int db = 0; db < kD / 16; ++db) acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    float mRun = -INFINITY, lRun = 0.f;

    // Software pipeline, two tiles deep: slot indices are fetched two tiles ahead, V rows and logits one tile ahead,
    // so that the dependent chain slot -> row address -> row never stalls the tile being multiplied.
    constexpr int NJ = kVTileTokens / 4;
    int64_t rowOff[NJ];
    auto fetchSlots = [&](int64_t ts) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            int64_t t = ts + 4 * j + kq;
            if (t > tEnd - 1) t = tEnd - 1;  // tail tokens alias the last valid one; their probability is zero
            int64_t slot = loadIndex(a.bLoc, locBase + t, a.loc64);
            slot = slot < 0 ? 0 : (slot >= a.numSlots ? a.numSlots - 1 : slot);
            rowOff[j] = slot * rowStride;
        }
    };
    auto fetchRows = [&](u32x4* dst) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) dst[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vHead + rowOff[j]));
    };
    auto fetchLogits = [&](int64_t ts, float* dst) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int64_t t = ts + 8 * kq + e;
            const int64_t col = start + t;
            dst[e] = -INFINITY;
            if (headOk && t < tEnd && col >= 0 && col < a.logitCols) dst[e] = static_cast<float>(logitRow[col]);
        }
    };
    u32x4 vv[NJ], vn[NJ];
    float x[8], xn[8];
    fetchSlots(t0);
    fetchRows(vv);
    fetchLogits(t0, x);
    if (t0 + kVTileTokens < tEnd) fetchSlots(t0 + kVTileTokens);

    for (int64_t ts = t0; ts < tEnd; ts += kVTileTokens) {
        if (ts + kVTileTokens < tEnd) {
            fetchRows(vn);
            fetchLogits(ts + kVTileTokens, xn);
            if (ts + 2 * kVTileTokens < tEnd) fetchSlots(ts + 2 * kVTileTokens);
        }
        float umax = -INFINITY;
#pragma unroll
        for (int e = 0; e < 8; ++e) umax = fmaxf(umax, x[e]);
        umax = fmaxf(umax, __shfl_xor(umax, 16, kWave));
        umax = fmaxf(umax, __shfl_xor(umax, 32, kWave));
        const float mNew = fmaxf(mRun, umax);
        const float alpha = (mRun == -INFINITY) ? 0.f : __expf(mRun - mNew);
        Frag pf;
        float psum = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float p = (x[e] == -INFINITY) ? 0.f : __expf(x[e] - mNew);
            psum += p;
            pf[e] = static_cast<T>(p);
        }
        lRun = lRun * alpha + psum;  // this lane's share; the four k blocks are added at the end
        mRun = mNew;
#pragma unroll
        for (int db = 0; db < kD / 16; ++db) {
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) acc[db][rr] *= alpha;
        }
        // ---- park the V block: row = token, 16-byte packet index XOR-ed with 2 * (token / 8) ----
#pragma unroll
        for (int j = 0; j < kVTileTokens / 4; ++j) {
            const int t = 4 * j + kq;
            *reinterpret_cast<u32x4*>(myTile + t * kVTilePitch + ((n ^ (((t >> 3) & 3) << 1)) * 8)) = vv[j];
        }
        __builtin_amdgcn_wave_barrier();
        // ---- out^T[16*db + m, g] += sum_t V[t, 16*db + m] * P[t, g] ----
#pragma unroll
        for (int db = 0; db < kD / 16; ++db) {
            Frag vf;
#pragma unroll
            for (int e = 0; e < 8; ++e) vf[e] = myTile[(8 * kq + e) * kVTilePitch + 16 * (db ^ kq) + n];
            acc[db] = Ops::mma(vf, pf, acc[db]);
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < NJ; ++j) vv[j] = vn[j];
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = xn[e];
    }

    // ---- this wave's partial: lane (n = head, kq) holds dims 16*db + 4*kq + rr ----
    lRun += __shfl_xor(lRun, 16, kWave);
    lRun += __shfl_xor(lRun, 32, kWave);
    if (!headOk) return;
    const bool single = L <= sp.TT;
    if (single) {
        const float inv = 1.0f / lRun;
        T* o = out + (static_cast<int64_t>(i) * a.H + qh) * kD;
#pragma unroll
        for (int db = 0; db < kD / 16; ++db) {
            T pk[4];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) pk[rr] = static_cast<T>(acc[db][rr] * inv);
            *reinterpret_cast<u32x2*>(o + 16 * db + 4 * kq) = *reinterpret_cast<const u32x2*>(pk);
        }
    } else {
        float* pa = sp.partAcc + ((static_cast<int64_t>(i) * sp.splits + split) * a.H + qh) * kD;
#pragma unroll
        for (int db = 0; db < kD / 16; ++db) *reinterpret_cast<f32x4*>(pa + 16 * db + 4 * kq) = acc[db];
        if (kq == 0) {
            float* ml = sp.partMl + ((static_cast<int64_t>(i) * sp.splits + split) * a.H + qh) * 2;
            ml[0] = mRun;
            ml[1] = lRun;
        }
    }
}

// out[i, h, :] = sum_j w_j acc_j / sum_j w_j l_j with w_j = exp(m_j - max_j m_j), over the ranges of sequence i.
template <typename T>
__global__ __launch_bounds__(kRvThreads) void softmaxReduceVMerge(T* __restrict__ out, DecodeArgs a, SplitArgs sp) {
    const int i = blockIdx.y;
    int64_t L = loadIndex(a.bSeqLen, i, a.len64);
    if (L > a.maxInputLen) L = a.maxInputLen;
    if (L <= sp.TT) return;  // finished by the split kernel (or empty)
    const int ns = static_cast<int>((L + sp.TT - 1) / sp.TT);
    const int idx = blockIdx.x * kRvThreads + threadIdx.x;
    if (idx >= a.H * a.D) return;
    const int qh = idx / a.D, d = idx % a.D;
    const float* ml = sp.partMl + (static_cast<int64_t>(i) * sp.splits * a.H + qh) * 2;
    const float* pa = sp.partAcc + (static_cast<int64_t>(i) * sp.splits * a.H + qh) * a.D + d;
    // ranges are visited in batches of 8 so that the loads of a batch are all in flight together
    constexpr int kBatch = 8;
    float m = -INFINITY;
    for (int j0 = 0; j0 < ns; j0 += kBatch) {
        float mj[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) mj[u] = (j0 + u < ns) ? ml[static_cast<int64_t>(j0 + u) * a.H * 2] : -INFINITY;
#pragma unroll
        for (int u = 0; u < kBatch; ++u) m = fmaxf(m, mj[u]);
    }
    float num = 0.f, den = 0.f;
    for (int j0 = 0; j0 < ns; j0 += kBatch) {
        float mj[kBatch], lj[kBatch], aj[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const bool ok = j0 + u < ns;
            mj[u] = ok ? ml[static_cast<int64_t>(j0 + u) * a.H * 2] : -INFINITY;
            lj[u] = ok ? ml[static_cast<int64_t>(j0 + u) * a.H * 2 + 1] : 0.f;
            aj[u] = ok ? pa[static_cast<int64_t>(j0 + u) * a.H * a.D] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const float w = (mj[u] == -INFINITY) ? 0.f : __expf(mj[u] - m);
            num += w * aj[u];
            den += w * lj[u];
        }
    }
    out[(static_cast<int64_t>(i) * a.H + qh) * a.D + d] = static_cast<T>(num / den);
}

// Any dtype / head size: one work-group per (sequence, query head); threads own output dims.
template <typename T, typename AccT>
__global__ __launch_bounds__(kRvThreads) void softmaxReduceVGeneric(T* __restrict__ out, const T* __restrict__ logits, const T* __restrict__ v, DecodeArgs a) {
    __shared__ AccT sRed[kRvThreads];
    const int i = blockIdx.y;
    const int qh = blockIdx.x;
    int64_t L = loadIndex(a.bSeqLen, i, a.len64);
    if (L > a.maxInputLen) L = a.maxInputLen;
    if (L <= 0) return;
    const int64_t start = loadIndex(a.bStartLoc, i, a.start64);
    const int64_t locBase = static_cast<int64_t>(i) * a.bLocStride + (a.maxInputLen - L);
    const T* row = logits + static_cast<int64_t>(qh) * a.logitCols;
    const int tid = threadIdx.x;
    auto logitAt = [&](int64_t t) -> AccT {
        const int64_t col = start + t;
        return (col >= 0 && col < a.logitCols) ? static_cast<AccT>(row[col]) : static_cast<AccT>(-INFINITY);
    };
    // maximum
    AccT m = static_cast<AccT>(-INFINITY);
    for (int64_t t = tid; t < L; t += kRvThreads) {
        const AccT x = logitAt(t);
        m = x > m ? x : m;
    }
    sRed[tid] = m;
    __syncthreads();
    for (int s = kRvThreads / 2; s > 0; s >>= 1) {
        if (tid < s) sRed[tid] = sRed[tid + s] > sRed[tid] ? sRed[tid + s] : sRed[tid];
        __syncthreads();
    }
    m = sRed[0];
    __syncthreads();
    // denominator
    AccT den = 0;
    for (int64_t t = tid; t < L; t += kRvThreads) {
        const AccT x = logitAt(t);
        den += (x == static_cast<AccT>(-INFINITY)) ? static_cast<AccT>(0) : static_cast<AccT>(exp(static_cast<double>(x - m)));
    }
    sRed[tid] = den;
    __syncthreads();
    for (int s = kRvThreads / 2; s > 0; s >>= 1) {
        if (tid < s) sRed[tid] += sRed[tid + s];
        __syncthreads();
    }
    den = sRed[0];
    // weighted sum, thread per output dim
    for (int d = tid; d < a.D; d += kRvThreads) {
        AccT acc = 0;
        for (int64_t t = 0; t < L; ++t) {
            int64_t slot = loadIndex(a.bLoc, locBase + t, a.loc64);
            slot = slot < 0 ? 0 : (slot >= a.numSlots ? a.numSlots - 1 : slot);
            const AccT x = logitAt(t);
            const AccT p = (x == static_cast<AccT>(-INFINITY)) ? static_cast<AccT>(0) : static_cast<AccT>(exp(static_cast<double>(x - m))) / den;
            // the reference rounds the probabilities to the element type before the product
            const AccT pr = static_cast<AccT>(static_cast<T>(p));
            acc += pr * static_cast<AccT>(v[(slot * a.Hkv + qh / a.G) * a.D + d]);
        }
        out[(static_cast<int64_t>(i) * a.H + qh) * a.D + d] = static_cast<T>(acc);
    }
}

int pow2Floor(int x) {
    int p = 1;
    while (p * 2 <= x) p *= 2;
    return p;
}

template <typename T>
diopiError_t launchSplit(diopiContextHandle_t ctx, hipStream_t stream, void* out, const void* logits, const void* v, const DecodeArgs& a) {
    SplitArgs sp;
    // Range length: the fp32 partial of a range (G*D*4 bytes per kv head) should stay near 1.5 % of the
    // V bytes the range streams (TT*D*2 per kv head)  =>  TT >= ~128*G; heads per group then chosen so
    // that a work-group streams roughly half a MiB.
    int TT = 128 * a.G;
    if (TT < 512) TT = 512;
    if (TT > 2048) TT = 2048;
    TT = envInt("DIOPI_ROCM_REDUCEV_TT", TT);
    TT = static_cast<int>(ceilDiv(TT, kSub)) * kSub;
    int HB = pow2Floor(static_cast<int>((512 * 1024) / (static_cast<int64_t>(TT) * kD * sizeof(T))));
    if (HB > 16) HB = 16;
    if (HB < 1) HB = 1;
    while (HB > 1 && HB * a.G > kMaxHeadsQ) HB /= 2;
    while (HB > 1 && HB > pow2Floor(a.Hkv) ) HB /= 2;
    HB = envInt("DIOPI_ROCM_REDUCEV_HB", HB);
    sp.TT = TT;
    sp.HB = HB;
    sp.splits = static_cast<int>(ceilDiv(a.maxInputLen, TT));
    sp.partAcc = nullptr;
    sp.partMl = nullptr;
    if (sp.splits > 1) {
        const int64_t accBytes = static_cast<int64_t>(a.batch) * sp.splits * a.H * kD * sizeof(float);
        const int64_t mlBytes = static_cast<int64_t>(a.batch) * sp.splits * a.H * 2 * sizeof(float);
        void* scratch = nullptr;
        ROCM_CALL(requireScratch(ctx, accBytes + mlBytes, &scratch));
        sp.partAcc = static_cast<float*>(scratch);
        sp.partMl = reinterpret_cast<float*>(static_cast<char*>(scratch) + accBytes);
    }
    const dim3 grid(static_cast<unsigned>(sp.splits), static_cast<unsigned>(a.batch), static_cast<unsigned>(ceilDiv(a.Hkv, HB)));
#define ROCM_RV_CASE(GC)                                                                                                                       \
    hipLaunchKernelGGL((softmaxReduceVSplit<T, GC>), grid, dim3(kRvThreads), 0, stream, static_cast<T*>(out), static_cast<const T*>(logits), \
                       static_cast<const T*>(v), a, sp)
    switch (a.G) {
        case 1: ROCM_RV_CASE(1); break;
        case 2: ROCM_RV_CASE(2); break;
        case 4: ROCM_RV_CASE(4); break;
        case 8: ROCM_RV_CASE(8); break;
        default: ROCM_CHECK(false, "unsupported group size %d in the split kernel", a.G);
    }
#undef ROCM_RV_CASE
    ROCM_LAUNCH_CHECK();
    if (sp.splits > 1) {
        const dim3 mgrid(static_cast<unsigned>(ceilDiv(static_cast<int64_t>(a.H) * a.D, kRvThreads)), static_cast<unsigned>(a.batch));
        hipLaunchKernelGGL(softmaxReduceVMerge<T>, mgrid, dim3(kRvThreads), 0, stream, static_cast<T*>(out), a, sp);
        ROCM_LAUNCH_CHECK();
    }
    return diopiSuccess;
}

template <typename T>
diopiError_t launchMfma(diopiContextHandle_t ctx, hipStream_t stream, void* out, const void* logits, const void* v, const DecodeArgs& a) {
    SplitArgs sp;
    // tokens per partial: the fp32 partial (G*D*4 bytes) against the V bytes it summarises (TT*D*2): about 1.5 % at TT = 128*G
    int TT = 128 * a.G;
    if (TT < 512) TT = 512;
    if (TT > 4096) TT = 4096;
    TT = envInt("DIOPI_ROCM_REDUCEV_TT", TT);
    TT = static_cast<int>(ceilDiv(TT, kVTileTokens)) * kVTileTokens;
    // one kv head per wave; with fewer than four kv heads the spare waves take further token ranges
    const int HS = a.Hkv >= 4 ? 4 : (a.Hkv >= 2 ? 2 : 1);
    const int TPH = kRvWaves / HS;
    sp.TT = TT;
    sp.HB = HS;
    sp.splits = static_cast<int>(ceilDiv(a.maxInputLen, TT));
    sp.partAcc = nullptr;
    sp.partMl = nullptr;
    if (sp.splits > 1) {
        const int64_t accBytes = static_cast<int64_t>(a.batch) * sp.splits * a.H * kD * sizeof(float);
        const int64_t mlBytes = static_cast<int64_t>(a.batch) * sp.splits * a.H * 2 * sizeof(float);
        void* scratch = nullptr;
        ROCM_CALL(requireScratch(ctx, accBytes + mlBytes, &scratch));
        sp.partAcc = static_cast<float*>(scratch);
        sp.partMl = reinterpret_cast<float*>(static_cast<char*>(scratch) + accBytes);
    }
    const dim3 grid(static_cast<unsigned>(ceilDiv(sp.splits, TPH)), static_cast<unsigned>(a.batch), static_cast<unsigned>(ceilDiv(a.Hkv, HS)));
    hipLaunchKernelGGL(softmaxReduceVMfma<T>, grid, dim3(kRvThreads), 0, stream, static_cast<T*>(out), static_cast<const T*>(logits),
                       static_cast<const T*>(v), a, sp, HS);
    ROCM_LAUNCH_CHECK();
    if (sp.splits > 1) {
        const dim3 mgrid(static_cast<unsigned>(ceilDiv(static_cast<int64_t>(a.H) * a.D, kRvThreads)), static_cast<unsigned>(a.batch));
        hipLaunchKernelGGL(softmaxReduceVMerge<T>, mgrid, dim3(kRvThreads), 0, stream, static_cast<T*>(out), a, sp);
        ROCM_LAUNCH_CHECK();
    }
    return diopiSuccess;
}

template <typename T, typename AccT>
diopiError_t launchGeneric(hipStream_t stream, void* out, const void* logits, const void* v, const DecodeArgs& a) {
    const dim3 grid(static_cast<unsigned>(a.H), static_cast<unsigned>(a.batch));
    hipLaunchKernelGGL((softmaxReduceVGeneric<T, AccT>), grid, dim3(kRvThreads), 0, stream, static_cast<T*>(out), static_cast<const T*>(logits),
                       static_cast<const T*>(v), a);
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

}  // namespace
}  // namespace rocm

extern "C" diopiError_t diopiTokenSoftmaxReduceVInference(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t logics,
                                                          diopiConstTensorHandle_t v, diopiConstTensorHandle_t b_loc, diopiConstTensorHandle_t b_start_loc,
                                                          diopiConstTensorHandle_t b_seq_len, int max_input_len, int other_kv_index) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    (void)other_kv_index;  // unused by the reference as well (functions_lightllm.cpp:82-107)
    TensorView vOut, vLogits, vV, vLoc, vStart, vLen;
    ROCM_CALL(unwrap(out, "out", &vOut));
    ROCM_CALL(unwrap(logics, "logics", &vLogits));
    ROCM_CALL(unwrap(v, "v", &vV));
    ROCM_CALL(unwrap(b_loc, "b_loc", &vLoc));
    ROCM_CALL(unwrap(b_start_loc, "b_start_loc", &vStart));
    ROCM_CALL(unwrap(b_seq_len, "b_seq_len", &vLen));
    DecodeArgs a;
    bool empty = false;
    ROCM_CALL(prepareDecode(vLogits, vOut, vV, vLoc, vStart, vLen, max_input_len, &a, &empty));
    if (empty) return diopiSuccess;

    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    const bool fast = a.D == kD && (a.G == 1 || a.G == 2 || a.G == 4 || a.G == 8) && (reinterpret_cast<uintptr_t>(vV.data) & 15) == 0 &&
                      envInt("DIOPI_ROCM_FORCE_GENERIC", 0) == 0;
    // The vector-ALU split kernel is instantiated for G in {1, 2, 4, 8}; other group sizes up to 16 (and any G at or
    // above DIOPI_ROCM_REDUCEV_MFMA_MIN_G) take the MFMA kernel.
    const int mfmaMinG = envInt("DIOPI_ROCM_REDUCEV_MFMA_MIN_G", 17);
    const bool mfma = a.D == kD && a.G <= 16 && (a.G >= mfmaMinG || !fast) && (reinterpret_cast<uintptr_t>(vV.data) & 15) == 0 &&
                      envInt("DIOPI_ROCM_FORCE_GENERIC", 0) == 0;
    switch (vOut.dtype) {
        case diopi_dtype_float16:
            if (mfma) return launchMfma<half_t>(ctx, stream, vOut.data, vLogits.data, vV.data, a);
            return fast ? launchSplit<half_t>(ctx, stream, vOut.data, vLogits.data, vV.data, a)
                        : launchGeneric<half_t, float>(stream, vOut.data, vLogits.data, vV.data, a);
        case diopi_dtype_bfloat16:
            if (mfma) return launchMfma<bf16_t>(ctx, stream, vOut.data, vLogits.data, vV.data, a);
            return fast ? launchSplit<bf16_t>(ctx, stream, vOut.data, vLogits.data, vV.data, a)
                        : launchGeneric<bf16_t, float>(stream, vOut.data, vLogits.data, vV.data, a);
        case diopi_dtype_float32: return launchGeneric<float, float>(stream, vOut.data, vLogits.data, vV.data, a);
        case diopi_dtype_float64: return launchGeneric<double, double>(stream, vOut.data, vLogits.data, vV.data, a);
        default: break;
    }
    setLastError("diopiTokenSoftmaxReduceVInference: dtype %s is not supported", dtypeName(vOut.dtype));
    return diopiDtypeNotSupported;
    ROCM_ENTRY_END
}
