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
// Kernel shape (16-bit types, D == 128, G <= 16): a split-K ("flash decoding") pass on the matrix cores followed
// by a small merge.  A work-group owns (kv head, token range, sequence); its four waves take the range's 128-token
// sub-tiles in turn, never meet at a barrier while they stream, and combine their (max, denominator, accumulator)
// triples in LDS at the end.  The range's triple goes to context-owned scratch and a merge kernel combines the
// ranges of a sequence; a sequence that fits one range is finished in place and skips the scratch round trip.
// V bytes are read exactly once.  Nothing on the host depends on the sequence lengths.
// Everything else (fp32 / fp64, other head sizes, G > 16) takes a shape-agnostic kernel.
#include <cmath>

#include "common.hpp"
#include "decode.hpp"
#include "device.hpp"

namespace rocm {
namespace {

constexpr int kRvThreads = 256;
constexpr int kRvWaves = kRvThreads / kWave;
constexpr int kSub = 128;          // tokens per sub-tile
constexpr int kD = 128;

struct SplitArgs {
    float* partAcc;  // [batch, splits, H, D]
    float* partMl;   // [batch, splits, H, 2]  (running max, denominator)
    int splits;      // ranges per sequence the scratch is sized for
    int TT;          // tokens per range (multiple of kSub)
};

// Matrix-core kernel (16-bit types, D == 128, any G <= 16): per kv head the weighted sum is the small product
//   out[g, d] += P[g, t] . V[t, d]      on v_mfma_f32_16x16x32 (16 query heads x 16 dims x 32 tokens),
// so the vector-ALU work per V byte does not grow with G.
// A wave works for the G query heads of its work-group's kv head and walks its share of the range (every fourth
// sub-tile of 128 tokens) without meeting another wave before the final hand-over:
//   * logits of the sub-tile: per query head two coalesced loads (lane = token), prefetched one sub-tile ahead
//     (tokens past the range alias its last one and become -inf by a select): no load sits inside a branch, so all of
//     them stay in flight until the next sub-tile's softmax;
//     running maximum / denominator per head are wave-uniform values (DPP row reduction + four lane reads);
//     the probabilities go to a wave-private LDS tile [G][128 + 8] in the element type;
//   * cache slots of the next sub-tile are fetched one sub-tile ahead and parked in wave-private LDS;
//   * V rows: the four 16-lane groups read the rows of 8 tokens each (one 16-byte load per lane and row, 8 rows in
//     flight per lane).  MFMA wants the contraction index (tokens) inside a lane's registers while a row is contiguous
//     along d; since 16-bit operands travel as pairs, interleaving the registers of rows (t, t+1) with two byte
//     permutes turns the 8 loaded rows into the B operands of the lane's 8 dims: 4 permutes per row, no LDS, no
//     second pass over the data.  The first rows of the next sub-tile are requested before its softmax work starts,
//     so the wave always has rows in flight;
//   * the A operand (8 consecutive tokens of query head l % 16) is one 16-byte read of the probability tile;
//   * C holds out[4 * (l / 16) + r][8 * (l % 16) + e] in acc[e][r]: a lane ends up with 8 consecutive dims of up to
//     four query heads; accumulator rows are rescaled only when some head's maximum moved (a wave-uniform test).
constexpr int kTilePitch = kSub + 8;  // elements per probability row; 272 bytes
constexpr int kMergePitch = kD + 4;   // floats per query head in the hand-over of a work-group's waves: 128 sums, maximum, denominator

// LDS that only one wave touches needs no barrier (the LDS executes a wave's operations in order), but the compiler
// must not move accesses of different types across the hand-over points.
__device__ __forceinline__ void waveLdsFence() {
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
}
__device__ __forceinline__ float laneValue(float v, int l) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
__device__ __forceinline__ float waveMaxUniform(float v) {
    v = rowMax16(v);
    return fmaxf(fmaxf(laneValue(v, 0), laneValue(v, 16)), fmaxf(laneValue(v, 32), laneValue(v, 48)));
}
__device__ __forceinline__ float waveSumUniform(float v) {
    v = rowSum16(v);
    return (laneValue(v, 0) + laneValue(v, 16)) + (laneValue(v, 32) + laneValue(v, 48));
}

// Which (sequence, range) is this work-group's?  The one whose token count has the rank of the work-group's index
// (y, then z: the order in which work-groups start), over all items when there are at most 256, else over the
// sequences of each range (a range's token counts fall with the sequence length like the lengths themselves);
// with more sequences than that the items are taken as they come, the sequence rotated by the range so that
// neighbouring work-groups mix ranges of different sequences.  Called by every thread of the work-group.
__device__ __forceinline__ void rankedItem(const DecodeArgs& a, const SplitArgs& sp, int waveId, int& i, int& zIdx) {
    __shared__ int sItem;
    const int nSeq = static_cast<int>(gridDim.y);
    const int nRanges = static_cast<int>(gridDim.z);
    i = static_cast<int>((blockIdx.y + blockIdx.z) % gridDim.y);
    zIdx = static_cast<int>(blockIdx.z);
    if (nSeq <= kRankedItems && nSeq * nRanges > 1) {  // at most 256 x 65535 items: no overflow
        if (waveId == 0) {
            auto lengthOf = [&](int seq) {
                const int64_t len = loadIndex(a.bSeqLen, seq, a.len64);
                return len > a.maxInputLen ? a.maxInputLen : (len < 0 ? int64_t{0} : len);
            };
            int picked;
            if (nSeq * nRanges <= kRankedItems) {
                picked = itemOfRank(static_cast<int>(blockIdx.z) * nSeq + static_cast<int>(blockIdx.y), nSeq * nRanges, sp.TT, [&](int j) {
                    const int64_t rest = lengthOf(j % nSeq) - static_cast<int64_t>(j / nSeq) * sp.TT;
                    return rest <= 0 ? 0 : (rest < sp.TT ? static_cast<int>(rest) : sp.TT);
                });
            } else {
                picked = static_cast<int>(blockIdx.z) * nSeq +
                         itemOfRank(static_cast<int>(blockIdx.y), nSeq, static_cast<int>(a.maxInputLen), [&](int j) { return static_cast<int>(lengthOf(j)); });
            }
            if (threadIdx.x == 0) sItem = picked;
        }
        __syncthreads();
        i = sItem % nSeq;
        zIdx = sItem / nSeq;
    }
}

template <typename T, int GC>
__global__ __launch_bounds__(kRvThreads, 2) void softmaxReduceVWave(T* __restrict__ out, const T* __restrict__ logits, const T* __restrict__ v, DecodeArgs a,
                                                                    SplitArgs sp) {
    using Ops = Mfma16<T>;
    using Frag = typename Ops::Frag;
    __shared__ __attribute__((aligned(16))) T sP[kRvWaves][GC * kTilePitch];
    __shared__ __attribute__((aligned(16))) int32_t sSlotW[kRvWaves][kSub];
    __shared__ __attribute__((aligned(16))) float sStat[kRvWaves][16];
    __shared__ __attribute__((aligned(16))) float sMerge[kRvWaves][GC][kMergePitch];  // per wave and query head: 128 sums, maximum, denominator

    // x runs over kv heads (neighbouring work-groups read neighbouring 256-byte pieces of the same cache rows at the same
    // time), y and z over the (sequence, range) items
    const int waveId = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    int i, zIdx;
    rankedItem(a, sp, waveId, i, zIdx);
    int64_t L = loadIndex(a.bSeqLen, i, a.len64);
    if (L > a.maxInputLen) L = a.maxInputLen;
    const int64_t t0 = static_cast<int64_t>(zIdx) * sp.TT;
    constexpr int HG = 1;  // kv heads per work-group (two and four side by side measured up to 8 % slower with grouped heads)
    const int phases = kRvWaves / HG;  // waves that share a kv head take the sub-tiles in turn
    const int hkRaw = blockIdx.x * HG + waveId % HG;
    const bool headLive = hkRaw < a.Hkv;
    const int hk = headLive ? hkRaw : a.Hkv - 1;  // a wave past the last kv head streams nothing and writes nothing
    const int phase = waveId / HG;
    if (t0 >= L) {
        // a sequence without tokens: the reference's product over an empty inner dimension gives zeros
        // (functions_lightllm.cpp:98-104); the work-groups of range 0 write them
        if (L <= 0 && zIdx == 0 && phase == 0 && headLive) {
            const int l = threadIdx.x % kWave;
            Pack16<T> z;
            z.raw = u32x4{0u, 0u, 0u, 0u};
            for (int g = l / 16; g < a.G; g += 4) storePack(out + (static_cast<int64_t>(i) * a.H + hk * a.G + g) * kD + (l % 16) * 8, z);
        }
        return;
    }
    // The range of the work-group, cut into sub-tiles of 128 tokens that the waves of a kv head take in turn (phase p the
    // sub-tiles p, p + phases, ...): several waves stream one (sequence, kv head, range) that many times as fast as one would,
    // and what leaves the work-group is one partial result per kv head.
    const int64_t tEnd = (t0 + sp.TT < L) ? t0 + sp.TT : L;
    const int nTokR = static_cast<int>(tEnd - t0);             // tokens of the work-group's range
    const int nSubAll = (nTokR + kSub - 1) / kSub;
    const int64_t start = loadIndex(a.bStartLoc, i, a.start64);
    const int64_t locBase = static_cast<int64_t>(i) * a.bLocStride + (a.maxInputLen - L) + t0;
    const int tid = threadIdx.x;
    const int lane = tid % kWave;
    const int wave = waveId;
    const int nSub = (headLive && phase < nSubAll) ? (nSubAll - phase + phases - 1) / phases : 0;  // sub-tiles of this wave
    auto subOff = [&](int sub) { return (sub * phases + phase) * kSub; };                           // first token of its sub-tile `sub`
    // lane group q takes tokens 8q .. 8q+7 of every 32-token step
    const int q = lane / 16;
    const int c = lane % 16;  // 16-byte packet of the row segment; also the row (query head) of the A operand
    const int G = a.G;
    const int R = G;          // query heads (rows of the A operand) of this wave, <= GC
    constexpr int kStep = 32;  // tokens per step
    const int64_t rowStride = static_cast<int64_t>(a.Hkv) * kD;
    T* tile = &sP[wave][0];
    int32_t* slotW = &sSlotW[wave][0];
    float* statW = &sStat[wave][0];
    const T* vHead = v + hk * kD + c * 8;
    const int64_t colBase = start + t0;
    // tokens of the range whose logits exist: the range may stick out of the logits columns only on invalid input
    int nLogit = 0;
    if (colBase >= 0 && colBase < a.logitCols) nLogit = (a.logitCols - colBase < nTokR) ? static_cast<int>(a.logitCols - colBase) : nTokR;
    // descriptor over the G logits rows of this kv head, from the first column of the range to the last valid one of
    // row G-1 (the launcher checks that this extent fits 31 bits); empty when no logit of the range exists
    const int xRowBytes = static_cast<int>(a.logitCols) * static_cast<int>(sizeof(T));
    const __amdgpu_buffer_rsrc_t xBuf = rawBuffer(uniformPointer(logits + static_cast<int64_t>(hk) * G * a.logitCols + colBase),
                                                  nLogit > 0 ? (R - 1) * xRowBytes + nLogit * static_cast<int>(sizeof(T)) : 0);

    // logits of sub-tile `sub`: xr[g][k] = logit of query head g, token 64k + lane (-inf outside the range).  Lanes
    // past the range re-read its last token (same cache line, nothing new is fetched) and select -inf; rows g >= R
    // re-read row 0 and are never looked at.  No condition guards a load: a guarded load is waited for on the spot,
    // an unguarded one stays in flight until the next sub-tile's softmax.
    float xr[GC][2];
    auto loadLogits = [&](int sub) {
#pragma unroll
        for (int g = 0; g < GC; ++g) {
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const int t = subOff(sub) + 64 * k + lane;
                const int tc = t < nLogit ? t : nLogit - 1;
                const unsigned short raw =
                    __builtin_amdgcn_raw_buffer_load_b16(xBuf, (g < R ? g : 0) * xRowBytes + tc * static_cast<int>(sizeof(T)), 0, 0);
                xr[g][k] = (t < nLogit) ? static_cast<float>(__builtin_bit_cast(T, raw)) : -INFINITY;
            }
        }
    };
    // Slot numbers of a sub-tile: requested as raw words through a descriptor over this range of b_loc (element j of a
    // 64-bit tensor is the word pair at byte 8j; for 32-bit storage the second read repeats the first) and only put
    // together, clamped and parked in LDS when the rows are about to be requested, so that the reads stay in flight
    // behind the logits instead of being waited for on the spot.
    const int locElem = a.loc64 ? 8 : 4;
    const __amdgpu_buffer_rsrc_t locBuf =
        rawBuffer(uniformPointer(reinterpret_cast<const char*>(a.bLoc) + locBase * locElem), nTokR * locElem);
    uint32_t slotLo[2], slotHi[2];
    auto loadSlots = [&](int sub) {
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            int t = subOff(sub) + 64 * k + lane;
            t = t < nTokR ? t : nTokR - 1;  // tokens past the end alias the last valid one (their probability is zero)
            slotLo[k] = __builtin_amdgcn_raw_buffer_load_b32(locBuf, t * locElem, 0, 0);
            slotHi[k] = __builtin_amdgcn_raw_buffer_load_b32(locBuf, t * locElem, a.loc64 ? 4 : 0, 0);
        }
    };
    auto storeSlots = [&]() {
        waveLdsFence();
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            int64_t slot = a.loc64 ? static_cast<int64_t>((static_cast<uint64_t>(slotHi[k]) << 32) | slotLo[k])
                                   : static_cast<int64_t>(static_cast<int32_t>(slotLo[k]));
            slot = slot < 0 ? 0 : (slot >= a.numSlots ? a.numSlots - 1 : slot);
            slotW[64 * k + lane] = static_cast<int32_t>(slot);
        }
        waveLdsFence();
    };
    // One set of 8 rows per lane, requested a step ahead; what hides the wait of a wave is the other waves of its SIMD, not a
    // second set in its own registers (two sets, requested two steps ahead, measured 0.8 % slower at 64 sequences of 512..2048
    // tokens and 0.4 % at 128 of 1024..8192 with grouped heads: fewer requests of a lane in flight stream faster here).
    u32x4 rowsV8[8];
    auto issueV = [&](int step, u32x4 (&rows)[8]) {
        const int first = 32 * step + 8 * q;
        const u32x4 s0 = *reinterpret_cast<const u32x4*>(slotW + first);
        const u32x4 s1 = *reinterpret_cast<const u32x4*>(slotW + first + 4);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            rows[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vHead + static_cast<int64_t>(static_cast<int32_t>(s0[r])) * rowStride));
            rows[4 + r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vHead + static_cast<int64_t>(static_cast<int32_t>(s1[r])) * rowStride));
        }
    };
    auto stepsOf = [&](int sub) {
        const int n = (nTokR - subOff(sub) < kSub) ? nTokR - subOff(sub) : kSub;
        return (n + kStep - 1) / kStep;
    };

    // the first logits are requested before the first rows: the softmax of sub-tile 0 then only waits for them, as
    // the softmax of every later sub-tile does, while rows are in flight
    if (nSub > 0) {  // a wave without sub-tiles (a short range) only takes part in the hand-over below
        loadSlots(0);
        loadLogits(0);
        storeSlots();
        issueV(0, rowsV8);
    }

    f32x4 acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = f32x4{0.f, 0.f, 0.f, 0.f};
    float mRun[GC], lRun[GC];  // wave-uniform
#pragma unroll
    for (int g = 0; g < GC; ++g) {
        mRun[g] = -INFINITY;
        lRun[g] = 0.f;
    }

    for (int sub = 0; sub < nSub; ++sub) {
        const int nTok = (nTokR - subOff(sub) < kSub) ? nTokR - subOff(sub) : kSub;
        const int nSteps = (nTok + kStep - 1) / kStep;
        // ---- softmax of the sub-tile ----
        waveLdsFence();
        bool moved = false;
#pragma unroll
        for (int g = 0; g < GC; ++g) {
            if (g < R) {
                const float mNew = fmaxf(mRun[g], waveMaxUniform(fmaxf(xr[g][0], xr[g][1])));
                const float mUse = (mNew == -INFINITY) ? 0.f : mNew;  // a head whose logits are all -inf keeps p = 0
                const float p0 = __expf(xr[g][0] - mUse);
                const float p1 = __expf(xr[g][1] - mUse);
                const float alpha = (mRun[g] == -INFINITY) ? 0.f : __expf(mRun[g] - mNew);
                moved = moved || (mNew != mRun[g]);
                lRun[g] = lRun[g] * alpha + waveSumUniform(p0 + p1);
                mRun[g] = mNew;
                tile[g * kTilePitch + lane] = static_cast<T>(p0);
                tile[g * kTilePitch + 64 + lane] = static_cast<T>(p1);
                if (lane == 0) statW[g] = alpha;
            }
        }
        // requested for every sub-tile, also the last one (nothing past the range is fetched: the reads alias the last
        // token), so that no load sits inside a branch
        loadLogits(sub + 1);
        loadSlots(sub + 1);
        waveLdsFence();
        if (moved) {
            const f32x4 al = *reinterpret_cast<const f32x4*>(statW + 4 * q);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] *= al;
        }
        // ---- P . V on the matrix cores ----
        // A operand: row c, the 8 tokens of this lane group's k slots; rows past the last query head are zeros
        const bool rowLive = c < G;
        const T* pRow = tile + (c < R ? c : 0) * kTilePitch + 8 * q;
        const int nStepsNext = (sub + 1 < nSub) ? stepsOf(sub + 1) : 0;
        auto pvStep = [&](int s, u32x4 (&rowsV)[8]) {
            union {
                u32x4 u;
                Frag f;
            } pa;
            pa.u = *reinterpret_cast<const u32x4*>(pRow + kStep * s);
            if (!rowLive) pa.u = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                union {
                    u32x4 u;
                    Frag f;
                } lo, hi;
#pragma unroll
                for (int pr = 0; pr < 4; ++pr) {
                    // dims 2j and 2j+1 of this lane's packet, tokens (2pr, 2pr+1) of the lane group
                    lo.u[pr] = __builtin_amdgcn_perm(rowsV[2 * pr + 1][j], rowsV[2 * pr][j], 0x05040100u);
                    hi.u[pr] = __builtin_amdgcn_perm(rowsV[2 * pr + 1][j], rowsV[2 * pr][j], 0x07060302u);
                }
                acc[2 * j] = Ops::mma(pa.f, lo.f, acc[2 * j]);
                acc[2 * j + 1] = Ops::mma(pa.f, hi.f, acc[2 * j + 1]);
            }
            // the row registers are free again: request the rows of the next step (of this sub-tile or of the next one,
            // whose slots take over the wave's LDS line once the last rows of this sub-tile are requested)
            if (s + 1 < nSteps) {
                issueV(s + 1, rowsV);
            } else if (s + 1 - nSteps < nStepsNext) {
                if (s + 1 == nSteps) storeSlots();
                issueV(s + 1 - nSteps, rowsV);
            }
        };
        for (int s = 0; s < nSteps; ++s) pvStep(s, rowsV8);
    }

    // ---- the waves of the work-group hand their (maximum, denominator, sums) over in LDS; all threads combine them ----
    {
        float* mine = &sMerge[wave][0][0];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int g = 4 * q + r;
            if (g < G) {
                *reinterpret_cast<f32x4*>(mine + g * kMergePitch + 8 * c) = f32x4{acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
                *reinterpret_cast<f32x4*>(mine + g * kMergePitch + 8 * c + 4) = f32x4{acc[4][r], acc[5][r], acc[6][r], acc[7][r]};
            }
        }
#pragma unroll
        for (int g = 0; g < GC; ++g) {
            if (lane == g && g < G) {
                mine[g * kMergePitch + kD] = mRun[g];
                mine[g * kMergePitch + kD + 1] = lRun[g];
            }
        }
    }
    __syncthreads();
    const bool single = L <= sp.TT;  // the whole sequence lives in this range
    for (int idx = tid; idx < HG * G * kD; idx += kRvThreads) {
        const int hl = idx / (G * kD);  // kv head of the work-group
        const int g = idx / kD % G, d = idx % kD;
        if (blockIdx.x * HG + hl >= a.Hkv) break;
        float mw[kRvWaves];
        float m = -INFINITY;
#pragma unroll
        for (int p = 0; p < kRvWaves; ++p) {
            mw[p] = p < phases ? sMerge[p * HG + hl][g][kD] : -INFINITY;
            m = fmaxf(m, mw[p]);
        }
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int p = 0; p < kRvWaves; ++p) {
            if (p < phases) {
                const float wgt = (mw[p] == -INFINITY) ? 0.f : __expf(mw[p] - m);  // a wave without tokens has maximum -inf and weighs nothing
                num += wgt * sMerge[p * HG + hl][g][d];
                den += wgt * sMerge[p * HG + hl][g][kD + 1];
            }
        }
        const int qh = (blockIdx.x * HG + hl) * G + g;
        if (single) {
            out[(static_cast<int64_t>(i) * a.H + qh) * kD + d] = static_cast<T>(num / den);
        } else {
            const int64_t slot = (static_cast<int64_t>(i) * sp.splits + zIdx) * a.H + qh;
            sp.partAcc[slot * kD + d] = num;
            if (d == 0) {
                sp.partMl[slot * 2] = m;
                sp.partMl[slot * 2 + 1] = den;
            }
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
    // One pass over the ranges, in batches of 8 whose loads are all in flight together (a sequence of up to 8 ranges costs
    // one memory round trip): the running maximum moves from batch to batch and the sums collected so far are rescaled.
    constexpr int kBatch = 8;
    float m = -INFINITY, num = 0.f, den = 0.f;
    for (int j0 = 0; j0 < ns; j0 += kBatch) {
        float mj[kBatch], lj[kBatch], aj[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const bool ok = j0 + u < ns;
            mj[u] = ok ? ml[static_cast<int64_t>(j0 + u) * a.H * 2] : -INFINITY;
            lj[u] = ok ? ml[static_cast<int64_t>(j0 + u) * a.H * 2 + 1] : 0.f;
            aj[u] = ok ? pa[static_cast<int64_t>(j0 + u) * a.H * a.D] : 0.f;
        }
        float mNew = m;
#pragma unroll
        for (int u = 0; u < kBatch; ++u) mNew = fmaxf(mNew, mj[u]);
        const float keep = (m == -INFINITY) ? 0.f : __expf(m - mNew);
        num *= keep;
        den *= keep;
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const float w = (mj[u] == -INFINITY) ? 0.f : __expf(mj[u] - mNew);
            num += w * aj[u];
            den += w * lj[u];
        }
        m = mNew;
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
    const int tid = threadIdx.x;
    if (L <= 0) {
        // no tokens: zeros, as the reference's product over an empty inner dimension (functions_lightllm.cpp:98-104)
        for (int d = tid; d < a.D; d += kRvThreads) out[(static_cast<int64_t>(i) * a.H + qh) * a.D + d] = static_cast<T>(0);
        return;
    }
    const int64_t start = loadIndex(a.bStartLoc, i, a.start64);
    const int64_t locBase = static_cast<int64_t>(i) * a.bLocStride + (a.maxInputLen - L);
    const T* row = logits + static_cast<int64_t>(qh) * a.logitCols;
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

template <typename T>
diopiError_t launchWave(diopiContextHandle_t ctx, hipStream_t stream, void* out, const void* logits, const void* v, const DecodeArgs& a) {
    SplitArgs sp;
    // tokens per work-group range.  What leaves a range is an fp32 partial of G*(D+2)*4 bytes per kv head, and those
    // writes are dear next to the row gather (8.5 MB of them cost 10 us of 111 at 64 sequences of 512..2048 tokens and
    // one query head per kv head; 19 MB cost 27 us of 236 at 128 sequences of 1024..8192 tokens and 8 query heads per
    // kv head): ranges are long, and the four waves of a work-group share one so that it still streams quickly.
    // Measured with the items taken longest first: ranges of 4096..6144 tokens 212-215 us at the second shape (8192: 218; 2048
    // and 3072, whose items are too many to be ranked together: 233 and 228), 2048 tokens 106 us at the first (1024: 111).
    int TT = 512 * a.G;
    if (TT < 2048) TT = 2048;
    if (TT > 8192) TT = 8192;
    TT = static_cast<int>(ceilDiv(TT, kSub)) * kSub;
    sp.TT = TT;
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
    ROCM_CHECK(a.batch <= 65535, "batch %d exceeds the launch limit of 65535 sequences", a.batch);
    ROCM_CHECK(sp.splits <= 65535, "max_input_len %d needs more than 65535 ranges of %d tokens", a.maxInputLen, TT);
    // kv heads per work-group: 1, 2 or 4 of the four waves' worth (the others are sub-tile phases of the same head); one
    // head per work-group measured best or equal at both shapes above (2 and 4 heads: up to 8 % slower with grouped heads)
    const int HG = 1;
    const dim3 grid(static_cast<unsigned>(ceilDiv(a.Hkv, HG)), static_cast<unsigned>(a.batch), static_cast<unsigned>(sp.splits));
#define ROCM_RVW_CASE(GC)                                                                                                                   \
    hipLaunchKernelGGL((softmaxReduceVWave<T, GC>), grid, dim3(kRvThreads), 0, stream, static_cast<T*>(out), static_cast<const T*>(logits), \
                       static_cast<const T*>(v), a, sp)
    if (a.G <= 1) {
        ROCM_RVW_CASE(1);
    } else if (a.G <= 2) {
        ROCM_RVW_CASE(2);
    } else if (a.G <= 4) {
        ROCM_RVW_CASE(4);
    } else if (a.G <= 8) {
        ROCM_RVW_CASE(8);
    } else {
        ROCM_RVW_CASE(16);
    }
#undef ROCM_RVW_CASE
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

namespace rocm {

diopiError_t tokenSoftmaxReduceV(diopiContextHandle_t ctx, const TensorView& vOut, const TensorView& vLogits, const TensorView& vV, const TensorView& vLoc,
                                 const TensorView& vStart, const TensorView& vLen, int max_input_len) {
    DecodeArgs a;
    bool empty = false;
    ROCM_CALL(prepareDecode(vLogits, vOut, vV, vLoc, vStart, vLen, max_input_len, &a, &empty));
    if (empty) return diopiSuccess;

    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    // the matrix-core kernel keeps slot numbers in 32 bits, reads V rows with 16-byte loads and addresses the G logits
    // rows of a kv head with a 32-bit byte offset
    const bool mfma = a.D == kD && a.G <= 16 && a.numSlots < (int64_t(1) << 31) && (reinterpret_cast<uintptr_t>(vV.data) & 15) == 0 &&
                      a.logitCols * 16 * 2 < (int64_t(1) << 31);
    switch (vOut.dtype) {
        case diopi_dtype_float16:
            return mfma ? launchWave<half_t>(ctx, stream, vOut.data, vLogits.data, vV.data, a)
                        : launchGeneric<half_t, float>(stream, vOut.data, vLogits.data, vV.data, a);
        case diopi_dtype_bfloat16:
            return mfma ? launchWave<bf16_t>(ctx, stream, vOut.data, vLogits.data, vV.data, a)
                        : launchGeneric<bf16_t, float>(stream, vOut.data, vLogits.data, vV.data, a);
        case diopi_dtype_float32: return launchGeneric<float, float>(stream, vOut.data, vLogits.data, vV.data, a);
        case diopi_dtype_float64: return launchGeneric<double, double>(stream, vOut.data, vLogits.data, vV.data, a);
        default: break;
    }
    setLastError("diopiTokenSoftmaxReduceVInference: dtype %s is not supported", dtypeName(vOut.dtype));
    return diopiDtypeNotSupported;
}

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
    return tokenSoftmaxReduceV(ctx, vOut, vLogits, vV, vLoc, vStart, vLen, max_input_len);
    ROCM_ENTRY_END
}
