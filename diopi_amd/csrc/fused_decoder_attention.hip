// diopiFusedDecoderAttentionInp for gfx950: one decode step of self-attention behind a single call, from the hidden
// states to the attention output, over a contiguous per-sequence KV cache.
//
// Interface: proto/include/diopi/functions_lmdeploy.h:104-135 of the reference.  The reference holds the prototype and
// five lines of prose, no implementation and no test; what the prose leaves open is decided here and listed below.
// For batch row b that is not finished, with L = sequence_lengths[b] tokens already cached:
//   1. qkv = T(inoutput[b, :] @ qkv_weight) + qkv_bias                  [(H + 2 Hkv) * D], fp32 accumulate
//   2. the first rot = rotary_embedding dims of q and k heads rotate at position step - 1 - total_padding_tokens[b] with the
//      half-split pairing of diopiRotaryEmbedding (dims j and j + rot/2, angle pos * rope_theta^(-2j/rot), formed in
//      double); the sums of 1 and the rotation are done in fp32 and rounded once to the element type
//   3. k and v go to key_cache / value_cache [layer_id, b, kv head, L % max_seq_len, :]
//   4. out[b, h, :] = sum_j p_j v_j over the last min(L + 1, max_seq_len) cached tokens (the new one included),
//      p_j = exp(s_j - max s) / (sum exp(s - max s) + 1e-6), s_j = (q_h . k_j) / sqrt(D), query head h reading kv head
//      h / (H / Hkv); fp32 scores and sums, probabilities rounded to the element type before the product with V
//   5. inoutput[b, 0 : H*D] = out[b] (H*D <= hidden_units; columns past H*D keep their values)
// Open in the prose, fixed here: the rotary pairing (2), a circular cache window once L reaches max_seq_len (3, 4),
// where the output lands when H*D < hidden_units (5), that finished rows are left untouched everywhere, and the caches'
// dimensions: the header writes [num_layer, batch, local_head_num, max_seq_len, size_per_head]; a cache holds kv heads, so
// dimension 2 is local_kv_head_num here, and dimension 1 may exceed this call's batch_size (an engine allocates for its
// largest batch): the layer stride is taken from the caches themselves.
//
// Four kernels for 16-bit tensors with heads of 128 (three plain ones further down for everything else), all on the
// context's stream:
//   fusedQkvPart     the projection, HBM-bound on the weights.  Its units (a 32-row step of the hidden dimension of one
//                    128-column head) go in equal runs to one work-group per compute unit: a compute unit draws a bounded
//                    share of the memory bandwidth, so all of them have to pull, whatever the number of heads.  The four
//                    waves of a work-group split a run's steps and each covers all 64 batch rows: a lane loads 8
//                    consecutive weight rows (16 bytes = 8 columns each); pairs of rows interleaved with two byte permutes
//                    become the B operands of v_mfma_f32_16x16x32 for the lane's 8 columns and serve four products (four
//                    blocks of 16 batch rows, whose A operands are 16 bytes of a hidden-state row each).  The waves meet
//                    in LDS (fp32, 132 KiB) and the work-group writes one fp32 partial tile per head its run touched.
//   fusedQkvFinish   adds the partial tiles of a head, rounds, adds the bias, rotates, and writes the head: q to the
//                    workspace, k and v straight into the cache.
//   fusedDecodeAttn  a work-group owns (batch row, kv head, range of 1024 cached tokens; the items longest first) and its four waves take the range's
//                    128-token chunks in turn, meeting only for a final hand-over in LDS; per 32 tokens 8 K loads that arrive in
//                    the B-operand layout of q.k^T (16 lanes x 16-byte pieces of 16 consecutive cache rows), online
//                    softmax on the 16 x 32 scores (row maxima and sums by DPP row reductions), probabilities through a
//                    wave-private LDS tile into the A-operand layout, 8 V loads permuted as above for P.V.  The scores
//                    never leave the chip: per cached token the kernel reads its K row and its V row and nothing else.
//   fusedDecodeMerge combines the ranges of a row (skipped when the window fits one range).
#include <diopi/functions_lmdeploy.h>

#include <algorithm>
#include <cmath>

#include "common.hpp"
#include "device.hpp"

namespace rocm {
namespace {

constexpr int kFD = 128;          // head size of the fast path
constexpr int kProjThreads = 256;
constexpr int kProjWaves = kProjThreads / kWave;  // each with its own steps of the hidden dimension
constexpr int kProjRB = 4;         // blocks of 16 batch rows per wave: all 64 rows of the work-group
constexpr int kProjDepth = 2;      // steps of a wave in flight
constexpr int kProjRows = 64;     // batch rows per work-group of the projection
constexpr int kProjPitch = kFD + 4;  // floats per row of a partial tile: rows 4 apart are 16 banks apart
constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = kAttnThreads / kWave;
constexpr int kAttnStep = 32;     // cached tokens per step of a wave
constexpr int kProbPitch = kAttnStep + 8;  // elements per row of the probability tile

struct FusedArgs {
    const void* finished;  // [B] one byte per row, or null
    const void* padding;   // [B] total_padding_tokens, or null
    const void* seqLen;    // [B] sequence_lengths
    bool pad64, len64;
    int B, hidden, H, Hkv, G;
    int64_t step;
    int maxSeq;
    int rot;               // rotating dims of a head: even, 0 .. head size
    float ropeTheta;
    int64_t layerOffset;   // elements from the start of a cache to the layer's [B, Hkv, maxSeq, D] block
};

__device__ __forceinline__ bool rowFinished(const FusedArgs& a, int b) {
    return a.finished != nullptr && reinterpret_cast<const unsigned char*>(a.finished)[b] != 0;
}
__device__ __forceinline__ int64_t rowLength(const FusedArgs& a, int b) {
    const int64_t L = loadIndex(a.seqLen, b, a.len64);
    return L < 0 ? 0 : L;
}

// The rotation angle of pair j of a head at position pos: pos * theta^(-2j/rot), formed in double so that positions in the
// hundreds of thousands keep their fraction of a turn (in fp32 the product alone is off by pos * 6e-8 radians).
__device__ __forceinline__ void rotaryAngle(const FusedArgs& a, int b, int j, float* sn, float* cs) {
    const int64_t pad = a.padding != nullptr ? loadIndex(a.padding, b, a.pad64) : 0;
    const double pos = static_cast<double>(a.step - 1 - pad);
    const double invFreq = exp2(-(2.0 * j / a.rot) * log2(static_cast<double>(a.ropeTheta)));
    double s, c;
    sincos(pos * invFreq, &s, &c);
    *sn = static_cast<float>(s);
    *cs = static_cast<float>(c);
}

// Finishes two elements of head `tile` of batch row b from the fp32 sums of the projection: rounding of the product, bias,
// rotation, and the store to where the head belongs (q to the workspace, k and v into the cache row of the new token).
// The 64 threads of a head: thread j < rot/2 takes the rotating pair (j, j + rot/2), the others two neighbours each of the
// dims past `rot`, which keep their values.
template <typename T>
__device__ __forceinline__ void finishPair(T* __restrict__ qOut, T* __restrict__ kCache, T* __restrict__ vCache, const T* __restrict__ bias, const FusedArgs& a,
                                           int tile, int b, int j, const float* __restrict__ sums, int parts, int64_t partStride) {
    const bool isQ = tile < a.H;
    const bool isK = !isQ && tile < a.H + a.Hkv;
    const int head = isQ ? tile : (isK ? tile - a.H : tile - a.H - a.Hkv);
    const int halfRot = a.rot / 2;
    const bool pair = j < halfRot;
    const int e0 = pair ? j : a.rot + 2 * (j - halfRot);
    const int e1 = pair ? j + halfRot : e0 + 1;
    float v0 = 0.f, v1 = 0.f;
    for (int p = 0; p < parts; ++p) {
        v0 += sums[p * partStride + e0];
        v1 += sums[p * partStride + e1];
    }
    // the product is rounded to the element type as a matrix product in that type would leave it
    float y0 = toFloat(fromFloat<T>(v0)), y1 = toFloat(fromFloat<T>(v1));
    if (bias != nullptr) {
        y0 += toFloat(bias[tile * kFD + e0]);
        y1 += toFloat(bias[tile * kFD + e1]);
    }
    if ((isQ || isK) && pair) {
        float sn, cs;
        rotaryAngle(a, b, j, &sn, &cs);
        const float o0 = y0 * cs - y1 * sn;
        const float o1 = y0 * sn + y1 * cs;
        y0 = o0;
        y1 = o1;
    }
    T* dst;
    if (isQ) {
        dst = qOut + (static_cast<int64_t>(b) * a.H + head) * kFD;
    } else {
        const int64_t slot = rowLength(a, b) % a.maxSeq;
        dst = (isK ? kCache : vCache) + a.layerOffset + ((static_cast<int64_t>(b) * a.Hkv + head) * a.maxSeq + slot) * kFD;
    }
    dst[e0] = fromFloat<T>(y0);
    dst[e1] = fromFloat<T>(y1);
}

// ---------------------------------------------------------------------------------------------------------------------
// How the projection is cut: a unit is one 32-row step of the hidden dimension of one 128-column head; the units, head
// after head, are dealt out in equal runs to as many work-groups as the device has compute units (a compute unit draws
// a bounded share of the memory bandwidth, so every one of them has to pull).  A run may end inside a head and go on in
// the next one: a work-group then writes one partial tile per head it touched, and a head gets its partial tiles from
// the work-groups first(t) .. last(t), in slots 0 .. last(t) - first(t).
struct ProjPlan {
    int tiles;         // heads of the projection: H + 2 Hkv
    int stepsPerTile;  // hidden / 32
    int unitsPerWg;
    int slots;         // partial tiles kept per head (the most any head gets)
};
__host__ __device__ __forceinline__ int projFirstWg(const ProjPlan& pl, int tile) { return tile * pl.stepsPerTile / pl.unitsPerWg; }
__host__ __device__ __forceinline__ int projLastWg(const ProjPlan& pl, int tile) { return ((tile + 1) * pl.stepsPerTile - 1) / pl.unitsPerWg; }

template <typename T>
__global__ __launch_bounds__(kProjThreads, 1) void fusedQkvPart(float* __restrict__ hiddenPart, const T* __restrict__ x, const T* __restrict__ w, FusedArgs a,
                                                               ProjPlan pl) {
    using Ops = Mfma16<T>;
    using Frag = typename Ops::Frag;
    extern __shared__ __attribute__((aligned(16))) float part[];  // [kProjWaves][64 rows][kProjPitch]
    const int rowBase = blockIdx.y * kProjRows;
    const int N = pl.tiles * kFD;
    const int lane = threadIdx.x % kWave;
    const int ks = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // this wave's share of a run's steps
    const int g4 = lane / 16;  // A, B: k slots 8 g4 .. + 7 of a 32-row step; C: rows 4 g4 .. + 3
    const int c = lane % 16;   // A: batch row of a block; loads: 16-byte packet (8 columns) of the panel; C: column
    const T* xRow[kProjRB];
#pragma unroll
    for (int rb = 0; rb < kProjRB; ++rb) {
        int row = rowBase + rb * 16 + c;
        row = row < a.B ? row : a.B - 1;
        xRow[rb] = x + static_cast<int64_t>(row) * a.hidden + 8 * g4;
    }
    struct Step {
        u32x4 w[8];
        u32x4 x[kProjRB];
    };
    const int units = pl.tiles * pl.stepsPerTile;
    const int uEnd = (blockIdx.x + 1) * pl.unitsPerWg < units ? (blockIdx.x + 1) * pl.unitsPerWg : units;
    for (int u = blockIdx.x * pl.unitsPerWg; u < uEnd;) {
        const int tile = u / pl.stepsPerTile;
        const int s0 = u % pl.stepsPerTile;
        const int n = pl.stepsPerTile - s0 < uEnd - u ? pl.stepsPerTile - s0 : uEnd - u;  // steps of this head in the run
        u += n;
        // the waves take consecutive quarters of the n steps; a wave without steps reads some valid step and adds zeros
        const int q = (n + kProjWaves - 1) / kProjWaves;
        int first = s0 + ks * q;
        const int steps = n - ks * q < 0 ? 0 : (n - ks * q < q ? n - ks * q : q);
        first = first < pl.stepsPerTile ? first : pl.stepsPerTile - 1;
        const T* wCol = w + static_cast<int64_t>(32 * first + 8 * g4) * N + tile * kFD + 8 * c;
        const int xOff = 32 * first;

        f32x4 acc[kProjRB][8];
#pragma unroll
        for (int rb = 0; rb < kProjRB; ++rb) {
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[rb][e] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        // every step issues the same loads (past the last step the last one again), so that the wait for one step's rows
        // leaves exactly the later steps' in flight
        auto issue = [&](int st, Step& r) {
            int sc = st < steps ? st : steps - 1;
            sc = sc < 0 ? 0 : sc;
#pragma unroll
            for (int i = 0; i < 8; ++i) r.w[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wCol + static_cast<int64_t>(32 * sc + i) * N));
#pragma unroll
            for (int rb = 0; rb < kProjRB; ++rb) r.x[rb] = *reinterpret_cast<const u32x4*>(xRow[rb] + xOff + 32 * sc);
        };
        // `live` is false for the steps past the last one (the ring is consumed in whole rounds): their products add zeros
        auto consume = [&](const Step& r, bool live) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                union {
                    u32x4 u;
                    Frag f;
                } lo, hi;
#pragma unroll
                for (int pr = 0; pr < 4; ++pr) {
                    // columns 2j and 2j+1 of this lane's packet, weight rows (2pr, 2pr+1) of the lane group
                    lo.u[pr] = __builtin_amdgcn_perm(r.w[2 * pr + 1][j], r.w[2 * pr][j], 0x05040100u);
                    hi.u[pr] = __builtin_amdgcn_perm(r.w[2 * pr + 1][j], r.w[2 * pr][j], 0x07060302u);
                }
#pragma unroll
                for (int rb = 0; rb < kProjRB; ++rb) {
                    union {
                        u32x4 u;
                        Frag f;
                    } pa;
                    pa.u = live ? r.x[rb] : u32x4{0u, 0u, 0u, 0u};
                    acc[rb][2 * j] = Ops::mma(pa.f, lo.f, acc[rb][2 * j]);
                    acc[rb][2 * j + 1] = Ops::mma(pa.f, hi.f, acc[rb][2 * j + 1]);
                }
            }
        };
        // The scheduling barriers keep the loads of the steps in step order, in the prologue as in the loop: a wait counts
        // in issue order, and the compiler's count at the loop head is the smaller of what the two ways into it allow.
        Step ring[kProjDepth];
#pragma unroll
        for (int d = 0; d < kProjDepth; ++d) {
            issue(d, ring[d]);
            __builtin_amdgcn_sched_barrier(0);
        }
        for (int st = 0; st < steps; st += kProjDepth) {
#pragma unroll
            for (int d = 0; d < kProjDepth; ++d) {
                consume(ring[d], st + d < steps);
                __builtin_amdgcn_sched_barrier(0);
                issue(st + d + kProjDepth, ring[d]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // acc[rb][e][r] is this wave's sum for batch row rb * 16 + 4 g4 + r, column 8c + e: every wave leaves its tile in LDS
        float* mine = part + (ks * kProjRows + 4 * g4) * kProjPitch + 8 * c;
#pragma unroll
        for (int rb = 0; rb < kProjRB; ++rb) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float* p = mine + (rb * 16 + r) * kProjPitch;
                *reinterpret_cast<f32x4*>(p) = f32x4{acc[rb][0][r], acc[rb][1][r], acc[rb][2][r], acc[rb][3][r]};
                *reinterpret_cast<f32x4*>(p + 4) = f32x4{acc[rb][4][r], acc[rb][5][r], acc[rb][6][r], acc[rb][7][r]};
            }
        }
        __syncthreads();
        // the head's partial tile of this work-group: 16-byte stores, a row of the tile is 512 consecutive bytes
        const int slot = static_cast<int>(blockIdx.x) - projFirstWg(pl, tile);
        float* dst = hiddenPart + (static_cast<int64_t>(slot) * a.B) * N + tile * kFD;
        for (int idx = threadIdx.x; idx < kProjRows * (kFD / 4); idx += kProjThreads) {
            const int r = idx / (kFD / 4), col = (idx % (kFD / 4)) * 4;
            if (rowBase + r >= a.B) continue;
            f32x4 v = *reinterpret_cast<const f32x4*>(part + r * kProjPitch + col);
#pragma unroll
            for (int k2 = 1; k2 < kProjWaves; ++k2) v += *reinterpret_cast<const f32x4*>(part + (k2 * kProjRows + r) * kProjPitch + col);
            *reinterpret_cast<f32x4*>(dst + static_cast<int64_t>(rowBase + r) * N + col) = v;
        }
        __syncthreads();  // the tile storage is free for the next head of the run
    }
}

// Adds the partial tiles of a head and finishes every pair: rounding, bias, rotation, and the stores of q, k and v.
template <typename T>
__global__ __launch_bounds__(256) void fusedQkvFinish(T* __restrict__ qOut, T* __restrict__ kCache, T* __restrict__ vCache, const float* __restrict__ hiddenPart,
                                                      const T* __restrict__ bias, FusedArgs a, ProjPlan pl) {
    const int tile = blockIdx.x;
    const int N = pl.tiles * kFD;
    const int parts = projLastWg(pl, tile) - projFirstWg(pl, tile) + 1;
    for (int idx = threadIdx.x; idx < 4 * (kFD / 2); idx += 256) {
        const int b = blockIdx.y * 4 + idx / (kFD / 2);
        const int j = idx % (kFD / 2);
        if (b >= a.B || rowFinished(a, b)) continue;
        finishPair<T>(qOut, kCache, vCache, bias, a, tile, b, j, hiddenPart + static_cast<int64_t>(b) * N + tile * kFD, parts, static_cast<int64_t>(a.B) * N);
    }
}

// ---------------------------------------------------------------------------------------------------------------------
struct AttnSplit {
    float* partAcc;  // [B, splits, H, D]
    float* partMl;   // [B, splits, H, 2]  (maximum, denominator)
    int splits;      // ranges per row the workspace is sized for
    int TT;          // cached tokens per range (a multiple of kAttnStep)
};

template <typename T>
__global__ __launch_bounds__(kAttnThreads, 2) void fusedDecodeAttn(T* __restrict__ out, const T* __restrict__ qIn, const T* __restrict__ kCache,
                                                                   const T* __restrict__ vCache, FusedArgs a, AttnSplit sp) {
    using Ops = Mfma16<T>;
    using Frag = typename Ops::Frag;
    __shared__ __attribute__((aligned(16))) T sP[kAttnWaves][16 * kProbPitch];
    // per wave and query head of the group: 128 sums, maximum, denominator; [kAttnWaves][G][kFD + 4] floats, sized by the launcher
    // (a fixed 16 heads would cost a group of one three quarters of the work-groups a compute unit can hold)
    extern __shared__ __attribute__((aligned(16))) float sMerge[];
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int hk = blockIdx.x;  // the kv head of this work-group
    // the (row, range) of this work-group: longest first when the items can be ranked (see itemOfRank), else as they come
    __shared__ int sItem;
    int b = static_cast<int>(blockIdx.y), split = static_cast<int>(blockIdx.z);
    if (a.B <= kRankedItems && a.B * sp.splits > 1) {  // at most 256 x 65535 items: no overflow
        if (wave == 0) {
            auto windowOf = [&](int row) {
                if (rowFinished(a, row)) return 0;
                const int64_t len = rowLength(a, row);
                return static_cast<int>(len + 1 < a.maxSeq ? len + 1 : a.maxSeq);
            };
            int picked;
            if (a.B * sp.splits <= kRankedItems) {
                picked = itemOfRank(split * a.B + b, a.B * sp.splits, sp.TT, [&](int j) {
                    const int rest = windowOf(j % a.B) - (j / a.B) * sp.TT;
                    return rest <= 0 ? 0 : (rest < sp.TT ? rest : sp.TT);
                });
            } else {
                picked = split * a.B + itemOfRank(b, a.B, a.maxSeq, windowOf);
            }
            if (threadIdx.x == 0) sItem = picked;
        }
        __syncthreads();
        b = sItem % a.B;
        split = sItem / a.B;
    }
    if (rowFinished(a, b)) return;
    const int64_t L = rowLength(a, b);
    const int nWin = static_cast<int>(L + 1 < a.maxSeq ? L + 1 : a.maxSeq);  // tokens in the window, the new one last
    const int t0 = split * sp.TT;
    if (t0 >= nWin) return;
    // The range of the work-group is cut into chunks of 128 tokens that its four waves take in turn (wave w the chunks
    // w, w + 4, ...): a (row, kv head) streams four times as fast as one wave would, and what leaves the work-group is one
    // result.  Local token i of a wave is token (4 * (i / 128) + w) * 128 + i % 128 of the range.
    constexpr int kChunk = 4 * kAttnStep;
    const int nTok = nWin - t0 < sp.TT ? nWin - t0 : sp.TT;  // tokens of the range
    const int nChunks = (nTok + kChunk - 1) / kChunk;
    const int myChunks = wave < nChunks ? (nChunks - wave + kAttnWaves - 1) / kAttnWaves : 0;
    int nSteps = 0;
    if (myChunks > 0) {
        const int lastStart = ((myChunks - 1) * kAttnWaves + wave) * kChunk;  // first token of this wave's last chunk
        const int lastTok = nTok - lastStart < kChunk ? nTok - lastStart : kChunk;
        nSteps = (myChunks - 1) * (kChunk / kAttnStep) + (lastTok + kAttnStep - 1) / kAttnStep;
    }
    const int firstPos = static_cast<int>((L + 1 - nWin) % a.maxSeq);  // cache row of the window's first token
    const int g4 = lane / 16;
    const int c = lane % 16;
    const int G = a.G;
    const int64_t headOff = a.layerOffset + (static_cast<int64_t>(b) * a.Hkv + hk) * a.maxSeq * kFD;
    const T* kHead = kCache + headOff + 8 * g4;  // + row * D + 32 s: 8 dims of k block g4
    const T* vHead = vCache + headOff + 8 * c;   // + row * D: packet c of a row
    T* tile = sP[wave];
    // token of the range behind local token i of this wave
    auto tokenOf = [&](int i) { return ((i / kChunk) * kAttnWaves + wave) * kChunk + i % kChunk; };
    // its cache row; tokens past the range repeat the range's last one (their scores become -inf)
    auto rowOf = [&](int i) {
        const int t = tokenOf(i);
        int p = firstPos + t0 + (t < nTok ? t : nTok - 1);
        p = p >= a.maxSeq ? p - a.maxSeq : p;
        return static_cast<int64_t>(p) * kFD;
    };
    // A fragments of q.k^T: row c is query head hk*G + c (zero beyond the group)
    Frag qa[kFD / 32];
#pragma unroll
    for (int s = 0; s < kFD / 32; ++s) {
        union {
            u32x4 raw;
            Frag f;
        } u;
        u.raw = u32x4{0u, 0u, 0u, 0u};
        if (c < G) u.raw = *reinterpret_cast<const u32x4*>(qIn + (static_cast<int64_t>(b) * a.H + hk * G + c) * kFD + 32 * s + 8 * g4);
        qa[s] = u.f;
    }
    u32x4 kb[2][kFD / 32], vb[8];
    auto issueK = [&](int st) {
#pragma unroll
        for (int tg = 0; tg < 2; ++tg) {
            const T* p = kHead + rowOf(kAttnStep * st + 16 * tg + c);
#pragma unroll
            for (int s = 0; s < kFD / 32; ++s) kb[tg][s] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p + 32 * s));
        }
    };
    auto issueV = [&](int st) {
#pragma unroll
        for (int r = 0; r < 8; ++r) vb[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vHead + rowOf(kAttnStep * st + 8 * g4 + r)));
    };
    // The scheduling barriers keep the requests in the order K, V, K, V ...: a wait for the K rows then leaves the V rows
    // in flight and the other way round (a wait is a count of younger requests).
    if (nSteps > 0) {  // a wave without chunks (a short range) only takes part in the hand-over below
        issueK(0);
        __builtin_amdgcn_sched_barrier(0);
        issueV(0);
        __builtin_amdgcn_sched_barrier(0);
    }

    f32x4 acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = f32x4{0.f, 0.f, 0.f, 0.f};
    float mRun[4], lRun[4];  // of query heads 4 g4 + r (the same in the 16 lanes of a row group)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        mRun[r] = -INFINITY;
        lRun[r] = 0.f;
    }
    const float scale = 1.0f / sqrtf(static_cast<float>(kFD));
    const bool rowLive = c < G;

    for (int st = 0; st < nSteps; ++st) {
        // ---- scores of 32 tokens: C holds query heads 4 g4 + r of token column c of each 16-token group
        f32x4 sc[2];
#pragma unroll
        for (int tg = 0; tg < 2; ++tg) {
            sc[tg] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < kFD / 32; ++s) {
                union {
                    u32x4 raw;
                    Frag f;
                } u;
                u.raw = kb[tg][s];
                sc[tg] = Ops::mma(qa[s], u.f, sc[tg]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        issueK(st + 1);  // the K registers are free: the next step's rows (past the range: its last row again)
        __builtin_amdgcn_sched_barrier(0);
        float alpha[4];
        bool moved = false;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const bool ok0 = tokenOf(kAttnStep * st + c) < nTok, ok1 = tokenOf(kAttnStep * st + 16 + c) < nTok;
            const float s0 = ok0 ? sc[0][r] * scale : -INFINITY;
            const float s1 = ok1 ? sc[1][r] * scale : -INFINITY;
            const float mNew = fmaxf(mRun[r], rowMax16(fmaxf(s0, s1)));  // finite: every step holds a token of the range
            const float p0 = __expf(s0 - mNew), p1 = __expf(s1 - mNew);
            alpha[r] = __expf(mRun[r] - mNew);  // 0 on the first step
            moved = moved || mNew != mRun[r];
            lRun[r] = lRun[r] * alpha[r] + rowSum16(p0 + p1);
            mRun[r] = mNew;
            tile[(4 * g4 + r) * kProbPitch + c] = static_cast<T>(p0);
            tile[(4 * g4 + r) * kProbPitch + 16 + c] = static_cast<T>(p1);
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        if (__any(moved)) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[e][r] *= alpha[r];
            }
        }
        // ---- P . V: A operand row c, tokens 8 g4 .. + 7; B operands from the lane's 8 V rows
        union {
            u32x4 u;
            Frag f;
        } pa;
        pa.u = *reinterpret_cast<const u32x4*>(tile + c * kProbPitch + 8 * g4);
        if (!rowLive) pa.u = u32x4{0u, 0u, 0u, 0u};
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            union {
                u32x4 u;
                Frag f;
            } lo, hi;
#pragma unroll
            for (int pr = 0; pr < 4; ++pr) {
                lo.u[pr] = __builtin_amdgcn_perm(vb[2 * pr + 1][j], vb[2 * pr][j], 0x05040100u);
                hi.u[pr] = __builtin_amdgcn_perm(vb[2 * pr + 1][j], vb[2 * pr][j], 0x07060302u);
            }
            acc[2 * j] = Ops::mma(pa.f, lo.f, acc[2 * j]);
            acc[2 * j + 1] = Ops::mma(pa.f, hi.f, acc[2 * j + 1]);
        }
        __builtin_amdgcn_sched_barrier(0);
        issueV(st + 1);
        __builtin_amdgcn_sched_barrier(0);
    }

    // ---- acc[e][r] is dim 8c + e of query head 4 g4 + r: the waves hand their (maximum, denominator, sums) over in LDS
    {
        float* mine = sMerge + wave * a.G * (kFD + 4);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int g = 4 * g4 + r;
            if (g < G) {
                *reinterpret_cast<f32x4*>(mine + g * (kFD + 4) + 8 * c) = f32x4{acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
                *reinterpret_cast<f32x4*>(mine + g * (kFD + 4) + 8 * c + 4) = f32x4{acc[4][r], acc[5][r], acc[6][r], acc[7][r]};
                if (c == 0) {
                    mine[g * (kFD + 4) + kFD] = mRun[r];
                    mine[g * (kFD + 4) + kFD + 1] = lRun[r];
                }
            }
        }
    }
    __syncthreads();
    const bool single = nWin <= sp.TT;
    for (int idx = threadIdx.x; idx < G * kFD; idx += kAttnThreads) {
        const int g = idx / kFD, d = idx % kFD;
        float mw[kAttnWaves];
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) {
            mw[w] = sMerge[(w * a.G + g) * (kFD + 4) + kFD];
            m = fmaxf(m, mw[w]);
        }
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) {
            const float wgt = (mw[w] == -INFINITY) ? 0.f : __expf(mw[w] - m);  // a wave without tokens weighs nothing
            num += wgt * sMerge[(w * a.G + g) * (kFD + 4) + d];
            den += wgt * sMerge[(w * a.G + g) * (kFD + 4) + kFD + 1];
        }
        const int qh = hk * G + g;
        if (single) {
            out[static_cast<int64_t>(b) * a.hidden + qh * kFD + d] = static_cast<T>(num / (den + 1e-6f));
        } else {
            const int64_t slot = (static_cast<int64_t>(b) * sp.splits + split) * a.H + qh;
            sp.partAcc[slot * kFD + d] = num;
            if (d == 0) {
                sp.partMl[slot * 2] = m;
                sp.partMl[slot * 2 + 1] = den;
            }
        }
    }
}

// out[b, h, :] = sum_j w_j acc_j / (sum_j w_j l_j + 1e-6), w_j = exp(m_j - max m), over the ranges of row b
template <typename T>
__global__ __launch_bounds__(256) void fusedDecodeMerge(T* __restrict__ out, FusedArgs a, AttnSplit sp) {
    const int b = blockIdx.y;
    if (rowFinished(a, b)) return;
    const int64_t L = rowLength(a, b);
    const int nWin = static_cast<int>(L + 1 < a.maxSeq ? L + 1 : a.maxSeq);
    if (nWin <= sp.TT) return;  // finished by the attention kernel
    const int ns = (nWin + sp.TT - 1) / sp.TT;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= a.H * kFD) return;
    const int qh = idx / kFD, d = idx % kFD;
    const float* ml = sp.partMl + (static_cast<int64_t>(b) * sp.splits * a.H + qh) * 2;
    const float* pa = sp.partAcc + (static_cast<int64_t>(b) * sp.splits * a.H + qh) * kFD + d;
    float m = -INFINITY;
    for (int j = 0; j < ns; ++j) m = fmaxf(m, ml[static_cast<int64_t>(j) * a.H * 2]);
    float num = 0.f, den = 0.f;
    for (int j = 0; j < ns; ++j) {
        const float wgt = __expf(ml[static_cast<int64_t>(j) * a.H * 2] - m);
        num += wgt * pa[static_cast<int64_t>(j) * a.H * kFD];
        den += wgt * ml[static_cast<int64_t>(j) * a.H * 2 + 1];
    }
    out[static_cast<int64_t>(b) * a.hidden + idx] = static_cast<T>(num / (den + 1e-6f));
}

// ---------------------------------------------------------------------------------------------------------------------
// The plain path: any of float32 / float16 / bfloat16, heads of up to kPlainMaxD dims, any even number of rotating dims, any
// grouping of query heads and any hidden size or alignment.  Three kernels with scalar accesses and fp32 arithmetic, the
// same five steps as above; what the fast path cannot take comes here, at a fraction of its speed.
constexpr int kPlainMaxD = 512;
constexpr int kPlainCols = 64;   // columns of the projection per work-group (one per lane of a wave)
constexpr int kPlainRows = 8;    // batch rows per work-group of the projection
constexpr int kPlainSplit = 4;   // waves of a work-group, each with every fourth row of the weights

// staged[b, c] = float(T(inoutput[b, :] . qkv_weight[:, c])) + bias[c]
template <typename T>
__global__ __launch_bounds__(kPlainCols * kPlainSplit) void plainQkv(float* __restrict__ staged, const T* __restrict__ x, const T* __restrict__ w,
                                                                    const T* __restrict__ bias, FusedArgs a, int N) {
    __shared__ float part[kPlainSplit][kPlainRows][kPlainCols];
    const int lane = threadIdx.x % kPlainCols, wave = threadIdx.x / kPlainCols;
    const int c = blockIdx.x * kPlainCols + lane;
    const int b0 = blockIdx.y * kPlainRows;
    const int rows = min(kPlainRows, a.B - b0);
    float acc[kPlainRows];
#pragma unroll
    for (int r = 0; r < kPlainRows; ++r) acc[r] = 0.f;
    if (c < N) {
        for (int h = wave; h < a.hidden; h += kPlainSplit) {
            const float wv = toFloat(w[static_cast<int64_t>(h) * N + c]);
#pragma unroll
            for (int r = 0; r < kPlainRows; ++r) {
                if (r < rows) acc[r] = fmaf(toFloat(x[static_cast<int64_t>(b0 + r) * a.hidden + h]), wv, acc[r]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < kPlainRows; ++r) part[wave][r][lane] = acc[r];
    __syncthreads();
    for (int r = wave; r < rows; r += kPlainSplit) {
        if (c >= N) continue;
        float sum = 0.f;
#pragma unroll
        for (int p = 0; p < kPlainSplit; ++p) sum += part[p][r][lane];
        float y = toFloat(fromFloat<T>(sum));
        if (bias != nullptr) y += toFloat(bias[c]);
        staged[static_cast<int64_t>(b0 + r) * N + c] = y;
    }
}

// Rotation and placement of one head of one batch row: q to the workspace, k and v into the cache row of the new token.
template <typename T>
__global__ __launch_bounds__(128) void plainFinish(T* __restrict__ qOut, T* __restrict__ kCache, T* __restrict__ vCache, const float* __restrict__ staged,
                                                  FusedArgs a, int D) {
    const int tile = blockIdx.x, b = blockIdx.y;
    if (rowFinished(a, b)) return;
    const bool isQ = tile < a.H;
    const bool isK = !isQ && tile < a.H + a.Hkv;
    const int head = isQ ? tile : (isK ? tile - a.H : tile - a.H - a.Hkv);
    const float* src = staged + (static_cast<int64_t>(b) * (a.H + 2 * a.Hkv) + tile) * D;
    T* dst;
    if (isQ) {
        dst = qOut + (static_cast<int64_t>(b) * a.H + head) * D;
    } else {
        const int64_t slot = rowLength(a, b) % a.maxSeq;
        dst = (isK ? kCache : vCache) + a.layerOffset + ((static_cast<int64_t>(b) * a.Hkv + head) * a.maxSeq + slot) * D;
    }
    const int halfRot = a.rot / 2;
    for (int j = threadIdx.x; j < D; j += blockDim.x) {
        float y = src[j];
        if ((isQ || isK) && j < a.rot) {
            const bool low = j < halfRot;
            float sn, cs;
            rotaryAngle(a, b, low ? j : j - halfRot, &sn, &cs);
            y = low ? y * cs - src[j + halfRot] * sn : src[j - halfRot] * sn + y * cs;
        }
        dst[j] = fromFloat<T>(y);
    }
}

// One wave per (query head, batch row): the lanes split the head's dims, the cached tokens of the window go by one at a
// time with a running maximum and denominator (fp32).
template <typename T>
__global__ __launch_bounds__(kWave) void plainDecodeAttn(T* __restrict__ out, const T* __restrict__ qIn, const T* __restrict__ kCache, const T* __restrict__ vCache,
                                                        FusedArgs a, int D) {
    constexpr int kPer = kPlainMaxD / kWave;
    const int h = blockIdx.x, b = blockIdx.y;
    if (rowFinished(a, b)) return;
    const int lane = threadIdx.x;
    const int64_t L = rowLength(a, b);
    const int64_t n = L + 1 < a.maxSeq ? L + 1 : a.maxSeq;
    const int64_t headOff = a.layerOffset + (static_cast<int64_t>(b) * a.Hkv + h / a.G) * a.maxSeq * D;
    const T* q = qIn + (static_cast<int64_t>(b) * a.H + h) * D;
    const float scale = 1.0f / sqrtf(static_cast<float>(D));
    float qv[kPer], acc[kPer];
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
        const int d = lane + kWave * i;
        qv[i] = d < D ? toFloat(q[d]) : 0.f;
        acc[i] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    for (int64_t t = 0; t < n; ++t) {
        const int64_t row = (L + 1 - n + t) % a.maxSeq;
        const T* kr = kCache + headOff + row * D;
        const T* vr = vCache + headOff + row * D;
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int d = lane + kWave * i;
            if (d < D) dot = fmaf(qv[i], toFloat(kr[d]), dot);
        }
        // the score as token attention leaves it: the dot product and its scaling each rounded to the element type
        const float sc = toFloat(fromFloat<T>(toFloat(fromFloat<T>(waveSum(dot))) * scale));
        const float mNew = fmaxf(m, sc);
        const float corr = expf(m - mNew);  // 0 at the first token
        const float p = expf(sc - mNew);
        l = l * corr + p;
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int d = lane + kWave * i;
            if (d < D) acc[i] = fmaf(p, toFloat(vr[d]), acc[i] * corr);
        }
        m = mNew;
    }
    const float inv = 1.0f / (l + 1e-6f);
    T* o = out + static_cast<int64_t>(b) * a.hidden + static_cast<int64_t>(h) * D;
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
        const int d = lane + kWave * i;
        if (d < D) o[d] = fromFloat<T>(acc[i] * inv);
    }
}

template <typename T>
diopiError_t launchPlain(hipStream_t stream, void* inout, const void* w, const void* bias, void* workspace, void* kCache, void* vCache, const FusedArgs& a, int D,
                         int64_t qBytes) {
    T* qBuf = static_cast<T*>(workspace);
    float* staged = reinterpret_cast<float*>(static_cast<char*>(workspace) + qBytes);
    const int tiles = a.H + 2 * a.Hkv;
    const int N = tiles * D;
    const dim3 pgrid(static_cast<unsigned>(ceilDiv(N, kPlainCols)), static_cast<unsigned>(ceilDiv(a.B, kPlainRows)));
    hipLaunchKernelGGL((plainQkv<T>), pgrid, dim3(kPlainCols * kPlainSplit), 0, stream, staged, static_cast<const T*>(inout), static_cast<const T*>(w),
                       static_cast<const T*>(bias), a, N);
    ROCM_LAUNCH_CHECK();
    hipLaunchKernelGGL((plainFinish<T>), dim3(static_cast<unsigned>(tiles), static_cast<unsigned>(a.B)), dim3(128), 0, stream, qBuf, static_cast<T*>(kCache),
                       static_cast<T*>(vCache), staged, a, D);
    ROCM_LAUNCH_CHECK();
    hipLaunchKernelGGL((plainDecodeAttn<T>), dim3(static_cast<unsigned>(a.H), static_cast<unsigned>(a.B)), dim3(kWave), 0, stream, static_cast<T*>(inout), qBuf,
                       static_cast<const T*>(kCache), static_cast<const T*>(vCache), a, D);
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

template <typename T>
diopiError_t launchFused(hipStream_t stream, void* inout, const void* w, const void* bias, void* workspace, void* kCache, void* vCache, const FusedArgs& a,
                         const AttnSplit& spIn, int64_t qBytes, const ProjPlan& pl) {
    T* qBuf = static_cast<T*>(workspace);
    AttnSplit sp = spIn;
    // the partial tiles of the projection share the storage of the attention partials: the attention kernel runs after the
    // finishing kernel has read them
    float* hiddenPart = reinterpret_cast<float*>(static_cast<char*>(workspace) + qBytes);
    sp.partAcc = hiddenPart;
    sp.partMl = sp.partAcc + static_cast<int64_t>(a.B) * sp.splits * a.H * kFD;
    const size_t projLds = static_cast<size_t>(kProjWaves) * kProjRows * kProjPitch * sizeof(float);
    ROCM_CALL(grantDynamicLds(reinterpret_cast<const void*>(fusedQkvPart<T>), static_cast<int>(projLds)));
    const int projWgs = static_cast<int>(ceilDiv(static_cast<int64_t>(pl.tiles) * pl.stepsPerTile, pl.unitsPerWg));
    const dim3 pgrid(static_cast<unsigned>(projWgs), static_cast<unsigned>(ceilDiv(a.B, kProjRows)));
    hipLaunchKernelGGL((fusedQkvPart<T>), pgrid, dim3(kProjThreads), projLds, stream, hiddenPart, static_cast<const T*>(inout), static_cast<const T*>(w), a, pl);
    ROCM_LAUNCH_CHECK();
    const dim3 fgrid(static_cast<unsigned>(pl.tiles), static_cast<unsigned>(ceilDiv(a.B, 4)));
    hipLaunchKernelGGL((fusedQkvFinish<T>), fgrid, dim3(256), 0, stream, qBuf, static_cast<T*>(kCache), static_cast<T*>(vCache), hiddenPart,
                       static_cast<const T*>(bias), a, pl);
    ROCM_LAUNCH_CHECK();
    const dim3 agrid(static_cast<unsigned>(a.Hkv), static_cast<unsigned>(a.B), static_cast<unsigned>(sp.splits));
    const size_t mergeLds = static_cast<size_t>(kAttnWaves) * a.G * (kFD + 4) * sizeof(float);
    hipLaunchKernelGGL((fusedDecodeAttn<T>), agrid, dim3(kAttnThreads), mergeLds, stream, static_cast<T*>(inout), qBuf, static_cast<const T*>(kCache),
                       static_cast<const T*>(vCache), a, sp);
    ROCM_LAUNCH_CHECK();
    if (sp.splits > 1) {
        const dim3 mgrid(static_cast<unsigned>(ceilDiv(static_cast<int64_t>(a.H) * kFD, 256)), static_cast<unsigned>(a.B));
        hipLaunchKernelGGL((fusedDecodeMerge<T>), mgrid, dim3(256), 0, stream, static_cast<T*>(inout), a, sp);
        ROCM_LAUNCH_CHECK();
    }
    return diopiSuccess;
}

diopiError_t fusedDecoderAttention(diopiContextHandle_t ctx, diopiTensorHandle_t inoutput, diopiConstTensorHandle_t qkv_weight, diopiConstTensorHandle_t qkv_bias,
                                   diopiTensorHandle_t workspace, int64_t* workspace_size, int64_t fusion_level, diopiTensorHandle_t key_cache,
                                   diopiTensorHandle_t value_cache, diopiConstTensorHandle_t finished, diopiConstTensorHandle_t total_padding_tokens,
                                   diopiConstTensorHandle_t sequence_lengths, int64_t step, int64_t layer_id, int64_t local_head_num,
                                   int64_t local_kv_head_num, int64_t size_per_head, int64_t max_seq_len, int64_t rotary_embedding, float rope_theta) {
    (void)fusion_level;  // every level gets the same kernels
    TensorView vX, vW, vB, vWs, vK, vV, vF, vP, vL;
    ROCM_CALL(unwrap(inoutput, "inoutput", &vX));
    ROCM_CALL(unwrap(qkv_weight, "qkv_weight", &vW));
    ROCM_CALL(unwrap(key_cache, "key_cache", &vK));
    ROCM_CALL(unwrap(value_cache, "value_cache", &vV));
    ROCM_CALL(unwrap(sequence_lengths, "sequence_lengths", &vL));
    ROCM_CALL(requireDeviceContiguous(vX, "inoutput"));
    ROCM_CALL(requireDeviceContiguous(vW, "qkv_weight"));
    ROCM_CALL(requireDeviceContiguous(vK, "key_cache"));
    ROCM_CALL(requireDeviceContiguous(vV, "value_cache"));
    ROCM_CALL(requireDeviceContiguous(vL, "sequence_lengths"));
    ROCM_CHECK(workspace_size != nullptr, "workspace_size must not be null");
    ROCM_CHECK(vX.ndim == 2, "inoutput must be [batch_size, hidden_units]");
    const int64_t B = vX.shape[0], hidden = vX.shape[1];
    const int64_t H = local_head_num, Hkv = local_kv_head_num, D = size_per_head;
    ROCM_CHECK(H > 0 && Hkv > 0 && H % Hkv == 0, "local_head_num %lld must be a positive multiple of local_kv_head_num %lld", static_cast<long long>(H),
               static_cast<long long>(Hkv));
    const int64_t N = (H + 2 * Hkv) * D;
    ROCM_CHECK(vW.ndim == 2 && vW.shape[0] == hidden && vW.shape[1] == N && vW.dtype == vX.dtype,
               "qkv_weight must be [hidden_units, (local_head_num + 2 local_kv_head_num) size_per_head] = [%lld, %lld] of dtype %s",
               static_cast<long long>(hidden), static_cast<long long>(N), dtypeName(vX.dtype));
    ROCM_CHECK(H * D <= hidden, "the attention output [local_head_num * size_per_head = %lld] does not fit hidden_units = %lld", static_cast<long long>(H * D),
               static_cast<long long>(hidden));
    ROCM_CHECK(max_seq_len > 0 && max_seq_len < (int64_t(1) << 31) / D, "max_seq_len %lld is out of range", static_cast<long long>(max_seq_len));
    // the caches may be allocated for more rows than this call's batch: the layer stride comes from their own batch dimension
    ROCM_CHECK(vK.ndim == 5 && vK.shape[1] >= B && vK.shape[2] == Hkv && vK.shape[3] == max_seq_len && vK.shape[4] == D && vK.dtype == vX.dtype,
               "key_cache must be [num_layer, batch >= batch_size, local_kv_head_num, max_seq_len, size_per_head] of dtype %s", dtypeName(vX.dtype));
    ROCM_CHECK(vV.sameShape(vK) && vV.dtype == vK.dtype, "value_cache must have the shape and dtype of key_cache");
    ROCM_CHECK(layer_id >= 0 && layer_id < vK.shape[0], "layer_id %lld is outside the %lld layers of the caches", static_cast<long long>(layer_id),
               static_cast<long long>(vK.shape[0]));
    ROCM_CHECK(isIndexDtype(vL.dtype) && vL.numel == B, "sequence_lengths must hold batch_size = %lld int32 or int64 values", static_cast<long long>(B));
    const void* biasPtr = nullptr;
    if (qkv_bias != nullptr) {
        ROCM_CALL(unwrap(qkv_bias, "qkv_bias", &vB));
        ROCM_CALL(requireDeviceContiguous(vB, "qkv_bias"));
        ROCM_CHECK(vB.numel == N && vB.dtype == vX.dtype, "qkv_bias must hold %lld elements of dtype %s", static_cast<long long>(N), dtypeName(vX.dtype));
        biasPtr = vB.data;
    }
    FusedArgs a;
    a.finished = nullptr;
    if (finished != nullptr) {
        ROCM_CALL(unwrap(finished, "finished", &vF));
        ROCM_CALL(requireDeviceContiguous(vF, "finished"));
        ROCM_CHECK(vF.numel == B && vF.itemsize() == 1, "finished must hold batch_size = %lld one-byte values", static_cast<long long>(B));
        a.finished = vF.data;
    }
    a.padding = nullptr;
    a.pad64 = false;
    if (total_padding_tokens != nullptr) {
        ROCM_CALL(unwrap(total_padding_tokens, "total_padding_tokens", &vP));
        ROCM_CALL(requireDeviceContiguous(vP, "total_padding_tokens"));
        ROCM_CHECK(isIndexDtype(vP.dtype) && vP.numel == B, "total_padding_tokens must hold batch_size = %lld int32 or int64 values", static_cast<long long>(B));
        a.padding = vP.data;
        a.pad64 = vP.dtype == diopi_dtype_int64;
    }
    ROCM_CHECK(vX.dtype == diopi_dtype_float16 || vX.dtype == diopi_dtype_bfloat16 || vX.dtype == diopi_dtype_float32,
               "inoutput must be float16, bfloat16 or float32, got %s", dtypeName(vX.dtype));
    ROCM_CHECK(D > 0 && D <= kPlainMaxD, "size_per_head %lld is outside 1..%d", static_cast<long long>(D), kPlainMaxD);
    ROCM_CHECK(rotary_embedding >= 0 && rotary_embedding <= D && rotary_embedding % 2 == 0, "rotary_embedding %lld must be even and within 0..size_per_head = %lld",
               static_cast<long long>(rotary_embedding), static_cast<long long>(D));
    ROCM_CHECK(B <= 65535 && H <= 65535, "batch %lld / local_head_num %lld exceed the launch limits", static_cast<long long>(B), static_cast<long long>(H));
    // the fast path: 16-bit elements, heads of 128, up to 16 query heads per kv head, a hidden size in whole 32-row steps for
    // each of a work-group's four waves, 16-byte aligned rows; everything else goes to the plain kernels
    const bool fast = (vX.dtype == diopi_dtype_float16 || vX.dtype == diopi_dtype_bfloat16) && D == kFD && H / Hkv <= 16 && hidden % 128 == 0 && hidden >= 256 &&
                      ((reinterpret_cast<uintptr_t>(vX.data) | reinterpret_cast<uintptr_t>(vW.data) | reinterpret_cast<uintptr_t>(vK.data) |
                        reinterpret_cast<uintptr_t>(vV.data)) & 15) == 0;
    // ranges of the attention kernel: 1024 cached tokens per work-group (its four waves share them), the workspace sized for
    // max_seq_len.  Measured at 64 rows of 512..2047 tokens, 32 kv heads, items taken longest first: 1024 tokens per range
    // 237-238 us per call in two harnesses, 512: 247-251, 2048 (no partials, no merge launch): 235 in one, 254 in the other
    AttnSplit sp;
    sp.TT = 1024;
    static_assert(1024 % kAttnStep == 0, "a range is a whole number of steps");
    sp.splits = static_cast<int>(ceilDiv(max_seq_len, sp.TT));
    sp.partAcc = nullptr;
    sp.partMl = nullptr;
    ROCM_CHECK(sp.splits <= 65535, "max_seq_len %lld exceeds the launch limits", static_cast<long long>(max_seq_len));
    const int64_t e = vX.itemsize();
    const int64_t qBytes = ceilDiv(B * H * D * e, 256) * 256;
    const int64_t attnBytes = sp.splits > 1 ? B * sp.splits * H * (D + 2) * static_cast<int64_t>(sizeof(float)) : 0;
    // the projection's units in equal runs over one work-group per compute unit (fewer when a run would leave a wave without
    // a step, or when several blocks of 64 batch rows multiply the work-groups)
    ProjPlan pl;
    pl.tiles = static_cast<int>(H + 2 * Hkv);
    pl.stepsPerTile = static_cast<int>(hidden / 32);
    pl.unitsPerWg = 1;
    pl.slots = 1;
    if (fast) {
        const int64_t units = static_cast<int64_t>(pl.tiles) * pl.stepsPerTile;
        const int64_t rowBlocks = ceilDiv(B > 0 ? B : 1, kProjRows);
        // when the heads are fewer than the compute units a head is cut into as many equal runs as fit (runs that end with
        // their head: 33.2 us at 96 heads x 4096 against 35.6 us for 256 runs that cross heads); otherwise equal runs
        int64_t wgs = std::max<int64_t>(1, deviceInfo().numCU / rowBlocks);
        if (pl.tiles <= wgs) wgs = pl.tiles * std::min<int64_t>(wgs / pl.tiles, ceilDiv(pl.stepsPerTile, kProjWaves));
        wgs = std::max<int64_t>(1, std::min<int64_t>(wgs, ceilDiv(units, kProjWaves)));
        pl.unitsPerWg = static_cast<int>(ceilDiv(units, wgs));
        if (pl.tiles <= wgs && pl.stepsPerTile % pl.unitsPerWg != 0 && pl.unitsPerWg < pl.stepsPerTile)
            pl.unitsPerWg = static_cast<int>(ceilDiv(pl.stepsPerTile, ceilDiv(pl.stepsPerTile, pl.unitsPerWg)));  // the same count of runs per head, evened out
        pl.slots = 1;
        for (int t = 0; t < pl.tiles; ++t) pl.slots = std::max(pl.slots, projLastWg(pl, t) - projFirstWg(pl, t) + 1);
    }
    const int64_t projBytes = static_cast<int64_t>(pl.slots) * B * N * static_cast<int64_t>(sizeof(float));
    const int64_t stagedBytes = B * N * static_cast<int64_t>(sizeof(float));  // the plain path's projection, fp32
    const int64_t need = qBytes + (fast ? (attnBytes > projBytes ? attnBytes : projBytes) : stagedBytes);
    if (*workspace_size < 0) {
        *workspace_size = need;  // size query: nothing else happens
        return diopiSuccess;
    }
    void* wsPtr = nullptr;
    if (workspace != nullptr) {
        ROCM_CALL(unwrap(workspace, "workspace", &vWs));
        ROCM_CALL(requireDeviceContiguous(vWs, "workspace"));
        ROCM_CHECK(vWs.nbytes() >= need && *workspace_size >= need, "workspace holds %lld bytes (workspace_size %lld), %lld are needed",
                   static_cast<long long>(vWs.nbytes()), static_cast<long long>(*workspace_size), static_cast<long long>(need));
        ROCM_CHECK((reinterpret_cast<uintptr_t>(vWs.data) & 15) == 0, "workspace must be 16-byte aligned");
        wsPtr = vWs.data;
    } else {
        ROCM_CALL(requireScratch(ctx, need, &wsPtr));  // a caller without a workspace tensor gets context scratch
    }
    if (B == 0) return diopiSuccess;
    a.seqLen = vL.data;
    a.len64 = vL.dtype == diopi_dtype_int64;
    a.B = static_cast<int>(B);
    a.hidden = static_cast<int>(hidden);
    a.H = static_cast<int>(H);
    a.Hkv = static_cast<int>(Hkv);
    a.G = static_cast<int>(H / Hkv);
    a.step = step;
    a.maxSeq = static_cast<int>(max_seq_len);
    a.rot = static_cast<int>(rotary_embedding);
    a.ropeTheta = rope_theta;
    a.layerOffset = layer_id * vK.shape[1] * Hkv * max_seq_len * D;
    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    if (!fast) {
        const int d = static_cast<int>(D);
        if (vX.dtype == diopi_dtype_float32) return launchPlain<float>(stream, vX.data, vW.data, biasPtr, wsPtr, vK.data, vV.data, a, d, qBytes);
        if (vX.dtype == diopi_dtype_float16) return launchPlain<half_t>(stream, vX.data, vW.data, biasPtr, wsPtr, vK.data, vV.data, a, d, qBytes);
        return launchPlain<bf16_t>(stream, vX.data, vW.data, biasPtr, wsPtr, vK.data, vV.data, a, d, qBytes);
    }
    if (vX.dtype == diopi_dtype_float16) return launchFused<half_t>(stream, vX.data, vW.data, biasPtr, wsPtr, vK.data, vV.data, a, sp, qBytes, pl);
    return launchFused<bf16_t>(stream, vX.data, vW.data, biasPtr, wsPtr, vK.data, vV.data, a, sp, qBytes, pl);
}

}  // namespace
}  // namespace rocm

extern "C" diopiError_t diopiFusedDecoderAttentionInp(diopiContextHandle_t ctx, diopiTensorHandle_t inoutput, diopiConstTensorHandle_t qkv_weight,
                                                      diopiConstTensorHandle_t qkv_bias, diopiTensorHandle_t workspace, int64_t* workspace_size,
                                                      int64_t fusion_level, diopiTensorHandle_t key_cache, diopiTensorHandle_t value_cache,
                                                      diopiConstTensorHandle_t finished, diopiConstTensorHandle_t total_padding_tokens,
                                                      diopiConstTensorHandle_t sequence_lengths, int64_t step, int64_t layer_id, int64_t local_head_num,
                                                      int64_t local_kv_head_num, int64_t size_per_head, int64_t max_seq_len, int64_t rotary_embedding,
                                                      float rope_theta) {
    ROCM_ENTRY_BEGIN
    return rocm::fusedDecoderAttention(ctx, inoutput, qkv_weight, qkv_bias, workspace, workspace_size, fusion_level, key_cache, value_cache, finished,
                                       total_padding_tokens, sequence_lengths, step, layer_id, local_head_num, local_kv_head_num, size_per_head, max_seq_len,
                                       rotary_embedding, rope_theta);
    ROCM_ENTRY_END
}
