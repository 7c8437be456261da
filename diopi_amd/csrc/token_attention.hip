// diopiTokenAttentionInference for gfx950: scaled q.k against every cached token of every sequence.
//
// Semantics: impl/torch/functions/functions_lightllm.cpp:53-80 of the reference (Python statement
// customized_test.py:698-713).  For sequence i with length L_i:
//   slots  = b_loc[i, max_input_len - L_i : max_input_len]           (right-aligned window)
//   out[h, b_start_loc[i] + t] = T( T(q[i,h,:] . k[slots[t], h/G, :]) / sqrt(D) )
// The dot product accumulates in fp32 and is rounded to the element type before the scaling, as
// the reference's matmul-then-divide does.  G = H / Hkv query heads share one kv head (the
// reference only has G = 1).  Columns of `out` outside every sequence are not written.
//
// Kernel shape (16-bit types, D in {64, 128}, G <= 16).  The contraction is tiny per byte of K
// (G dot products per 2*D bytes), so the kernel is an HBM stream of K rows; the arithmetic goes
// to one MFMA per 32 head-dim elements so that no VALU time is spent on conversions or
// cross-lane reductions:
//   v_mfma_f32_16x16x32: A = the G query heads of one kv head (rows >= G are zero) x 32 dims,
//                        B = 32 dims x 16 tokens, C = 16 heads x 16 tokens.
// Lane l of the wave supplies 8 consecutive head-dim elements (one 16-byte load straight from the
// token's cache row) for token l % 16 and dim block l / 16.  A wave keeps the A fragments of one
// kv head in registers and sweeps the token tile, with the slot indices of the tile prefetched
// into registers, so every K byte is loaded exactly once and never staged.
// Work-group = (token tile, sequence, kv-head group); tiles past the end of a sequence exit at once,
// so no host-side knowledge of the lengths (and no device-to-host copy) is needed.
#include <cmath>

#include "common.hpp"
#include "decode.hpp"
#include "device.hpp"

namespace rocm {
namespace {

constexpr int kAttThreads = 256;
constexpr int kAttWaves = kAttThreads / kWave;
constexpr int kTokGroup = 16;  // tokens per MFMA column block

template <typename T>
struct MfmaOps;

template <>
struct MfmaOps<half_t> {
    using Frag = f16x8;
    static __device__ __forceinline__ f32x4 mma(Frag a, Frag b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};
template <>
struct MfmaOps<bf16_t> {
    using Frag = bf16x8;
    static __device__ __forceinline__ f32x4 mma(Frag a, Frag b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};

template <typename Frag>
__device__ __forceinline__ Frag loadFrag(const void* p) {
    union {
        u32x4 raw;
        Frag f;
    } u;
    u.raw = *reinterpret_cast<const u32x4*>(p);
    return u.f;
}

template <typename Frag>
__device__ __forceinline__ Frag loadFragStream(const void* p) {
    union {
        u32x4 raw;
        Frag f;
    } u;
    u.raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return u.f;
}

template <typename Frag>
__device__ __forceinline__ Frag zeroFrag() {
    union {
        u32x4 raw;
        Frag f;
    } u;
    u.raw = u32x4{0u, 0u, 0u, 0u};
    return u.f;
}

// TT tokens per tile, HB kv heads per work-group, KSTEPS = D / 32.
template <typename T, int KSTEPS, int TT>
__global__ __launch_bounds__(kAttThreads) void tokenAttMfma(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k, DecodeArgs a, int HB,
                                                            float scale) {
    using Ops = MfmaOps<T>;
    using Frag = typename Ops::Frag;
    constexpr int kGroups = TT / kTokGroup;
    // x runs over head groups (neighbouring work-groups read neighbouring pieces of the same cache rows at the same
    // time), y over sequences, z over token tiles, with the sequence rotated by the tile index so that consecutive
    // work-groups (which the dispatcher deals round-robin to the 8 XCDs) mix tiles of different sequences: with
    // ragged lengths no XCD is left with only the sparsely populated late tiles
    const int i = static_cast<int>((blockIdx.y + blockIdx.z) % gridDim.y);
    int64_t L = loadIndex(a.bSeqLen, i, a.len64);
    if (L > a.maxInputLen) L = a.maxInputLen;
    const int64_t t0 = static_cast<int64_t>(blockIdx.z) * TT;
    if (t0 >= L) return;
    const int64_t start = loadIndex(a.bStartLoc, i, a.start64);
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int n = lane % 16;   // token column inside a group / query-head row of A
    const int kq = lane / 16;  // which 8-element block of a 32-wide k step
    const int D = KSTEPS * 32;
    const int64_t rowStride = static_cast<int64_t>(a.Hkv) * D;

    // slot of token (g*16 + n) of this tile, clamped so that every load stays inside the cache
    const int64_t locBase = static_cast<int64_t>(i) * a.bLocStride + (a.maxInputLen - L);
    int64_t slotOff[kGroups];
#pragma unroll
    for (int g = 0; g < kGroups; ++g) {
        int64_t t = t0 + g * kTokGroup + n;
        if (t > L - 1) t = L - 1;
        int64_t slot = loadIndex(a.bLoc, locBase + t, a.loc64);
        slot = slot < 0 ? 0 : (slot >= a.numSlots ? a.numSlots - 1 : slot);
        slotOff[g] = slot * rowStride;
    }

    const int hkBegin = blockIdx.x * HB;
    const int hkEnd = (hkBegin + HB < a.Hkv) ? hkBegin + HB : a.Hkv;
    for (int hk = hkBegin + wave; hk < hkEnd; hk += kAttWaves) {
        // A fragments: row n is query head hk*G + n (zero beyond the group)
        Frag qa[KSTEPS];
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            qa[s] = (n < a.G) ? loadFrag<Frag>(q + (static_cast<int64_t>(i) * a.H + hk * a.G + n) * D + s * 32 + kq * 8) : zeroFrag<Frag>();
        }
        const T* kHead = k + hk * D + kq * 8;
#pragma unroll
        for (int g0 = 0; g0 < kGroups; g0 += 4) {
            // 4 token groups x KSTEPS loads in flight
            Frag kb[4][KSTEPS];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (g0 + u < kGroups && t0 + (g0 + u) * kTokGroup < L) {
#pragma unroll
                    for (int s = 0; s < KSTEPS; ++s) kb[u][s] = loadFragStream<Frag>(kHead + slotOff[g0 + u] + s * 32);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (g0 + u < kGroups && t0 + (g0 + u) * kTokGroup < L) {
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < KSTEPS; ++s) acc = Ops::mma(qa[s], kb[u][s], acc);
                    // C: lane holds rows 4*kq + r (query head inside the group) of column n (token)
                    const int64_t t = t0 + (g0 + u) * kTokGroup + n;
                    const int64_t col = start + t;
                    if (t < L && col >= 0 && col < a.logitCols) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int gh = 4 * kq + r;
                            if (gh < a.G) {
                                const T dot = static_cast<T>(acc[r]);
                                out[static_cast<int64_t>(hk * a.G + gh) * a.logitCols + col] = static_cast<T>(static_cast<float>(dot) * scale);
                            }
                        }
                    }
                }
            }
        }
    }
}

// LDS-staged variant for D == 128.  The direct kernel above asks the memory pipeline for 16 different
// cache rows per load instruction (64 bytes of each); this one loads the way the cache is laid out
// and lets LDS do the re-shaping:
//   * 16 consecutive lanes read one head row (256 contiguous bytes) of one token; a wave owns HW
//     adjacent kv heads, so it reads HW*256 contiguous bytes per token and the waves of a work-group
//     cover adjacent head ranges of the same tokens;
//   * the loads a lane issues per unit (TU = UNIT/HW tokens x HW heads: 16 loads for UNIT = 64, 4 for UNIT = 16; the launcher
//     says which) are all in flight before the first use; each [16 tokens x 128 dims] block then goes through a wave-private LDS tile
//     (row pitch 272 bytes: conflict-free for both the 16-byte row writes and the 16-byte
//     column-block reads) and comes back in the MFMA B-operand layout;
//   * LDS operations of one wave execute in order, so the private tile needs no barrier;
//   * the scores of the whole tile wait in LDS, one line per query head, and the work-group writes them out at the end
//     in 16-byte packets along the token axis (the MFMA result layout would send every wave store to two or four
//     far-apart 32-byte pieces of the logits).
// Waves are mapped to (head slot, token phase): with few kv heads the spare waves take other units.
// What bounds this kernel when several query heads share a kv head is the logits themselves: on 128 sequences of
// 1024..8192 tokens, 8 kv heads and 8 query heads each, the rows alone stream in 176 us, and the 6 % of the bytes
// that are logits add 60..75 us whatever their layout, cache policy or place in the instruction stream (a copy of this
// kernel's access pattern without arithmetic shows the same).
constexpr int kStagePitch = 136;  // elements per staged row: 128 + 8

template <typename T, int HW, int UNIT>
__global__ __launch_bounds__(kAttThreads) void tokenAttStaged(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k, DecodeArgs a, int TT,
                                                              int HS, float scale, int order) {
    using Ops = MfmaOps<T>;
    using Frag = typename Ops::Frag;
    constexpr int D = 128;
    constexpr int KSTEPS = D / 32;
    constexpr int TU = UNIT / HW;  // tokens per unit
    constexpr int NJ = TU / 4;    // loads per head per lane in a unit (4 tokens per load instruction)
    constexpr int NG = TU / 16;   // MFMA column groups per unit
    __shared__ __attribute__((aligned(16))) T stage[kAttWaves][16 * kStagePitch];
    __shared__ int sSlot[1024];   // slot index of every token of the tile (TT <= 1024)
    extern __shared__ __attribute__((aligned(16))) unsigned char dynLds[];  // scores of the tile: HS*HW*G rows of TT + 8

    // x runs over head groups (neighbouring work-groups read neighbouring pieces of the same cache rows at the same
    // time); the launcher says how y and z map to (sequence, token tile)
    int i, tileIdx;
    if (order == 1) {  // y = tile, z = sequence: the tiles of a sequence one after the other
        i = static_cast<int>(blockIdx.z);
        tileIdx = static_cast<int>(blockIdx.y);
    } else {  // y = sequence, z = tile, the sequence rotated by the tile index: consecutive work-groups mix tiles of different sequences
        i = static_cast<int>((blockIdx.y + blockIdx.z) % gridDim.y);
        tileIdx = static_cast<int>(blockIdx.z);
    }
    int64_t L = loadIndex(a.bSeqLen, i, a.len64);
    if (L > a.maxInputLen) L = a.maxInputLen;
    const int64_t t0 = static_cast<int64_t>(tileIdx) * TT;
    if (t0 >= L) return;
    const int nTok = static_cast<int>((L - t0 < TT) ? L - t0 : TT);
    const int64_t start = loadIndex(a.bStartLoc, i, a.start64);
    const int64_t locBase = static_cast<int64_t>(i) * a.bLocStride + (a.maxInputLen - L) + t0;
    for (int t = threadIdx.x; t < TT; t += kAttThreads) {
        const int tc = t < nTok ? t : nTok - 1;  // tail tokens alias the last valid one; their results are not stored
        int64_t slot = loadIndex(a.bLoc, locBase + tc, a.loc64);
        slot = slot < 0 ? 0 : (slot >= a.numSlots ? a.numSlots - 1 : slot);
        sSlot[t] = static_cast<int>(slot);
    }
    __syncthreads();

    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int r = lane / 16;  // loads: token inside a quad; MFMA: k block (kq)
    const int c = lane % 16;  // loads: 16-byte packet of the head row; MFMA: token column / query-head row (n)
    const int TPH = kAttWaves / HS;
    const int hs = wave % HS;
    const int tph = wave / HS;
    const int hkGroup = blockIdx.x * HS * HW;  // first kv head of the work-group
    const int hk0 = hkGroup + hs * HW;
    const int64_t rowStride = static_cast<int64_t>(a.Hkv) * D;
    T* myStage = stage[wave];

    // The scores of the tile are collected in LDS, one row per query head, and written out afterwards in 16-byte
    // packets along the token axis: the MFMA result layout would send every wave store to two or four far-apart
    // 32-byte pieces.  Element t of local row j sits at sOut[j * outPitch + mis(j) + t], where mis(j) is the offset
    // of the row's first logits element inside its 16-byte packet in global memory, so that packets of the LDS row
    // and packets of the logits row coincide.
    T* sOut = reinterpret_cast<T*>(dynLds);
    const int outPitch = TT + 8;  // (TT + 8) / 2 banks: 4 rows apart is 16 banks apart for TT a multiple of 64
    const int64_t col0 = start + t0;
    const int64_t elem0 = static_cast<int64_t>(reinterpret_cast<uintptr_t>(out) / sizeof(T)) + col0;

    if (hk0 < a.Hkv) {
        // A fragments of this wave's heads: row c is query head (hk0+u)*G + c, k slot (r, e) <-> dim 32*s + 8*r + e
        Frag qa[HW][KSTEPS];
#pragma unroll
        for (int u = 0; u < HW; ++u) {
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) {
                const bool valid = c < a.G && hk0 + u < a.Hkv;
                qa[u][s] = valid ? loadFrag<Frag>(q + (static_cast<int64_t>(i) * a.H + (hk0 + u) * a.G + c) * D + s * 32 + r * 8) : zeroFrag<Frag>();
            }
        }
        // where this lane's four result rows (query heads 4*r + rr of head u) start in sOut
        int outBase[HW][4];
#pragma unroll
        for (int u = 0; u < HW; ++u) {
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const int j = (hs * HW + u) * a.G + 4 * r + rr;
                const int64_t hq = static_cast<int64_t>(hk0 + u) * a.G + 4 * r + rr;
                outBase[u][rr] = j * outPitch + static_cast<int>((elem0 + hq * a.logitCols) & 7);
            }
        }

        const int numUnits = (nTok + TU - 1) / TU;
        for (int unit = tph; unit < numUnits; unit += TPH) {
            const int tu0 = unit * TU;
            // every load of the unit is issued before the first use
            u32x4 kv[NJ][HW];
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int64_t rowOff = static_cast<int64_t>(sSlot[tu0 + 4 * j + r]) * rowStride;
#pragma unroll
                for (int u = 0; u < HW; ++u) {
                    const int hk = (hk0 + u < a.Hkv) ? hk0 + u : a.Hkv - 1;
                    kv[j][u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(k + rowOff + hk * D + c * 8));
                }
            }
#pragma unroll
            for (int u = 0; u < HW; ++u) {
#pragma unroll
                for (int g = 0; g < NG; ++g) {
                    // 16 tokens x 128 dims of head u: rows 4*jj + r of the private tile
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) *reinterpret_cast<u32x4*>(myStage + (4 * jj + r) * kStagePitch + c * 8) = kv[4 * g + jj][u];
                    __builtin_amdgcn_wave_barrier();  // keep the tile writes ahead of the reads in program order
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < KSTEPS; ++s) {
                        const Frag kb = loadFrag<Frag>(myStage + c * kStagePitch + s * 32 + r * 8);
                        acc = Ops::mma(qa[u][s], kb, acc);
                    }
                    __builtin_amdgcn_wave_barrier();  // ... and the reads ahead of the next tile's writes
                    // C: this lane holds query heads 4*r + rr of token column c
                    const int t = tu0 + g * 16 + c;
                    if (hk0 + u < a.Hkv) {
#pragma unroll
                        for (int rr = 0; rr < 4; ++rr) {
                            if (4 * r + rr < a.G) {
                                const T dot = static_cast<T>(acc[rr]);
                                sOut[outBase[u][rr] + t] = static_cast<T>(static_cast<float>(dot) * scale);
                            }
                        }
                    }
                }
            }
        }
    }
    __syncthreads();

    // write-out: local row j is query head hkGroup*G + j; columns outside the logits tensor are dropped
    const int rowsHere = ((hkGroup + HS * HW < a.Hkv) ? HS * HW : a.Hkv - hkGroup) * a.G;
    int tLo = 0, tHi = nTok;
    if (col0 < 0) tLo = static_cast<int>(-col0 < nTok ? -col0 : nTok);
    if (col0 + nTok > a.logitCols) tHi = static_cast<int>(a.logitCols - col0 > 0 ? a.logitCols - col0 : 0);
    const int packets = (TT + 8) / 8;
    for (int item = threadIdx.x; item < rowsHere * packets; item += kAttThreads) {
        const int j = item / packets;
        const int p = item - j * packets;
        const int64_t rowElem = (static_cast<int64_t>(hkGroup) * a.G + j) * a.logitCols + col0;  // of token 0 of the tile
        const int mis = static_cast<int>((elem0 + (static_cast<int64_t>(hkGroup) * a.G + j) * a.logitCols) & 7);
        const int tFirst = 8 * p - mis;  // token of the packet's first element
        if (tFirst + 8 <= tLo || tFirst >= tHi) continue;
        const T* src = sOut + j * outPitch + 8 * p;
        T* dst = out + rowElem + tFirst;
        if (tFirst >= tLo && tFirst + 8 <= tHi) {
            *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(src);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                if (tFirst + e >= tLo && tFirst + e < tHi) dst[e] = src[e];
            }
        }
    }
}

// Any dtype / head size / grouping: one thread per (token, query head) pair of a tile.
template <typename T, typename AccT>
__global__ __launch_bounds__(kAttThreads) void tokenAttGeneric(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k, DecodeArgs a, int TT,
                                                               AccT scale) {
    // x runs over head groups (neighbouring work-groups read neighbouring pieces of the same cache rows at the same
    // time), y over sequences, z over token tiles, with the sequence rotated by the tile index so that consecutive
    // work-groups (which the dispatcher deals round-robin to the 8 XCDs) mix tiles of different sequences: with
    // ragged lengths no XCD is left with only the sparsely populated late tiles
    const int i = static_cast<int>((blockIdx.y + blockIdx.z) % gridDim.y);
    int64_t L = loadIndex(a.bSeqLen, i, a.len64);
    if (L > a.maxInputLen) L = a.maxInputLen;
    const int64_t t0 = static_cast<int64_t>(blockIdx.z) * TT;
    if (t0 >= L) return;
    const int64_t start = loadIndex(a.bStartLoc, i, a.start64);
    const int64_t locBase = static_cast<int64_t>(i) * a.bLocStride + (a.maxInputLen - L);
    const int64_t tEnd = (t0 + TT < L) ? t0 + TT : L;
    const int64_t pairs = (tEnd - t0) * a.H;
    for (int64_t p = threadIdx.x; p < pairs; p += kAttThreads) {
        // token is the fastest index so that lanes write consecutive columns of one head
        const int64_t t = t0 + p % (tEnd - t0);
        const int h = static_cast<int>(p / (tEnd - t0));
        int64_t slot = loadIndex(a.bLoc, locBase + t, a.loc64);
        slot = slot < 0 ? 0 : (slot >= a.numSlots ? a.numSlots - 1 : slot);
        const T* qv = q + (static_cast<int64_t>(i) * a.H + h) * a.D;
        const T* kv = k + (slot * a.Hkv + h / a.G) * a.D;
        AccT acc = 0;
        for (int d = 0; d < a.D; ++d) acc += static_cast<AccT>(qv[d]) * static_cast<AccT>(kv[d]);
        const int64_t col = start + t;
        if (col >= 0 && col < a.logitCols) {
            const T dot = static_cast<T>(acc);
            out[static_cast<int64_t>(h) * a.logitCols + col] = static_cast<T>(static_cast<AccT>(dot) * scale);
        }
    }
}

template <typename T>
diopiError_t launchMfma(hipStream_t stream, void* out, const void* q, const void* k, const DecodeArgs& a, float scale) {
    constexpr int TT = 128;
    // kv heads per work-group: about 256 KiB of K per group, at least one head per wave
    const int HB = a.Hkv < 8 ? a.Hkv : 8;
    ROCM_CHECK(a.batch <= 65535 && ceilDiv(a.maxInputLen, TT) <= 65535, "batch %d / max_input_len %d exceed the launch limits (65535 sequences, 65535 tiles of %d tokens)", a.batch, a.maxInputLen, static_cast<int>(TT));
    const dim3 grid(static_cast<unsigned>(ceilDiv(a.Hkv, HB)), static_cast<unsigned>(a.batch), static_cast<unsigned>(ceilDiv(a.maxInputLen, TT)));
    // head size 64 (128 goes through the staged kernel)
    hipLaunchKernelGGL((tokenAttMfma<T, 2, TT>), grid, dim3(kAttThreads), 0, stream, static_cast<T*>(out), static_cast<const T*>(q),
                       static_cast<const T*>(k), a, HB, scale);
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

template <typename T>
diopiError_t launchStaged(hipStream_t stream, void* out, const void* q, const void* k, const DecodeArgs& a, float scale) {
    // heads per wave, head slots per work-group (waves beyond the head slots take other token units).  One head per
    // wave and short token tiles measured best once the head groups of a tile are dispatched next to each other:
    // neighbouring work-groups then stream neighbouring pieces of the same cache rows at the same time.
    constexpr int HW = 1;
    const int slots = static_cast<int>(ceilDiv(a.Hkv, HW));
    const int HS = slots >= 4 ? 4 : (slots >= 2 ? 2 : 1);
    // tokens per work-group: with one query head per kv head, tiles of 64 tokens measured 1.7 % faster than 128 (64
    // sequences of 512..2048 tokens, 32 heads); with 8 query heads per kv head (128 sequences of 1024..8192 tokens, 8 kv
    // heads) 256 is 4 % faster than 128 and 512 is 1 % slower than 256: longer pieces of every logits row per write-out
    int TT = a.G == 1 ? 64 : 256;
    // the scores of a tile wait in LDS for the write-out: at most 40 KiB of them
    const int outRows = HS * HW * a.G;
    while (TT > 64 && outRows * (TT + 8) * static_cast<int>(sizeof(T)) > 40 * 1024) TT -= 64;
    const size_t outLds = static_cast<size_t>(outRows) * (TT + 8) * sizeof(T);
    ROCM_CHECK(a.batch <= 65535 && ceilDiv(a.maxInputLen, TT) <= 65535, "batch %d / max_input_len %d exceed the launch limits (65535 sequences, 65535 tiles of %d tokens)", a.batch, a.maxInputLen, static_cast<int>(TT));
    // Work-groups go round-robin to the 8 XCDs in index order.  When the head groups (x) are a multiple of 8, a work-group's XCD
    // depends on its head group alone and every XCD gets the same share whatever the order of the rest: the tiles of a
    // sequence then run one after the other, y = tile, z = sequence (cfg3: 100.3 us against 103.1).  Otherwise a
    // sequence would stay on a few XCDs and ragged lengths would unbalance them: y = sequence, z = tile, the sequence rotated by
    // the tile index (cfg5, 2 head groups: 242 us; unrotated 264, tiles in sequence order 268).
    const int gridX = static_cast<int>(ceilDiv(a.Hkv, HS * HW));
    const int order = gridX % kNumXcd == 0 ? 1 : 0;
    const dim3 grid = order == 1 ? dim3(static_cast<unsigned>(ceilDiv(a.Hkv, HS * HW)), static_cast<unsigned>(ceilDiv(a.maxInputLen, TT)), static_cast<unsigned>(a.batch))
                                 : dim3(static_cast<unsigned>(ceilDiv(a.Hkv, HS * HW)), static_cast<unsigned>(a.batch), static_cast<unsigned>(ceilDiv(a.maxInputLen, TT)));
    // Loads a lane has in flight per unit of tokens: 16 with one query head per kv head; with grouped heads 4, where the rows
    // compete with the logits being written (128 sequences of 1024..8192 tokens, 8 kv heads of 8 query heads: 234.3 us against
    // 242.9 with 16 and 243.6 with 8; with one query head per kv head 4 and 8 are 1 % slower than 16)
    if (a.G == 1) {
        hipLaunchKernelGGL((tokenAttStaged<T, HW, 64>), grid, dim3(kAttThreads), outLds, stream, static_cast<T*>(out), static_cast<const T*>(q),
                           static_cast<const T*>(k), a, TT, HS, scale, order);
    } else {
        hipLaunchKernelGGL((tokenAttStaged<T, HW, 16>), grid, dim3(kAttThreads), outLds, stream, static_cast<T*>(out), static_cast<const T*>(q),
                           static_cast<const T*>(k), a, TT, HS, scale, order);
    }
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

template <typename T, typename AccT>
diopiError_t launchGeneric(hipStream_t stream, void* out, const void* q, const void* k, const DecodeArgs& a) {
    const int TT = 64;
    ROCM_CHECK(a.batch <= 65535 && ceilDiv(a.maxInputLen, TT) <= 65535, "batch %d / max_input_len %d exceed the launch limits (65535 sequences, 65535 tiles of %d tokens)", a.batch, a.maxInputLen, static_cast<int>(TT));
    const dim3 grid(1, static_cast<unsigned>(a.batch), static_cast<unsigned>(ceilDiv(a.maxInputLen, TT)));
    const AccT scale = static_cast<AccT>(1.0 / std::sqrt(static_cast<double>(a.D)));
    hipLaunchKernelGGL((tokenAttGeneric<T, AccT>), grid, dim3(kAttThreads), 0, stream, static_cast<T*>(out), static_cast<const T*>(q),
                       static_cast<const T*>(k), a, TT, scale);
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

}  // namespace
}  // namespace rocm

namespace rocm {

diopiError_t tokenAttention(diopiContextHandle_t ctx, const TensorView& vOut, const TensorView& vQ, const TensorView& vK, const TensorView& vLoc,
                            const TensorView& vStart, const TensorView& vLen, int max_input_len) {
    DecodeArgs a;
    bool empty = false;
    ROCM_CALL(prepareDecode(vOut, vQ, vK, vLoc, vStart, vLen, max_input_len, &a, &empty));
    if (empty) return diopiSuccess;
    const int64_t D = a.D;

    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    const bool fast = (D == 128 || D == 64) && a.G <= 16 && ((reinterpret_cast<uintptr_t>(vQ.data) | reinterpret_cast<uintptr_t>(vK.data)) & 15) == 0;
    // the element type's matmul rounds the fp32 dot to T, then the division by sqrt(D) rounds again
    const float scale = 1.0f / static_cast<float>(std::sqrt(static_cast<double>(D)));
    const bool staged = fast && D == 128;
    switch (vQ.dtype) {
        case diopi_dtype_float16:
            if (staged) return launchStaged<half_t>(stream, vOut.data, vQ.data, vK.data, a, scale);
            return fast ? launchMfma<half_t>(stream, vOut.data, vQ.data, vK.data, a, scale) : launchGeneric<half_t, float>(stream, vOut.data, vQ.data, vK.data, a);
        case diopi_dtype_bfloat16:
            if (staged) return launchStaged<bf16_t>(stream, vOut.data, vQ.data, vK.data, a, scale);
            return fast ? launchMfma<bf16_t>(stream, vOut.data, vQ.data, vK.data, a, scale) : launchGeneric<bf16_t, float>(stream, vOut.data, vQ.data, vK.data, a);
        case diopi_dtype_float32: return launchGeneric<float, float>(stream, vOut.data, vQ.data, vK.data, a);
        case diopi_dtype_float64: return launchGeneric<double, double>(stream, vOut.data, vQ.data, vK.data, a);
        default: break;
    }
    setLastError("diopiTokenAttentionInference: dtype %s is not supported", dtypeName(vQ.dtype));
    return diopiDtypeNotSupported;
}

}  // namespace rocm

extern "C" diopiError_t diopiTokenAttentionInference(diopiContextHandle_t ctx, diopiTensorHandle_t token_attention_out, diopiConstTensorHandle_t q,
                                                     diopiConstTensorHandle_t k, diopiConstTensorHandle_t b_loc, diopiConstTensorHandle_t b_start_loc,
                                                     diopiConstTensorHandle_t b_seq_len, int max_input_len) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    TensorView vOut, vQ, vK, vLoc, vStart, vLen;
    ROCM_CALL(unwrap(token_attention_out, "token_attention_out", &vOut));
    ROCM_CALL(unwrap(q, "q", &vQ));
    ROCM_CALL(unwrap(k, "k", &vK));
    ROCM_CALL(unwrap(b_loc, "b_loc", &vLoc));
    ROCM_CALL(unwrap(b_start_loc, "b_start_loc", &vStart));
    ROCM_CALL(unwrap(b_seq_len, "b_seq_len", &vLen));
    return tokenAttention(ctx, vOut, vQ, vK, vLoc, vStart, vLen, max_input_len);
    ROCM_ENTRY_END
}
