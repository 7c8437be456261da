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
    const int i = blockIdx.y;
    int64_t L = loadIndex(a.bSeqLen, i, a.len64);
    if (L > a.maxInputLen) L = a.maxInputLen;
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * TT;
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

    const int hkBegin = blockIdx.z * HB;
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

// Any dtype / head size / grouping: one thread per (token, query head) pair of a tile.
template <typename T, typename AccT>
__global__ __launch_bounds__(kAttThreads) void tokenAttGeneric(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k, DecodeArgs a, int TT,
                                                               AccT scale) {
    const int i = blockIdx.y;
    int64_t L = loadIndex(a.bSeqLen, i, a.len64);
    if (L > a.maxInputLen) L = a.maxInputLen;
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * TT;
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
    int HB = a.Hkv < 8 ? a.Hkv : 8;
    HB = envInt("DIOPI_ROCM_TOKATT_HB", HB);
    const dim3 grid(static_cast<unsigned>(ceilDiv(a.maxInputLen, TT)), static_cast<unsigned>(a.batch), static_cast<unsigned>(ceilDiv(a.Hkv, HB)));
    if (a.D == 128) {
        hipLaunchKernelGGL((tokenAttMfma<T, 4, TT>), grid, dim3(kAttThreads), 0, stream, static_cast<T*>(out), static_cast<const T*>(q),
                           static_cast<const T*>(k), a, HB, scale);
    } else {
        hipLaunchKernelGGL((tokenAttMfma<T, 2, TT>), grid, dim3(kAttThreads), 0, stream, static_cast<T*>(out), static_cast<const T*>(q),
                           static_cast<const T*>(k), a, HB, scale);
    }
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

template <typename T, typename AccT>
diopiError_t launchGeneric(hipStream_t stream, void* out, const void* q, const void* k, const DecodeArgs& a) {
    const int TT = 64;
    const dim3 grid(static_cast<unsigned>(ceilDiv(a.maxInputLen, TT)), static_cast<unsigned>(a.batch));
    const AccT scale = static_cast<AccT>(1.0 / std::sqrt(static_cast<double>(a.D)));
    hipLaunchKernelGGL((tokenAttGeneric<T, AccT>), grid, dim3(kAttThreads), 0, stream, static_cast<T*>(out), static_cast<const T*>(q),
                       static_cast<const T*>(k), a, TT, scale);
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

}  // namespace
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
    DecodeArgs a;
    bool empty = false;
    ROCM_CALL(prepareDecode(vOut, vQ, vK, vLoc, vStart, vLen, max_input_len, &a, &empty));
    if (empty) return diopiSuccess;
    const int64_t D = a.D;

    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    const bool fast = (D == 128 || D == 64) && a.G <= 16 && ((reinterpret_cast<uintptr_t>(vQ.data) | reinterpret_cast<uintptr_t>(vK.data)) & 15) == 0 &&
                      envInt("DIOPI_ROCM_FORCE_GENERIC", 0) == 0;
    // the element type's matmul rounds the fp32 dot to T, then the division by sqrt(D) rounds again
    const float scale = 1.0f / static_cast<float>(std::sqrt(static_cast<double>(D)));
    switch (vQ.dtype) {
        case diopi_dtype_float16:
            return fast ? launchMfma<half_t>(stream, vOut.data, vQ.data, vK.data, a, scale) : launchGeneric<half_t, float>(stream, vOut.data, vQ.data, vK.data, a);
        case diopi_dtype_bfloat16:
            return fast ? launchMfma<bf16_t>(stream, vOut.data, vQ.data, vK.data, a, scale) : launchGeneric<bf16_t, float>(stream, vOut.data, vQ.data, vK.data, a);
        case diopi_dtype_float32: return launchGeneric<float, float>(stream, vOut.data, vQ.data, vK.data, a);
        case diopi_dtype_float64: return launchGeneric<double, double>(stream, vOut.data, vQ.data, vK.data, a);
        default: break;
    }
    setLastError("diopiTokenAttentionInference: dtype %s is not supported", dtypeName(vQ.dtype));
    return diopiDtypeNotSupported;
    ROCM_ENTRY_END
}
