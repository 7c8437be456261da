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
        for (int t = tid; t < nTok; t += kRvThreads) {
            int64_t slot = loadIndex(a.bLoc, locBase + ts + t, a.loc64);
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
                sP[h][t] = p;
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
    float m = -INFINITY;
    for (int j = 0; j < ns; ++j) m = fmaxf(m, ml[static_cast<int64_t>(j) * a.H * 2]);
    float num = 0.f, den = 0.f;
    for (int j = 0; j < ns; ++j) {
        const float mj = ml[static_cast<int64_t>(j) * a.H * 2];
        const float w = (mj == -INFINITY) ? 0.f : __expf(mj - m);
        num += w * pa[static_cast<int64_t>(j) * a.H * a.D];
        den += w * ml[static_cast<int64_t>(j) * a.H * 2 + 1];
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
    if (TT < 256) TT = 256;
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
    switch (vOut.dtype) {
        case diopi_dtype_float16:
            return fast ? launchSplit<half_t>(ctx, stream, vOut.data, vLogits.data, vV.data, a)
                        : launchGeneric<half_t, float>(stream, vOut.data, vLogits.data, vV.data, a);
        case diopi_dtype_bfloat16:
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
