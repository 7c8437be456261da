// diopiApplyPenalty and diopiApplyPenaltyV2 for gfx950: the sampling prologue of lightllm, a sparse in-place update of
// the logits of the tokens a sequence has already generated.
//
// diopiApplyPenalty (functions_ext.h:527-529; impl/torch/functions/functions_lightllm.cpp:28-51; Python statement
// customized_test.py:667-692).  Sequence i owns entries [cum[i], cum[i+1]) of p_token_ids / p_token_counts:
//   logits[i, id_j] <- logits[i, id_j] - count_j * frequency_penalty[i] - presence_penalty[i]
// p_max_len_in_batch is not read by the reference either.
// diopiApplyPenaltyV2 (functions_ext.h:547-549; statement customized_test.py:823-841; no torch body).  p_token_ids are
// flat indices into logits.view(-1) and every penalty tensor has one entry per generated token:
//   x = logits[id_j];  x <- x > 0 ? x / repetition_j : x * repetition_j;  x <- x - count_j * frequency_j - presence_j
// Both follow the reference's rounding: the expressions are evaluated left to right in the logits dtype (every product,
// quotient and difference is rounded to it; ATen computes each of them in fp32 for 16-bit tensors).  Indices outside
// the tensor are skipped; an id that occurs twice in one sequence is written by either occurrence, as with the
// reference's non-accumulating index_put.
// One thread per generated token: these launches are a few microseconds whatever the kernel does (a batch of 64
// sequences with a few hundred generated tokens each touches a few hundred KiB).
#include <utility>

#include "common.hpp"
#include "device.hpp"

namespace rocm {
namespace {

constexpr int kPenThreads = 256;

// The reference rounds the product and both differences to the logits dtype one after the other.  Device code is
// compiled with floating-point contraction allowed, which would fuse the product into the first subtraction and drop
// its rounding: contraction is switched off for the rest of this file.
#pragma clang fp contract(off)

// The arithmetic type ATen uses for an element type: fp32 for everything narrower than fp64.
template <typename T>
__device__ __forceinline__ T roundTo(typename AccType<T>::type v) {
    return static_cast<T>(v);
}

template <typename T>
__global__ __launch_bounds__(kPenThreads) void applyPenaltyKernel(T* __restrict__ logits, const T* __restrict__ presence, const T* __restrict__ frequency,
                                                                  const void* __restrict__ ids, bool ids64, const void* __restrict__ counts, bool counts64,
                                                                  const void* __restrict__ cum, bool cum64, int64_t tokens, int batch, int64_t vocab) {
    using Acc = typename AccType<T>::type;
    const int64_t j = static_cast<int64_t>(blockIdx.x) * kPenThreads + threadIdx.x;
    if (j >= tokens) return;
    // the sequence that owns entry j: the last i with cum[i] <= j (entries before cum[0] or past cum[batch] belong to nobody)
    int lo = 0, hi = batch;  // cum has batch + 1 entries
    if (j < loadIndex(cum, 0, cum64) || j >= loadIndex(cum, batch, cum64)) return;
    while (hi - lo > 1) {
        const int mid = (lo + hi) / 2;
        if (loadIndex(cum, mid, cum64) <= j) {
            lo = mid;
        } else {
            hi = mid;
        }
    }
    const int i = lo;
    const int64_t id = loadIndex(ids, j, ids64);
    if (id < 0 || id >= vocab) return;
    T* p = logits + static_cast<int64_t>(i) * vocab + id;
    const T count = roundTo<T>(static_cast<Acc>(loadIndex(counts, j, counts64)));  // the count enters the product in the logits dtype
    const T prod = roundTo<T>(static_cast<Acc>(count) * static_cast<Acc>(frequency[i]));
    const T diff = roundTo<T>(static_cast<Acc>(*p) - static_cast<Acc>(prod));
    *p = roundTo<T>(static_cast<Acc>(diff) - static_cast<Acc>(presence[i]));
}

template <typename T>
__global__ __launch_bounds__(kPenThreads) void applyPenaltyV2Kernel(T* __restrict__ logits, const T* __restrict__ presence, const T* __restrict__ frequency,
                                                                    const T* __restrict__ repetition, const void* __restrict__ ids, bool ids64,
                                                                    const void* __restrict__ counts, bool counts64, int64_t tokens, int64_t numel) {
    using Acc = typename AccType<T>::type;
    const int64_t j = static_cast<int64_t>(blockIdx.x) * kPenThreads + threadIdx.x;
    if (j >= tokens) return;
    const int64_t id = loadIndex(ids, j, ids64);
    if (id < 0 || id >= numel) return;
    const Acc x = static_cast<Acc>(logits[id]), rep = static_cast<Acc>(repetition[j]);
    const T scaled = roundTo<T>(x > static_cast<Acc>(0) ? x / rep : x * rep);
    const T count = roundTo<T>(static_cast<Acc>(loadIndex(counts, j, counts64)));
    const T prod = roundTo<T>(static_cast<Acc>(count) * static_cast<Acc>(frequency[j]));
    const T diff = roundTo<T>(static_cast<Acc>(scaled) - static_cast<Acc>(prod));
    logits[id] = roundTo<T>(static_cast<Acc>(diff) - static_cast<Acc>(presence[j]));
}

}  // namespace
}  // namespace rocm

extern "C" diopiError_t diopiApplyPenalty(diopiContextHandle_t ctx, diopiTensorHandle_t logits, diopiConstTensorHandle_t presence_penalty,
                                          diopiConstTensorHandle_t frequency_penalty, diopiConstTensorHandle_t p_token_ids,
                                          diopiConstTensorHandle_t p_token_counts, diopiConstTensorHandle_t p_cumsum_seq_len, int p_max_len_in_batch) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    (void)p_max_len_in_batch;  // unused by the reference as well (functions_lightllm.cpp:28-51)
    TensorView vL, vP, vF, vIds, vCnt, vCum;
    ROCM_CALL(unwrap(logits, "logits", &vL));
    ROCM_CALL(unwrap(presence_penalty, "presence_penalty", &vP));
    ROCM_CALL(unwrap(frequency_penalty, "frequency_penalty", &vF));
    ROCM_CALL(unwrap(p_token_ids, "p_token_ids", &vIds));
    ROCM_CALL(unwrap(p_token_counts, "p_token_counts", &vCnt));
    ROCM_CALL(unwrap(p_cumsum_seq_len, "p_cumsum_seq_len", &vCum));
    for (const auto& tv : {std::make_pair(&vL, "logits"), std::make_pair(&vP, "presence_penalty"), std::make_pair(&vF, "frequency_penalty"),
                           std::make_pair(&vIds, "p_token_ids"), std::make_pair(&vCnt, "p_token_counts"), std::make_pair(&vCum, "p_cumsum_seq_len")}) {
        ROCM_CALL(requireDeviceContiguous(*tv.first, tv.second));
    }
    ROCM_CHECK(vL.ndim == 2, "logits must be [batch, vocabulary], got rank %d", vL.ndim);
    ROCM_CHECK(isFloatDtype(vL.dtype), "logits dtype %s is not supported", dtypeName(vL.dtype));
    ROCM_CHECK(vP.dtype == vL.dtype && vF.dtype == vL.dtype, "the penalties must have the dtype of logits (%s)", dtypeName(vL.dtype));
    ROCM_CHECK(isIndexDtype(vIds.dtype) && isIndexDtype(vCnt.dtype) && isIndexDtype(vCum.dtype), "p_token_ids, p_token_counts and p_cumsum_seq_len must be int32 or int64");
    const int64_t batch = vL.shape[0], vocab = vL.shape[1];
    ROCM_CHECK(vP.numel == batch && vF.numel == batch, "presence_penalty (%lld) and frequency_penalty (%lld) need one entry per sequence (%lld)",
               static_cast<long long>(vP.numel), static_cast<long long>(vF.numel), static_cast<long long>(batch));
    ROCM_CHECK(vCum.numel == batch + 1, "p_cumsum_seq_len must hold batch + 1 = %lld entries, got %lld", static_cast<long long>(batch + 1),
               static_cast<long long>(vCum.numel));
    ROCM_CHECK(vIds.numel == vCnt.numel, "p_token_ids (%lld) and p_token_counts (%lld) must have the same length", static_cast<long long>(vIds.numel),
               static_cast<long long>(vCnt.numel));
    ROCM_CHECK(batch <= INT32_MAX - 1, "too many sequences");
    const int64_t tokens = vIds.numel;
    if (tokens == 0 || batch == 0 || vocab == 0) return diopiSuccess;
    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    const int64_t blocks = ceilDiv(tokens, kPenThreads);
    ROCM_CHECK(blocks <= INT32_MAX, "too many generated tokens for one launch");
#define ROCM_PEN_CASE(T)                                                                                                                            \
    hipLaunchKernelGGL(applyPenaltyKernel<T>, dim3(static_cast<unsigned>(blocks)), dim3(kPenThreads), 0, stream, static_cast<T*>(vL.data),          \
                       static_cast<const T*>(vP.data), static_cast<const T*>(vF.data), vIds.data, vIds.dtype == diopi_dtype_int64, vCnt.data,       \
                       vCnt.dtype == diopi_dtype_int64, vCum.data, vCum.dtype == diopi_dtype_int64, tokens, static_cast<int>(batch), vocab)
    switch (vL.dtype) {
        case diopi_dtype_float16: ROCM_PEN_CASE(half_t); break;
        case diopi_dtype_bfloat16: ROCM_PEN_CASE(bf16_t); break;
        case diopi_dtype_float32: ROCM_PEN_CASE(float); break;
        case diopi_dtype_float64: ROCM_PEN_CASE(double); break;
        default: setLastError("diopiApplyPenalty: dtype %s is not supported", dtypeName(vL.dtype)); return diopiDtypeNotSupported;
    }
#undef ROCM_PEN_CASE
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
    ROCM_ENTRY_END
}

extern "C" diopiError_t diopiApplyPenaltyV2(diopiContextHandle_t ctx, diopiTensorHandle_t logits, diopiConstTensorHandle_t presence_penalty,
                                            diopiConstTensorHandle_t frequency_penalty, diopiConstTensorHandle_t repetition_penalty,
                                            diopiConstTensorHandle_t p_token_ids, diopiConstTensorHandle_t p_token_counts) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    TensorView vL, vP, vF, vR, vIds, vCnt;
    ROCM_CALL(unwrap(logits, "logits", &vL));
    ROCM_CALL(unwrap(presence_penalty, "presence_penalty", &vP));
    ROCM_CALL(unwrap(frequency_penalty, "frequency_penalty", &vF));
    ROCM_CALL(unwrap(repetition_penalty, "repetition_penalty", &vR));
    ROCM_CALL(unwrap(p_token_ids, "p_token_ids", &vIds));
    ROCM_CALL(unwrap(p_token_counts, "p_token_counts", &vCnt));
    for (const auto& tv : {std::make_pair(&vL, "logits"), std::make_pair(&vP, "presence_penalty"), std::make_pair(&vF, "frequency_penalty"),
                           std::make_pair(&vR, "repetition_penalty"), std::make_pair(&vIds, "p_token_ids"), std::make_pair(&vCnt, "p_token_counts")}) {
        ROCM_CALL(requireDeviceContiguous(*tv.first, tv.second));
    }
    ROCM_CHECK(isFloatDtype(vL.dtype), "logits dtype %s is not supported", dtypeName(vL.dtype));
    ROCM_CHECK(vP.dtype == vL.dtype && vF.dtype == vL.dtype && vR.dtype == vL.dtype, "the penalties must have the dtype of logits (%s)", dtypeName(vL.dtype));
    ROCM_CHECK(isIndexDtype(vIds.dtype) && isIndexDtype(vCnt.dtype), "p_token_ids and p_token_counts must be int32 or int64");
    const int64_t tokens = vIds.numel;
    ROCM_CHECK(vCnt.numel == tokens && vP.numel == tokens && vF.numel == tokens && vR.numel == tokens,
               "p_token_counts and the three penalties need one entry per generated token (%lld)", static_cast<long long>(tokens));
    if (tokens == 0 || vL.numel == 0) return diopiSuccess;
    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    const int64_t blocks = ceilDiv(tokens, kPenThreads);
    ROCM_CHECK(blocks <= INT32_MAX, "too many generated tokens for one launch");
#define ROCM_PEN2_CASE(T)                                                                                                                          \
    hipLaunchKernelGGL(applyPenaltyV2Kernel<T>, dim3(static_cast<unsigned>(blocks)), dim3(kPenThreads), 0, stream, static_cast<T*>(vL.data),       \
                       static_cast<const T*>(vP.data), static_cast<const T*>(vF.data), static_cast<const T*>(vR.data), vIds.data,                  \
                       vIds.dtype == diopi_dtype_int64, vCnt.data, vCnt.dtype == diopi_dtype_int64, tokens, vL.numel)
    switch (vL.dtype) {
        case diopi_dtype_float16: ROCM_PEN2_CASE(half_t); break;
        case diopi_dtype_bfloat16: ROCM_PEN2_CASE(bf16_t); break;
        case diopi_dtype_float32: ROCM_PEN2_CASE(float); break;
        case diopi_dtype_float64: ROCM_PEN2_CASE(double); break;
        default: setLastError("diopiApplyPenaltyV2: dtype %s is not supported", dtypeName(vL.dtype)); return diopiDtypeNotSupported;
    }
#undef ROCM_PEN2_CASE
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
    ROCM_ENTRY_END
}
