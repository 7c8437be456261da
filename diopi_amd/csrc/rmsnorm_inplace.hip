// diopiRootMeanSquareNormInp / diopiFusedAddRootMeanSquareNormInp for gfx950: the in-place RMS normalisation of the
// lmdeploy operator set, alone or fused with the residual and bias addition that precedes it in a decoder layer.
//
// Interface: proto/include/diopi/functions_lmdeploy.h:31-49 of the reference.  The reference tree holds no
// implementation and no test of these two operators; their statement there is the header's sentence
//   "1.(res + inout + bias) = new_res  2.RMSNorm(new_res) = inout",  eps guards the division.
// The arithmetic below follows the kernels the interface was written for (lmdeploy's turbomind decoder,
// llama_kernels.cu: rootMeanSquareNorm and fusedAddBiasResidualNorm), as published:
//
//   diopiRootMeanSquareNormInp          inv = rsqrt(sum_l x[r,l]^2 / n + eps)           fp32 sums over the stored values
//                                       x[r,l] <- T(x[r,l] * inv) * scale[l]            product of two T values, rounded
//   diopiFusedAddRootMeanSquareNormInp  s = float(res[r,l]) + float(x[r,l]) + float(bias[l])
//                                       inv = rsqrt(sum_l s^2 / n + eps)                 squares of the unrounded sums
//                                       res[r,l] <- T(s)
//                                       x[r,l]   <- T(float(T(s)) * (inv * float(scale[l])))
//
// Layout: inoutput and residual [tokens, hidden] dense, scale and bias [hidden]; bias may be a null handle.
// One group of 256 threads (512 with the residual addition) owns a row and keeps it in registers as 16-byte packets, so every element is read once and
// written once: 2 (alone) or 4 (fused) passes over the matrix, which is what bounds the operator.  Many short-lived
// groups, each touching one contiguous row, is the launch shape the memory system sustains its highest rate for.
// Rows that do not fit that form (length not a multiple of a packet, more than 4 packets per thread, unaligned base)
// go through a wave-per-row kernel that sweeps the row twice.
#include <diopi/functions_lmdeploy.h>

#include "common.hpp"
#include "device.hpp"

namespace rocm {
namespace {

constexpr int kRowThreads = 256;  // threads of a group of the wave-per-row kernel, and of a row's group in the plain form
constexpr int kRowWaves = kRowThreads / kWave;
// Threads that own a row.  The plain form keeps the 256 of diopiRMSNorm's kernel, so that the two sum a row's squares in the
// same order and give the same bits; with the residual addition 256 / 512 / 1024 measured 86.4 / 84.3 / 86.0 us at bf16
// [16384, 4096].
constexpr int rowThreads(bool fuseAdd) { return fuseAdd ? 512 : 256; }

template <typename T, int NVT, bool FUSE_ADD, bool HAS_BIAS>
__global__ __launch_bounds__(rowThreads(FUSE_ADD)) void rmsNormInpBlockRow(T* __restrict__ inout, T* __restrict__ residual, const T* __restrict__ bias,
                                                                            const T* __restrict__ scale, int64_t rows, int n, float eps) {
    constexpr int EPV = Pack16<T>::N;
    constexpr int kThreads = rowThreads(FUSE_ADD);
    __shared__ float red[kThreads / kWave];
    const int tid = threadIdx.x;
    const int lane = tid % kWave;
    const int wave = tid / kWave;
    const int nvec = n / EPV;
    const int64_t row = blockIdx.x;
    T* xr = inout + row * n;
    T* rr = FUSE_ADD ? residual + row * n : nullptr;

    // the row first, the per-column vectors behind it
    Pack16<T> xv[NVT], rv[FUSE_ADD ? NVT : 1];
#pragma unroll
    for (int j = 0; j < NVT; ++j) {
        const int v = j * kThreads + tid;
        if (v < nvec) {
            xv[j] = loadPackStream(xr + v * EPV);
            if constexpr (FUSE_ADD) rv[j] = loadPackStream(rr + v * EPV);
        }
    }
    Pack16<T> sv[NVT], bv[HAS_BIAS ? NVT : 1];
#pragma unroll
    for (int j = 0; j < NVT; ++j) {
        const int v = j * kThreads + tid;
        if (v < nvec) {
            sv[j] = loadPack(scale + v * EPV);
            if constexpr (HAS_BIAS) bv[j] = loadPack(bias + v * EPV);
        }
    }

    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NVT; ++j) {
        const int v = j * kThreads + tid;
        if (v < nvec) {
            if constexpr (FUSE_ADD) {
                Pack16<T> nr;
#pragma unroll
                for (int e = 0; e < EPV; ++e) {
                    float s = toFloat(rv[j].e[e]) + toFloat(xv[j].e[e]);
                    if constexpr (HAS_BIAS) s += toFloat(bv[j].e[e]);
                    ss += s * s;
                    nr.e[e] = fromFloat<T>(s);
                }
                storePackStream(rr + v * EPV, nr);
                xv[j] = nr;  // the normalisation reads the stored residual
            } else {
#pragma unroll
                for (int e = 0; e < EPV; ++e) {
                    const float f = toFloat(xv[j].e[e]);
                    ss += f * f;
                }
            }
        }
    }
    ss = waveSum(ss);
    if (lane == 0) red[wave] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int i = 0; i < kThreads / kWave; ++i) tot += red[i];
    const float inv = 1.0f / sqrtf(tot / static_cast<float>(n) + eps);

#pragma unroll
    for (int j = 0; j < NVT; ++j) {
        const int v = j * kThreads + tid;
        if (v < nvec) {
            Pack16<T> o;
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                if (FUSE_ADD) {
                    o.e[e] = fromFloat<T>(toFloat(xv[j].e[e]) * (inv * toFloat(sv[j].e[e])));
                } else {
                    const T normed = fromFloat<T>(toFloat(xv[j].e[e]) * inv);
                    o.e[e] = fromFloat<T>(toFloat(normed) * toFloat(sv[j].e[e]));
                }
            }
            storePackStream(xr + v * EPV, o);
        }
    }
}

// Any row length and alignment: one wavefront per row, two sweeps (the second one hits in cache).
template <typename T, bool FUSE_ADD>
__global__ __launch_bounds__(kRowThreads) void rmsNormInpGeneric(T* __restrict__ inout, T* __restrict__ residual, const T* __restrict__ bias,
                                                                  const T* __restrict__ scale, int64_t rows, int64_t n, float eps) {
    const int lane = threadIdx.x % kWave;
    const int64_t wavesTotal = static_cast<int64_t>(gridDim.x) * kRowWaves;
    for (int64_t row = static_cast<int64_t>(blockIdx.x) * kRowWaves + threadIdx.x / kWave; row < rows; row += wavesTotal) {
        T* xr = inout + row * n;
        T* rr = FUSE_ADD ? residual + row * n : nullptr;
        float ss = 0.f;
        for (int64_t l = lane; l < n; l += kWave) {
            if (FUSE_ADD) {
                float s = toFloat(rr[l]) + toFloat(xr[l]);
                if (bias != nullptr) s += toFloat(bias[l]);
                ss += s * s;
                rr[l] = fromFloat<T>(s);
            } else {
                const float f = toFloat(xr[l]);
                ss += f * f;
            }
        }
        ss = waveSum(ss);
        const float inv = 1.0f / sqrtf(ss / static_cast<float>(n) + eps);
        // a lane reads back only what it wrote itself: no ordering between lanes is needed
        for (int64_t l = lane; l < n; l += kWave) {
            if (FUSE_ADD) {
                xr[l] = fromFloat<T>(toFloat(rr[l]) * (inv * toFloat(scale[l])));
            } else {
                const T normed = fromFloat<T>(toFloat(xr[l]) * inv);
                xr[l] = fromFloat<T>(toFloat(normed) * toFloat(scale[l]));
            }
        }
    }
}

bool aligned16(const void* p) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T, bool FUSE_ADD>
diopiError_t launchTyped(hipStream_t stream, void* inout, void* residual, const void* bias, const void* scale, int64_t rows, int64_t n, float eps) {
    constexpr int EPV = Pack16<T>::N;
    T* px = static_cast<T*>(inout);
    T* pr = static_cast<T*>(residual);
    const T* pb = static_cast<const T*>(bias);
    const T* ps = static_cast<const T*>(scale);
    const int64_t nvec = n / EPV;
    constexpr int kThreads = rowThreads(FUSE_ADD);
    const bool fast = n % EPV == 0 && nvec <= 4 * kThreads && rows <= INT32_MAX && aligned16(inout) && aligned16(residual) && aligned16(bias) &&
                      aligned16(scale);
    if (!fast) {
        int64_t blocks = ceilDiv(rows, kRowWaves);
        const int64_t cap = static_cast<int64_t>(deviceInfo().numCU) * 8;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL((rmsNormInpGeneric<T, FUSE_ADD>), dim3(static_cast<unsigned>(blocks)), dim3(kRowThreads), 0, stream, px, pr, pb, ps, rows, n, eps);
        ROCM_LAUNCH_CHECK();
        return diopiSuccess;
    }
    const int nvt = static_cast<int>(ceilDiv(nvec, kThreads));
    const dim3 grid(static_cast<unsigned>(rows));
    const int ni = static_cast<int>(n);
#define ROCM_INP_CASE(NVC)                                                                                                                        \
    if (FUSE_ADD && bias != nullptr) {                                                                                                            \
        hipLaunchKernelGGL((rmsNormInpBlockRow<T, NVC, FUSE_ADD, FUSE_ADD>), grid, dim3(kThreads), 0, stream, px, pr, pb, ps, rows, ni, eps);   \
    } else {                                                                                                                                      \
        hipLaunchKernelGGL((rmsNormInpBlockRow<T, NVC, FUSE_ADD, false>), grid, dim3(kThreads), 0, stream, px, pr, pb, ps, rows, ni, eps);      \
    }
    if (nvt <= 1) {
        ROCM_INP_CASE(1)
    } else if (nvt <= 2) {
        ROCM_INP_CASE(2)
    } else {
        ROCM_INP_CASE(4)
    }
#undef ROCM_INP_CASE
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

diopiError_t normInPlace(diopiContextHandle_t ctx, diopiTensorHandle_t inoutput, diopiTensorHandle_t residual, bool fuseAdd, diopiConstTensorHandle_t bias,
                         diopiConstTensorHandle_t scale, float eps) {
    TensorView vX, vR, vB, vS;
    ROCM_CALL(unwrap(inoutput, "inoutput", &vX));
    ROCM_CALL(unwrap(scale, "scale", &vS));
    ROCM_CALL(requireDeviceContiguous(vX, "inoutput"));
    ROCM_CALL(requireDeviceContiguous(vS, "scale"));
    ROCM_CHECK(vX.ndim >= 1, "inoutput must be [tokens, hidden]");
    const int64_t n = vX.shape[vX.ndim - 1];
    ROCM_CHECK(vX.dtype == diopi_dtype_float32 || vX.dtype == diopi_dtype_float16 || vX.dtype == diopi_dtype_bfloat16,
               "inoutput dtype %s is not supported (float32, float16, bfloat16)", dtypeName(vX.dtype));
    ROCM_CHECK(vS.numel == n && vS.dtype == vX.dtype, "scale must hold hidden = %lld elements of dtype %s", static_cast<long long>(n), dtypeName(vX.dtype));
    if (fuseAdd) {
        ROCM_CALL(unwrap(residual, "residual", &vR));
        ROCM_CALL(requireDeviceContiguous(vR, "residual"));
        ROCM_CHECK(vR.sameShape(vX) && vR.dtype == vX.dtype, "residual must have the shape and dtype of inoutput");
        ROCM_CHECK(vR.data != vX.data || vX.numel == 0, "residual and inoutput must be different tensors");
        if (bias != nullptr) {
            ROCM_CALL(unwrap(bias, "bias", &vB));
            ROCM_CALL(requireDeviceContiguous(vB, "bias"));
            ROCM_CHECK(vB.numel == n && vB.dtype == vX.dtype, "bias must hold hidden = %lld elements of dtype %s", static_cast<long long>(n),
                       dtypeName(vX.dtype));
        }
    }
    if (vX.numel == 0) return diopiSuccess;
    const int64_t rows = vX.numel / n;
    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    void* pr = fuseAdd ? vR.data : nullptr;
    const void* pb = (fuseAdd && bias != nullptr) ? vB.data : nullptr;
    if (fuseAdd) {
        if (vX.dtype == diopi_dtype_float32) return launchTyped<float, true>(stream, vX.data, pr, pb, vS.data, rows, n, eps);
        if (vX.dtype == diopi_dtype_float16) return launchTyped<half_t, true>(stream, vX.data, pr, pb, vS.data, rows, n, eps);
        return launchTyped<bf16_t, true>(stream, vX.data, pr, pb, vS.data, rows, n, eps);
    }
    if (vX.dtype == diopi_dtype_float32) return launchTyped<float, false>(stream, vX.data, pr, pb, vS.data, rows, n, eps);
    if (vX.dtype == diopi_dtype_float16) return launchTyped<half_t, false>(stream, vX.data, pr, pb, vS.data, rows, n, eps);
    return launchTyped<bf16_t, false>(stream, vX.data, pr, pb, vS.data, rows, n, eps);
}

}  // namespace
}  // namespace rocm

extern "C" diopiError_t diopiRootMeanSquareNormInp(diopiContextHandle_t ctx, diopiTensorHandle_t inoutput, diopiConstTensorHandle_t scale, float eps) {
    ROCM_ENTRY_BEGIN
    return rocm::normInPlace(ctx, inoutput, nullptr, false, nullptr, scale, eps);
    ROCM_ENTRY_END
}

extern "C" diopiError_t diopiFusedAddRootMeanSquareNormInp(diopiContextHandle_t ctx, diopiTensorHandle_t inoutput, diopiTensorHandle_t residual,
                                                           diopiConstTensorHandle_t bias, diopiConstTensorHandle_t scale, float eps) {
    ROCM_ENTRY_BEGIN
    return rocm::normInPlace(ctx, inoutput, residual, true, bias, scale, eps);
    ROCM_ENTRY_END
}
