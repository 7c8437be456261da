// diopiRotaryEmbedding for gfx950.
//
// Semantics: impl/torch/functions/functions_ext.cpp:43-64 and
// impl/torch/functions/functions_ext/rotary.cu:14-46 of the reference (Python statement:
// customized_test.py:374-390).  The last dimension of x is split into halves x1 | x2;
// cos and sin broadcast, right-aligned, against x1; the products are formed in fp32 (also for
// fp64 tensors, which the reference narrows with static_cast<float>) and rounded once:
//   conj == false: o1 = x1*c - x2*s,  o2 = x1*s + x2*c
//   conj == true : o1 = x1*c + x2*s,  o2 = -x1*s + x2*c
// interleaved == true is not implemented by the reference and returns diopiNoImplement here too.
//
// Two kernels:
//  * rotaryRows: the LLaMA layout.  x is viewed as [outer, A, B, D]; cos/sin are dense [A, D/2]
//    tables shared by the B heads of a position (and by every `outer` slice).  A lane owns one
//    16-byte packet position of the half-row of one head (kHeadsPerLane heads; one measured
//    fastest: short-lived lanes with two loads of x in flight each), so every global access is a
//    128-bit one and the small tables come from the cache.
//  * rotaryGeneric: any right-aligned broadcast of cos/sin, element by element.
#include "common.hpp"
#include "device.hpp"

namespace rocm {
namespace {

constexpr int kRotThreads = 256;
constexpr int kHeadsPerLane = 1;  // heads a lane rotates with one pair of table packets: 1 / 2 / 4 / 8 measured 85.4 / 86.3 / 89.0 / 90.1 us at [16384, 32, 128] bf16 x 2 tensors

template <typename T>
__device__ __forceinline__ void rotatePair(float x1, float x2, float c, float s, bool conj, T* o1, T* o2) {
    if (!conj) {
        *o1 = static_cast<T>(x1 * c - x2 * s);
        *o2 = static_cast<T>(x1 * s + x2 * c);
    } else {
        *o1 = static_cast<T>(x1 * c + x2 * s);
        *o2 = static_cast<T>(-x1 * s + x2 * c);
    }
}

// x, out: [rowsA * B, D] dense, where row r uses table row (r / B) % A.  packetsPerHalf = (D/2) / EPV.
template <typename T>
__global__ __launch_bounds__(kRotThreads) void rotaryRows(T* __restrict__ out, const T* __restrict__ x, const T* __restrict__ cosT, const T* __restrict__ sinT,
                                                          int64_t posTotal, int64_t A, int B, int half, int packetsPerHalf, int headChunks, bool conj) {
    constexpr int EPV = Pack16<T>::N;
    // work item = (position, head chunk, packet); packet is the fastest index so that lanes of a wave
    // read consecutive 16-byte packets of one half-row
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kRotThreads + threadIdx.x;
    const int64_t itemsTotal = posTotal * headChunks * packetsPerHalf;
    if (item >= itemsTotal) return;
    const int pk = static_cast<int>(item % packetsPerHalf);
    const int64_t rest = item / packetsPerHalf;
    const int hc = static_cast<int>(rest % headChunks);
    const int64_t pos = rest / headChunks;
    const int64_t tableRow = pos % A;

    const Pack16<T> cv = loadPack(cosT + tableRow * half + pk * EPV);
    const Pack16<T> sv = loadPack(sinT + tableRow * half + pk * EPV);
    float c[EPV], s[EPV];
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
        c[e] = static_cast<float>(cv.e[e]);
        s[e] = static_cast<float>(sv.e[e]);
    }
    const int D = 2 * half;
    const int h0 = hc * kHeadsPerLane;
    Pack16<T> a[kHeadsPerLane], b[kHeadsPerLane];
#pragma unroll
    for (int i = 0; i < kHeadsPerLane; ++i) {
        if (h0 + i < B) {
            const T* row = x + (pos * B + h0 + i) * D;
            a[i] = loadPackStream(row + pk * EPV);
            b[i] = loadPackStream(row + half + pk * EPV);
        }
    }
#pragma unroll
    for (int i = 0; i < kHeadsPerLane; ++i) {
        if (h0 + i < B) {
            Pack16<T> o1, o2;
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                rotatePair<T>(static_cast<float>(a[i].e[e]), static_cast<float>(b[i].e[e]), c[e], s[e], conj, &o1.e[e], &o2.e[e]);
            }
            T* orow = out + (pos * B + h0 + i) * D;
            storePackStream(orow + pk * EPV, o1);
            storePackStream(orow + half + pk * EPV, o2);
        }
    }
}

struct BroadcastDims {
    int ndim;
    int64_t shape[kMaxDims];      // shape of x1 (x with the last extent halved)
    int64_t cosStride[kMaxDims];  // element strides of cos / sin per x1 dimension, 0 where broadcast
    int64_t sinStride[kMaxDims];
};

template <typename T>
__global__ __launch_bounds__(kRotThreads) void rotaryGeneric(T* __restrict__ out, const T* __restrict__ x, const T* __restrict__ cosT, const T* __restrict__ sinT,
                                                             BroadcastDims dims, int64_t total, bool conj) {
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kRotThreads + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * kRotThreads) {
        int64_t rem = i, co = 0, so = 0, col = 0, row = 0;
        int64_t rowMul = 1;
        for (int d = dims.ndim - 1; d >= 0; --d) {
            const int64_t idx = rem % dims.shape[d];
            rem /= dims.shape[d];
            co += idx * dims.cosStride[d];
            so += idx * dims.sinStride[d];
            if (d == dims.ndim - 1) {
                col = idx;
            } else {
                row += idx * rowMul;
                rowMul *= dims.shape[d];
            }
        }
        const int64_t half = dims.shape[dims.ndim - 1];
        const int64_t base = row * 2 * half + col;
        T o1, o2;
        rotatePair<T>(static_cast<float>(x[base]), static_cast<float>(x[base + half]), static_cast<float>(cosT[co]), static_cast<float>(sinT[so]), conj, &o1,
                      &o2);
        out[base] = o1;
        out[base + half] = o2;
    }
}

// Strides of `t` seen from the dimensions of x1 (right-aligned), 0 where t broadcasts.
diopiError_t broadcastStrides(const TensorView& t, const char* name, int ndim, const int64_t* x1Shape, int64_t* strides) {
    ROCM_CHECK(t.ndim <= ndim, "%s has rank %d, more than x (%d)", name, t.ndim, ndim);
    for (int d = 0; d < ndim; ++d) {
        const int td = d - (ndim - t.ndim);
        if (td < 0) {
            strides[d] = 0;
            continue;
        }
        if (t.shape[td] == x1Shape[d]) {
            strides[d] = t.shape[td] == 1 ? 0 : t.stride[td];
        } else {
            ROCM_CHECK(t.shape[td] == 1, "%s extent %lld in dimension %d does not broadcast against %lld", name, static_cast<long long>(t.shape[td]), td,
                       static_cast<long long>(x1Shape[d]));
            strides[d] = 0;
        }
    }
    return diopiSuccess;
}

// Recognises cos (and sin) as a dense [A, half] table indexed by x1's dimension `ia`, shared by the
// B = prod(dims between ia and the last) heads and by everything outside.
bool tableLayout(const BroadcastDims& d, int64_t* A, int64_t* B) {
    const int n = d.ndim;
    const int64_t half = d.shape[n - 1];
    for (int which = 0; which < 2; ++which) {
        const int64_t* st = which ? d.sinStride : d.cosStride;
        if (half != 1 && st[n - 1] != 1) return false;
    }
    // find the innermost non-last dimension that cos actually varies along
    int ia = -1;
    for (int i = n - 2; i >= 0; --i) {
        if (d.shape[i] != 1 && (d.cosStride[i] != 0 || d.sinStride[i] != 0)) {
            ia = i;
            break;
        }
    }
    int64_t b = 1;
    for (int i = n - 2; i > ia; --i) b *= d.shape[i];
    if (ia < 0) {
        *A = 1;
        *B = b;
        return true;
    }
    // dimensions ia, ia-1, ... must form one dense run over the table (row stride = half), possibly followed by
    // pure broadcast dimensions further out
    int64_t a = 1;
    int i = ia;
    for (; i >= 0; --i) {
        if (d.shape[i] == 1) continue;
        if (d.cosStride[i] == 0 && d.sinStride[i] == 0) break;
        if (d.cosStride[i] != a * half || d.sinStride[i] != a * half) return false;
        a *= d.shape[i];
    }
    for (; i >= 0; --i) {
        if (d.shape[i] != 1 && (d.cosStride[i] != 0 || d.sinStride[i] != 0)) return false;
    }
    *A = a;
    *B = b;
    return true;
}

template <typename T>
diopiError_t launchTyped(hipStream_t stream, const TensorView& out, const TensorView& x, const TensorView& cosT, const TensorView& sinT,
                         const BroadcastDims& dims, bool conj) {
    constexpr int EPV = Pack16<T>::N;
    const int64_t half = dims.shape[dims.ndim - 1];
    const int64_t total = x.numel / 2;
    int64_t A = 0, B = 0;
    const bool aligned = ((reinterpret_cast<uintptr_t>(x.data) | reinterpret_cast<uintptr_t>(out.data) | reinterpret_cast<uintptr_t>(cosT.data) |
                           reinterpret_cast<uintptr_t>(sinT.data)) &
                          15) == 0;
    if (aligned && half % EPV == 0 && half <= (1 << 20) && tableLayout(dims, &A, &B) && B <= INT32_MAX) {
        const int packetsPerHalf = static_cast<int>(half / EPV);
        const int headChunks = static_cast<int>(ceilDiv(B, kHeadsPerLane));
        const int64_t posTotal = total / half / B;
        const int64_t items = posTotal * headChunks * packetsPerHalf;
        const int64_t blocks = ceilDiv(items, kRotThreads);
        ROCM_CHECK(blocks <= INT32_MAX, "rotary embedding: tensor too large for one launch");
        hipLaunchKernelGGL(rotaryRows<T>, dim3(static_cast<unsigned>(blocks)), dim3(kRotThreads), 0, stream, static_cast<T*>(out.data),
                           static_cast<const T*>(x.data), static_cast<const T*>(cosT.data), static_cast<const T*>(sinT.data), posTotal, A,
                           static_cast<int>(B), static_cast<int>(half), packetsPerHalf, headChunks, conj);
        ROCM_LAUNCH_CHECK();
        return diopiSuccess;
    }
    int64_t blocks = ceilDiv(total, kRotThreads);
    const int64_t cap = static_cast<int64_t>(deviceInfo().numCU) * 32;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(rotaryGeneric<T>, dim3(static_cast<unsigned>(blocks)), dim3(kRotThreads), 0, stream, static_cast<T*>(out.data),
                       static_cast<const T*>(x.data), static_cast<const T*>(cosT.data), static_cast<const T*>(sinT.data), dims, total, conj);
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

}  // namespace
}  // namespace rocm

extern "C" diopiError_t diopiRotaryEmbedding(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t x, diopiConstTensorHandle_t cos,
                                             diopiConstTensorHandle_t sin, const bool conj, const bool interleaved) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    if (interleaved) {
        // same behaviour and wording as functions_ext.cpp:45-48 of the reference
        setLastError("interleaved rotary embedding is not supported yet");
        return diopiNoImplement;
    }
    TensorView vOut, vX, vCos, vSin;
    ROCM_CALL(unwrap(out, "out", &vOut));
    ROCM_CALL(unwrap(x, "x", &vX));
    ROCM_CALL(unwrap(cos, "cos", &vCos));
    ROCM_CALL(unwrap(sin, "sin", &vSin));
    ROCM_CALL(requireDeviceContiguous(vOut, "out"));
    ROCM_CALL(requireDeviceContiguous(vX, "x"));
    ROCM_CHECK(vCos.device == diopi_device && vSin.device == diopi_device, "cos and sin must live in device memory");
    ROCM_CHECK(isFloatDtype(vX.dtype), "dtype %s is not supported", dtypeName(vX.dtype));
    ROCM_CHECK(vOut.dtype == vX.dtype && vCos.dtype == vX.dtype && vSin.dtype == vX.dtype, "out, x, cos and sin must share one dtype (x is %s)",
               dtypeName(vX.dtype));
    ROCM_CHECK(vOut.sameShape(vX), "out must have the shape of x");
    ROCM_CHECK(vX.ndim >= 1, "x must have at least one dimension");
    ROCM_CHECK(vX.shape[vX.ndim - 1] % 2 == 0, "the last dimension of x (%lld) must be even", static_cast<long long>(vX.shape[vX.ndim - 1]));

    BroadcastDims dims;
    dims.ndim = vX.ndim;
    for (int d = 0; d < vX.ndim; ++d) dims.shape[d] = vX.shape[d];
    dims.shape[vX.ndim - 1] /= 2;
    ROCM_CALL(broadcastStrides(vCos, "cos", dims.ndim, dims.shape, dims.cosStride));
    ROCM_CALL(broadcastStrides(vSin, "sin", dims.ndim, dims.shape, dims.sinStride));
    if (vX.numel == 0) return diopiSuccess;

    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    switch (vX.dtype) {
        case diopi_dtype_float16: return launchTyped<half_t>(stream, vOut, vX, vCos, vSin, dims, conj);
        case diopi_dtype_bfloat16: return launchTyped<bf16_t>(stream, vOut, vX, vCos, vSin, dims, conj);
        case diopi_dtype_float32: return launchTyped<float>(stream, vOut, vX, vCos, vSin, dims, conj);
        case diopi_dtype_float64: return launchTyped<double>(stream, vOut, vX, vCos, vSin, dims, conj);
        default: break;
    }
    setLastError("diopiRotaryEmbedding: dtype %s is not supported", dtypeName(vX.dtype));
    return diopiDtypeNotSupported;
    ROCM_ENTRY_END
}
