// diopiRotaryEmbeddingV2 for gfx950: rotates query and key in place, both in one launch.
//
// Semantics: proto/include/diopi/functions_ext.h:649-650 of the reference; its statement is the Python function
// rotary_emb_v2 (diopi_test/python/conformance/customized_test.py:843-852), the torch implementation has no body for
// this operator.  query [T, Hq * dim] and key [T, Hk * dim] are viewed as [T, heads, dim]; cos and sin hold T * dim
// elements ([T, 1, dim] in the reference's cases, diopi_configs.py:9107-9135) and are shared by the heads of a token:
//   out[.., d]         = x[.., d]         * cos[d]         - x[.., d + dim/2] * sin[d]              d < dim/2
//   out[.., d + dim/2] = x[.., d + dim/2] * cos[d + dim/2] + x[.., d]         * sin[d + dim/2]
// i.e. x * cos + rotate_half(x) * sin with full-width tables (the two halves of cos / sin need not be equal).
// Products and the sum are formed in fp32 (fp64 for fp64 tensors) and rounded once; the Python statement rounds each
// product and the sum in the tensor dtype, which differs by at most two roundings of the element type.
//
// Kernel: a lane owns one 16-byte packet position p of the half-row (dims p*EPV .. +EPV-1 and the same + dim/2) of one
// head of query or key and reads the four table packets of its token for it (the tables are small and stay in cache): every
// global access is a 128-bit one, and a lane has two loads of the tensor in flight, not more, which is what the memory
// system streams fastest here (see kRot2HeadsPerLane).  Shapes that do not fit take an element-wise kernel.
#include "common.hpp"
#include "device.hpp"

namespace rocm {
namespace {

constexpr int kRot2Threads = 256;
constexpr int kRot2HeadsPerLane = 1;  // heads a lane rotates with one pair of table packets: 1 / 2 / 4 measured 83.1 / 88.7 / 91.0 us at [16384, 32, 128] bf16, query and key

template <typename T>
__device__ __forceinline__ T* headRow(T* q, T* k, int64_t t, int h, int hq, int hk, int dim) {
    return h < hq ? q + (t * hq + h) * dim : k + (t * hk + (h - hq)) * dim;
}

template <typename T>
__global__ __launch_bounds__(kRot2Threads) void rotaryV2Rows(T* __restrict__ q, T* __restrict__ k, const T* __restrict__ cosT, const T* __restrict__ sinT,
                                                            int64_t tokens, int hq, int hk, int dim, int packetsPerHalf, int headChunks) {
    using Acc = typename AccType<T>::type;
    constexpr int EPV = Pack16<T>::N;
    // work item = (token, head chunk, packet); packet is the fastest index so that lanes read consecutive packets
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kRot2Threads + threadIdx.x;
    if (item >= tokens * headChunks * packetsPerHalf) return;
    const int pk = static_cast<int>(item % packetsPerHalf);
    const int64_t rest = item / packetsPerHalf;
    const int hc = static_cast<int>(rest % headChunks);
    const int64_t t = rest / headChunks;
    const int half = dim / 2;

    const Pack16<T> c1 = loadPack(cosT + t * dim + pk * EPV), c2 = loadPack(cosT + t * dim + half + pk * EPV);
    const Pack16<T> s1 = loadPack(sinT + t * dim + pk * EPV), s2 = loadPack(sinT + t * dim + half + pk * EPV);
    const int h0 = hc * kRot2HeadsPerLane;
    Pack16<T> a[kRot2HeadsPerLane], b[kRot2HeadsPerLane];
#pragma unroll
    for (int i = 0; i < kRot2HeadsPerLane; ++i) {
        if (h0 + i < hq + hk) {
            const T* row = headRow<T>(q, k, t, h0 + i, hq, hk, dim);
            a[i] = loadPackStream(row + pk * EPV);
            b[i] = loadPackStream(row + half + pk * EPV);
        }
    }
#pragma unroll
    for (int i = 0; i < kRot2HeadsPerLane; ++i) {
        if (h0 + i < hq + hk) {
            Pack16<T> o1, o2;
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                const Acc x1 = static_cast<Acc>(a[i].e[e]), x2 = static_cast<Acc>(b[i].e[e]);
                o1.e[e] = static_cast<T>(x1 * static_cast<Acc>(c1.e[e]) - x2 * static_cast<Acc>(s1.e[e]));
                o2.e[e] = static_cast<T>(x1 * static_cast<Acc>(s2.e[e]) + x2 * static_cast<Acc>(c2.e[e]));
            }
            T* row = headRow<T>(q, k, t, h0 + i, hq, hk, dim);
            storePackStream(row + pk * EPV, o1);
            storePackStream(row + half + pk * EPV, o2);
        }
    }
}

// Any even dim, any alignment: one thread per (token, head, d < dim/2).
template <typename T>
__global__ __launch_bounds__(kRot2Threads) void rotaryV2Generic(T* __restrict__ q, T* __restrict__ k, const T* __restrict__ cosT, const T* __restrict__ sinT,
                                                               int64_t tokens, int hq, int hk, int dim) {
    using Acc = typename AccType<T>::type;
    const int half = dim / 2;
    const int64_t total = tokens * (hq + hk) * half;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kRot2Threads + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * kRot2Threads) {
        const int d = static_cast<int>(i % half);
        const int64_t rest = i / half;
        const int h = static_cast<int>(rest % (hq + hk));
        const int64_t t = rest / (hq + hk);
        T* row = headRow<T>(q, k, t, h, hq, hk, dim);
        const Acc x1 = static_cast<Acc>(row[d]), x2 = static_cast<Acc>(row[d + half]);
        row[d] = static_cast<T>(x1 * static_cast<Acc>(cosT[t * dim + d]) - x2 * static_cast<Acc>(sinT[t * dim + d]));
        row[d + half] = static_cast<T>(x1 * static_cast<Acc>(sinT[t * dim + half + d]) + x2 * static_cast<Acc>(cosT[t * dim + half + d]));
    }
}

template <typename T>
diopiError_t launchV2(hipStream_t stream, const TensorView& q, const TensorView& k, const TensorView& c, const TensorView& s, int64_t tokens, int hq, int hk,
                      int dim) {
    constexpr int EPV = Pack16<T>::N;
    const int half = dim / 2;
    const bool aligned = ((reinterpret_cast<uintptr_t>(q.data) | reinterpret_cast<uintptr_t>(k.data) | reinterpret_cast<uintptr_t>(c.data) |
                           reinterpret_cast<uintptr_t>(s.data)) & 15) == 0;
    if (aligned && half % EPV == 0) {
        const int packetsPerHalf = half / EPV;
        const int headChunks = static_cast<int>(ceilDiv(hq + hk, kRot2HeadsPerLane));
        const int64_t items = tokens * headChunks * packetsPerHalf;
        const int64_t blocks = ceilDiv(items, kRot2Threads);
        ROCM_CHECK(blocks <= INT32_MAX, "rotary embedding: too many elements for one launch");
        hipLaunchKernelGGL(rotaryV2Rows<T>, dim3(static_cast<unsigned>(blocks)), dim3(kRot2Threads), 0, stream, static_cast<T*>(q.data),
                           static_cast<T*>(k.data), static_cast<const T*>(c.data), static_cast<const T*>(s.data), tokens, hq, hk, dim, packetsPerHalf,
                           headChunks);
    } else {
        const int64_t total = tokens * (hq + hk) * half;
        int64_t blocks = ceilDiv(total, kRot2Threads);
        if (blocks > 65536) blocks = 65536;
        hipLaunchKernelGGL(rotaryV2Generic<T>, dim3(static_cast<unsigned>(blocks)), dim3(kRot2Threads), 0, stream, static_cast<T*>(q.data),
                           static_cast<T*>(k.data), static_cast<const T*>(c.data), static_cast<const T*>(s.data), tokens, hq, hk, dim);
    }
    ROCM_LAUNCH_CHECK();
    return diopiSuccess;
}

}  // namespace
}  // namespace rocm

extern "C" diopiError_t diopiRotaryEmbeddingV2(diopiContextHandle_t ctx, diopiTensorHandle_t query, diopiTensorHandle_t key, diopiConstTensorHandle_t cos,
                                               diopiConstTensorHandle_t sin, int64_t dim) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    TensorView vQ, vK, vCos, vSin;
    ROCM_CALL(unwrap(query, "query", &vQ));
    ROCM_CALL(unwrap(key, "key", &vK));
    ROCM_CALL(unwrap(cos, "cos", &vCos));
    ROCM_CALL(unwrap(sin, "sin", &vSin));
    ROCM_CALL(requireDeviceContiguous(vQ, "query"));
    ROCM_CALL(requireDeviceContiguous(vK, "key"));
    ROCM_CALL(requireDeviceContiguous(vCos, "cos"));
    ROCM_CALL(requireDeviceContiguous(vSin, "sin"));
    ROCM_CHECK(isFloatDtype(vQ.dtype), "dtype %s is not supported", dtypeName(vQ.dtype));
    ROCM_CHECK(vK.dtype == vQ.dtype && vCos.dtype == vQ.dtype && vSin.dtype == vQ.dtype, "query, key, cos and sin must share one dtype (query is %s)",
               dtypeName(vQ.dtype));
    ROCM_CHECK(dim > 0 && dim % 2 == 0 && dim <= (1 << 20), "dim %lld must be positive and even", static_cast<long long>(dim));
    ROCM_CHECK(vQ.ndim >= 1 && vK.ndim >= 1 && vQ.shape[0] == vK.shape[0], "query and key must have the same number of tokens in dimension 0");
    const int64_t tokens = vQ.shape[0];
    if (tokens == 0 || (vQ.numel == 0 && vK.numel == 0)) return diopiSuccess;
    const int64_t perTokenQ = vQ.numel / tokens, perTokenK = vK.numel / tokens;
    ROCM_CHECK(perTokenQ % dim == 0 && perTokenK % dim == 0, "query (%lld per token) and key (%lld per token) must hold whole heads of %lld elements",
               static_cast<long long>(perTokenQ), static_cast<long long>(perTokenK), static_cast<long long>(dim));
    ROCM_CHECK(vCos.numel == tokens * dim && vSin.numel == tokens * dim, "cos and sin must hold tokens * dim = %lld elements (cos %lld, sin %lld)",
               static_cast<long long>(tokens * dim), static_cast<long long>(vCos.numel), static_cast<long long>(vSin.numel));
    const int64_t hq = perTokenQ / dim, hk = perTokenK / dim;
    ROCM_CHECK(hq + hk <= INT32_MAX / 2, "too many heads");

    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    const int ihq = static_cast<int>(hq), ihk = static_cast<int>(hk), idim = static_cast<int>(dim);
    switch (vQ.dtype) {
        case diopi_dtype_float16: return launchV2<half_t>(stream, vQ, vK, vCos, vSin, tokens, ihq, ihk, idim);
        case diopi_dtype_bfloat16: return launchV2<bf16_t>(stream, vQ, vK, vCos, vSin, tokens, ihq, ihk, idim);
        case diopi_dtype_float32: return launchV2<float>(stream, vQ, vK, vCos, vSin, tokens, ihq, ihk, idim);
        case diopi_dtype_float64: return launchV2<double>(stream, vQ, vK, vCos, vSin, tokens, ihq, ihk, idim);
        default: break;
    }
    setLastError("diopiRotaryEmbeddingV2: dtype %s is not supported", dtypeName(vQ.dtype));
    return diopiDtypeNotSupported;
    ROCM_ENTRY_END
}
