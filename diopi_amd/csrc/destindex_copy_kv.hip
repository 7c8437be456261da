// diopiDestIndexCopyKV for gfx950: out[dest_loc[t], :, :] = k[t, :, :].
//
// Semantics follow impl/torch/functions/functions_lightllm.cpp:18-26 of the reference
// (a non-accumulating index_put_ along dimension 0) and its Python statement
// customized_test.py:694-696 (out[dest_loc] = k).  The copy is bit-exact: rows are moved as
// raw bytes, never through an arithmetic type.
//
// Layout: k is [T, ...] and out is [R, ...] with identical trailing dimensions, both dense, so a
// token is one contiguous row of `rowBytes` bytes.  One work-group column copies one row with
// 16-byte accesses; consecutive lanes touch consecutive 16-byte packets, so both the gather side
// and the scatter side are fully coalesced within a row.
#include "common.hpp"
#include "device.hpp"

namespace rocm {
namespace {

constexpr int kCopyThreads = 256;

// UNIT is the widest power-of-two access (16, 8, 4, 2 or 1 bytes) that divides the row size and
// both base addresses.
template <typename UNIT>
__global__ __launch_bounds__(kCopyThreads) void destIndexCopyKernel(UNIT* __restrict__ out, const UNIT* __restrict__ src, const void* __restrict__ destLoc,
                                                                    bool idx64, int64_t numTokens, int64_t numRows, int64_t unitsPerRow) {
    const int64_t t = blockIdx.y;
    if (t >= numTokens) return;
    int64_t dest = loadIndex(destLoc, t, idx64);
    if (dest < 0) dest += numRows;             // index_put_ wraps negative indices once
    if (dest < 0 || dest >= numRows) return;   // never write outside the cache
    const UNIT* s = src + t * unitsPerRow;
    UNIT* d = out + dest * unitsPerRow;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kCopyThreads + threadIdx.x; i < unitsPerRow; i += static_cast<int64_t>(gridDim.x) * kCopyThreads) {
        d[i] = s[i];
    }
}

template <typename UNIT>
diopiError_t launchCopy(hipStream_t stream, void* out, const void* src, const void* destLoc, bool idx64, int64_t numTokens, int64_t numRows,
                        int64_t rowBytes) {
    const int64_t unitsPerRow = rowBytes / static_cast<int64_t>(sizeof(UNIT));
    int64_t gx = ceilDiv(unitsPerRow, kCopyThreads);
    if (gx > 64) gx = 64;
    // gridDim.y is limited to 65535: walk the token axis in slabs
    const int64_t kMaxY = 65535;
    for (int64_t t0 = 0; t0 < numTokens; t0 += kMaxY) {
        const int64_t ny = (numTokens - t0 < kMaxY) ? numTokens - t0 : kMaxY;
        const void* loc = idx64 ? static_cast<const void*>(static_cast<const int64_t*>(destLoc) + t0)
                                : static_cast<const void*>(static_cast<const int32_t*>(destLoc) + t0);
        hipLaunchKernelGGL(destIndexCopyKernel<UNIT>, dim3(static_cast<unsigned>(gx), static_cast<unsigned>(ny)), dim3(kCopyThreads), 0, stream,
                           static_cast<UNIT*>(out), static_cast<const UNIT*>(src) + t0 * unitsPerRow, loc, idx64, ny, numRows, unitsPerRow);
        ROCM_LAUNCH_CHECK();
    }
    return diopiSuccess;
}

}  // namespace
}  // namespace rocm

extern "C" diopiError_t diopiDestIndexCopyKV(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t k, diopiConstTensorHandle_t dest_loc) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    TensorView vOut, vK, vLoc;
    ROCM_CALL(unwrap(out, "out", &vOut));
    ROCM_CALL(unwrap(k, "k", &vK));
    ROCM_CALL(unwrap(dest_loc, "dest_loc", &vLoc));
    ROCM_CALL(requireDeviceContiguous(vOut, "out"));
    ROCM_CALL(requireDeviceContiguous(vK, "k"));
    ROCM_CALL(requireDeviceContiguous(vLoc, "dest_loc"));
    ROCM_CHECK(vOut.dtype == vK.dtype, "out (%s) and k (%s) must have the same dtype", dtypeName(vOut.dtype), dtypeName(vK.dtype));
    ROCM_CHECK(vOut.itemsize() > 0, "dtype %s is not supported", dtypeName(vOut.dtype));
    ROCM_CHECK(isIndexDtype(vLoc.dtype), "dest_loc must be int32 or int64, got %s", dtypeName(vLoc.dtype));
    ROCM_CHECK(vLoc.ndim == 1, "dest_loc must be one-dimensional, got rank %d", vLoc.ndim);
    ROCM_CHECK(vK.ndim >= 1 && vOut.ndim == vK.ndim, "k and out must have the same rank (>= 1), got %d and %d", vK.ndim, vOut.ndim);
    ROCM_CHECK(vLoc.shape[0] == vK.shape[0], "dest_loc has %lld entries but k has %lld rows", static_cast<long long>(vLoc.shape[0]),
               static_cast<long long>(vK.shape[0]));
    int64_t rowElems = 1;
    for (int i = 1; i < vK.ndim; ++i) {
        ROCM_CHECK(vK.shape[i] == vOut.shape[i], "k and out differ in dimension %d (%lld vs %lld)", i, static_cast<long long>(vK.shape[i]),
                   static_cast<long long>(vOut.shape[i]));
        rowElems *= vK.shape[i];
    }
    const int64_t numTokens = vK.shape[0];
    const int64_t numRows = vOut.shape[0];
    const int64_t rowBytes = rowElems * vK.itemsize();
    if (numTokens == 0 || rowBytes == 0 || numRows == 0) return diopiSuccess;

    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    const bool idx64 = vLoc.dtype == diopi_dtype_int64;
    const uintptr_t align = reinterpret_cast<uintptr_t>(vOut.data) | reinterpret_cast<uintptr_t>(vK.data) | static_cast<uintptr_t>(rowBytes);
    if (align % 16 == 0) return launchCopy<u32x4>(stream, vOut.data, vK.data, vLoc.data, idx64, numTokens, numRows, rowBytes);
    if (align % 8 == 0) return launchCopy<uint64_t>(stream, vOut.data, vK.data, vLoc.data, idx64, numTokens, numRows, rowBytes);
    if (align % 4 == 0) return launchCopy<uint32_t>(stream, vOut.data, vK.data, vLoc.data, idx64, numTokens, numRows, rowBytes);
    if (align % 2 == 0) return launchCopy<uint16_t>(stream, vOut.data, vK.data, vLoc.data, idx64, numTokens, numRows, rowBytes);
    return launchCopy<uint8_t>(stream, vOut.data, vK.data, vLoc.data, idx64, numTokens, numRows, rowBytes);
    ROCM_ENTRY_END
}
