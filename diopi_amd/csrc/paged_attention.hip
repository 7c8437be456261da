// diopiPagedAttention for gfx950: one decode step of attention over a KV cache that is cut into blocks.
//
// Interface: proto/include/diopi/functions_ext.h:602-618 of the reference; Python statement
// customized_test.py:782-821 (the only implementation the reference holds is the Ascend one).  query and out are
// [batch, num_heads * dim]; key and value are [rows, num_kv_heads * dim]; token t of sequence i lives in row
//   block_table[i, t / block_size] * block_size + t % block_size
// and sequence i has actual_seq_lengths[i] tokens (a host-side list).  out[i, h] = softmax(q[i, h] . K_i^T / sqrt(dim)) V_i.
// The statement covers one sequence whose blocks are 0, 1, ... in order (its token t is row t), which is what the rule
// above gives for the reference's case (block table [[0, 1]]).  Like the statement, attenMask is not read: a decode
// step attends to every cached token.
//
// The work is the two decode kernels of the lightllm operators (score rows, then softmax and the product with V): a
// small kernel expands the block table into the per-token row table those kernels read, and the scores of all heads
// go through a scratch tensor of the element type, as they do between the two lightllm operators.  Nothing is copied
// from the device to the host and the host never waits; the sequence lengths travel in kernel arguments.
#include <vector>

#include "common.hpp"
#include "decode.hpp"
#include "device.hpp"

namespace rocm {
namespace {

constexpr int kSeqPerLaunch = 64;  // sequence lengths and score offsets a launch carries in its arguments
constexpr int kSlotThreads = 256;

struct PagedChunk {
    int32_t len[kSeqPerLaunch];
    int32_t start[kSeqPerLaunch];
};

// Row table of the decode kernels: sequence i owns loc[i, maxLen - L_i : maxLen], oldest token first.
__global__ __launch_bounds__(kSlotThreads) void pagedSlots(int32_t* __restrict__ loc, int32_t* __restrict__ startOut, int32_t* __restrict__ lenOut,
                                                           const void* __restrict__ table, bool table64, int64_t tableStride, PagedChunk c, int base,
                                                           int maxLen, int64_t blockSize, int64_t rows) {
    const int i = blockIdx.y;
    const int seq = base + i;
    const int L = c.len[i];
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        startOut[seq] = c.start[i];
        lenOut[seq] = L;
    }
    for (int t = blockIdx.x * kSlotThreads + threadIdx.x; t < maxLen; t += gridDim.x * kSlotThreads) {
        const int tok = t - (maxLen - L);
        int64_t row = 0;
        if (tok >= 0) {
            row = loadIndex(table, seq * tableStride + tok / blockSize, table64) * blockSize + tok % blockSize;
            row = row < 0 ? 0 : (row >= rows ? rows - 1 : row);  // a bad block number must not leave the cache
        }
        loc[static_cast<int64_t>(seq) * maxLen + t] = static_cast<int32_t>(row);
    }
}

TensorView viewOf(void* data, diopiDtype_t dtype, std::initializer_list<int64_t> dims) {
    TensorView v;
    v.data = data;
    v.dtype = dtype;
    v.device = diopi_device;
    v.ndim = static_cast<int>(dims.size());
    int d = 0;
    v.numel = 1;
    for (int64_t s : dims) {
        v.shape[d++] = s;
        v.numel *= s;
    }
    int64_t stride = 1;
    for (int k = v.ndim - 1; k >= 0; --k) {
        v.stride[k] = stride;
        stride *= v.shape[k];
    }
    return v;
}

int64_t roundUp256(int64_t x) { return (x + 255) / 256 * 256; }

}  // namespace
}  // namespace rocm

extern "C" diopiError_t diopiPagedAttention(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t q, diopiConstTensorHandle_t k,
                                            diopiConstTensorHandle_t v, diopiConstTensorHandle_t attenMask, diopiSize_t actual_seq_lengths, int64_t num_heads,
                                            int64_t num_kv_heads, int64_t dim, diopiConstTensorHandle_t block_table, int64_t block_size) {
    ROCM_ENTRY_BEGIN
    using namespace rocm;
    (void)attenMask;  // not read by the reference's statement either (customized_test.py:782-821)
    TensorView vOut, vQ, vK, vV, vTable;
    ROCM_CALL(unwrap(out, "out", &vOut));
    ROCM_CALL(unwrap(q, "q", &vQ));
    ROCM_CALL(unwrap(k, "k", &vK));
    ROCM_CALL(unwrap(v, "v", &vV));
    ROCM_CALL(unwrap(block_table, "block_table", &vTable));
    ROCM_CALL(requireDeviceContiguous(vOut, "out"));
    ROCM_CALL(requireDeviceContiguous(vQ, "q"));
    ROCM_CALL(requireDeviceContiguous(vK, "k"));
    ROCM_CALL(requireDeviceContiguous(vV, "v"));
    ROCM_CALL(requireDeviceContiguous(vTable, "block_table"));
    ROCM_CHECK(num_heads > 0 && num_kv_heads > 0 && dim > 0 && num_heads % num_kv_heads == 0 && num_heads <= 65535 && dim <= 65535,
               "num_heads %lld must be a positive multiple of num_kv_heads %lld, dim %lld positive", static_cast<long long>(num_heads),
               static_cast<long long>(num_kv_heads), static_cast<long long>(dim));
    ROCM_CHECK(block_size > 0, "block_size must be positive, got %lld", static_cast<long long>(block_size));
    ROCM_CHECK(actual_seq_lengths.len >= 0 && (actual_seq_lengths.len == 0 || actual_seq_lengths.data != nullptr), "actual_seq_lengths is malformed");
    const int64_t batch = actual_seq_lengths.len;
    ROCM_CHECK(batch <= 65535, "batch size %lld exceeds the launch limit of 65535", static_cast<long long>(batch));
    ROCM_CHECK(vQ.ndim == 2 && vQ.shape[0] == batch && vQ.shape[1] == num_heads * dim, "q must be [batch, num_heads * dim] = [%lld, %lld]",
               static_cast<long long>(batch), static_cast<long long>(num_heads * dim));
    ROCM_CHECK(vOut.sameShape(vQ), "out must have the shape of q");
    ROCM_CHECK(vK.ndim == 2 && vK.shape[1] == num_kv_heads * dim && vV.sameShape(vK), "k and v must be [rows, num_kv_heads * dim] = [rows, %lld]",
               static_cast<long long>(num_kv_heads * dim));
    ROCM_CHECK(vK.shape[0] <= INT32_MAX, "the cache has too many rows for 32-bit row numbers");
    ROCM_CHECK(isFloatDtype(vQ.dtype) && vK.dtype == vQ.dtype && vV.dtype == vQ.dtype && vOut.dtype == vQ.dtype,
               "q, k, v and out must share one floating dtype (q is %s)", dtypeName(vQ.dtype));
    ROCM_CHECK(vTable.ndim == 2 && vTable.shape[0] == batch && isIndexDtype(vTable.dtype), "block_table must be an int32 or int64 tensor [batch, blocks]");
    if (batch == 0) return diopiSuccess;
    ROCM_CHECK(vK.shape[0] > 0, "the cache has no rows");

    // per-sequence bookkeeping of the decode kernels, worked out on the host from the host-side list
    std::vector<int32_t> lens(batch), starts(batch);
    int64_t total = 0, maxLen = 0;
    for (int64_t i = 0; i < batch; ++i) {
        const int64_t L = actual_seq_lengths.data[i];
        ROCM_CHECK(L >= 0 && L <= vTable.shape[1] * block_size, "sequence %lld has %lld tokens but block_table holds %lld blocks of %lld",
                   static_cast<long long>(i), static_cast<long long>(L), static_cast<long long>(vTable.shape[1]), static_cast<long long>(block_size));
        ROCM_CHECK(total + L <= INT32_MAX, "the sequences hold too many tokens for one call");
        lens[i] = static_cast<int32_t>(L);
        starts[i] = static_cast<int32_t>(total);
        total += L;
        maxLen = L > maxLen ? L : maxLen;
    }
    hipStream_t stream;
    ROCM_CALL(getStream(ctx, &stream));
    if (total == 0) return zeroFill(stream, vOut.data, vOut.nbytes());  // nothing cached: nothing to attend to

    const int64_t locBytes = roundUp256(batch * maxLen * 4), metaBytes = roundUp256(batch * 4);
    const int64_t logitBytes = roundUp256(num_heads * total * vQ.itemsize());
    void* scratch = nullptr;
    ROCM_CALL(requireScratch(ctx, locBytes + 2 * metaBytes + logitBytes, &scratch));
    unsigned char* base = static_cast<unsigned char*>(scratch);
    int32_t* loc = reinterpret_cast<int32_t*>(base);
    int32_t* startDev = reinterpret_cast<int32_t*>(base + locBytes);
    int32_t* lenDev = reinterpret_cast<int32_t*>(base + locBytes + metaBytes);
    void* logits = base + locBytes + 2 * metaBytes;

    int64_t slotBlocks = ceilDiv(maxLen, kSlotThreads);
    if (slotBlocks > 64) slotBlocks = 64;
    for (int64_t first = 0; first < batch; first += kSeqPerLaunch) {
        const int count = static_cast<int>(batch - first < kSeqPerLaunch ? batch - first : kSeqPerLaunch);
        PagedChunk c = {};
        for (int i = 0; i < count; ++i) {
            c.len[i] = lens[first + i];
            c.start[i] = starts[first + i];
        }
        hipLaunchKernelGGL(pagedSlots, dim3(static_cast<unsigned>(slotBlocks), static_cast<unsigned>(count)), dim3(kSlotThreads), 0, stream, loc, startDev, lenDev,
                           vTable.data, vTable.dtype == diopi_dtype_int64, vTable.shape[1], c, static_cast<int>(first), static_cast<int>(maxLen), block_size,
                           vK.shape[0]);
        ROCM_LAUNCH_CHECK();
    }

    const TensorView q3 = viewOf(vQ.data, vQ.dtype, {batch, num_heads, dim});
    const TensorView o3 = viewOf(vOut.data, vOut.dtype, {batch, num_heads, dim});
    const TensorView k3 = viewOf(vK.data, vK.dtype, {vK.shape[0], num_kv_heads, dim});
    const TensorView v3 = viewOf(vV.data, vV.dtype, {vV.shape[0], num_kv_heads, dim});
    const TensorView lg = viewOf(logits, vQ.dtype, {num_heads, total});
    const TensorView tLoc = viewOf(loc, diopi_dtype_int32, {batch, maxLen});
    const TensorView tStart = viewOf(startDev, diopi_dtype_int32, {batch});
    const TensorView tLen = viewOf(lenDev, diopi_dtype_int32, {batch});
    ROCM_CALL(tokenAttention(ctx, lg, q3, k3, tLoc, tStart, tLen, static_cast<int>(maxLen)));
    return tokenSoftmaxReduceV(ctx, o3, lg, v3, tLoc, tStart, tLen, static_cast<int>(maxLen));
    ROCM_ENTRY_END
}
