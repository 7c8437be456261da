// Arguments shared by the two decode-attention operators (diopiTokenAttentionInference and
// diopiTokenSoftmaxReduceVInference): the KV-slot table and the per-sequence bookkeeping tensors.
// All of them are read on the device; nothing here is copied to the host.
#ifndef DIOPI_ROCM_CSRC_DECODE_HPP_
#define DIOPI_ROCM_CSRC_DECODE_HPP_

#include "common.hpp"

namespace rocm {

struct DecodeArgs {
    const void* bLoc;       // [batch, bLocStride] slot of every token of every sequence
    const void* bStartLoc;  // [batch] first logits column of a sequence
    const void* bSeqLen;    // [batch] number of cached tokens of a sequence
    int64_t bLocStride;     // elements per row of b_loc
    int64_t numSlots;       // rows of the kv cache
    int64_t logitCols;      // columns of the logits tensor [H, logitCols]
    int batch;
    int H, Hkv, G, D;       // query heads, kv heads, H / Hkv, head size
    int maxInputLen;        // window of b_loc in use: sequence i owns b_loc[i, maxInputLen - L_i : maxInputLen]
    bool loc64, start64, len64;
};

// Validates the tensors both operators share and fills `args`.  `logits` is [H, cols]; `qOrOut` is
// [B, H, D] (q for the first operator, out for the second); `cache` is [slots, Hkv, D].
// Sets *empty when there is nothing to do.
diopiError_t prepareDecode(const TensorView& logits, const TensorView& qOrOut, const TensorView& cache, const TensorView& bLoc, const TensorView& bStartLoc,
                           const TensorView& bSeqLen, int maxInputLen, DecodeArgs* args, bool* empty);

// The two decode operators on tensor views (what the C entry points call after unwrapping their handles, and what
// diopiPagedAttention calls on views of its own scratch tensors).  `out`/`logits` is [H, cols], q/out is [B, H, D],
// the cache is [slots, Hkv, D].
diopiError_t tokenAttention(diopiContextHandle_t ctx, const TensorView& out, const TensorView& q, const TensorView& k, const TensorView& bLoc,
                            const TensorView& bStartLoc, const TensorView& bSeqLen, int maxInputLen);
diopiError_t tokenSoftmaxReduceV(diopiContextHandle_t ctx, const TensorView& out, const TensorView& logits, const TensorView& v, const TensorView& bLoc,
                                 const TensorView& bStartLoc, const TensorView& bSeqLen, int maxInputLen);

}  // namespace rocm

#endif  // DIOPI_ROCM_CSRC_DECODE_HPP_
