/*
 * The operators of the lmdeploy operator set that the gfx950 library implements: the two in-place normalisations and
 * the fused decoder attention step.
 *
 * reference: proto/include/diopi/functions_lmdeploy.h:31-49, 104-135.  The reference tree declares these operators and
 * holds neither an implementation nor a test of them; the library follows the header's statement and the published
 * kernels the interface was written for (see diopi_amd/csrc/rmsnorm_inplace.hip and fused_decoder_attention.hip for the
 * exact arithmetic).  The other declarations of that header (the context attention block, the FFN block, sampling, batch
 * bookkeeping) are not implemented: a caller that tests the weak symbols' addresses gets diopiNoImplement from its
 * adaptor, as for any absent operator.
 */
#ifndef DIOPI_ROCM_INCLUDE_DIOPI_FUNCTIONS_LMDEPLOY_H_
#define DIOPI_ROCM_INCLUDE_DIOPI_FUNCTIONS_LMDEPLOY_H_

#include <diopi/diopirt.h>

#if defined(__cplusplus)
extern "C" {
#endif

/*
 * In-place RMS normalisation of every row (reference: functions_lmdeploy.h:31-38).
 *   inoutput [tokens, hidden] float32 / float16 (bfloat16 accepted as an extension), dense, on the device
 *   scale    [hidden], same dtype
 *   inoutput[r, :] <- inoutput[r, :] * rsqrt(mean(inoutput[r, :]^2) + eps) * scale
 * Sums in fp32.  HBM-bound: one read and one write of the matrix.
 */
DIOPI_API diopiError_t diopiRootMeanSquareNormInp(diopiContextHandle_t ctx, diopiTensorHandle_t inoutput, diopiConstTensorHandle_t scale, float eps);

/*
 * Residual and bias addition fused with the RMS normalisation that follows it (reference: functions_lmdeploy.h:40-49):
 *   residual <- residual + inoutput + bias          (the sum is formed in fp32 and rounded once)
 *   inoutput <- RMSNorm(residual) * scale
 *   residual [tokens, hidden], same dtype as inoutput, a different tensor; bias [hidden] or a null handle
 * HBM-bound: one read and one write of each of the two matrices, instead of the three reads and two writes that an
 * addition followed by diopiRMSNorm costs.
 */
DIOPI_API diopiError_t diopiFusedAddRootMeanSquareNormInp(diopiContextHandle_t ctx, diopiTensorHandle_t inoutput, diopiTensorHandle_t residual,
                                                          diopiConstTensorHandle_t bias, diopiConstTensorHandle_t scale, float eps);

/*
 * One decode step of self-attention behind a single call (reference: functions_lmdeploy.h:104-135): QKV projection,
 * bias, rotary embedding, insertion of the new key/value rows into the caches, and attention of the new token over its
 * sequence's cached tokens, without any intermediate tensor in HBM but the projected query.
 *   inoutput   [batch_size, hidden_units] float16 / bfloat16 / float32; in: hidden states, out: columns 0 .. H*D-1 hold the
 *              attention output of every row that is not finished (H*D <= hidden_units)
 *   qkv_weight [hidden_units, (H + 2 Hkv) * D], qkv_bias [(H + 2 Hkv) * D] or a null handle: query heads, then key
 *              heads, then value heads along the second axis
 *   workspace / workspace_size: *workspace_size < 0 only writes the bytes the call needs into *workspace_size; else
 *              `workspace` (any dtype, 16-byte aligned) must hold that many bytes.  A null workspace handle with a
 *              non-negative size takes the bytes from the context (diopiRequireBuffer)
 *   key_cache, value_cache [num_layer, rows >= batch_size, Hkv, max_seq_len, D]: row sequence_lengths[b] % max_seq_len of
 *              layer layer_id receives the new key / value of row b
 *   finished [batch_size] bool or null; total_padding_tokens [batch_size] int32/int64 or null (zeros);
 *   sequence_lengths [batch_size] int32/int64: tokens already cached; step: the rotary position is
 *              step - 1 - total_padding_tokens[b]; rotary_embedding: rotating dims of a head (even, 0 .. D: the
 *              first rotary_embedding dims pair up as j and j + rotary_embedding/2, the rest keep their values); rope_theta: base
 * Attention runs over the last min(sequence_lengths[b] + 1, max_seq_len) tokens, scores scaled by 1/sqrt(D), softmax
 * denominator + 1e-6.  fusion_level is accepted and ignored.  Two sets of kernels: float16 / bfloat16 with D = 128,
 * H / Hkv <= 16, hidden_units a multiple of 128 and 16-byte aligned tensors run on the matrix cores, HBM-bound (the weight
 * matrix once, then one K row and one V row per cached token); every other combination (float32, D up to 512, any grouping,
 * size or alignment) runs plain kernels with the same results at a fraction of that speed.  An odd rotary_embedding,
 * D > 512 or another dtype is an error (diopiErrorOccurred).
 */
DIOPI_API diopiError_t diopiFusedDecoderAttentionInp(diopiContextHandle_t ctx, diopiTensorHandle_t inoutput, diopiConstTensorHandle_t qkv_weight,
                                                     diopiConstTensorHandle_t qkv_bias, diopiTensorHandle_t workspace, int64_t* workspace_size,
                                                     int64_t fusion_level, diopiTensorHandle_t key_cache, diopiTensorHandle_t value_cache,
                                                     diopiConstTensorHandle_t finished, diopiConstTensorHandle_t total_padding_tokens,
                                                     diopiConstTensorHandle_t sequence_lengths, int64_t step, int64_t layer_id, int64_t local_head_num,
                                                     int64_t local_kv_head_num, int64_t size_per_head, int64_t max_seq_len, int64_t rotary_embedding,
                                                     float rope_theta);

#if defined(__cplusplus)
}
#endif

#endif /* DIOPI_ROCM_INCLUDE_DIOPI_FUNCTIONS_LMDEPLOY_H_ */
