/*
 * The LLaMA-inference operator family of the DIOPI extension ABI, as exported
 * by the gfx950 build of libdiopi_impl.so.  Signatures restate
 * proto/include/diopi/functions_ext.h of the reference (line numbers cited at
 * each prototype) and must stay declaration-compatible with it.
 *
 * Common rules for every operator here:
 *  - all tensors live on the device, are contiguous, and are allocated by the
 *    caller (outputs included); optional tensors are passed as NULL;
 *  - work is enqueued on the stream of `ctx` and the call returns without
 *    waiting for it;
 *  - index tensors (dest_loc, b_loc, b_start_loc, b_seq_len) may be int32 or
 *    int64 and are read on the device only: no host synchronisation;
 *  - the return value is a diopiError_t; on failure the text is available
 *    from diopiGetLastErrorString().
 */
#ifndef DIOPI_ROCM_INCLUDE_DIOPI_FUNCTIONS_EXT_H_
#define DIOPI_ROCM_INCLUDE_DIOPI_FUNCTIONS_EXT_H_

#include <diopi/diopirt.h>
#include <stdbool.h>
#include <stdint.h>

#if defined(__cplusplus)
extern "C" {
#endif

/*
 * Rotary position embedding on the two halves of the last dimension.
 * reference: functions_ext.h:31-32.
 *   x1 = x[..., :D/2], x2 = x[..., D/2:]; cos/sin broadcast (right-aligned) against x1.
 *   conj == false: out1 = x1*cos - x2*sin, out2 = x1*sin + x2*cos
 *   conj == true : out1 = x1*cos + x2*sin, out2 = -x1*sin + x2*cos
 * Arithmetic is fp32 with one rounding to the element type (fp64 inputs too).
 * interleaved == true returns diopiNoImplement, as the reference does.
 * dtypes: float16, bfloat16, float32, float64 (out, x, cos, sin share one dtype).
 */
DIOPI_API diopiError_t diopiRotaryEmbedding(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t x, diopiConstTensorHandle_t cos,
                                            diopiConstTensorHandle_t sin, const bool conj, const bool interleaved);

/*
 * Rotary position embedding of query and key, in place, with full-width tables (the lightllm form).
 * reference: functions_ext.h:649-650 (statement: customized_test.py:843-852).
 *   query [T, Hq*dim] and key [T, Hk*dim] are viewed as [T, heads, dim]; cos, sin hold T*dim elements ([T, 1, dim]).
 *   x[.., d]         <- x[.., d]*cos[d]             - x[.., d + dim/2]*sin[d]              (d < dim/2)
 *   x[.., d + dim/2] <- x[.., d + dim/2]*cos[d + dim/2] + x[.., d]*sin[d + dim/2]
 * Arithmetic is fp32 (fp64 for fp64 tensors) with one rounding to the element type.
 * dtypes: float16, bfloat16, float32, float64 (query, key, cos, sin share one dtype).
 */
DIOPI_API diopiError_t diopiRotaryEmbeddingV2(diopiContextHandle_t ctx, diopiTensorHandle_t query, diopiTensorHandle_t key, diopiConstTensorHandle_t cos,
                                              diopiConstTensorHandle_t sin, int64_t dim);

/*
 * Presence / frequency penalty on the logits of already generated tokens, in place.
 * reference: functions_ext.h:527-529 (impl/torch/functions/functions_lightllm.cpp:28-51).
 *   sequence i owns entries [cum[i], cum[i+1]) of p_token_ids / p_token_counts:
 *   logits[i, id_j] <- logits[i, id_j] - count_j * frequency_penalty[i] - presence_penalty[i]
 * evaluated left to right in the logits dtype.  logits [batch, vocabulary]; penalties [batch] in the logits dtype;
 * ids, counts, cumulative lengths int32 or int64.  p_max_len_in_batch is not read (the reference ignores it too).
 */
DIOPI_API diopiError_t diopiApplyPenalty(diopiContextHandle_t ctx, diopiTensorHandle_t logits, diopiConstTensorHandle_t presence_penalty,
                                         diopiConstTensorHandle_t frequency_penalty, diopiConstTensorHandle_t p_token_ids,
                                         diopiConstTensorHandle_t p_token_counts, diopiConstTensorHandle_t p_cumsum_seq_len, int p_max_len_in_batch);

/*
 * Repetition / frequency / presence penalty with one penalty entry per generated token, in place.
 * reference: functions_ext.h:547-549 (statement: customized_test.py:823-841).
 *   x = logits.view(-1)[id_j];  x <- x > 0 ? x / repetition_j : x * repetition_j;  x <- x - count_j * frequency_j - presence_j
 * p_token_ids are flat indices into logits; all penalty tensors and p_token_counts have the length of p_token_ids.
 */
DIOPI_API diopiError_t diopiApplyPenaltyV2(diopiContextHandle_t ctx, diopiTensorHandle_t logits, diopiConstTensorHandle_t presence_penalty,
                                           diopiConstTensorHandle_t frequency_penalty, diopiConstTensorHandle_t repetition_penalty,
                                           diopiConstTensorHandle_t p_token_ids, diopiConstTensorHandle_t p_token_counts);

/*
 * RMS normalisation over the trailing `normalized_shape` dimensions.
 * reference: functions_ext.h:45-46.
 *   inv_rms[row] = rsqrt(mean(x[row]^2) + eps)         (fp32 accumulate; fp64 for fp64 input)
 *   out[row]     = weight * round_to_out_dtype(inv_rms[row] * x[row])  (+ bias if bias != NULL)
 * inv_rms has the leading dimensions of input and dtype float32 (float64 for float64 input).
 * out/weight/bias share one dtype; input may be the same dtype, or float32 with a 16-bit out.
 */
DIOPI_API diopiError_t diopiRMSNorm(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiTensorHandle_t inv_rms, diopiConstTensorHandle_t input,
                                    diopiSize_t normalized_shape, diopiConstTensorHandle_t weight, diopiConstTensorHandle_t bias, double eps);

/*
 * Gradient of diopiRMSNorm.  reference: functions_ext.h:62-65.
 *   g = grad_output * weight;  s = sum_l g_l * x_l * inv_rms          (per row)
 *   grad_input_l  = (inv_rms / n2) * (n2 * g_l - x_l * inv_rms * s)
 *   grad_weight_j = sum_rows grad_output * x * inv_rms
 *   grad_bias     = grad_output summed over the leading dimensions (only if grad_bias != NULL)
 * `bias` and `eps` are accepted and unused, as in the reference.  Needs one
 * scratch buffer from diopiRequireBuffer for the partial column sums.
 */
DIOPI_API diopiError_t diopiRMSNormBackward(diopiContextHandle_t ctx, diopiTensorHandle_t grad_input, diopiTensorHandle_t grad_weight,
                                            diopiTensorHandle_t grad_bias, diopiConstTensorHandle_t grad_output, diopiConstTensorHandle_t input,
                                            diopiConstTensorHandle_t weight, diopiConstTensorHandle_t bias, diopiConstTensorHandle_t inv_rms,
                                            diopiSize_t normalized_shape, double eps);

/*
 * KV-cache row scatter: out[dest_loc[t], :, :] = k[t, :, :].  reference: functions_ext.h:563.
 * Bit-exact copy, no dtype conversion; rows of `out` not named by dest_loc are
 * untouched.  Negative indices wrap once (index + rows); indices still out of
 * range are skipped.  Duplicate indices: one of the rows wins, unspecified which.
 */
DIOPI_API diopiError_t diopiDestIndexCopyKV(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t k, diopiConstTensorHandle_t dest_loc);

/*
 * Decode attention, first half: scaled q.k for every cached token of every sequence.
 * reference: functions_ext.h:579-581.
 *   slots_i = b_loc[i, max_input_len - L_i : max_input_len]           (right-aligned window)
 *   token_attention_out[h, b_start_loc[i] + t] = dot(q[i, h, :], k[slots_i[t], h / G, :]) / sqrt(D)
 * q [B, H, D]; k [slots, Hkv, D] with H = G * Hkv (G = 1 is the reference's case);
 * out [H, sum L].  Columns not covered by any sequence are left untouched.
 */
DIOPI_API diopiError_t diopiTokenAttentionInference(diopiContextHandle_t ctx, diopiTensorHandle_t token_attention_out, diopiConstTensorHandle_t q,
                                                    diopiConstTensorHandle_t k, diopiConstTensorHandle_t b_loc, diopiConstTensorHandle_t b_start_loc,
                                                    diopiConstTensorHandle_t b_seq_len, int max_input_len);

/*
 * Decode attention, second half: softmax over each sequence's logits, then the weighted sum of V.
 * reference: functions_ext.h:597-599.
 *   P = softmax(logics[h, b_start_loc[i] : b_start_loc[i] + L_i])     (fp32 inside)
 *   out[i, h, :] = sum_t P[t] * v[slots_i[t], h / G, :]
 * other_kv_index is accepted and ignored, as in the reference.  Needs scratch from
 * diopiRequireBuffer when a sequence is split over several work-groups.
 */
DIOPI_API diopiError_t diopiTokenSoftmaxReduceVInference(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t logics,
                                                         diopiConstTensorHandle_t v, diopiConstTensorHandle_t b_loc, diopiConstTensorHandle_t b_start_loc,
                                                         diopiConstTensorHandle_t b_seq_len, int max_input_len, int other_kv_index);

/*
 * Prefill attention: causal softmax(q k^T / sqrt(D)) v per packed sequence.
 * reference: functions_ext.h:634-636.
 * q, k, v, out [sum L, H, D]; sequence i owns rows [b_start_loc[i], b_start_loc[i] + b_seq_len[i]).
 * Rows outside every sequence are left untouched.  max_input_len is only an upper
 * bound used to size the launch (the reference never reads it).
 */
DIOPI_API diopiError_t diopiContextAttentionInference(diopiContextHandle_t ctx, diopiTensorHandle_t context_attention_out, diopiConstTensorHandle_t q,
                                                      diopiConstTensorHandle_t k, diopiConstTensorHandle_t v, diopiConstTensorHandle_t b_start_loc,
                                                      diopiConstTensorHandle_t b_seq_len, int max_input_len);

/*
 * diopiContextAttentionInference for callers that cannot allocate.
 * No counterpart in the reference: this entry point exists for code that runs under HIP graph capture, tight serving
 * loops and harnesses that forbid hipMalloc.  Same arguments, checks and results as diopiContextAttentionInference,
 * but it never calls diopiRequireBuffer / diopiRequireTensor or any other allocating routine: the visiting order of
 * the query tiles is kept in a static device array of the library (128 KiB per device, held until the process ends).
 * Limit: ceil(rows / BM) + batch <= 8192 (BM = 256 query rows once the sequences average 1024 rows or more, else
 * 128); a larger call returns diopiErrorOccurred with a message.  All calls on one device share the array: calls that
 * overlap on one device (different streams or threads) race on it and must be serialised by the caller.  The first
 * call on a device looks the array's address up (hipGetSymbolAddress) and reads the device's properties, neither of
 * which may be recorded into a graph: make one ordinary call on each device before the first capture.
 */
DIOPI_API diopiError_t diopiContextAttentionInferenceNoAlloc(diopiContextHandle_t ctx, diopiTensorHandle_t context_attention_out, diopiConstTensorHandle_t q,
                                                             diopiConstTensorHandle_t k, diopiConstTensorHandle_t v, diopiConstTensorHandle_t b_start_loc,
                                                             diopiConstTensorHandle_t b_seq_len, int max_input_len);

/*
 * Variable-length flash attention, forward.
 * reference: functions_ext.h:355-359 (Python statement customized_test.py:525-588, 36-57).
 * q [total, Hq, D]; k, v [total, Hkv, D] with Hq a multiple of Hkv (query head h reads key/value head h / (Hq/Hkv));
 * sequence i owns tokens [cum_seq_q[i], cum_seq_q[i+1]) of q, k and v (cum_seq_kv must describe the same tokens, as in
 * the reference's statement; it is not read).  attention_out = softmax(softmax_scale * q k^T [+ causal mask]) v,
 * softmax_lse [batch, Hq, max_seqlen_q] (float32, may be null) receives the log-sum-exp of every query row's scaled
 * scores; entries past a sequence's length are left untouched.  softmax_scale == 0 means 1/sqrt(D).
 * With float16 tensors at D == 128 the query is multiplied by the scale once and rounded to float16 (2^-11 relative);
 * the output and softmax_lse both belong to those scores, so softmax_lse can differ from the log-sum-exp of unrounded
 * scores by about 2^-12 of the largest scaled score of a row (5e-3 at a score of 35).  bfloat16 and float32 tensors scale
 * every score in float32 instead.
 * Not implemented (error 13): p_dropout != 0, alibi_slopes, sliding windows (window sizes >= 0).  gen is not used.
 * dtypes: float16, bfloat16 (matrix cores at D == 128), float32, float64; cum_seq int32 or int64.
 */
DIOPI_API diopiError_t diopiFlashAttentionVarLen(diopiContextHandle_t ctx, diopiTensorHandle_t attention_out, diopiTensorHandle_t softmax_lse,
                                                 diopiGeneratorHandle_t gen, diopiConstTensorHandle_t q, diopiConstTensorHandle_t k, diopiConstTensorHandle_t v,
                                                 diopiConstTensorHandle_t cum_seq_q, diopiConstTensorHandle_t cum_seq_kv, diopiConstTensorHandle_t alibi_slopes,
                                                 int32_t max_seqlen_q, int32_t max_seqlen_kv, float p_dropout, float softmax_scale, bool is_causal,
                                                 int32_t window_size_left, int32_t window_size_right);

/*
 * Flash attention on padded batches, forward.
 * reference: functions_ext.h:209-212 (Python statement customized_test.py:462-485).
 * q [batch, seq_len, Hq, D]; k, v [batch, seq_len, Hkv, D] (same seq_len, as in the reference's statement), Hq a
 * multiple of Hkv; softmax_lse [batch, Hq, seq_len] float32, may be null.  Everything else as diopiFlashAttentionVarLen.
 */
DIOPI_API diopiError_t diopiFlashAttention(diopiContextHandle_t ctx, diopiTensorHandle_t attention_out, diopiTensorHandle_t softmax_lse,
                                           diopiGeneratorHandle_t gen, diopiConstTensorHandle_t q, diopiConstTensorHandle_t k, diopiConstTensorHandle_t v,
                                           diopiConstTensorHandle_t alibi_slopes, float p_dropout, float softmax_scale, bool is_causal,
                                           int32_t window_size_left, int32_t window_size_right);

/*
 * The older names of the two operators above (reference: functions_ext.h:93-95 and 150-153, marked deprecated there;
 * Python statements customized_test.py:416-460).  q, k, v are not modified.  dropout_p != 0 or return_debug_mask answer
 * 13; gen and debug_attn_mask are not used.  scale == 0 means 1/sqrt(D).
 */
DIOPI_API diopiError_t diopiMultiHeadAttention(diopiContextHandle_t ctx, diopiTensorHandle_t q, diopiTensorHandle_t k, diopiTensorHandle_t v, double dropout_p,
                                               bool is_causal, bool return_debug_mask, double scale, diopiTensorHandle_t out, diopiTensorHandle_t softmax_lse,
                                               diopiGeneratorHandle_t gen, diopiTensorHandle_t debug_attn_mask);
DIOPI_API diopiError_t diopiMultiHeadAttentionVarLen(diopiContextHandle_t ctx, diopiTensorHandle_t q, diopiTensorHandle_t k, diopiTensorHandle_t v,
                                                     diopiConstTensorHandle_t cum_seq_q, diopiConstTensorHandle_t cum_seq_k, int64_t max_q, int64_t max_k,
                                                     double dropout_p, bool is_causal, bool return_debug_mask, double scale, diopiTensorHandle_t out,
                                                     diopiTensorHandle_t softmax_lse, diopiGeneratorHandle_t gen, diopiTensorHandle_t debug_attn_mask);

/*
 * One decode step of attention over a KV cache cut into blocks.
 * reference: functions_ext.h:602-618 (Python statement customized_test.py:782-821; case diopi_configs.py:9425-9468).
 * q, out [batch, num_heads * dim]; k, v [rows, num_kv_heads * dim]; num_heads a multiple of num_kv_heads; block_table
 * int32 or int64 [batch, blocks]; actual_seq_lengths a host list of batch token counts.  Token t of sequence i is row
 * block_table[i, t / block_size] * block_size + t % block_size of k and v; out[i, h] = softmax(q[i, h] . K^T / sqrt(dim)) V
 * over that sequence's tokens.  attenMask is not read (the statement does not read it either).  Asynchronous on the
 * context's stream; the host list is consumed before the call returns.
 */
DIOPI_API diopiError_t diopiPagedAttention(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t q, diopiConstTensorHandle_t k,
                                           diopiConstTensorHandle_t v, diopiConstTensorHandle_t attenMask, diopiSize_t actual_seq_lengths, int64_t num_heads,
                                           int64_t num_kv_heads, int64_t dim, diopiConstTensorHandle_t block_table, int64_t block_size);

/*
 * Causal prefill attention on a padded batch with flattened heads.
 * reference: functions_ext.h:684-686 (Python statement customized_test.py:751-780; case diopi_configs.py:9383-9423).
 * query, out [batch * max_input_len, num_heads * dim]; key, value [batch * max_input_len, num_kv_heads * dim]; batch is
 * the length of the host list actual_seq_lengths.  Row r of sequence i attends to rows 0..r of that sequence, scale
 * 1/sqrt(dim).  As in the statement every row is computed and atten_mask is not read.
 */
DIOPI_API diopiError_t diopiPromptFlashAttention(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t query,
                                                 diopiConstTensorHandle_t key, diopiConstTensorHandle_t value, diopiConstTensorHandle_t atten_mask,
                                                 diopiSize_t actual_seq_lengths, int64_t max_input_len, int64_t num_heads, int64_t num_kv_heads, int64_t dim);

#if defined(__cplusplus)
}
#endif

#endif /* DIOPI_ROCM_INCLUDE_DIOPI_FUNCTIONS_EXT_H_ */
