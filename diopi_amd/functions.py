"""Python callers of the seven LLaMA-inference operators, through the C ABI.

Each function mirrors the wrapper of the same name in
``diopi_test/python/conformance/diopi_functions.py`` of the reference
(rotary_emb 7030-7037, rms_norm 7040-7070, rms_norm_backward 7073-7109,
destindex_copy_kv 7896-7902, token_attention 7905-7911,
token_softmax_reducev 7914-7939, context_attention 7942-7948): same argument
order and meaning, outputs allocated by the caller side with the reference's
shape/dtype rules, return code checked with the reference's policy.

Arguments are torch tensors on the GPU; they are wrapped as diopiTensor handles
for the duration of the call.  The operators run on the context's stream; the
wrappers order that stream after torch's current stream on entry and torch's
current stream after it on exit, so results can be used by torch code directly.
"""
from __future__ import annotations

from typing import Optional, Sequence

import math

import ctypes

import torch

from . import runtime as rt
from .runtime import Sizes, Tensor, as_handle, check_returncode

# inv_rms of the last rms_norm call, consumed by rms_norm_backward
# (reference: GLOBAL_STATE["rms_norm_inv_rms"], diopi_functions.py:7069, 7087)
GLOBAL_STATE = {}


def _ctx(ctx: Optional[rt.Context]) -> rt.Context:
    return ctx if ctx is not None else rt.default_context()


class _on_stream:
    """Orders the context's stream with torch's current stream around a call."""

    def __init__(self, ctx: rt.Context, *tensors):
        self.ctx = ctx
        on_device = any(t is not None and t.is_cuda for t in tensors)
        self.cuda = ctx.torch_stream is not None and on_device
        # a context that made its own native stream has no torch stream to order against: the host waits instead, before
        # the call for what torch has queued (fills and copies of the arguments) and after it for the operator
        self.foreign = ctx.torch_stream is None and on_device

    def __enter__(self):
        if self.cuda:
            self.ctx.torch_stream.wait_stream(torch.cuda.current_stream())
        elif self.foreign:
            torch.cuda.current_stream().synchronize()
        return self

    def __exit__(self, *exc):
        if self.cuda:
            torch.cuda.current_stream().wait_stream(self.ctx.torch_stream)
        elif self.foreign:
            self.ctx.synchronize()
        # scratch an operator took from the context (partial sums, tile plans, score buffers) belongs to that call:
        # hand it back to the context's pool, as the reference harness does after every case (litert.hpp:268-276);
        # the pool is reused in stream order, so a later call on this context may overwrite it safely
        self.ctx.clear_tensors()
        return False


def _handles(*tensors):
    """Wraps torch tensors as diopiTensor handles.  Returns (keepalive, handles): the wrappers own the
    handles, so `keepalive` must stay referenced until the call has returned."""
    keep = [None if t is None else Tensor(t) for t in tensors]
    return keep, [as_handle(k) for k in keep]


def rotary_emb(input: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, conj: bool, interleaved: bool, ctx: Optional[rt.Context] = None) -> torch.Tensor:
    ctx = _ctx(ctx)
    out = torch.empty_like(input, memory_format=torch.contiguous_format)
    with _on_stream(ctx, input):
        keep, h = _handles(out, input, cos, sin)
        ret = rt.libs().impl.diopiRotaryEmbedding(ctx.handle, *h, bool(conj), bool(interleaved))
    check_returncode(ret, "diopiRotaryEmbedding")
    return out


def rotary_emb_v2(query: torch.Tensor, key: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, dim: int, ctx: Optional[rt.Context] = None):
    """In place on query and key, like the reference wrapper (diopi_functions.py:8051-8056)."""
    ctx = _ctx(ctx)
    with _on_stream(ctx, query):
        keep, h = _handles(query, key, cos, sin)
        ret = rt.libs().impl.diopiRotaryEmbeddingV2(ctx.handle, *h, int(dim))
    check_returncode(ret, "diopiRotaryEmbeddingV2")
    return query, key


def apply_penalty(logits: torch.Tensor, presence_penalty: torch.Tensor, frequency_penalty: torch.Tensor, p_token_ids: torch.Tensor,
                  p_token_counts: torch.Tensor, p_cumsum_seq_len: torch.Tensor, p_max_len_in_batch: int, ctx: Optional[rt.Context] = None) -> torch.Tensor:
    """In place on logits, like the reference wrapper (diopi_functions.py:7851-7895)."""
    ctx = _ctx(ctx)
    with _on_stream(ctx, logits):
        keep, h = _handles(logits, presence_penalty, frequency_penalty, p_token_ids, p_token_counts, p_cumsum_seq_len)
        ret = rt.libs().impl.diopiApplyPenalty(ctx.handle, *h, int(p_max_len_in_batch))
    check_returncode(ret, "diopiApplyPenalty")
    return logits


def apply_penalty_v2(logits: torch.Tensor, presence_penalty: torch.Tensor, frequency_penalty: torch.Tensor, repetition_penalty: torch.Tensor,
                     p_token_ids: torch.Tensor, p_token_counts: torch.Tensor, ctx: Optional[rt.Context] = None) -> torch.Tensor:
    """In place on logits, like the reference wrapper (diopi_functions.py:8019-8049)."""
    ctx = _ctx(ctx)
    with _on_stream(ctx, logits):
        keep, h = _handles(logits, presence_penalty, frequency_penalty, repetition_penalty, p_token_ids, p_token_counts)
        ret = rt.libs().impl.diopiApplyPenaltyV2(ctx.handle, *h)
    check_returncode(ret, "diopiApplyPenaltyV2")
    return logits


def rms_norm(input: torch.Tensor, normalized_shape: Sequence[int], weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float,
             ctx: Optional[rt.Context] = None, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    ctx = _ctx(ctx)
    out = torch.empty(input.shape, dtype=out_dtype or input.dtype, device=input.device)
    n = len(normalized_shape)
    inv_shape = list(input.shape)[: input.dim() - n]
    # 16-bit and fp32 inputs keep their statistics in fp32, fp64 inputs in fp64
    inv_dtype = torch.float64 if input.dtype == torch.float64 else torch.float32
    inv_rms = torch.empty(inv_shape, dtype=inv_dtype, device=input.device)
    sizes = Sizes(normalized_shape)
    with _on_stream(ctx, input):
        keep, h = _handles(out, inv_rms, input, weight, bias)
        ret = rt.libs().impl.diopiRMSNorm(ctx.handle, h[0], h[1], h[2], sizes.c, h[3], h[4], float(eps))
    check_returncode(ret, "diopiRMSNorm")
    GLOBAL_STATE["rms_norm_inv_rms"] = inv_rms
    return out


def rms_norm_backward(grad_outputs: Sequence[torch.Tensor], input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                      normalized_shape: Sequence[int], eps: float, ctx: Optional[rt.Context] = None, inv_rms: Optional[torch.Tensor] = None) -> dict:
    ctx = _ctx(ctx)
    grad_input = torch.empty_like(input)
    grad_weight = torch.empty_like(weight)
    grad_bias = torch.empty_like(bias) if bias is not None else None
    if inv_rms is None:
        inv_rms = GLOBAL_STATE.pop("rms_norm_inv_rms")
    sizes = Sizes(normalized_shape)
    with _on_stream(ctx, input):
        keep, h = _handles(grad_input, grad_weight, grad_bias, grad_outputs[0], input, weight, bias, inv_rms)
        ret = rt.libs().impl.diopiRMSNormBackward(ctx.handle, *h, sizes.c, float(eps))
    check_returncode(ret, "diopiRMSNormBackward")
    out = {"input": grad_input, "weight": grad_weight}
    if bias is not None:
        out["bias"] = grad_bias
    return out


def root_mean_square_norm_inp(inoutput: torch.Tensor, scale: torch.Tensor, eps: float, ctx: Optional[rt.Context] = None) -> torch.Tensor:
    """In-place RMS normalisation of every row (functions_lmdeploy.h:31-38 of the reference)."""
    ctx = _ctx(ctx)
    with _on_stream(ctx, inoutput):
        keep, h = _handles(inoutput, scale)
        ret = rt.libs().impl.diopiRootMeanSquareNormInp(ctx.handle, h[0], h[1], float(eps))
    check_returncode(ret, "diopiRootMeanSquareNormInp")
    return inoutput


def fused_add_root_mean_square_norm_inp(inoutput: torch.Tensor, residual: torch.Tensor, bias: Optional[torch.Tensor], scale: torch.Tensor, eps: float,
                                        ctx: Optional[rt.Context] = None):
    """residual += inoutput + bias; inoutput = RMSNorm(residual) * scale (functions_lmdeploy.h:40-49 of the reference)."""
    ctx = _ctx(ctx)
    with _on_stream(ctx, inoutput):
        keep, h = _handles(inoutput, residual, bias, scale)
        ret = rt.libs().impl.diopiFusedAddRootMeanSquareNormInp(ctx.handle, h[0], h[1], h[2], h[3], float(eps))
    check_returncode(ret, "diopiFusedAddRootMeanSquareNormInp")
    return inoutput, residual


def fused_decoder_attention_inp(inoutput: torch.Tensor, qkv_weight: torch.Tensor, qkv_bias: Optional[torch.Tensor], workspace: Optional[torch.Tensor],
                                fusion_level: int, key_cache: torch.Tensor, value_cache: torch.Tensor, finished: Optional[torch.Tensor],
                                total_padding_tokens: Optional[torch.Tensor], sequence_lengths: torch.Tensor, step: int, layer_id: int, local_head_num: int,
                                local_kv_head_num: int, size_per_head: int, max_seq_len: int, rotary_embedding: int, rope_theta: float,
                                ctx: Optional[rt.Context] = None) -> torch.Tensor:
    """One decode step of self-attention, from hidden states to attention output (functions_lmdeploy.h:104-135 of the reference).

    `workspace` None allocates one of the size the operator asks for (the header's size query: workspace_size < 0)."""
    ctx = _ctx(ctx)
    with _on_stream(ctx, inoutput):
        keep, h = _handles(inoutput, qkv_weight, qkv_bias, key_cache, value_cache, finished, total_padding_tokens, sequence_lengths)
        args = (int(fusion_level), h[3], h[4], h[5], h[6], h[7], int(step), int(layer_id), int(local_head_num), int(local_kv_head_num), int(size_per_head),
                int(max_seq_len), int(rotary_embedding), float(rope_theta))
        if workspace is None:
            size = ctypes.c_int64(-1)
            ret = rt.libs().impl.diopiFusedDecoderAttentionInp(ctx.handle, h[0], h[1], h[2], None, ctypes.byref(size), *args)
            check_returncode(ret, "diopiFusedDecoderAttentionInp (size query)")
            workspace = torch.empty(max(int(size.value), 16), dtype=torch.int8, device=inoutput.device)
        size = ctypes.c_int64(workspace.numel() * workspace.element_size())
        keep_ws, hw = _handles(workspace)
        ret = rt.libs().impl.diopiFusedDecoderAttentionInp(ctx.handle, h[0], h[1], h[2], hw[0], ctypes.byref(size), *args)
    check_returncode(ret, "diopiFusedDecoderAttentionInp")
    ctx.clear_tensors()
    return inoutput


def destindex_copy_kv(k: torch.Tensor, dest_loc: torch.Tensor, out: torch.Tensor, ctx: Optional[rt.Context] = None) -> torch.Tensor:
    ctx = _ctx(ctx)
    with _on_stream(ctx, out):
        keep, h = _handles(out, k, dest_loc)
        ret = rt.libs().impl.diopiDestIndexCopyKV(ctx.handle, *h)
    check_returncode(ret, "diopiDestIndexCopyKV")
    return out


def token_attention(q: torch.Tensor, k: torch.Tensor, out: torch.Tensor, b_loc: torch.Tensor, b_start_loc: torch.Tensor, b_seq_len: torch.Tensor,
                    max_input_len: int, ctx: Optional[rt.Context] = None) -> torch.Tensor:
    ctx = _ctx(ctx)
    with _on_stream(ctx, out):
        keep, h = _handles(out, q, k, b_loc, b_start_loc, b_seq_len)
        ret = rt.libs().impl.diopiTokenAttentionInference(ctx.handle, *h, int(max_input_len))
    check_returncode(ret, "diopiTokenAttentionInference")
    return out


def token_softmax_reducev(logics: torch.Tensor, v: torch.Tensor, out: torch.Tensor, b_loc: torch.Tensor, b_start_loc: torch.Tensor,
                          b_seq_len: torch.Tensor, max_input_len: int, other_kv_index: int, ctx: Optional[rt.Context] = None) -> torch.Tensor:
    ctx = _ctx(ctx)
    with _on_stream(ctx, out):
        keep, h = _handles(out, logics, v, b_loc, b_start_loc, b_seq_len)
        ret = rt.libs().impl.diopiTokenSoftmaxReduceVInference(ctx.handle, *h, int(max_input_len), int(other_kv_index))
    check_returncode(ret, "diopiTokenSoftmaxReduceVInference")
    return out


def context_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, b_start_loc: torch.Tensor, b_seq_len: torch.Tensor,
                      max_input_len: int, ctx: Optional[rt.Context] = None) -> torch.Tensor:
    ctx = _ctx(ctx)
    with _on_stream(ctx, out):
        keep, h = _handles(out, q, k, v, b_start_loc, b_seq_len)
        ret = rt.libs().impl.diopiContextAttentionInference(ctx.handle, *h, int(max_input_len))
    check_returncode(ret, "diopiContextAttentionInference")
    return out


def context_attention_no_alloc(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, b_start_loc: torch.Tensor, b_seq_len: torch.Tensor,
                               max_input_len: int, ctx: Optional[rt.Context] = None) -> torch.Tensor:
    """context_attention through the entry point that allocates nothing (no counterpart in the reference): the tile plan
    lives in a static device array of the library, so calls on one device must not overlap."""
    ctx = _ctx(ctx)
    with _on_stream(ctx, out):
        keep, h = _handles(out, q, k, v, b_start_loc, b_seq_len)
        ret = rt.libs().impl.diopiContextAttentionInferenceNoAlloc(ctx.handle, *h, int(max_input_len))
    check_returncode(ret, "diopiContextAttentionInferenceNoAlloc")
    return out


def flash_attention_varlen(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens_q: torch.Tensor, cu_seqlens_kv: torch.Tensor, alibi_slopes,
                           max_seqlen_q: int, max_seqlen_kv: int, p_dropout: float, softmax_scale, is_causal: bool, window_size_left: int = -1,
                           window_size_right: int = -1, ctx: Optional[rt.Context] = None) -> torch.Tensor:
    """diopi_functions.py:7530-7590 of the reference: allocates out and softmax_lse [batch, heads, max_seqlen_q] (kept in
    GLOBAL_STATE["flash_attention_varlen_softmax_lse"]), replaces a missing scale by 1/sqrt(head_dim), returns out."""
    ctx = _ctx(ctx)
    out = torch.empty_like(q)
    batch = cu_seqlens_q.numel() - 1
    lse = torch.zeros(batch, q.shape[1], int(max_seqlen_q), dtype=torch.float32, device=q.device)
    scale = 1.0 / math.sqrt(q.shape[-1]) if not softmax_scale else float(softmax_scale)
    with _on_stream(ctx, out):
        keep, h = _handles(out, lse, q, k, v, cu_seqlens_q, cu_seqlens_kv)
        alibi = None
        if alibi_slopes is not None:
            keep2, (alibi,) = _handles(alibi_slopes)
        ret = rt.libs().impl.diopiFlashAttentionVarLen(ctx.handle, h[0], h[1], None, h[2], h[3], h[4], h[5], h[6], alibi, int(max_seqlen_q),
                                                       int(max_seqlen_kv), float(p_dropout), scale, bool(is_causal), int(window_size_left),
                                                       int(window_size_right))
    check_returncode(ret, "diopiFlashAttentionVarLen")
    GLOBAL_STATE["flash_attention_varlen_softmax_lse"] = lse
    return out


def flash_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, alibi_slopes, p_dropout: float, softmax_scale, is_causal: bool,
                    window_size_left: int = -1, window_size_right: int = -1, ctx: Optional[rt.Context] = None) -> torch.Tensor:
    """diopi_functions.py flash_attention of the reference: allocates out and softmax_lse [batch, heads, seq_len] (kept in
    GLOBAL_STATE["flash_attention_softmax_lse"]), replaces a missing scale by 1/sqrt(head_dim), returns out."""
    ctx = _ctx(ctx)
    out = torch.empty_like(q)
    lse = torch.zeros(q.shape[0], q.shape[2], q.shape[1], dtype=torch.float32, device=q.device)
    scale = 1.0 / math.sqrt(q.shape[-1]) if not softmax_scale else float(softmax_scale)
    with _on_stream(ctx, out):
        keep, h = _handles(out, lse, q, k, v, alibi_slopes)
        ret = rt.libs().impl.diopiFlashAttention(ctx.handle, h[0], h[1], None, h[2], h[3], h[4], h[5], float(p_dropout), scale, bool(is_causal),
                                                 int(window_size_left), int(window_size_right))
    check_returncode(ret, "diopiFlashAttention")
    GLOBAL_STATE["flash_attention_softmax_lse"] = lse
    return out


def multihead_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, dropout_p: float, is_causal: bool, return_debug_mask: bool, scale,
                        ctx: Optional[rt.Context] = None) -> torch.Tensor:
    """diopi_functions.py:7112-7149 of the reference (softmax_lse kept in GLOBAL_STATE["multihead_attention_softmax_lse"])."""
    ctx = _ctx(ctx)
    out = torch.empty_like(q)
    lse = torch.zeros(q.shape[0], q.shape[2], q.shape[1], dtype=torch.float32, device=q.device)
    softmax_scale = 1.0 / math.sqrt(q.shape[-1]) if not scale else float(scale)
    with _on_stream(ctx, out):
        keep, h = _handles(q, k, v, out, lse)
        ret = rt.libs().impl.diopiMultiHeadAttention(ctx.handle, h[0], h[1], h[2], float(dropout_p), bool(is_causal), bool(return_debug_mask), softmax_scale,
                                                     h[3], h[4], None, None)
    check_returncode(ret, "diopiMultiHeadAttention")
    GLOBAL_STATE["multihead_attention_softmax_lse"] = lse
    return out


def multihead_attention_varlen(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens: torch.Tensor, max_seqlen: int, dropout_p: float,
                               is_causal: bool, return_debug_mask: bool, scale, ctx: Optional[rt.Context] = None) -> torch.Tensor:
    """diopi_functions.py:7195-7250 of the reference (softmax_lse kept in GLOBAL_STATE["multihead_attention_varlen_softmax_lse"])."""
    ctx = _ctx(ctx)
    out = torch.empty_like(q)
    lse = torch.zeros(cu_seqlens.numel() - 1, q.shape[1], int(max_seqlen), dtype=torch.float32, device=q.device)
    softmax_scale = 1.0 / math.sqrt(q.shape[-1]) if not scale else float(scale)
    with _on_stream(ctx, out):
        keep, h = _handles(q, k, v, cu_seqlens, out, lse)
        ret = rt.libs().impl.diopiMultiHeadAttentionVarLen(ctx.handle, h[0], h[1], h[2], h[3], h[3], int(max_seqlen), int(max_seqlen), float(dropout_p),
                                                           bool(is_causal), bool(return_debug_mask), softmax_scale, h[4], h[5], None, None)
    check_returncode(ret, "diopiMultiHeadAttentionVarLen")
    GLOBAL_STATE["multihead_attention_varlen_softmax_lse"] = lse
    return out


def prompt_flash_attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, attenMask: Optional[torch.Tensor], actualSeqLengths: Sequence[int],
                           maxInputLen: int, numHeads: int, numKeyValueHeads: int, dim: int, ctx: Optional[rt.Context] = None) -> torch.Tensor:
    """diopi_functions.py:7951-7981 of the reference."""
    ctx = _ctx(ctx)
    out = torch.empty_like(query)
    sizes = Sizes(actualSeqLengths)
    with _on_stream(ctx, out):
        keep, h = _handles(out, query, key, value, attenMask)
        ret = rt.libs().impl.diopiPromptFlashAttention(ctx.handle, h[0], h[1], h[2], h[3], h[4], sizes.c, int(maxInputLen), int(numHeads),
                                                       int(numKeyValueHeads), int(dim))
    check_returncode(ret, "diopiPromptFlashAttention")
    return out


def paged_attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, attenMask: Optional[torch.Tensor], actualSeqLengths: Sequence[int],
                    numHeads: int, numKeyValueHeads: int, dim: int, blockTable: torch.Tensor, blockSize: int,
                    ctx: Optional[rt.Context] = None) -> torch.Tensor:
    """diopi_functions.py:7984-8016 of the reference."""
    ctx = _ctx(ctx)
    out = torch.empty_like(query)
    sizes = Sizes(actualSeqLengths)
    with _on_stream(ctx, out):
        keep, h = _handles(out, query, key, value, attenMask, blockTable)
        ret = rt.libs().impl.diopiPagedAttention(ctx.handle, h[0], h[1], h[2], h[3], h[4], sizes.c, int(numHeads), int(numKeyValueHeads), int(dim), h[5],
                                                 int(blockSize))
    check_returncode(ret, "diopiPagedAttention")
    return out
