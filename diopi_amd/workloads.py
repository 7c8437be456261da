"""Seeded synthetic inputs for the five benchmark configurations, and their algorithmic work.

Shapes, distributions and byte/flop formulas are the ones the benchmark definition fixes:
  cfg1  RMSNorm forward+backward, fp32 [8192, 4096]
  cfg2  LLaMA-7B prologue, bf16: RMSNorm [16384, 4096], rotary on q and k [16384, 32, 128]
  cfg3  decode step, fp16: batch 64, 32 heads, head 128, cache [131072, 32, 128], L ~ U(512, 2048)
  cfg4  prefill, fp16: causal varlen, batch 8, L ~ U(1024, 4096), 32 heads, head 128
  cfg5  GQA decode, bf16: 64 q heads / 8 kv heads, batch 128, cache [1048576, 8, 128], L ~ U(1024, 8192)
Every `scale` argument shrinks the problem for parity tests (1.0 = the configured size).

Small index tensors come from numpy's PCG64 with the recorded seed; large value tensors are drawn on
the target device with a torch generator seeded from the same number (drawing 2 GiB caches on the
host would dominate the run).
"""
from __future__ import annotations

import math
from typing import Dict

import numpy as np
import torch

E = {torch.float16: 2, torch.bfloat16: 2, torch.float32: 4, torch.float64: 8}


def _gen(device, seed):
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def _randn(shape, dtype, device, g, std=1.0, chunk=1 << 26):
    """N(0, std) in `dtype`, drawn in fp32 chunks so that the temporary stays small."""
    out = torch.empty(shape, dtype=dtype, device=device)
    flat = out.view(-1)
    for s in range(0, flat.numel(), chunk):
        n = min(chunk, flat.numel() - s)
        flat[s:s + n] = (torch.randn(n, device=device, generator=g, dtype=torch.float32) * std).to(dtype)
    return out


def cfg1(device="cuda", seed=1, scale=1.0) -> Dict:
    n1, n2 = max(1, int(8192 * scale)), 4096
    g = _gen(device, seed)
    return dict(
        x=_randn((n1, n2), torch.float32, device, g),
        weight=(torch.rand(n2, device=device, generator=g) + 0.5),
        grad_out=_randn((n1, n2), torch.float32, device, g),
        eps=1e-6, normalized_shape=(n2,), n1=n1, n2=n2, seed=seed)


def rmsnorm_fwd_bytes(n1, n2, e):
    return 2 * n1 * n2 * e + n2 * e + 4 * n1


def rmsnorm_bwd_bytes(n1, n2, e):
    return 3 * n1 * n2 * e + 4 * n1 + 2 * n2 * e


def cfg2(device="cuda", seed=2, scale=1.0) -> Dict:
    T, H, D, n2 = max(1, int(16384 * scale)), 32, 128, 4096
    g = _gen(device, seed)
    rng = np.random.Generator(np.random.PCG64(seed))
    pos = torch.from_numpy(rng.integers(0, 4096, size=T)).to(device)
    inv_freq = 10000.0 ** (-2.0 * torch.arange(D // 2, device=device, dtype=torch.float32) / D)
    ang = pos.to(torch.float32)[:, None] * inv_freq[None, :]
    return dict(
        x=_randn((T, n2), torch.bfloat16, device, g),
        weight=(torch.rand(n2, device=device, generator=g) + 0.5).to(torch.bfloat16),
        q=_randn((T, H, D), torch.bfloat16, device, g),
        k=_randn((T, H, D), torch.bfloat16, device, g),
        cos=ang.cos().to(torch.bfloat16).reshape(T, 1, D // 2),
        sin=ang.sin().to(torch.bfloat16).reshape(T, 1, D // 2),
        eps=1e-6, normalized_shape=(n2,), T=T, H=H, D=D, n2=n2, seed=seed)


def rotary_bytes(T, H, D, e):
    return 2 * T * H * D * e + 2 * T * (D // 2) * e


def _decode(device, seed, dtype, B, H, Hkv, D, slots, lo, hi, new_tokens):
    g = _gen(device, seed)
    rng = np.random.Generator(np.random.PCG64(seed))
    seq_len = rng.integers(lo, hi + 1, size=B).astype(np.int32)
    max_len = int(seq_len.max())
    width = hi
    perm = rng.permutation(slots)
    b_loc = perm[: B * width].reshape(B, width).astype(np.int32)  # all slots distinct
    start = np.concatenate(([0], np.cumsum(seq_len)[:-1])).astype(np.int32)
    total = int(seq_len.sum())
    dest = rng.permutation(slots)[:new_tokens].astype(np.int32)
    return dict(
        k_cache=_randn((slots, Hkv, D), dtype, device, g),
        v_cache=_randn((slots, Hkv, D), dtype, device, g),
        q=_randn((B, H, D), dtype, device, g),
        new_k=_randn((new_tokens, Hkv, D), dtype, device, g),
        new_v=_randn((new_tokens, Hkv, D), dtype, device, g),
        dest_loc=torch.from_numpy(dest).to(device),
        b_loc=torch.from_numpy(b_loc).to(device),
        b_seq_len=torch.from_numpy(seq_len).to(device),
        b_start_loc=torch.from_numpy(start).to(device),
        max_input_len=max_len, total_len=total, B=B, H=H, Hkv=Hkv, D=D, slots=slots, dtype=dtype, seed=seed)


def cfg3(device="cuda", seed=3, scale=1.0) -> Dict:
    B = max(1, int(64 * scale))
    slots = max(B * 2048, int(131072 * scale))
    return _decode(device, seed, torch.float16, B, 32, 32, 128, slots, 512, 2048, B)


def cfg5(device="cuda", seed=5, scale=1.0) -> Dict:
    B = max(1, int(128 * scale))
    slots = max(B * 8192, int(1048576 * scale))
    return _decode(device, seed, torch.bfloat16, B, 64, 8, 128, slots, 1024, 8192, B)


def destindex_bytes(T, H, D, e):
    return 2 * T * H * D * e + 4 * T


def token_attention_bytes(total_len, B, H, Hkv, D, e):
    return total_len * (Hkv * D * e + 4) + B * H * D * e + H * total_len * e + 8 * B


def softmax_reducev_bytes(total_len, B, H, Hkv, D, e):
    return total_len * (Hkv * D * e + 4) + H * total_len * e + B * H * D * e + 8 * B


def cfg4(device="cuda", seed=4, scale=1.0) -> Dict:
    B, H, D = 8, 32, 128
    g = _gen(device, seed)
    rng = np.random.Generator(np.random.PCG64(seed))
    lo, hi = max(1, int(1024 * scale)), max(2, int(4096 * scale))
    seq_len = rng.integers(lo, hi + 1, size=B).astype(np.int32)
    start = np.concatenate(([0], np.cumsum(seq_len)[:-1])).astype(np.int32)
    T = int(seq_len.sum())
    return dict(
        q=_randn((T, H, D), torch.float16, device, g, std=0.5),
        k=_randn((T, H, D), torch.float16, device, g, std=0.5),
        v=_randn((T, H, D), torch.float16, device, g, std=0.5),
        b_seq_len=torch.from_numpy(seq_len).to(device),
        b_start_loc=torch.from_numpy(start).to(device),
        max_input_len=int(seq_len.max()), T=T, B=B, H=H, D=D, seq_len_host=seq_len, seed=seed)


def context_attention_flops(seq_len, H, D):
    """sum_i H * 4 * D * L_i (L_i + 1) / 2: the causal half of QK^T and PV, 2 flops per multiply-add."""
    return int(sum(H * 4 * D * int(L) * (int(L) + 1) // 2 for L in seq_len))
