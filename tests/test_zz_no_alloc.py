"""The entry point that allocates nothing (diopiContextAttentionInferenceNoAlloc), through the C ABI on the GPU.

It has no counterpart in the reference; its bar is the existing entry point: same kernels, so the outputs must be
bit-identical, on two calls in a row of which the second is smaller (the static plan array keeps the first call's
contents), while the context is never asked for memory.
"""
import numpy as np
import pytest
import torch

from diopi_amd import functions as F
from diopi_amd import runtime as rt
from tests.helpers import assert_bit_equal, assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _packed(lens, H, dtype, seed, gap=0):
    g = torch.Generator().manual_seed(seed)
    starts, pos = [], gap
    for L in lens:
        starts.append(pos)
        pos += L + gap
    T = pos
    q, k, v = ((torch.randn(T, H, 128, generator=g) * 0.5).to(dtype).to(DEV) for _ in range(3))
    return q, k, v, torch.tensor(starts, dtype=torch.int32, device=DEV), torch.tensor(lens, dtype=torch.int32, device=DEV), max(lens)


def _both(case, ctx, what):
    q, k, v, bs, bl, ml = case
    want = F.context_attention(q, k, v, torch.full_like(q, 55.0), bs, bl, ml)
    got = F.context_attention_no_alloc(q, k, v, torch.full_like(q, 55.0), bs, bl, ml, ctx=ctx)
    ctx.synchronize()
    assert_bit_equal(got, want, what)
    return got


def test_no_alloc_entry_point_matches_the_allocating_one_twice_in_a_row():
    print("no-alloc prefill: fp16, 4 ragged sequences then 2 short ones", flush=True)
    ctx = rt.Context(own_stream=True)
    big = _packed([300, 1500, 64, 700], 4, torch.float16, 901, gap=3)      # 21 query tiles of 128 rows + 4
    small = _packed([33, 129], 2, torch.float16, 902)                      # 3 tiles + 2: most plan entries stay from `big`
    out_big = _both(big, ctx, "no-alloc vs allocating entry point, first call")
    out_small = _both(small, ctx, "no-alloc vs allocating entry point, second (smaller) call")
    # and once more the large one after the small one, in bf16 with 256-row tiles (sequences of 1024 rows and more)
    wide = _packed([1024, 2100], 2, torch.bfloat16, 903)
    _both(wide, ctx, "no-alloc vs allocating entry point, 256-row tiles")
    # the context was never asked for memory
    assert ctx.malloc_count == 0 and ctx.scratch_peak == 0, (ctx.malloc_count, ctx.scratch_peak)
    # first token of a sequence returns its own value row, rows in the gaps stay untouched
    q, k, v, bs, bl, _ = big
    for s in bs.tolist():
        assert_bit_equal(out_big[s], v[s], "first token of a sequence")
    assert bool((out_big[:3] == 55.0).all())
    assert out_small.shape == small[0].shape
    ctx.close()


def test_no_alloc_entry_point_other_kernels_and_limit():
    print("no-alloc prefill: fp32 (no plan needed) and a call beyond the plan's capacity", flush=True)
    ctx = rt.Context(own_stream=True)
    g = torch.Generator().manual_seed(904)
    q, k, v = (torch.randn(70, 2, 64, generator=g).to(DEV) for _ in range(3))
    bs, bl = torch.tensor([0, 40], dtype=torch.int32, device=DEV), torch.tensor([40, 30], dtype=torch.int32, device=DEV)
    want = F.context_attention(q, k, v, torch.zeros_like(q), bs, bl, 40)
    got = F.context_attention_no_alloc(q, k, v, torch.zeros_like(q), bs, bl, 40, ctx=ctx)
    assert_close(got, want, rtol=0, atol=0, what="fp32 head size 64 through the no-alloc entry point")
    # 2500 sequences over 760000 rows: 5938 tiles of 128 rows + 2500 > 8192 entries -> rejected before any launch
    B, T = 2500, 760000
    qe = torch.empty(T, 1, 128, dtype=torch.float16, device=DEV)
    lens = torch.full((B,), T // B, dtype=torch.int32, device=DEV)
    starts = (torch.arange(B, dtype=torch.int32, device=DEV) * (T // B)).int()
    with pytest.raises(rt.DiopiException) as e:
        F.context_attention_no_alloc(qe, qe, qe, torch.empty_like(qe), starts, lens, T // B, ctx=ctx)
    assert "at most 8192" in str(e.value)
    assert ctx.malloc_count == 0
    ctx.close()
