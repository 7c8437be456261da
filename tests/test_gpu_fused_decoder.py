"""Parity of diopiFusedDecoderAttentionInp (called through the C ABI) against the CPU oracle's composition of the
reference's pinned parts.  Bar: 16-bit tensors within atol = rtol = 1e-2, float32 tensors within atol = rtol = 1e-5, of the
dtype-faithful composition and of float64; the cache rows the call writes are compared the same way, every other cache row
bit for bit."""
import ctypes
import math

import pytest
import torch

from diopi_amd import functions as F
from diopi_amd import runtime as rt
from oracle import ref_ops as O
from tests.helpers import TOL, assert_bit_equal, assert_close, report

pytestmark = pytest.mark.gpu
DEV = "cuda"


def say(*a):
    print(*a, flush=True)


def _case(B, H, Hkv, S, seq, dt, seed, hidden=None, layers=2, layer=1, pad=None, finished=None, step=None, bias=True, rot=128, idt=torch.int32,
          theta=10000.0, what="", out_mismatch=0.0, D=128, cache_rows=None, misalign=False):
    """cache_rows: batch dimension of the caches when larger than B (rows past B must stay untouched); misalign: every
    tensor starts one element past a 16-byte boundary."""
    g = torch.Generator().manual_seed(seed)
    hid = H * D if hidden is None else hidden
    N = (H + 2 * Hkv) * D
    x = torch.randn(B, hid, generator=g).to(dt)
    w = (torch.randn(hid, N, generator=g) / math.sqrt(hid)).to(dt)
    b = torch.randn(N, generator=g).to(dt) if bias else None
    CB = B if cache_rows is None else cache_rows
    kc = torch.randn(layers, CB, Hkv, S, D, generator=g).to(dt)
    vc = torch.randn(layers, CB, Hkv, S, D, generator=g).to(dt)
    seq_t = torch.tensor(seq, dtype=idt)
    pad_t = None if pad is None else torch.tensor(pad, dtype=idt)
    fin_t = None if finished is None else torch.tensor(finished, dtype=torch.bool)
    step = max(seq) + 1 if step is None else step
    say("fused decoder attention", what, dict(B=B, H=H, Hkv=Hkv, D=D, S=S, hidden=hid, rot=rot, dtype=str(dt), seq=seq[:8], step=step))
    # oracle, dtype-faithful and float64 (each on its own copy of the caches)
    rk, rv = kc.clone(), vc.clone()
    ref = O.fused_decoder_attention_inp(x, w, b, rk, rv, fin_t, pad_t, seq_t, step, layer, H, Hkv, D, S, rot, theta)
    ek, ev = kc.double(), vc.double()
    ex = O.fused_decoder_attention_inp(x, w, b, ek, ev, fin_t, pad_t, seq_t, step, layer, H, Hkv, D, S, rot, theta, exact=True)
    # device
    def put(t):
        if t is None or not misalign:
            return None if t is None else t.to(DEV)
        buf = torch.empty(t.numel() + 1, dtype=t.dtype, device=DEV)
        view = buf[1:].view(t.shape)
        view.copy_(t)
        assert view.data_ptr() % 16 != 0
        return view

    xd, wd, bd, kd, vd = put(x), put(w), put(b), put(kc), put(vc)
    args = [t if t is None else t.to(DEV) for t in (fin_t, pad_t, seq_t)]
    w_before = wd.clone()
    out = F.fused_decoder_attention_inp(xd, wd, bd, None, 0, kd, vd, args[0], args[1], args[2], step, layer, H, Hkv, D, S, rot, theta)
    assert_bit_equal(wd, w_before, "qkv_weight was modified")
    tol = TOL[dt]
    assert_close(out, ref, what=what + " output vs reference composition", mismatch_ratio=out_mismatch, **tol)
    assert_close(out, ex, what=what + " output vs float64", mismatch_ratio=out_mismatch, **tol)
    say(what, "max_abs/rel vs f64: %.3e %.3e" % report(out, ex))
    # caches: the written rows within tolerance, every other row untouched
    written = torch.zeros(layers, CB, Hkv, S, dtype=torch.bool)
    for i in range(B):
        if finished is None or not finished[i]:
            written[layer, i, :, seq[i] % S] = True
    for name, dev, r, e, orig in (("key_cache", kd, rk, ek, kc), ("value_cache", vd, rv, ev, vc)):
        devc = dev.cpu()
        assert_bit_equal(devc[~written], orig[~written], f"{what}: {name} rows outside the insertion were modified")
        assert_close(devc[written], r[written], what=f"{what} {name} new rows vs reference composition", **tol)
        assert_close(devc[written], e[written], what=f"{what} {name} new rows vs float64", **tol)
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_decoder_attention_small(dtype):
    # multi-head, one range; lengths 0 (nothing cached), mid, last row of the cache
    _case(B=5, H=4, Hkv=4, S=64, seq=[0, 1, 31, 40, 63], dt=dtype, seed=1, what="MHA")
    # grouped heads, several ranges (S > 256), int64 index tensors, padding offsets, a finished row, no bias
    _case(B=4, H=8, Hkv=2, S=700, seq=[5, 300, 699, 450], dt=dtype, seed=2, pad=[0, 3, 10, 1], finished=[False, False, False, True], bias=False,
          idt=torch.int64, what="GQA 4, ranges")
    # three query heads on one kv head; a hidden size the projection cannot cut across work-groups (384 = 3 x 128)
    _case(B=6, H=3, Hkv=1, S=40, seq=[0, 39, 7, 20, 33, 12], dt=dtype, seed=6, what="GQA 3, hidden 384")
    # multi-query, hidden wider than H*D, no rotation, layer 0
    _case(B=3, H=16, Hkv=1, S=96, seq=[95, 10, 50], dt=dtype, seed=3, hidden=16 * 128 + 256, layer=0, rot=0, what="MQA 16, wide hidden")


def test_fused_decoder_attention_circular_cache_and_many_rows():
    # sequences past max_seq_len wrap around; more than 64 batch rows take a second row group of the projection
    _case(B=70, H=4, Hkv=2, S=48, seq=[(7 * i) % 200 for i in range(70)], dt=torch.float16, seed=4, step=260, what="wrap, 70 rows")


def test_fused_decoder_attention_projection_runs_that_cross_heads():
    # 2200 rows are 35 blocks of 64: the projection then has fewer work-groups per block (256 // 35 = 7) than heads (8), and its
    # equal runs of (head, 32-row step) units end inside heads: a work-group writes partial tiles of two heads
    _case(B=2200, H=4, Hkv=2, S=24, seq=[(5 * i) % 24 for i in range(2200)], dt=torch.float16, seed=9, layers=1, layer=0, what="2200 rows")


def test_fused_decoder_attention_random_shapes():
    """Twelve seeded random combinations of batch, head grouping, cache length, hidden size, lengths (before and past the wrap),
    finished rows, padding offsets, rotation on or off, bias or none, index width and dtype.  With bf16 tensors 2 in 1000
    output elements may miss the bar: over a window of a handful of tokens nothing averages out, and one bf16 rounding of a score
    of size 4 (the composition keeps its scores in the tensor type; the device rounds q and k to it) moves a probability by 2 %."""
    rng = torch.Generator().manual_seed(1234)

    def pick(*vals):
        return vals[int(torch.randint(len(vals), (1,), generator=rng))]

    for n in range(12):
        Hkv = pick(1, 2, 3, 4)
        G = pick(1, 2, 4, 5, 8, 16)
        H = Hkv * G
        B = pick(1, 2, 7, 33, 65)
        S = pick(16, 31, 100, 257, 600, 1100)
        extra = pick(0, 0, 128, 384)
        hidden = max(H * 128 + extra, 256)
        wrap = pick(False, False, True)
        hi = 3 * S if wrap else S - 1
        seq = torch.randint(0, hi + 1, (B,), generator=rng).tolist()
        finished = None if pick(True, False) else (torch.rand(B, generator=rng) < 0.3).tolist()
        pad = None if pick(True, False) else torch.randint(0, 5, (B,), generator=rng).tolist()
        dt = pick(torch.float16, torch.bfloat16)
        _case(B=B, H=H, Hkv=Hkv, S=S, seq=seq, dt=dt, seed=100 + n, hidden=hidden, layers=pick(1, 3), layer=0,
              pad=pad, finished=finished, step=max(seq) + 1 + (0 if pad is None else 5), bias=pick(True, False), rot=pick(0, 128),
              idt=pick(torch.int32, torch.int64), what=f"random case {n}", out_mismatch=2e-3 if dt is torch.bfloat16 else 0.0)


def test_fused_decoder_attention_decode_shape_sampled():
    """The decode benchmark's shape (batch 64, 32 heads of 128, hidden 4096, lengths 512..2047 in a 2048-row cache): the whole
    output against the oracle."""
    g = torch.Generator().manual_seed(5)
    seq = torch.randint(512, 2048, (64,), generator=g).tolist()
    _case(B=64, H=32, Hkv=32, S=2048, seq=seq, dt=torch.float16, seed=5, layers=1, layer=0, what="decode shape")


def test_fused_decoder_attention_workspace_protocol_and_errors():
    impl = rt.libs().impl
    ctx = rt.Context()
    B, H, Hkv, D, S = 2, 4, 4, 128, 512
    x = torch.randn(B, H * D, dtype=torch.float16, device=DEV)
    w = torch.randn(H * D, 3 * H * D, dtype=torch.float16, device=DEV)
    kc = torch.zeros(1, B, Hkv, S, D, dtype=torch.float16, device=DEV)
    vc = torch.zeros_like(kc)
    seq = torch.tensor([3, 9], dtype=torch.int32, device=DEV)
    hx, hw, hk, hv, hs = (rt.Tensor(t) for t in (x, w, kc, vc, seq))
    tail = (0, hk.handle, hv.handle, None, None, hs.handle, 10, 0, H, Hkv, D, S, D, 10000.0)
    # size query: nothing is computed
    size = ctypes.c_int64(-1)
    x0 = x.clone()
    assert impl.diopiFusedDecoderAttentionInp(ctx.handle, hx.handle, hw.handle, None, None, ctypes.byref(size), *tail) == 0
    ctx.synchronize()
    assert size.value >= B * H * D * 2 and torch.equal(x, x0) and int(kc.abs().sum()) == 0
    # a workspace that is too small is refused with a message
    small = torch.empty(16, dtype=torch.int8, device=DEV)
    hsm = rt.Tensor(small)
    sz = ctypes.c_int64(16)
    assert impl.diopiFusedDecoderAttentionInp(ctx.handle, hx.handle, hw.handle, None, hsm.handle, ctypes.byref(sz), *tail) != 0
    assert b"workspace" in impl.diopiGetLastErrorString()
    # an exact-size workspace and the context's own scratch give the same bits
    ws = torch.empty(size.value, dtype=torch.int8, device=DEV)
    hws = rt.Tensor(ws)
    x1, k1 = x.clone(), kc.clone()
    hx1, hk1 = rt.Tensor(x1), rt.Tensor(k1)
    assert impl.diopiFusedDecoderAttentionInp(ctx.handle, hx1.handle, hw.handle, None, hws.handle, ctypes.byref(size), *((0, hk1.handle) + tail[2:])) == 0
    x2, k2 = x.clone(), kc.clone()
    hx2, hk2 = rt.Tensor(x2), rt.Tensor(k2)
    zero = ctypes.c_int64(0)
    assert impl.diopiFusedDecoderAttentionInp(ctx.handle, hx2.handle, hw.handle, None, None, ctypes.byref(zero), *((0, hk2.handle) + tail[2:])) == 0
    ctx.synchronize()
    ctx.clear_tensors()
    assert_bit_equal(x1, x2, "workspace tensor vs context scratch")
    assert_bit_equal(k1, k2, "workspace tensor vs context scratch: key cache")
    # an odd number of rotating dims is refused with a message
    r = impl.diopiFusedDecoderAttentionInp(ctx.handle, hx.handle, hw.handle, None, None, ctypes.byref(ctypes.c_int64(-1)), *(tail[:-2] + (33, 10000.0)))
    assert r != 0 and b"rotary_embedding" in impl.diopiGetLastErrorString()
    # float64 tensors are refused
    x64, w64, k64 = x.double(), w.double(), kc.double()
    v64 = k64.clone()
    hx64, hw64, hk64, hv64 = (rt.Tensor(t) for t in (x64, w64, k64, v64))
    r = impl.diopiFusedDecoderAttentionInp(ctx.handle, hx64.handle, hw64.handle, None, None, ctypes.byref(ctypes.c_int64(-1)), 0, hk64.handle, hv64.handle,
                                           *tail[3:])
    assert r != 0 and b"float16, bfloat16 or float32" in impl.diopiGetLastErrorString()


def test_fused_decoder_attention_partial_rotation_on_heads_of_128():
    # the first 64 (32, 2) dims of a head rotate, the rest keep their values
    for dt, rot, seed in ((torch.float16, 64, 21), (torch.bfloat16, 32, 22), (torch.float16, 2, 23)):
        _case(B=5, H=4, Hkv=2, S=300, seq=[0, 17, 299, 150, 64], dt=dt, seed=seed, rot=rot, pad=[0, 1, 2, 3, 4], step=310, what=f"rotary {rot} of 128")


def test_fused_decoder_attention_float32_and_other_head_sizes():
    """What the fast kernels do not take goes through the plain kernels: float32 tensors, heads of 64 / 80 / 256 dims, partial
    rotation there, more than 16 query heads per kv head, a hidden size that is no multiple of 128, unaligned tensors."""
    _case(B=5, H=4, Hkv=4, S=64, seq=[0, 1, 31, 40, 63], dt=torch.float32, seed=31, what="float32 MHA")
    _case(B=9, H=6, Hkv=2, S=50, seq=[0, 49, 120, 7, 50, 51, 99, 100, 3], dt=torch.float32, seed=32, D=64, rot=32, pad=[0, 1, 0, 2, 0, 3, 0, 4, 0],
          finished=[False] * 8 + [True], step=130, idt=torch.int64, what="float32 heads of 64, rotary 32, wrap")
    _case(B=3, H=4, Hkv=2, S=40, seq=[5, 39, 0], dt=torch.float16, seed=33, D=80, rot=40, hidden=4 * 80 + 8, what="fp16 heads of 80, rotary 40")
    _case(B=2, H=2, Hkv=1, S=33, seq=[32, 8], dt=torch.bfloat16, seed=34, D=256, rot=256, bias=False, what="bf16 heads of 256")
    _case(B=4, H=32, Hkv=1, S=70, seq=[69, 0, 33, 12], dt=torch.float16, seed=35, what="32 query heads on one kv head")
    _case(B=3, H=1, Hkv=1, S=20, seq=[19, 3, 10], dt=torch.float16, seed=36, hidden=200, what="hidden 200")
    _case(B=3, H=2, Hkv=2, S=20, seq=[19, 3, 10], dt=torch.float16, seed=37, misalign=True, what="unaligned tensors")
    _case(B=3, H=2, Hkv=2, S=20, seq=[19, 3, 10], dt=torch.float32, seed=38, rot=0, layers=3, layer=2, what="float32 no rotation, layer 2")


def test_fused_decoder_attention_caches_with_more_rows_than_the_batch():
    # the layer stride follows the caches' own batch dimension; rows past the batch stay as they are
    _case(B=3, H=4, Hkv=2, S=40, seq=[5, 39, 0], dt=torch.float16, seed=41, cache_rows=7, layers=3, layer=2, what="cache of 7 rows, fast path")
    _case(B=3, H=4, Hkv=2, S=40, seq=[5, 39, 0], dt=torch.float32, seed=42, cache_rows=5, layers=2, layer=1, D=64, rot=64, what="cache of 5 rows, plain path")


def test_fused_decoder_attention_far_positions():
    # position 100000: the angle needs more than fp32 (100000 * 6e-8 = 6e-3 radians of error otherwise)
    _case(B=3, H=4, Hkv=2, S=40, seq=[5, 39, 0], dt=torch.float16, seed=51, pad=[0, 7, 50000], step=100001, what="position 1e5, fast path")
    _case(B=3, H=4, Hkv=2, S=40, seq=[5, 39, 0], dt=torch.float32, seed=52, pad=[0, 7, 50000], step=100001, D=64, rot=64, what="position 1e5, float32")


def test_fused_decoder_attention_long_caches():
    # caches of 40000 to 70000 positions, nearly full, next to a short and an empty history; the plain kernels on 50000
    _case(2, 8, 2, 40000, [39998, 12345], torch.float16, 5, hidden=1024, layers=1, layer=0, what="long cache fp16")
    _case(3, 4, 4, 70000, [69999, 0, 35000], torch.bfloat16, 6, hidden=512, layers=1, layer=0, what="long cache bf16", step=70001)
    _case(1, 16, 1, 50000, [49999], torch.float32, 7, hidden=1024, layers=1, layer=0, what="long cache fp32, plain kernels", D=64, rot=32)


def test_fused_decoder_attention_more_items_than_the_ranking_takes():
    # 200 rows x 2 ranges of 1024 tokens are 400 items per kv head: past the 256 that are taken longest first, the plain order
    g = torch.Generator().manual_seed(61)
    seq = torch.randint(0, 2048, (200,), generator=g).tolist()
    seq[0], seq[1], seq[2] = 2047, 0, 1024
    _case(B=200, H=2, Hkv=1, S=2048, seq=seq, dt=torch.float16, seed=61, layers=1, layer=0, hidden=256, what="200 rows, 2 ranges")
