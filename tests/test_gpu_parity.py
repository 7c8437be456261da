"""Parity of the HIP operators (called through the C ABI of libdiopi_impl.so) against the CPU oracle.

Bars (north star): bit-exact for DestIndexCopyKV and all index handling; fp32 within rtol 1e-5
(atol 1e-5, the reference harness's own default); fp16/bf16 within atol = rtol = 1e-2.  Every case
also checks that the inputs were not modified, as the reference harness does (case_template.py:205-207).
"""
import math

import numpy as np
import pytest
import torch

from diopi_amd import functions as F
from diopi_amd import runtime as rt
from diopi_amd import workloads as W
from oracle import ref_ops as O
from tests.conftest import TORCH_DTYPES
from tests.helpers import TOL, assert_bit_equal, assert_close, report

pytestmark = pytest.mark.gpu
DEV = "cuda"


def say(*a):
    print(*a, flush=True)


def gen(seed):
    return torch.Generator().manual_seed(seed)


def snapshot(*tensors):
    return [None if t is None else t.clone() for t in tensors]


def assert_unmodified(before, *tensors):
    for b, t in zip(before, tensors):
        if b is not None:
            assert_bit_equal(t, b, "an input tensor was modified")


def test_library_identity():
    impl = rt.libs().impl
    assert b"Device" in impl.diopiGetVendorName()
    assert b"DIOPI Version: 1.0.0" in impl.diopiGetImplVersion()
    assert rt.device_count() >= 1


# ----------------------------------------------------------------------------- DestIndexCopyKV
def test_destindex_copy_kv_reference_fixtures(golden):
    g = gen(100)
    for case in golden["destindex_copy_kv"]["cases"]:
        for dt in (TORCH_DTYPES[case["dtype"]], torch.bfloat16):
            for idt in (torch.int32, torch.int64):
                k = torch.randn(*case["k_shape"], generator=g).to(dt)
                out = torch.randn(*case["out_shape"], generator=g).to(dt)
                dest = torch.tensor(case["dest_loc"], dtype=idt)
                want = O.destindex_copy_kv(k, dest, out.clone())
                kd, dd, od = k.to(DEV), dest.to(DEV), out.to(DEV)
                before = snapshot(kd, dd)
                F.destindex_copy_kv(kd, dd, od)
                assert_bit_equal(od, want, f"destindex {case['k_shape']} {dt} {idt}")
                assert_unmodified(before, kd, dd)


def test_destindex_copy_kv_config3_shape_bit_exact():
    w = W.cfg3(DEV, seed=3)
    for src, cache in ((w["new_k"], w["k_cache"]), (w["new_v"], w["v_cache"])):
        before_rows = cache[w["dest_loc"].long()].clone()
        ref = cache.clone()
        ref[w["dest_loc"].long()] = src  # torch's own scatter on the device as a second opinion
        sample = torch.randint(0, cache.shape[0], (4096,), generator=gen(1)).to(DEV)
        untouched_before = cache[sample].clone()
        F.destindex_copy_kv(src, w["dest_loc"], cache)
        assert torch.equal(cache.view(torch.int16), ref.view(torch.int16)), "full 1 GiB cache differs from the scatter"
        # oracle (numpy, CPU) on the touched rows and a sample of untouched ones
        assert_bit_equal(cache[w["dest_loc"].long()], src, "scattered rows")
        mask = ~torch.isin(sample, w["dest_loc"].long())
        assert_bit_equal(cache[sample][mask], untouched_before[mask], "untouched rows")
        del before_rows


def test_destindex_copy_kv_edge_cases():
    g = gen(101)
    # odd row sizes exercise every access width; negative indices wrap; out-of-range indices are dropped
    for shape, dt in (((7, 3, 5), torch.float16), ((6, 1, 3), torch.float32), ((5, 2, 2), torch.float64), ((9, 1, 1), torch.int8), ((4, 33), torch.bfloat16)):
        k = (torch.randn(*shape, generator=g) * 10).to(dt)
        rows = 23
        out = (torch.randn(rows, *shape[1:], generator=g) * 10).to(dt)
        dest = torch.randperm(rows, generator=g)[: shape[0]].int()
        want = O.destindex_copy_kv(k, dest, out.clone())
        od = out.to(DEV)
        F.destindex_copy_kv(k.to(DEV), dest.to(DEV), od)
        assert_bit_equal(od, want, f"odd shape {shape} {dt}")
    k = torch.randn(3, 4, 8, generator=g).half()
    out = torch.zeros(10, 4, 8).half()
    od = out.to(DEV)
    F.destindex_copy_kv(k.to(DEV), torch.tensor([-1, 2, 99], dtype=torch.int32).to(DEV), od)
    want = out.clone()
    want[9], want[2] = k[0], k[1]
    assert_bit_equal(od, want, "negative index wraps, out-of-range index is skipped")
    # empty token list
    F.destindex_copy_kv(torch.zeros(0, 4, 8, dtype=torch.float16, device=DEV), torch.zeros(0, dtype=torch.int32, device=DEV), od)
    assert_bit_equal(od, want, "empty scatter")


def test_destindex_copy_kv_repeated_destinations():
    """Several tokens sent to one row: the reference's non-accumulating index_put_ leaves the winner unspecified
    (functions_lightllm.cpp:18-26).  Every element of such a row must come from one of the tokens sent there, rows that
    receive one token get exactly that token, and all other rows stay as they were."""
    g = gen(150)
    for dt in (torch.float16, torch.float32):
        k = torch.randn(64, 32, 128, generator=g).to(dt).to(DEV)
        cache = torch.randn(40, 32, 128, generator=g).to(dt).to(DEV)
        before = cache.clone()
        dest = torch.tensor([3] * 20 + [7] * 30 + list(range(20, 33)) + [39], dtype=torch.int32, device=DEV)
        F.destindex_copy_kv(k, dest, cache)
        for row, senders in ((3, range(0, 20)), (7, range(20, 50))):
            from_some_sender = torch.zeros(32, 128, dtype=torch.bool, device=DEV)
            for t in senders:
                from_some_sender |= cache[row].view(torch.int16 if dt == torch.float16 else torch.int32) == k[t].view(
                    torch.int16 if dt == torch.float16 else torch.int32)
            assert bool(from_some_sender.all()), f"row {row} holds bytes that none of its tokens carries"
        assert_bit_equal(cache[20:33], k[50:63], "rows with a single token")
        assert_bit_equal(cache[39], k[63], "last row")
        rest = [r for r in range(40) if r not in (3, 7, 39) and not 20 <= r < 33]
        assert_bit_equal(cache[rest], before[rest], "rows that no token was sent to")


def test_destindex_copy_kv_large_round_trip():
    # encode -> scatter -> gather round trip over a full permutation of 65536 rows of 8 KiB
    T = 65536
    src = torch.randint(-32768, 32767, (T, 32, 128), dtype=torch.int16, device=DEV).view(torch.float16)
    perm = torch.randperm(T, device=DEV).int()
    cache = torch.zeros_like(src)
    F.destindex_copy_kv(src, perm, cache)
    assert torch.equal(cache[perm.long()].view(torch.int16), src.view(torch.int16))


# ----------------------------------------------------------------------------- RMSNorm
def _rms_case(shape, ns, eps, dt, with_bias, seed, ones_grad):
    g = gen(seed)
    x = torch.randn(*shape, generator=g).to(dt)
    w = (torch.rand(*ns, generator=g) + 0.5).to(dt)
    b = torch.randn(*ns, generator=g).to(dt) if with_bias else None
    go = torch.ones(*shape).to(dt) if ones_grad else torch.randn(*shape, generator=g).to(dt)
    xd, wd, bd, god = x.to(DEV), w.to(DEV), (b.to(DEV) if with_bias else None), go.to(DEV)
    before = snapshot(xd, wd, bd, god)
    out = F.rms_norm(xd, ns, wd, bd, eps)
    inv = F.GLOBAL_STATE["rms_norm_inv_rms"]
    grads = F.rms_norm_backward([god], xd, wd, bd, ns, eps)
    assert_unmodified(before, xd, wd, bd, god)
    ref_out, ref_inv = O.rms_norm(x, ns, w, b, eps)
    ex_out, ex_inv = O.rms_norm(x, ns, w, b, eps, exact=True)
    tol = TOL[dt]
    what = f"rms_norm {shape} ns={ns} {dt} bias={with_bias}"
    assert inv.dtype == (torch.float64 if dt == torch.float64 else torch.float32) and tuple(inv.shape) == tuple(ref_inv.shape)
    assert_close(inv, ex_inv, 1e-6 if dt != torch.float64 else 1e-12, 0, what + " inv_rms")
    assert_close(out, ref_out, what=what + " out vs reference composition", **tol)
    if dt == torch.float32 and not with_bias:
        # a product of three rounded factors keeps its relative accuracy down to the smallest element: the stated fp32
        # bar (rtol 1e-5) holds without any absolute term.  With a bias the final sum can cancel, hence atol above.
        assert_close(out, ref_out, rtol=1e-5, atol=0, what=what + " out vs reference composition, relative only")
    if with_bias and dt in (torch.float16, torch.bfloat16):
        # the reference rounds weight*normed to 16 bits before adding the bias: where the sum cancels, the distance to the
        # float64 value is one rounding of the larger intermediate, not of the result
        mag = float((ex_out - b.double()).abs().max())
        assert_close(out, ex_out, rtol=tol["rtol"], atol=max(tol["atol"], mag * 2.0 ** -8), what=what + " out vs float64")
    else:
        assert_close(out, ex_out, what=what + " out vs float64", **tol)
    # backward is checked with the inv_rms the device produced, as the harness feeds it back
    r_gi, r_gw, r_gb = O.rms_norm_backward(go, x, w, inv.cpu(), ns, with_bias=with_bias)
    e_gi, e_gw, e_gb = O.rms_norm_backward(go, x, w, inv.cpu(), ns, with_bias=with_bias, exact=True)
    n1 = x.numel() // int(np.prod(ns))
    assert_close(grads["input"], r_gi, what=what + " grad_input", **tol)
    assert_close(grads["input"], e_gi, what=what + " grad_input vs float64", **tol)
    # a column sum over n1 rows: the reference's own fp32 summation order moves the result by ~1e-7*sqrt(n1)*|terms|,
    # so the fp32 comparison against the float64 sum carries an absolute term scaled by the size of the sum
    scale = float((go.double() * x.double()).abs().sum(tuple(range(x.dim() - len(ns)))).max()) if n1 > 0 else 1.0
    atol_w = tol["atol"] if dt != torch.float32 else max(1e-5, 2e-7 * scale)
    assert_close(grads["weight"], e_gw, rtol=tol["rtol"], atol=atol_w, what=what + " grad_weight vs float64")
    if dt in (torch.float16, torch.bfloat16):
        # 16-bit outputs of sums over many rows: one rounding of the exact sum
        assert_close(grads["weight"], r_gw, rtol=1e-2, atol=max(1e-2, 8e-3 * float(e_gw.abs().max())), what=what + " grad_weight vs reference")
    if with_bias:
        assert_close(grads["bias"], e_gb, rtol=tol["rtol"], atol=max(atol_w, tol["atol"]), what=what + " grad_bias")
    return out


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32", "float64"])
def test_rms_norm_reference_cases(golden, dtype):
    dt = TORCH_DTYPES[dtype]
    for i, case in enumerate(golden["rms_norm"]["cases"]):
        for with_bias in (False, True):
            say("rms_norm case", case, dtype, with_bias)
            _rms_case(tuple(case["input"]), tuple(case["normalized_shape"]), case["eps"], dt, with_bias, 200 + i, ones_grad=(i % 2 == 0))


@pytest.mark.parametrize("shape,dtype", [((512, 4096), "float32"), ((300, 4096), "bfloat16"), ((129, 8192), "float16"), ((64, 1024), "float32"),
                                         ((33, 2048), "float16"), ((17, 4104), "float32"), ((8, 16384), "float32"), ((5, 40000), "float16"), ((130, 8192), "float32"), ((1100, 6144), "float32"),
                                         ((1030, 8192), "bfloat16")])
def test_rms_norm_wide_rows(shape, dtype):
    say("rms_norm wide", shape, dtype)
    _rms_case(shape, (shape[-1],), 1e-6, TORCH_DTYPES[dtype], with_bias=(shape[0] % 2 == 1), seed=300, ones_grad=False)


def test_rms_norm_config1_full_size():
    w = W.cfg1(DEV, seed=1)
    x, wt, go = w["x"], w["weight"], w["grad_out"]
    out = F.rms_norm(x, w["normalized_shape"], wt, None, w["eps"])
    inv = F.GLOBAL_STATE["rms_norm_inv_rms"]
    grads = F.rms_norm_backward([go], x, wt, None, w["normalized_shape"], w["eps"])
    xc, wc, goc = x.cpu(), wt.cpu(), go.cpu()
    ref_out, ref_inv = O.rms_norm(xc, w["normalized_shape"], wc, None, w["eps"])
    assert_close(out, ref_out, rtol=1e-5, atol=0, what="cfg1 out")  # a product: the relative bar holds for every element
    assert_close(inv, ref_inv, rtol=1e-5, atol=0, what="cfg1 inv_rms")
    e_gi, e_gw, _ = O.rms_norm_backward(goc, xc, wc, inv.cpu(), w["normalized_shape"], exact=True)
    r_gi, r_gw, _ = O.rms_norm_backward(goc, xc, wc, inv.cpu(), w["normalized_shape"])
    # grad_input is a difference of two terms of similar size: where they cancel, the result's error is one rounding of the
    # terms, so this comparison keeps the reference harness's absolute term
    assert_close(grads["input"], r_gi, rtol=1e-5, atol=1e-5, what="cfg1 grad_input")
    # grad_weight: against the float64 column sum at rtol 1e-5 with an absolute floor of one part in 1e7 of sum|terms|
    floor = 2e-7 * float((goc.double() * xc.double() * inv.cpu().double()[:, None]).abs().sum(0).max())
    assert_close(grads["weight"], e_gw, rtol=1e-5, atol=floor, what="cfg1 grad_weight vs float64")
    say("cfg1 grad_weight: max_abs/max_rel vs float64 %.3e %.3e ; reference fp32 order vs float64 %.3e %.3e" %
        (report(grads["weight"], e_gw) + report(r_gw, e_gw)))
    # the reference harness's own bar for rms_norm (atol = rtol = 1e-4) against the fp32 ATen result
    assert_close(grads["weight"], r_gw, rtol=1e-4, atol=1e-4, what="cfg1 grad_weight vs fp32 ATen")


def test_rms_norm_config2_full_size():
    w = W.cfg2(DEV, seed=2)
    out = F.rms_norm(w["x"], w["normalized_shape"], w["weight"], None, w["eps"])
    ref_out, ref_inv = O.rms_norm(w["x"].cpu(), w["normalized_shape"], w["weight"].cpu(), None, w["eps"])
    assert_close(out, ref_out, rtol=1e-2, atol=1e-2, what="cfg2 rms_norm bf16")
    assert_close(F.GLOBAL_STATE["rms_norm_inv_rms"], ref_inv, rtol=1e-5, atol=0, what="cfg2 inv_rms")
    # mixed precision pair of the reference: fp32 input, 16-bit output and weight
    x32 = w["x"][:257].float()
    o16 = F.rms_norm(x32, w["normalized_shape"], w["weight"], None, w["eps"], out_dtype=torch.bfloat16)
    r16, _ = O.rms_norm(x32.cpu(), w["normalized_shape"], w["weight"].cpu(), None, w["eps"], out_dtype=torch.bfloat16)
    assert_close(o16, r16, rtol=1e-2, atol=1e-2, what="fp32 -> bf16 rms_norm")


# ----------------------------------------------------------------------------- in-place RMS normalisations (lmdeploy set)
def _inplace_norm_case(shape, dt, with_bias, seed, eps=1e-6, offset=0):
    g = gen(seed)
    n = shape[-1]

    def dense(*sh):
        # offset > 0: a dense view whose first element is not 16-byte aligned
        flat = torch.randn(int(np.prod(sh)) + offset, generator=g).to(dt).to(DEV)
        return flat[offset:].view(*sh)

    x, r = dense(*shape), dense(*shape)
    b = dense(n) if with_bias else None
    w = (dense(n).abs() + 0.5).to(dt)
    xc, rc, bc, wc = x.cpu(), r.cpu(), (None if b is None else b.cpu()), w.cpu()
    before = snapshot(b, w)
    # plain form on a copy of x
    y = x.clone() if offset == 0 else dense(*shape).copy_(x)
    F.root_mean_square_norm_inp(y, w, eps)
    assert_close(y, O.root_mean_square_norm_inp(xc, wc, eps), what=f"plain {shape} {dt}", **TOL[dt])
    assert_close(y, O.root_mean_square_norm_inp(xc, wc, eps, exact=True), what=f"plain {shape} {dt} vs float64", **TOL[dt])
    # fused form
    F.fused_add_root_mean_square_norm_inp(x, r, b, w, eps)
    want_out, want_res = O.fused_add_root_mean_square_norm_inp(xc, rc, bc, wc, eps)
    e_out, e_res = O.fused_add_root_mean_square_norm_inp(xc, rc, bc, wc, eps, exact=True)
    if dt == torch.float32:
        assert_close(r, want_res, rtol=0, atol=0, what=f"fused {shape} {dt}: residual (fp32 sum, same order)")
    else:
        assert_bit_equal(r, want_res, f"fused {shape} {dt}: residual is the sum rounded once")
    assert_close(x, want_out, what=f"fused {shape} {dt} bias={with_bias}", **TOL[dt])
    assert_close(x, e_out, what=f"fused {shape} {dt} vs float64", **TOL[dt])
    assert_close(r, e_res, what=f"fused residual {shape} {dt} vs float64", **TOL[dt])
    assert_unmodified(before, b, w)


@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16"])
def test_inplace_norms_shapes(dtype):
    dt = TORCH_DTYPES[dtype]
    # the reference's rms_norm case shape, the model widths, rows with a tail, rows that are no packet multiple,
    # rows longer than the register form holds, a 3-d input, unaligned views
    for i, shape in enumerate([(12, 32), (7, 4096), (33, 8192), (5, 100), (3, 4104), (4, 11008), (2, 40000), (2, 3, 256), (1, 8)]):
        for with_bias in (False, True):
            say("in-place norm", shape, dtype, with_bias)
            _inplace_norm_case(shape, dt, with_bias, 500 + i)
    for shape in [(9, 4096), (4, 512)]:
        say("in-place norm, unaligned", shape, dtype)
        _inplace_norm_case(shape, dt, True, 520, offset=1)


def test_inplace_norms_full_size_and_against_the_separate_operators():
    w = W.cfg2(DEV, seed=2)  # bf16 [16384, 4096]
    x, wt, eps = w["x"], w["weight"], w["eps"]
    g = gen(530)
    res = torch.randn(x.shape, generator=g).to(x.dtype).to(DEV)
    x0, r0 = x.clone(), res.clone()
    F.fused_add_root_mean_square_norm_inp(x, res, None, wt, eps)
    want_out, want_res = O.fused_add_root_mean_square_norm_inp(x0.cpu(), r0.cpu(), None, wt.cpu(), eps)
    assert_bit_equal(res, want_res, "full size: residual")
    assert_close(x, want_out, what="full size: fused output", **TOL[torch.bfloat16])
    # the same step from the separate operators: an addition, then diopiRMSNorm on the stored sum
    two_step = F.rms_norm(want_res.to(DEV), w["normalized_shape"], wt, None, eps)
    assert_close(x, two_step, what="fused vs addition + diopiRMSNorm", **TOL[torch.bfloat16])
    # the plain form is diopiRMSNorm in place: same roundings, so the same bits
    y = x0.clone()
    F.root_mean_square_norm_inp(y, wt, eps)
    assert_bit_equal(y, F.rms_norm(x0, w["normalized_shape"], wt, None, eps), "plain form vs diopiRMSNorm")


def test_inplace_norms_empty_and_argument_errors():
    wt = torch.ones(64, device=DEV)
    x = torch.zeros(0, 64, device=DEV)
    F.root_mean_square_norm_inp(x, wt, 1e-6)
    F.fused_add_root_mean_square_norm_inp(x, torch.zeros(0, 64, device=DEV), None, wt, 1e-6)
    x = torch.randn(4, 64, device=DEV)
    with pytest.raises(rt.DiopiException):
        F.fused_add_root_mean_square_norm_inp(x, x, None, wt, 1e-6)  # one tensor in both roles
    with pytest.raises(rt.DiopiException):
        F.fused_add_root_mean_square_norm_inp(x, torch.randn(4, 32, device=DEV), None, wt, 1e-6)
    with pytest.raises(rt.DiopiException):
        F.root_mean_square_norm_inp(x, wt.half(), 1e-6)
    with pytest.raises(rt.DiopiException):
        F.root_mean_square_norm_inp(x.double(), wt.double(), 1e-6)
    torch.cuda.synchronize()


# ----------------------------------------------------------------------------- Rotary
@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32", "float64"])
def test_rotary_reference_cases(golden, dtype):
    dt = TORCH_DTYPES[dtype]
    g = gen(400)
    for case in golden["rotary_emb"]["cases"] + golden["rotary_emb"]["empty_cases"]:
        say("rotary case", case, dtype)
        x = torch.randn(*case["input"], generator=g).to(dt)
        cos = torch.randn(*case["cos"], generator=g).to(dt)
        sin = torch.randn(*case["cos"], generator=g).to(dt)
        xd, cd, sd = x.to(DEV), cos.to(DEV), sin.to(DEV)
        before = snapshot(xd, cd, sd)
        if case["interleaved"]:
            with pytest.raises(rt.FunctionNotImplementedError):  # the harness turns code 13 into a skip
                F.rotary_emb(xd, cd, sd, case["conj"], True)
            continue
        out = F.rotary_emb(xd, cd, sd, case["conj"], False)
        assert_unmodified(before, xd, cd, sd)
        ref = O.rotary_emb(x, cos, sin, case["conj"])
        if dt == torch.float64:
            # fp32 products, as the reference computes them: ten times tighter than the stated fp32 bar.  The absolute
            # term stays because o1 = x1*cos - x2*sin cancels: near zero the result carries one rounding of the products
            assert_close(out, ref, rtol=1e-6, atol=1e-6, what=f"rotary {case}")
        else:
            assert_close(out, ref, what=f"rotary {case}", **TOL[dt])


def test_rotary_position_zero_identity_and_inverse():
    g = gen(401)
    x = torch.randn(64, 32, 128, generator=g).half().to(DEV)
    one = torch.ones(64, 1, 64, dtype=torch.float16, device=DEV)
    zero = torch.zeros_like(one)
    assert_bit_equal(F.rotary_emb(x, one, zero, False, False), x, "angle 0 is the identity")
    ang = torch.rand(64, 1, 64, generator=g) * 6.28
    xf = x.float()
    y = F.rotary_emb(xf, ang.cos().to(DEV), ang.sin().to(DEV), False, False)
    back = F.rotary_emb(y, ang.cos().to(DEV), ang.sin().to(DEV), True, False)
    assert_close(back, xf, rtol=1e-5, atol=1e-5, what="conj inverts the rotation")


def test_rotary_config2_full_size():
    w = W.cfg2(DEV, seed=2)
    for name in ("q", "k"):
        out = F.rotary_emb(w[name], w["cos"], w["sin"], False, False)
        ref = O.rotary_emb(w[name].cpu(), w["cos"].cpu(), w["sin"].cpu(), False)
        # one rounding of an fp32 result on both sides: the results agree to the last bit almost everywhere
        assert_close(out, ref, rtol=1e-2, atol=1e-2, what=f"cfg2 rotary {name}")
        same = float((out.cpu().view(torch.int16) == ref.view(torch.int16)).float().mean())
        say(f"cfg2 rotary {name}: bit-identical fraction {same:.6f}")
        assert same > 0.999


def _rotary_v2_case(T, Hq, Hk, dim, dt, what, true_rotation=True):
    g = gen(700 + T)
    q = torch.randn(T, Hq * dim, generator=g).to(dt).to(DEV)
    k = torch.randn(T, Hk * dim, generator=g).to(dt).to(DEV)
    if true_rotation:
        ang = torch.rand(T, 1, dim // 2, generator=g) * 6.28
        cos, sin = torch.cat((ang.cos(), ang.cos()), -1).to(dt).to(DEV), torch.cat((ang.sin(), ang.sin()), -1).to(dt).to(DEV)
    else:
        cos, sin = torch.randn(T, 1, dim, generator=g).to(dt).to(DEV), torch.randn(T, 1, dim, generator=g).to(dt).to(DEV)
    q0, k0 = q.clone(), k.clone()
    before = snapshot(cos, sin)
    F.rotary_emb_v2(q, k, cos, sin, dim)
    assert_unmodified(before, cos, sin)
    rq, rk = O.rotary_emb_v2(q0.cpu(), k0.cpu(), cos.cpu(), sin.cpu(), dim)
    eq, ek = O.rotary_emb_v2(q0.cpu(), k0.cpu(), cos.cpu(), sin.cpu(), dim, exact=True)
    tol = TOL[dt]
    for got, ref, ex, name in ((q, rq, eq, "query"), (k, rk, ek, "key")):
        assert_close(got.cpu(), ref, what=f"{what} {name} vs reference composition", **tol)
        assert_close(got.cpu(), ex, what=f"{what} {name} vs float64", **tol)
    say(what, "query max_abs/rel vs f64: %.3e %.3e" % report(q.cpu(), eq))


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32", "float64"])
def test_rotary_v2_reference_case_and_variants(dtype):
    dt = TORCH_DTYPES[dtype]
    _rotary_v2_case(8, 32, 32, 128, dt, f"rotary v2 reference case (8, 4096) {dtype}")  # diopi_configs.py:9107-9135
    _rotary_v2_case(5, 8, 2, 64, dt, f"rotary v2 grouped heads {dtype}")
    _rotary_v2_case(3, 3, 1, 12, dt, f"rotary v2 odd sizes (element-wise kernel) {dtype}", true_rotation=False)
    _rotary_v2_case(4, 5, 3, 128, dt, f"rotary v2 unrelated table halves {dtype}", true_rotation=False)


def test_rotary_v2_matches_two_rotary_calls_at_config2_size():
    w = W.cfg2(DEV, seed=2)
    T, H, D = w["T"], w["H"], w["D"]
    cos, sin = torch.cat((w["cos"], w["cos"]), -1).contiguous(), torch.cat((w["sin"], w["sin"]), -1).contiguous()
    q, k = w["q"].reshape(T, H * D).clone(), w["k"].reshape(T, H * D).clone()
    F.rotary_emb_v2(q, k, cos, sin, D)
    q1 = F.rotary_emb(w["q"], w["cos"], w["sin"], False, False)
    k1 = F.rotary_emb(w["k"], w["cos"], w["sin"], False, False)
    assert_bit_equal(q.reshape(T, H, D).cpu(), q1.cpu(), "query: one fused launch equals the separate operator")
    assert_bit_equal(k.reshape(T, H, D).cpu(), k1.cpu(), "key: one fused launch equals the separate operator")


def test_rotary_v2_argument_errors():
    q = torch.randn(4, 64, device=DEV)
    k = torch.randn(4, 32, device=DEV)
    c = torch.randn(4, 1, 32, device=DEV)
    with pytest.raises(rt.DiopiException):
        F.rotary_emb_v2(q, k, c, c, 31)  # odd dim
    with pytest.raises(rt.DiopiException):
        F.rotary_emb_v2(q, k, c[:3], c, 32)  # table with the wrong number of tokens
    with pytest.raises(rt.DiopiException):
        F.rotary_emb_v2(q, k.half(), c, c, 32)  # mixed dtypes


# ----------------------------------------------------------------------------- sampling penalties
PENALTY_LOGITS = [[0.1, 0.5, 0.4, 0.3, 0.5], [0.2, 0.4, 0.0, 0.0, 0.0], [0.3, 0.4, 0.5, 0.3, 0.0]]
PENALTY_COUNTS = [3, 3, 2, 2, 1, 3, 3, 3, 3, 2, 2]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32", "float64"])
def test_apply_penalty_reference_fixture_and_random(dtype):
    dt = TORCH_DTYPES[dtype]
    for idt in (torch.int32, torch.int64):
        logits = torch.tensor(PENALTY_LOGITS, dtype=dt, device=DEV)  # diopi_configs.py:9265-9312
        pres, freq = torch.tensor([0.1, 0.8, 1.0], dtype=dt, device=DEV), torch.tensor([0.3, 0.5, 0.4], dtype=dt, device=DEV)
        ids = torch.tensor([0, 1, 2, 3, 4, 0, 1, 0, 1, 2, 3], dtype=idt, device=DEV)
        cnt = torch.tensor(PENALTY_COUNTS, dtype=idt, device=DEV)
        cum = torch.tensor([0, 5, 7, 11], dtype=idt, device=DEV)
        want = O.apply_penalty(logits.cpu().clone(), pres.cpu(), freq.cpu(), ids.cpu(), cnt.cpu(), cum.cpu(), 5)
        before = snapshot(pres, freq, ids, cnt, cum)
        F.apply_penalty(logits, pres, freq, ids, cnt, cum, 5)
        assert_unmodified(before, pres, freq, ids, cnt, cum)
        assert_bit_equal(logits.cpu(), want, f"apply_penalty fixture {dtype} {idt}: the reference's rounding sequence is reproduced exactly")
    # a batch of 37 sequences over a 32000-entry vocabulary, distinct ids per sequence, one empty sequence
    rng = np.random.Generator(np.random.PCG64(91))
    B, V = 37, 32000
    lens = rng.integers(0, 400, size=B)
    lens[11] = 0
    cum = np.concatenate(([0], np.cumsum(lens)))
    ids = np.concatenate([rng.permutation(V)[:n] for n in lens]).astype(np.int32)
    cnt = rng.integers(1, 50, size=int(cum[-1])).astype(np.int32)
    g = gen(92)
    logits = torch.randn(B, V, generator=g).to(dt).to(DEV)
    pres, freq = torch.rand(B, generator=g).to(dt).to(DEV), torch.rand(B, generator=g).to(dt).to(DEV)
    want = O.apply_penalty(logits.cpu().clone(), pres.cpu(), freq.cpu(), torch.from_numpy(ids), torch.from_numpy(cnt), torch.from_numpy(cum.astype(np.int32)), 400)
    F.apply_penalty(logits, pres, freq, torch.from_numpy(ids).to(DEV), torch.from_numpy(cnt).to(DEV), torch.from_numpy(cum.astype(np.int32)).to(DEV), 400)
    assert_bit_equal(logits.cpu(), want, f"apply_penalty random batch {dtype}")


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32", "float64"])
def test_apply_penalty_v2_reference_fixture_and_random(dtype):
    dt = TORCH_DTYPES[dtype]
    pen = torch.tensor([0.1] * 4 + [0.8] * 4 + [1.0] * 3, dtype=dt, device=DEV)  # diopi_configs.py:9468-9515
    ids = torch.tensor([0, 1, 2, 3, 4, 5, 6, 8, 9, 10, 11], dtype=torch.int32, device=DEV)
    cnt = torch.tensor(PENALTY_COUNTS, dtype=torch.int32, device=DEV)
    logits = torch.tensor(PENALTY_LOGITS, dtype=dt, device=DEV)
    want = O.apply_penalty_v2(logits.cpu().clone(), pen.cpu(), pen.cpu(), pen.cpu(), ids.cpu(), cnt.cpu())
    F.apply_penalty_v2(logits, pen, pen, pen, ids, cnt)
    assert_bit_equal(logits.cpu(), want, f"apply_penalty_v2 fixture {dtype}")
    rng = np.random.Generator(np.random.PCG64(93))
    B, V, n = 16, 32000, 5000
    flat_ids = rng.permutation(B * V)[:n].astype(np.int64)
    g = gen(94)
    logits = torch.randn(B, V, generator=g).to(dt).to(DEV)
    pres, freq = torch.rand(n, generator=g).to(dt).to(DEV), torch.rand(n, generator=g).to(dt).to(DEV)
    rep = (torch.rand(n, generator=g) + 0.5).to(dt).to(DEV)
    cnt = torch.from_numpy(rng.integers(1, 50, size=n).astype(np.int32))
    want = O.apply_penalty_v2(logits.cpu().clone(), pres.cpu(), freq.cpu(), rep.cpu(), torch.from_numpy(flat_ids), cnt)
    F.apply_penalty_v2(logits, pres, freq, rep, torch.from_numpy(flat_ids).to(DEV), cnt.to(DEV))
    assert_bit_equal(logits.cpu(), want, f"apply_penalty_v2 random {dtype}")


def test_apply_penalty_argument_errors_and_out_of_range_ids():
    logits = torch.zeros(2, 8, device=DEV)
    p = torch.ones(2, device=DEV)
    ids = torch.tensor([1, 100, -3], dtype=torch.int32, device=DEV)  # two ids outside the vocabulary are skipped
    cnt = torch.ones(3, dtype=torch.int32, device=DEV)
    F.apply_penalty(logits, p, p, ids, cnt, torch.tensor([0, 2, 3], dtype=torch.int32, device=DEV), 3)
    want = torch.zeros(2, 8)
    want[0, 1] = -2.0
    assert_bit_equal(logits.cpu(), want, "ids outside the vocabulary")
    with pytest.raises(rt.DiopiException):
        F.apply_penalty(logits, p, p, ids, cnt, torch.tensor([0, 3], dtype=torch.int32, device=DEV), 3)  # cumulative lengths too short
    with pytest.raises(rt.DiopiException):
        F.apply_penalty(logits, p.half(), p, ids, cnt, torch.tensor([0, 2, 3], dtype=torch.int32, device=DEV), 3)  # penalty dtype


# ----------------------------------------------------------------------------- decode attention
def _decode_case(w, dtype, what, seq_subset=None):
    """token_attention then token_softmax_reducev on workload dict `w`; oracle on the CPU for `seq_subset` sequences."""
    q, kc, vc = w["q"], w["k_cache"], w["v_cache"]
    H, total = q.shape[1], w["total_len"]
    tol = TOL[dtype]
    logits = torch.full((H, total), -12288.0, dtype=dtype, device=DEV)
    before = snapshot(q, w["b_loc"], w["b_start_loc"], w["b_seq_len"])
    F.token_attention(q, kc, logits, w["b_loc"], w["b_start_loc"], w["b_seq_len"], w["max_input_len"])
    out = torch.full_like(q, 7.0)  # every row must be written, also the zeros of a sequence without tokens
    F.token_softmax_reducev(logits, vc, out, w["b_loc"], w["b_start_loc"], w["b_seq_len"], w["max_input_len"], 0)
    assert_unmodified(before, q, w["b_loc"], w["b_start_loc"], w["b_seq_len"])
    idx = list(range(q.shape[0])) if seq_subset is None else seq_subset
    sel = torch.tensor(idx)
    # the oracle gathers only the cache rows it needs: remap slots of the chosen sequences to a compact cache
    b_loc_c, b_len_c, b_start_c = w["b_loc"].cpu()[sel], w["b_seq_len"].cpu()[sel], w["b_start_loc"].cpu()[sel]
    used = torch.unique(b_loc_c.long())
    remap = torch.zeros(int(used.max()) + 1, dtype=torch.int32)
    remap[used] = torch.arange(used.numel(), dtype=torch.int32)
    loc_small = remap[b_loc_c.long()]
    k_small, v_small = kc[used.to(DEV)].cpu(), vc[used.to(DEV)].cpu()
    ref_logits = torch.full((H, total), -12288.0, dtype=dtype)
    O.token_attention(q.cpu()[sel], k_small, ref_logits, loc_small, b_start_c, b_len_c, w["max_input_len"])
    ex_logits = torch.full((H, total), -12288.0, dtype=torch.float64)
    O.token_attention(q.cpu()[sel], k_small, ex_logits, loc_small, b_start_c, b_len_c, w["max_input_len"], exact=True)
    cols = torch.cat([torch.arange(int(s), int(s) + int(L)) for s, L in zip(b_start_c, b_len_c)])
    dev_logits = logits.cpu()
    assert_close(dev_logits[:, cols], ref_logits[:, cols], what=what + " logits vs reference composition", **tol)
    assert_close(dev_logits[:, cols], ex_logits[:, cols], what=what + " logits vs float64", **tol)
    if seq_subset is None:
        assert_bit_equal(dev_logits, torch.where(ref_logits == -12288.0, ref_logits, dev_logits), what + ": columns outside every sequence were written")
    # second operator: feed the oracle the device's logits so that the two checks are independent
    ref_out = torch.full((len(idx), H, q.shape[2]), -3.0, dtype=dtype)
    O.token_softmax_reducev(dev_logits, v_small, ref_out, loc_small, b_start_c, b_len_c, w["max_input_len"], 0)
    ex_out = torch.full((len(idx), H, q.shape[2]), -3.0, dtype=torch.float64)
    O.token_softmax_reducev(dev_logits, v_small, ex_out, loc_small, b_start_c, b_len_c, w["max_input_len"], 0, exact=True)
    assert_close(out.cpu()[sel], ref_out, what=what + " out vs reference composition", **tol)
    assert_close(out.cpu()[sel], ex_out, what=what + " out vs float64", **tol)
    say(what, "logits max_abs/rel vs f64: %.3e %.3e" % report(dev_logits[:, cols], ex_logits[:, cols]), " out: %.3e %.3e" % report(out.cpu()[sel], ex_out))
    return logits, out


@pytest.mark.parametrize("dtype", ["float16", "float32", "bfloat16", "float64"])
def test_decode_reference_fixture(golden, dtype):
    dt = TORCH_DTYPES[dtype]
    fx = golden["token_attention"]
    g = gen(500)
    w = dict(q=torch.randn(*fx["q_shape"], generator=g).to(dt).to(DEV), k_cache=torch.randn(*fx["k_shape"], generator=g).to(dt).to(DEV),
             v_cache=torch.randn(*fx["k_shape"], generator=g).to(dt).to(DEV), b_loc=torch.tensor(fx["b_loc"], dtype=torch.int32, device=DEV),
             b_start_loc=torch.tensor(fx["b_start_loc"], dtype=torch.int32, device=DEV), b_seq_len=torch.tensor(fx["b_seq_len"], dtype=torch.int32, device=DEV),
             max_input_len=fx["max_input_len"], total_len=13)
    _decode_case(w, dt, f"decode fixture {dtype}")


@pytest.mark.parametrize("dtype,Hq,Hkv", [("float16", 32, 32), ("bfloat16", 16, 2)])
def test_decode_sequences_sharing_cache_rows(dtype, Hq, Hkv):
    """Sequences with a common prefix point at the same cache rows (the row table is a table, not a partition): four
    sequences share their first 600 rows and differ in their tails; one row table also names a row twice."""
    dt = TORCH_DTYPES[dtype]
    g = gen(560)
    D, slots, maxlen = 128, 4096, 900
    prefix = torch.randperm(slots, generator=g)[:600]
    lens = [600, 731, 899, 655]
    b_loc = torch.zeros(len(lens), maxlen, dtype=torch.int32)
    for i, L in enumerate(lens):
        tail = torch.randint(0, slots, (L - 600,), generator=g)
        b_loc[i, maxlen - L:] = torch.cat((prefix, tail)).int()
    b_loc[2, maxlen - 1] = b_loc[2, maxlen - 2]  # the same row twice in one sequence
    starts = torch.tensor([0] + list(np.cumsum(lens)[:-1]), dtype=torch.int32)
    w = dict(q=torch.randn(len(lens), Hq, D, generator=g).to(dt).to(DEV), k_cache=torch.randn(slots, Hkv, D, generator=g).to(dt).to(DEV),
             v_cache=torch.randn(slots, Hkv, D, generator=g).to(dt).to(DEV), b_loc=b_loc.to(DEV), b_start_loc=starts.to(DEV),
             b_seq_len=torch.tensor(lens, dtype=torch.int32, device=DEV), max_input_len=maxlen, total_len=sum(lens))
    _decode_case(w, dt, f"decode with shared rows {dtype} {Hq}/{Hkv}")


def test_decode_range_length_follows_each_call_not_the_first_one():
    """The range length of the split decode kernel depends on the head grouping of the call at hand.  The scratch a call
    asks for shows it: B * ceil(max_len / range) * H * (D + 2) * 4 bytes with range = max(2048, 512 * G)."""
    g = gen(570)
    D, slots, maxlen, B = 128, 8192, 8192, 2

    def scratch_of(Hq, Hkv):
        ctx = rt.Context(own_stream=True)
        q = torch.randn(B, Hq, D, generator=g).half().to(DEV)
        v = torch.randn(slots, Hkv, D, generator=g).half().to(DEV)
        b_loc = torch.stack([torch.randperm(slots, generator=g)[:maxlen] for _ in range(B)]).int().to(DEV)
        lens = torch.tensor([maxlen, maxlen], dtype=torch.int32, device=DEV)
        starts = torch.tensor([0, maxlen], dtype=torch.int32, device=DEV)
        logits = torch.randn(Hq, B * maxlen, generator=g).half().to(DEV)
        out = torch.zeros(B, Hq, D, dtype=torch.float16, device=DEV)
        F.token_softmax_reducev(logits, v, out, b_loc, starts, lens, maxlen, 0, ctx=ctx)
        ctx.synchronize()
        peak = ctx.scratch_peak
        ctx.close()
        return peak

    def expected(Hq, Hkv):
        rng_len = max(2048, 512 * (Hq // Hkv))
        return B * math.ceil(maxlen / rng_len) * Hq * (D + 2) * 4

    for Hq, Hkv in ((4, 4), (8, 1), (4, 4), (8, 2)):  # ungrouped first, then grouped, and back
        peak = scratch_of(Hq, Hkv)
        want = expected(Hq, Hkv)
        assert want <= peak < want + 2048, f"{Hq}/{Hkv} heads: scratch {peak} bytes, expected {want} (+ rounding)"


def test_decode_index_exactness_and_int64():
    # k[slot] = slot pattern: the logits are exact small integers times a constant, so any wrong slot shows up exactly
    D, H = 128, 32
    slots = 300
    k = (torch.arange(slots, dtype=torch.float32) % 61).reshape(slots, 1, 1).expand(slots, H, D).contiguous().half().to(DEV)
    k = k * (torch.arange(D, device=DEV) == 0)  # only dim 0 is non-zero -> q.k = slot % 61 exactly
    q = torch.ones(3, H, D, dtype=torch.float16, device=DEV)
    rng = np.random.Generator(np.random.PCG64(7))
    b_len = np.array([1, 130, 77])
    b_start = np.array([0, 1, 131])
    b_loc = rng.permutation(slots)[: 3 * 90].reshape(3, 90)
    b_loc = np.concatenate([b_loc, rng.permutation(slots)[: 3 * 60].reshape(3, 60)], axis=1)  # width 150
    for idt in (torch.int32, torch.int64):
        out = torch.zeros(H, 208, dtype=torch.float16, device=DEV)
        F.token_attention(q, k, out, torch.from_numpy(b_loc).to(idt).to(DEV), torch.from_numpy(b_start).to(idt).to(DEV),
                          torch.from_numpy(b_len).to(idt).to(DEV), 140)
        want = np.concatenate([b_loc[i, 140 - L:140] % 61 for i, L in enumerate(b_len)]).astype(np.float32)
        want = torch.tensor(want).half().float() * (1.0 / math.sqrt(D))
        # a wrong slot moves a logit by at least 1/sqrt(128) = 0.088
        assert_close(out.cpu(), want.half().expand(H, 208), rtol=0, atol=1e-3, what=f"slot pattern {idt}")


def test_decode_config3_scaled_and_ragged():
    w = W.cfg3(DEV, seed=3, scale=0.125)  # 8 sequences of 512..2048 tokens
    _decode_case(w, torch.float16, "cfg3 x 1/8")
    # ragged: lengths 1, 15, 16, 17, 127, 128, 129, 257 and one empty sequence
    lens = np.array([1, 15, 16, 17, 0, 127, 128, 129, 257], dtype=np.int32)
    B = len(lens)
    w2 = W._decode(DEV, 33, torch.float16, B, 32, 32, 128, 4096, 1, 300, B)
    w2["b_seq_len"] = torch.from_numpy(lens).to(DEV)
    w2["b_start_loc"] = torch.from_numpy(np.concatenate(([0], np.cumsum(lens)[:-1])).astype(np.int32)).to(DEV)
    w2["total_len"] = int(lens.sum())
    w2["max_input_len"] = 260
    _decode_case(w2, torch.float16, "ragged lengths")


def test_decode_work_order_with_many_sequences_and_many_ranges():
    """The second decode operator hands its (sequence, range) items to the work-groups longest first when it can rank them:
    all items up to 256, the sequences of each range up to 256 sequences, nothing beyond.  Each of the three ways must give
    every item to exactly one work-group: the whole output against the oracle, with ties among the lengths and empty
    sequences in every case."""
    rng = np.random.Generator(np.random.PCG64(91))

    def case(B, lo, hi, what, fixed=()):
        lens = rng.integers(lo, hi + 1, size=B).astype(np.int32)
        for pos, val in fixed:
            lens[pos] = val
        w = W._decode(DEV, 90 + B, torch.float16, B, 2, 2, 128, B * hi, 1, hi, B)
        w["b_seq_len"] = torch.from_numpy(lens).to(DEV)
        w["b_start_loc"] = torch.from_numpy(np.concatenate(([0], np.cumsum(lens)[:-1])).astype(np.int32)).to(DEV)
        w["total_len"] = int(lens.sum())
        w["max_input_len"] = int(hi)
        _decode_case(w, torch.float16, what)

    # 3 ranges of 2048 tokens x 100 sequences = 300 items: ranked per range
    case(100, 1, 5000, "100 sequences x 3 ranges", fixed=((0, 0), (1, 2048), (2, 2048), (3, 2049), (4, 4096), (5, 5000), (6, 5000), (99, 0)))
    # 300 sequences of one range: taken as they come
    case(300, 1, 200, "300 short sequences", fixed=((0, 0), (7, 200), (8, 200), (299, 0)))
    # 2 ranges x 128 sequences = 256 items: all ranked together, many ties
    case(128, 2040, 2056, "128 sequences x 2 ranges, lengths within 16 of each other", fixed=((5, 0), (6, 1)))


def test_decode_gqa_config5_scaled():
    w = W.cfg5(DEV, seed=5, scale=1 / 32)  # 4 sequences of 1024..8192 tokens, 64 q heads over 8 kv heads
    _decode_case(w, torch.bfloat16, "cfg5 x 1/32")
    for G, Hkv in ((2, 4), (4, 2), (16, 1), (3, 2)):
        w3 = W._decode(DEV, 55 + G, torch.float16, 3, G * Hkv, Hkv, 128, 2048, 5, 600, 3)
        _decode_case(w3, torch.float16, f"GQA G={G} Hkv={Hkv}")


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_decode_head_size_64(dtype):
    """Head size 64 takes the matrix-core kernel that reads its operands straight from the cache rows (score operator)
    and the shape-agnostic reduce kernel: one query head per cache head and grouped heads, ragged lengths that are no
    multiple of 16 or 128 (and an empty sequence), 32- and 64-bit index tensors."""
    dt = TORCH_DTYPES[dtype]
    for (H, Hkv, idt) in ((8, 8, torch.int32), (12, 3, torch.int64), (16, 1, torch.int32)):
        lens = np.array([1, 15, 16, 17, 0, 127, 128, 129, 300, 77], dtype=np.int64)
        B = len(lens)
        w = W._decode(DEV, 640 + H, dt, B, H, Hkv, 64, 4096, 1, 320, B)
        w["b_seq_len"] = torch.from_numpy(lens).to(idt).to(DEV)
        w["b_start_loc"] = torch.from_numpy(np.concatenate(([0], np.cumsum(lens)[:-1]))).to(idt).to(DEV)
        w["b_loc"] = w["b_loc"].to(idt)
        w["total_len"] = int(lens.sum())
        w["max_input_len"] = 310
        _decode_case(w, dt, f"decode D=64 {dtype} H={H} Hkv={Hkv} {idt}")


def test_context_attention_scratch_returns_to_the_pool():
    """The tile plan of a prefill call is context scratch: repeated calls through the Python wrappers must reuse one
    block of the context's pool instead of growing it."""
    g = gen(641)
    T = 700
    q, k, v = ((torch.randn(T, 2, 128, generator=g) * 0.5).half().to(DEV) for _ in range(3))
    bs, bl = torch.tensor([0, 300], dtype=torch.int32, device=DEV), torch.tensor([300, 400], dtype=torch.int32, device=DEV)
    ctx = rt.Context(own_stream=True)
    out = torch.zeros_like(q)
    F.context_attention(q, k, v, out, bs, bl, 400, ctx=ctx)
    first = ctx.malloc_count
    assert first == 1
    for _ in range(20):
        F.context_attention(q, k, v, out, bs, bl, 400, ctx=ctx)
        F.flash_attention_varlen(q, k, v, torch.tensor([0, 300, 700], dtype=torch.int32, device=DEV), torch.tensor([0, 300, 700], dtype=torch.int32, device=DEV),
                                 None, 400, 400, 0.0, None, True, ctx=ctx)
    ctx.synchronize()
    assert ctx.malloc_count == first, f"the pool grew: {ctx.malloc_count} allocations"
    ctx.close()


def test_decode_config3_full_size_sampled():
    w = W.cfg3(DEV, seed=3)
    logits, out = _decode_case(w, torch.float16, "cfg3 full, 16 sequences checked", seq_subset=[0, 3, 7, 12, 16, 21, 25, 30, 34, 40, 45, 49, 54, 58, 62, 63])
    # size-independent properties over the whole batch: constant logits give the mean of the gathered rows,
    # and the result is invariant under a relabelling of the cache slots
    const = torch.zeros_like(logits)
    o2 = torch.zeros_like(out)
    F.token_softmax_reducev(const, w["v_cache"], o2, w["b_loc"], w["b_start_loc"], w["b_seq_len"], w["max_input_len"], 0)
    i = 17
    L = int(w["b_seq_len"][i])
    rows = w["b_loc"][i, w["max_input_len"] - L: w["max_input_len"]].long()
    assert_close(o2[i], w["v_cache"][rows].float().mean(0), rtol=1e-2, atol=1e-2, what="uniform softmax = mean of rows")
    perm = torch.randperm(w["slots"], device=DEV)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(w["slots"], device=DEV)
    k2 = torch.empty_like(w["k_cache"])
    k2[perm] = w["k_cache"]
    l2 = torch.zeros_like(logits)
    F.token_attention(w["q"], k2, l2, perm[w["b_loc"].long()].int(), w["b_start_loc"], w["b_seq_len"], w["max_input_len"])
    assert_bit_equal(l2, logits, "relabelling the cache slots changes nothing")


def _whole_batch_decode_checks(w, logits, out, what):
    """Checks of a full-size decode step that cover every sequence of the batch without the CPU oracle: the logits and the
    output against a float32 statement of the operator evaluated with torch on the device (gather, matmul, softmax, one
    sequence at a time), the uniform-softmax closed form, and invariance under a relabelling of the cache slots."""
    q, kc, vc = w["q"], w["k_cache"], w["v_cache"]
    B, H, D = q.shape
    Hkv = kc.shape[1]
    G = H // Hkv
    n = w["max_input_len"]
    lens, starts = w["b_seq_len"].tolist(), w["b_start_loc"].tolist()
    tol = TOL[q.dtype]
    const = torch.zeros_like(logits)
    mean_out = torch.zeros_like(out)
    F.token_softmax_reducev(const, vc, mean_out, w["b_loc"], w["b_start_loc"], w["b_seq_len"], n, 0)
    worst_l = worst_o = worst_m = 0.0
    for i in range(B):
        L, s0 = lens[i], starts[i]
        rows = w["b_loc"][i, n - L: n].long()
        k_rows = kc[rows].float()                                   # [L, Hkv, D]
        qi = q[i].float().reshape(Hkv, G, D)
        # the reference's own roundings: the dot product to the tensor dtype, then the division by sqrt(D)
        dots = torch.einsum("hgd,lhd->hgl", qi, k_rows).to(q.dtype).float()
        want_l = (dots / math.sqrt(D)).to(q.dtype).reshape(H, L)
        got_l = logits[:, s0: s0 + L]
        bad = ((got_l.float() - want_l.float()).abs() > tol["atol"] + tol["rtol"] * want_l.float().abs()).sum().item()
        assert bad == 0, f"{what}: sequence {i} (length {L}): {bad} logits outside tolerance of the float32 statement"
        worst_l = max(worst_l, float((got_l.float() - want_l.float()).abs().max()))
        v_rows = vc[rows].float()
        p = torch.softmax(got_l.float(), dim=-1).to(q.dtype).float().reshape(Hkv, G, L)
        want_o = torch.einsum("hgl,lhd->hgd", p, v_rows).reshape(H, D)
        assert_close(out[i], want_o, what=f"{what}: sequence {i} (length {L}) output vs the float32 statement", **tol)
        worst_o = max(worst_o, float((out[i].float() - want_o).abs().max()))
        want_m = v_rows.mean(0).repeat_interleave(G, dim=0)
        assert_close(mean_out[i], want_m, what=f"{what}: sequence {i}: uniform softmax = mean of rows", **tol)
        worst_m = max(worst_m, float((mean_out[i].float() - want_m).abs().max()))
    say(what, "all %d sequences: max abs error logits %.3e, output %.3e, uniform %.3e" % (B, worst_l, worst_o, worst_m))
    del const, mean_out
    perm = torch.randperm(w["slots"], device=DEV)
    k2 = torch.empty_like(kc)
    k2[perm] = kc
    l2 = torch.full_like(logits, -12288.0)
    F.token_attention(q, k2, l2, perm[w["b_loc"].long()].int(), w["b_start_loc"], w["b_seq_len"], n)
    assert_bit_equal(l2, logits, what + ": relabelling the cache slots changes nothing")


def test_decode_pair_random_shapes_against_float64_on_the_device():
    """120 seeded random draws of batch, head grouping (1 to 16 query heads per kv head), ragged lengths (empty sequences among
    them), dtype and the spread of q and k: TokenAttention against the scaled dot products in float64, SoftmaxReduceV against
    the float64 softmax of the logits the first operator wrote (probabilities rounded to the element type, as the reference
    does), both evaluated on the device."""
    g = gen(913)

    def pick(*vals):
        return vals[int(torch.randint(len(vals), (1,), generator=g))]

    for case in range(120):
        Hkv, G = pick(1, 2, 3, 8), pick(1, 2, 4, 5, 8, 16)
        H = Hkv * G
        B = pick(1, 2, 5, 17, 64)
        hi = pick(5, 70, 300, 1000, 2500, 5000, 9000)
        lens = torch.randint(0 if pick(0, 1) else 1, hi + 1, (B,), generator=g)
        dt = pick(torch.float16, torch.bfloat16)
        std = pick(0.5, 1.0, 3.0)
        maxlen = max(1, int(lens.max()))
        slots = int(lens.sum()) + 64
        kc = (torch.randn(slots, Hkv, 128, generator=g) * std).to(dt).to(DEV)
        vc = torch.randn(slots, Hkv, 128, generator=g).to(dt).to(DEV)
        q = (torch.randn(B, H, 128, generator=g) * std).to(dt).to(DEV)
        perm = torch.randperm(slots, generator=g)
        b_loc = torch.zeros(B, maxlen, dtype=torch.int32)
        start = torch.zeros(B, dtype=torch.int32)
        pos = 0
        for i, L in enumerate(lens.tolist()):
            b_loc[i, maxlen - L:] = perm[pos:pos + L].int()
            start[i] = pos
            pos += L
        total = max(1, pos)
        b_loc, start, ln = b_loc.to(DEV), start.to(DEV), lens.int().to(DEV)
        what = f"random decode case {case}: B={B} H={H} Hkv={Hkv} lengths {lens.tolist()[:8]} {dt} spread {std}"
        logits = torch.full((H, total), -77.0, dtype=dt, device=DEV)
        F.token_attention(q, kc, logits, b_loc, start, ln, maxlen)
        out = torch.full_like(q, 5.0)
        F.token_softmax_reducev(logits, vc, out, b_loc, start, ln, maxlen, 0)
        assert bool(torch.isfinite(out.float()).all()), what + ": non-finite output"
        for i, L in enumerate(lens.tolist()):
            if L == 0:
                assert int(out[i].count_nonzero()) == 0, what + ": an empty sequence gives zeros"
                continue
            sl = b_loc[i, maxlen - L:].long()
            kk = kc[sl].double().repeat_interleave(G, dim=1)
            vv = vc[sl].double().repeat_interleave(G, dim=1)
            sc = torch.einsum("hd,lhd->hl", q[i].double(), kk) / math.sqrt(128.0)
            got = logits[:, int(start[i]):int(start[i]) + L]
            assert_close(got, sc, rtol=2e-2, atol=1e-2, what=what + f": logits of sequence {i}")  # two roundings to the element type
            p = got.double().softmax(-1).to(dt).double()
            assert_close(out[i], torch.einsum("hl,lhd->hd", p, vv), what=what + f": output of sequence {i}", **TOL[dt])


@pytest.mark.parametrize("Hkv,G,lens,dtype,index_dtype", [
    (1, 16, [70001, 3, 20000], torch.bfloat16, torch.int64),
    (8, 8, [33000, 1, 66000, 0, 127], torch.float16, torch.int32),
    (2, 4, [262144], torch.bfloat16, torch.int32),
])
def test_decode_pair_very_long_sequences(Hkv, G, lens, dtype, index_dtype):
    """Contexts far beyond the benchmark's (up to 262144 tokens: 32 or more ranges per sequence, the merge kernel's batches of 8
    more than once) next to very short and empty ones, against float64 on the device in chunks of 16384 tokens."""
    g = gen(915)
    H, B = Hkv * G, len(lens)
    maxlen, slots = max(lens), sum(lens) + 64
    kc = torch.randn(slots, Hkv, 128, generator=g).to(dtype).to(DEV)
    vc = torch.randn(slots, Hkv, 128, generator=g).to(dtype).to(DEV)
    q = torch.randn(B, H, 128, generator=g).to(dtype).to(DEV)
    perm = torch.randperm(slots, generator=g)
    b_loc = torch.zeros(B, maxlen, dtype=index_dtype)
    start = torch.zeros(B, dtype=index_dtype)
    pos = 0
    for i, L in enumerate(lens):
        b_loc[i, maxlen - L:] = perm[pos:pos + L].to(index_dtype)
        start[i] = pos
        pos += L
    b_loc, start, ln = b_loc.to(DEV), start.to(DEV), torch.tensor(lens, dtype=index_dtype, device=DEV)
    logits = torch.full((H, pos), -77.0, dtype=dtype, device=DEV)
    F.token_attention(q, kc, logits, b_loc, start, ln, maxlen)
    out = torch.full_like(q, 5.0)
    F.token_softmax_reducev(logits, vc, out, b_loc, start, ln, maxlen, 0)
    for i, L in enumerate(lens):
        what = f"long decode Hkv={Hkv} G={G} {dtype}: sequence {i} of {L} tokens"
        if L == 0:
            assert int(out[i].count_nonzero()) == 0, what + ": an empty sequence gives zeros"
            continue
        sl = b_loc[i, maxlen - L:].long()
        got = logits[:, int(start[i]):int(start[i]) + L]
        p = got.double().softmax(-1).to(dtype).double()
        ref = torch.zeros(H, 128, dtype=torch.float64, device=DEV)
        for c0 in range(0, L, 16384):
            rows = sl[c0:c0 + 16384]
            kk = kc[rows].double().repeat_interleave(G, dim=1)
            vv = vc[rows].double().repeat_interleave(G, dim=1)
            sc = torch.einsum("hd,lhd->hl", q[i].double(), kk) / math.sqrt(128.0)
            assert_close(got[:, c0:c0 + 16384], sc, rtol=2e-2, atol=1e-2, what=what + f": logits from token {c0}")
            ref += torch.einsum("hl,lhd->hd", p[:, c0:c0 + 16384], vv)
        assert_close(out[i], ref, what=what + ": output", **TOL[dtype])


def test_decode_config5_full_size_sampled():
    w = W.cfg5(DEV, seed=5)
    lens = w["b_seq_len"].tolist()
    longest, shortest = max(range(len(lens)), key=lens.__getitem__), min(range(len(lens)), key=lens.__getitem__)
    subset = sorted(set([0, 9, 17, 26, 38, 47, 55, 64, 72, 81, 90, 99, 106, 113, 120, 127, longest, shortest]))
    logits, out = _decode_case(w, torch.bfloat16, f"cfg5 full, {len(subset)} sequences checked (longest and shortest among them)", seq_subset=subset)
    _whole_batch_decode_checks(w, logits, out, "cfg5 full, whole batch")


# ----------------------------------------------------------------------------- prefill attention
def _context_case(q, k, v, b_start, b_len, max_len, dt, what, check_rows=None):
    T = q.shape[0]
    out = torch.full_like(q, 77.0)
    before = snapshot(q, k, v, b_start, b_len)
    F.context_attention(q, k, v, out, b_start, b_len, max_len)
    assert_unmodified(before, q, k, v, b_start, b_len)
    tol = TOL[dt]
    outc = out.cpu()
    covered = torch.zeros(T, dtype=torch.bool)
    for s, L in zip(b_start.tolist(), b_len.tolist()):
        covered[s:s + L] = True
        if L > 0:
            assert_bit_equal(outc[s], v[s].cpu(), what + ": the first token of a sequence returns its own v row")
    assert bool((outc[~covered] == 77.0).all()), what + ": rows outside every sequence were written"
    if check_rows is None:
        ref = torch.full(q.shape, 77.0, dtype=dt)
        O.context_attention(q.cpu(), k.cpu(), v.cpu(), ref, b_start.cpu(), b_len.cpu(), max_len)
        ex = torch.full(q.shape, 77.0, dtype=torch.float64)
        O.context_attention(q.cpu(), k.cpu(), v.cpu(), ex, b_start.cpu(), b_len.cpu(), max_len, exact=True)
        # the reference narrows the scores to fp32 for its softmax whatever the tensor dtype (functions_lightllm.cpp:122),
        # so for float64 tensors its own result is only fp32-accurate
        rtol_ref = dict(rtol=1e-6, atol=1e-6) if dt == torch.float64 else tol
        assert_close(outc, ref, what=what + " vs reference composition", **rtol_ref)
        assert_close(outc, ex, what=what + " vs float64", **tol)
        say(what, "max_abs/rel vs f64: %.3e %.3e" % report(outc, ex))
    else:
        # full-size inputs: float64 attention for sampled rows only (decode formulation of the same row)
        kc, vc = k.cpu(), v.cpu()
        for (i, r) in check_rows:
            s = int(b_start[i])
            qq = q[s + r: s + r + 1].cpu()
            loc = torch.arange(s, s + r + 1, dtype=torch.int32).reshape(1, -1)
            lg = torch.zeros(q.shape[1], r + 1, dtype=torch.float64)
            O.token_attention(qq, kc, lg, loc, torch.tensor([0]), torch.tensor([r + 1]), r + 1, exact=True)
            ex = torch.zeros(1, q.shape[1], q.shape[2], dtype=torch.float64)
            O.token_softmax_reducev(lg, vc, ex, loc, torch.tensor([0]), torch.tensor([r + 1]), r + 1, 0, exact=True)
            assert_close(outc[s + r], ex[0], what=f"{what} sequence {i} row {r} vs float64", **tol)
    return out


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32", "float64"])
def test_context_attention_reference_fixtures(golden, dtype):
    dt = TORCH_DTYPES[dtype]
    g = gen(600)
    for case in golden["context_attention"]["cases"]:
        say("context case", case, dtype)
        q, k, v = ((torch.randn(*case["shape"], generator=g) * 0.5).to(dt).to(DEV) for _ in range(3))
        bs = torch.tensor(case["b_start_loc"], dtype=torch.int32, device=DEV)
        bl = torch.tensor(case["b_seq_len"], dtype=torch.int32, device=DEV)
        _context_case(q, k, v, bs, bl, case["max_input_len"], dt, f"context {case['shape']} {dtype}")


def test_context_attention_ragged_lengths():
    g = gen(601)
    lens = [1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 191, 193, 300]
    starts, pos = [], 3  # a gap before the first sequence and between some of them
    for i, L in enumerate(lens):
        starts.append(pos)
        pos += L + (5 if i % 3 == 0 else 0)
    T = pos + 4
    for dt in (torch.float16, torch.bfloat16):
        q, k, v = ((torch.randn(T, 4, 128, generator=g) * 0.5).to(dt).to(DEV) for _ in range(3))
        for idt in (torch.int32, torch.int64):
            _context_case(q, k, v, torch.tensor(starts, dtype=idt, device=DEV), torch.tensor(lens, dtype=idt, device=DEV), max(lens), dt,
                          f"ragged {dt} {idt}")


def test_context_attention_many_short_sequences():
    # more sequences than lanes in a wave or threads in the planning group's first pass, empty ones included
    rng = np.random.Generator(np.random.PCG64(77))
    lens = rng.integers(0, 40, size=1100).tolist()
    lens[5], lens[700] = 300, 129
    starts = np.concatenate(([0], np.cumsum(lens)[:-1])).tolist()
    T = int(sum(lens))
    g = gen(602)
    q, k, v = ((torch.randn(T, 2, 128, generator=g) * 0.5).to(torch.float16).to(DEV) for _ in range(3))
    _context_case(q, k, v, torch.tensor(starts, dtype=torch.int32, device=DEV), torch.tensor(lens, dtype=torch.int32, device=DEV), max(lens),
                  torch.float16, "1100 short sequences")


def test_context_attention_long_odd_lengths_whole_output():
    # long enough for the 256-row query tiles; lengths that are no multiple of any tile size; every row checked
    lens = [1531, 1099]
    starts = [0, 1531]
    g = gen(603)
    for dt in (torch.float16, torch.bfloat16):
        q, k, v = ((torch.randn(sum(lens), 2, 128, generator=g) * 0.5).to(dt).to(DEV) for _ in range(3))
        _context_case(q, k, v, torch.tensor(starts, dtype=torch.int32, device=DEV), torch.tensor(lens, dtype=torch.int32, device=DEV), max(lens), dt,
                      f"two long sequences {dt}")


def _rising_case(L, H, dt, profile, what, support=slice(0, 128)):
    """Scores that climb along the sequence: q = a * u + noise, k_j = b_j * u + noise with u a unit vector, so that the
    score of key j is about a * b_j (in powers of two after the softmax scale: `profile(j)`).  `support`: the head dims u
    lives on (the last 16 are the last of the eight products a score is summed from)."""
    g = gen(604)
    u = torch.zeros(128)
    u[support] = 1.0
    u = u / u.norm()
    a = 8.0
    to_raw = math.sqrt(128.0) / math.log2(math.e)  # from powers of two to the unscaled dot product
    b = torch.tensor([profile(j) * to_raw / a for j in range(L)])
    q = (a * u + 0.05 * torch.randn(L, H, 128, generator=g)).to(dt).to(DEV)
    k = (b.reshape(L, 1, 1) * u + 0.05 * torch.randn(L, H, 128, generator=g)).to(dt).to(DEV)
    v = torch.randn(L, H, 128, generator=g).to(dt).to(DEV)
    bs = torch.tensor([0], dtype=torch.int32, device=DEV)
    bl = torch.tensor([L], dtype=torch.int32, device=DEV)
    out = torch.full_like(q, 77.0)
    F.context_attention(q, k, v, out, bs, bl, L)
    ex = torch.full(q.shape, 77.0, dtype=torch.float64)
    O.context_attention(q.cpu(), k.cpu(), v.cpu(), ex, bs.cpu(), bl.cpu(), L, exact=True)
    assert bool(torch.isfinite(out.float()).all()), what + ": non-finite output"
    assert_close(out.cpu(), ex, what=what + " vs float64", **TOL[dt])


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_context_attention_rising_scores_move_the_softmax_reference(dtype):
    # The prefill kernels keep a lazily updated reference maximum per query row; seeded normal tensors never move it after
    # the first keys.  Here the scores climb by 2^60 along the sequence, steadily (the reference moves every few tiles) or
    # in single jumps that land in the lower and in the upper half of a 64-key tile, early and late in a query tile's keys.
    dt = TORCH_DTYPES[dtype]
    for L in (700, 1100):  # 128-row and 256-row query tiles
        _rising_case(L, 2, dt, lambda j: 60.0 * j / L, f"steady climb L={L} {dtype}")
        _rising_case(L, 2, dt, lambda j: (40.0 if j >= 100 else 0.0), f"jump at key 100 (upper half of tile 1) L={L} {dtype}")
        _rising_case(L, 2, dt, lambda j: (40.0 if j >= 200 else 0.0) + (30.0 if j >= 457 else 0.0),
                     f"jumps at keys 200 (lower half of tile 3) and 457 L={L} {dtype}")
        _rising_case(L, 2, dt, lambda j: 30.0 * (j % 64 == 63) + 20.0 * (j // 64), f"staircase with spikes L={L} {dtype}")


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_context_attention_second_rise_after_the_pipeline_was_left(dtype):
    """A first rise of the scores makes a wave leave its pipelined loop; a second one, by more than the 16 bits of headroom a
    16-bit probability has, then lands in the plain loop, in the upper half of a key tile, on each of the positions whose scores
    are the first to be read after the products (a read that came too early once moved the reference too little: NaN rows).
    Steps (every later key stays high) and isolated spikes, the second one 18-30 powers of two above the first, with the whole
    score carried by the last 16 head dims, i.e. by the last of the eight products it is summed from."""
    dt = TORCH_DTYPES[dtype]
    last = slice(112, 128)
    for pos in (0, 1, 2, 3, 6, 7, 12, 31):
        second = 64 * 9 + 32 + pos
        _rising_case(700, 1, dt, lambda j: (40.0 if j >= 100 else 0.0) + (30.0 if j >= second else 0.0), f"steps at 100 and {second} {dtype}", last)
        _rising_case(700, 1, dt, lambda j: 21.0 * (j < 32) + 42.0 * (j == 120) + 60.2 * (j == second), f"spikes at 120 and {second} {dtype}", last)
    # the shape the fault was found at: spikes deep in a long sequence, rows far below them
    _rising_case(2600, 1, dt, lambda j: 21.0 * (j < 32) + 42.0 * (j == 696) + 60.2 * (j == 1766), f"spikes at 696 and 1766, L=2600 {dtype}", last)
    _rising_case(1100, 2, dt, lambda j: 60.0 * j / 1100, f"steady climb on the last dims {dtype}", last)


def test_context_attention_random_shapes_two_kernels_and_float64():
    """160 seeded random draws of batch, ragged lengths (with lengths on and next to the tile sizes), heads, dtype and the spread
    of q and k (up to three times the configured one: sharply peaked softmax rows).  The lightllm operator must agree with
    diopiFlashAttentionVarLen on the same tokens (another kernel) to a few roundings, both must be finite, and for modest sizes
    both must match a float64 statement evaluated on the device.  bf16 draws with the widest spread are only checked for finite
    results: there the reference's own composition is 0.19 off float64 (rounded scores of size 40 move probabilities by 10 %)."""
    g = gen(911)

    def pick(*vals):
        return vals[int(torch.randint(len(vals), (1,), generator=g))]

    for case in range(160):
        B = pick(1, 2, 3, 5, 8, 12)
        hi = pick(3, 40, 130, 300, 700, 1500, 3000)
        lens = torch.randint(1, hi + 1, (B,), generator=g)
        if pick(0, 1):
            lens[int(torch.randint(B, (1,), generator=g))] = pick(1, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513, 1024, 1025)
        H = pick(1, 2, 5, 8)
        dt = pick(torch.float16, torch.bfloat16)
        std = pick(0.5, 1.0, 3.0)
        T = int(lens.sum())
        q = (torch.randn(T, H, 128, generator=g) * std).to(dt).to(DEV)
        k = (torch.randn(T, H, 128, generator=g) * std).to(dt).to(DEV)
        v = torch.randn(T, H, 128, generator=g).to(dt).to(DEV)
        start = torch.cat((torch.zeros(1, dtype=torch.long), lens.cumsum(0)[:-1])).int().to(DEV)
        ln = lens.int().to(DEV)
        what = f"random prefill case {case}: lengths {lens.tolist()}, {H} heads, {dt}, spread {std}"
        out = torch.full_like(q, 7.0)
        F.context_attention(q, k, v, out, start, ln, int(lens.max()))
        cu = torch.cat((start, (start[-1:] + ln[-1:]))).int()
        flash = F.flash_attention_varlen(q, k, v, cu, cu, None, int(lens.max()), int(lens.max()), 0.0, None, True)
        assert bool(torch.isfinite(out.float()).all()) and bool(torch.isfinite(flash.float()).all()), what + ": non-finite output"
        if dt is torch.bfloat16 and std > 2:
            continue
        tol = 4e-3 if dt is torch.float16 else 2e-2
        assert_close(out, flash, rtol=tol, atol=tol, what=what + ": the two kernels")
        if T <= 4000 and std < 2:
            s0 = 0
            for L in lens.tolist():
                qq, kk, vv = (t[s0:s0 + L].double().transpose(0, 1) for t in (q, k, v))
                sc = qq @ kk.transpose(1, 2) / math.sqrt(128.0)
                sc = sc.masked_fill(torch.triu(torch.ones(L, L, dtype=torch.bool, device=DEV), 1), float("-inf"))
                ref = (sc.softmax(-1) @ vv).transpose(0, 1)
                assert_close(out[s0:s0 + L], ref, what=what + " vs float64 on the device", **TOL[dt])
                s0 += L


@pytest.mark.parametrize("B,longest,H,dtype", [(4200, 40, 2, torch.float16), (20000, 5, 1, torch.float16), (4000, 300, 1, torch.bfloat16)])
def test_context_attention_thousands_of_short_sequences(B, longest, H, dtype):
    """More sequences than the planning kernel of the matrix-core path keeps in LDS (the call then takes the one-wave-per-row
    kernel), empty ones among them, and a batch just under that bound: every row against float64 on the device."""
    g = gen(917)
    lens = torch.randint(0, longest + 1, (B,), generator=g)
    T = int(lens.sum())
    q, k, v = (torch.randn(T, H, 128, generator=g).to(dtype).to(DEV) for _ in range(3))
    start = torch.cat((torch.zeros(1, dtype=torch.long), lens.cumsum(0)[:-1])).int().to(DEV)
    ln = lens.int().to(DEV)
    out = torch.full_like(q, 7.0)
    F.context_attention(q, k, v, out, start, ln, longest)
    steps = torch.arange(longest, device=DEV)
    valid = steps[None, :] < ln.long()[:, None]
    rows = torch.where(valid, start.long()[:, None] + steps[None, :], torch.zeros_like(valid, dtype=torch.long))
    causal = torch.tril(torch.ones(longest, longest, dtype=torch.bool, device=DEV))[None, None]
    for b0 in range(0, B, 1000):
        ii, live = rows[b0:b0 + 1000], valid[b0:b0 + 1000]
        sc = torch.einsum("bthd,bshd->bhts", q[ii].double(), k[ii].double()) / math.sqrt(128.0)
        sc = sc.masked_fill(~(causal & live[:, None, None, :]), float("-inf"))
        ref = torch.einsum("bhts,bshd->bthd", sc.softmax(-1).nan_to_num(0.0), v[ii].double())
        assert_close(out[ii][live], ref[live], what=f"{B} sequences of up to {longest} rows, {dtype}: sequences from {b0}", **TOL[dtype])


def test_context_attention_config4_scaled():
    w = W.cfg4(DEV, seed=4, scale=0.125)  # 8 sequences of 128..512 tokens
    _context_case(w["q"], w["k"], w["v"], w["b_start_loc"], w["b_seq_len"], w["max_input_len"], torch.float16, "cfg4 x 1/8")


@pytest.mark.timeout(900)
def test_context_attention_config4_half_scale_whole_sequences():
    """The prefill configuration at half its lengths (8 sequences of 512..2048 tokens) in one call; every row of every head of
    the two shortest sequences (636 and 1297 tokens) against the CPU restatement of the reference and against float64 (the CPU
    path needs about 100 seconds for a 2000-token sequence, which is what bounds the sample)."""
    w = W.cfg4(DEV, seed=4, scale=0.5)
    lens = w["seq_len_host"].tolist()
    say("cfg4 x 1/2 lengths", lens)
    q, k, v = w["q"], w["k"], w["v"]
    out = torch.full_like(q, 77.0)
    F.context_attention(q, k, v, out, w["b_start_loc"], w["b_seq_len"], w["max_input_len"])
    order = sorted(range(len(lens)), key=lambda i: lens[i])
    tol = TOL[torch.float16]
    for i in (order[0], order[1]):
        s0, L = int(w["b_start_loc"][i]), lens[i]
        qc, kc, vc = (t[s0:s0 + L].cpu() for t in (q, k, v))
        one = (torch.tensor([0]), torch.tensor([L]), L)
        ref = torch.zeros(L, q.shape[1], q.shape[2], dtype=torch.float16)
        O.context_attention(qc, kc, vc, ref, *one)
        say("  sequence", i, "length", L, ": reference composition done")
        ex = torch.zeros(L, q.shape[1], q.shape[2], dtype=torch.float64)
        O.context_attention(qc, kc, vc, ex, *one, exact=True)
        got = out[s0:s0 + L].cpu()
        assert_close(got, ref, what=f"cfg4 x 1/2 sequence {i} vs reference composition", **tol)
        assert_close(got, ex, what=f"cfg4 x 1/2 sequence {i} vs float64", **tol)
        say("  sequence", i, "max_abs/rel vs f64: %.3e %.3e" % report(got, ex))


def test_context_attention_config4_full_size_sampled():
    w = W.cfg4(DEV, seed=4)
    rows = []
    rng = np.random.Generator(np.random.PCG64(9))
    for i, L in enumerate(w["seq_len_host"].tolist()):
        rows += [(i, L - 1), (i, int(rng.integers(0, L))), (i, min(L - 1, 127)), (i, min(L - 1, 128))]
    out = _context_case(w["q"], w["k"], w["v"], w["b_start_loc"], w["b_seq_len"], w["max_input_len"], torch.float16, "cfg4 full", check_rows=rows)
    # constant V per head => the output equals V whatever the scores are
    vconst = w["v"][:1].expand_as(w["v"]).contiguous()
    o2 = torch.zeros_like(out)
    F.context_attention(w["q"], w["k"], vconst, o2, w["b_start_loc"], w["b_seq_len"], w["max_input_len"])
    assert_close(o2, vconst, rtol=1e-2, atol=1e-3, what="cfg4 full, constant V")


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_context_attention_config4_full_size_two_kernels_agree(dtype):
    """cfg4 at full size, every row of every head: the lightllm operator (the pipelined kernel) against
    diopiFlashAttentionVarLen on the same tokens (the kernel's general form: another loop, cumulative lengths, its own
    softmax-scale path).  Each is within 1e-2 of the exact result on the rows the oracle samples; here the whole tensors must
    agree to a few roundings of the element type, which a wrong tile, half or row anywhere in either kernel would break."""
    dt = TORCH_DTYPES[dtype]
    w = W.cfg4(DEV, seed=4)
    q, k, v = (w[x].to(dt) for x in ("q", "k", "v"))
    out = torch.full_like(q, 55.0)
    F.context_attention(q, k, v, out, w["b_start_loc"], w["b_seq_len"], w["max_input_len"])
    cu = torch.cat((w["b_start_loc"], (w["b_start_loc"][-1:] + w["b_seq_len"][-1:]))).int()
    flash = F.flash_attention_varlen(q, k, v, cu, cu, None, w["max_input_len"], w["max_input_len"], 0.0, None, True)
    assert not torch.isnan(out).any() and not torch.isnan(flash).any()
    tol = 2e-3 if dt is torch.float16 else 1.6e-2  # measured: 1.2e-4 in fp16, one bf16 step (7.8e-3) in bf16
    assert_close(out, flash, rtol=tol, atol=tol, what=f"cfg4 full size {dtype}: lightllm prefill vs flash varlen")
    say("cfg4 full size", dtype, "two kernels: max_abs/rel %.3e %.3e" % report(out.cpu(), flash.cpu()))


# ----------------------------------------------------------------------------- variable-length flash attention
# the reference's cases (diopi_configs.py:9854-9945): (q shape, key/value heads of the grouped case, cumulative lengths,
# max_seqlen, is_causal, softmax_scale)
FLASH_VARLEN_CASES = [
    ((32, 32, 128), 4, [0, 32], 32, True, None),
    ((64, 64, 128), 4, [0, 16, 48, 64], 32, True, 0.0883),
    ((256, 16, 128), 2, [0, 32, 64, 128, 256], 128, False, None),
    ((128, 8, 64), 2, [0, 16, 48, 64, 128], 64, True, 0.125),
    ((512, 8, 64), 2, [0, 2, 7, 19, 32, 64, 96, 128, 256, 512], 256, False, None),
    ((2784, 8, 64), 2, [0, 32, 96, 224, 2784], 2560, True, None),
]


def _flash_varlen_case(q, k, v, cu, max_seqlen, causal, scale, dt, what):
    before = snapshot(q, k, v, cu)
    out = F.flash_attention_varlen(q, k, v, cu, cu, None, max_seqlen, max_seqlen, 0, scale, causal, -1, -1)
    lse = F.GLOBAL_STATE["flash_attention_varlen_softmax_lse"]
    assert_unmodified(before, q, k, v, cu)
    # the C interface carries the scale as a float (functions_ext.h:355-359): the oracle gets the value that arrives
    scale = float(np.float32(scale if scale else 1.0 / math.sqrt(q.shape[-1])))
    exact, lse64 = O.flash_attention_varlen(q.cpu(), k.cpu(), v.cpu(), cu.cpu(), cu.cpu(), None, max_seqlen, max_seqlen, 0, scale, causal, exact=True,
                                            return_lse=True)
    assert_close(out, exact, **TOL[dt], what=f"{what}: out vs float64")
    if dt in (torch.float16, torch.bfloat16):
        faithful = O.flash_attention_varlen(q.cpu(), k.cpu(), v.cpu(), cu.cpu(), cu.cpu(), None, max_seqlen, max_seqlen, 0, scale, causal)
        # that composition rounds the scores and the probabilities to the 16-bit type, which moves single elements by
        # more than the tolerance; the reference's own checker allows 1e-3 of the elements to miss (check_result.py:138-149)
        assert_close(out, faithful, **TOL[dt], what=f"{what}: out vs the reference's composition", mismatch_ratio=1e-3)
    # the log-sum-exp is a float32 output computed from fp32 scores of 16-bit inputs
    assert_close(lse, lse64.float(), rtol=1e-4, atol=2e-3 if dt != torch.float32 else 1e-4, what=f"{what}: softmax_lse")
    return out


@pytest.mark.parametrize("case", range(len(FLASH_VARLEN_CASES)))
@pytest.mark.parametrize("grouped", [False, True])
def test_flash_attention_varlen_reference_cases(case, grouped):
    shape, hkv_grouped, cu, max_seqlen, causal, scale = FLASH_VARLEN_CASES[case]
    hkv = hkv_grouped if grouped else shape[1]
    g = gen(800 + case)
    for dt in (torch.float16, torch.bfloat16):
        q = torch.randn(*shape, generator=g).to(dt).to(DEV)
        k, v = (torch.randn(shape[0], hkv, shape[2], generator=g).to(dt).to(DEV) for _ in range(2))
        cu_t = torch.tensor(cu, dtype=torch.int32, device=DEV)
        _flash_varlen_case(q, k, v, cu_t, max_seqlen, causal, scale, dt, f"varlen case {case} grouped={grouped} {dt}")


def test_flash_attention_varlen_long_sequences_and_int64_lengths():
    # long enough for the 256-row query tiles, lengths that are no multiple of any tile size, full and causal attention
    cu = [0, 1531, 2630, 2631]
    g = gen(811)
    for causal in (True, False):
        q = (torch.randn(cu[-1], 8, 128, generator=g) * 0.5).half().to(DEV)
        k, v = ((torch.randn(cu[-1], 2, 128, generator=g) * 0.5).half().to(DEV) for _ in range(2))
        _flash_varlen_case(q, k, v, torch.tensor(cu, dtype=torch.int64, device=DEV), 1531, causal, None, torch.float16, f"long grouped causal={causal}")


def test_flash_attention_varlen_matches_context_attention_and_other_dtypes():
    w = W.cfg4(DEV, seed=4, scale=0.125)
    cu = torch.cat((w["b_start_loc"], (w["b_start_loc"][-1:] + w["b_seq_len"][-1:]))).to(torch.int32)
    ref = torch.zeros_like(w["q"])
    F.context_attention(w["q"], w["k"], w["v"], ref, w["b_start_loc"], w["b_seq_len"], w["max_input_len"])
    out = F.flash_attention_varlen(w["q"], w["k"], w["v"], cu, cu, None, w["max_input_len"], w["max_input_len"], 0, None, True)
    assert_close(out, ref, rtol=1e-3, atol=1e-3, what="causal multi-head varlen attention vs diopiContextAttentionInference")
    g = gen(812)
    for dt in (torch.float32, torch.float64):
        q = torch.randn(40, 4, 48, generator=g, dtype=dt).to(DEV)
        k, v = (torch.randn(40, 2, 48, generator=g, dtype=dt).to(DEV) for _ in range(2))
        _flash_varlen_case(q, k, v, torch.tensor([0, 7, 7, 40], dtype=torch.int32, device=DEV), 33, False, 0.2, dt, f"{dt} with an empty sequence")


def test_flash_attention_varlen_unsupported_modes_and_argument_errors():
    q = torch.randn(8, 2, 128, device=DEV).half()
    cu = torch.tensor([0, 8], dtype=torch.int32, device=DEV)
    for kwargs in (dict(p_dropout=0.1), dict(window_size_left=4), dict(alibi_slopes=torch.ones(2, device=DEV))):
        args = dict(alibi_slopes=None, p_dropout=0, window_size_left=-1)
        args.update(kwargs)
        with pytest.raises(rt.FunctionNotImplementedError):  # dropout, ALiBi and sliding windows answer with diopiNoImplement (13)
            F.flash_attention_varlen(q, q, q, cu, cu, args["alibi_slopes"], 8, 8, args["p_dropout"], None, True, args["window_size_left"], -1)
    with pytest.raises(rt.DiopiException):
        F.flash_attention_varlen(q, q[:, :1].contiguous().repeat(1, 3, 1), q, cu, cu, None, 8, 8, 0, None, True)  # 2 query heads over 3 key heads
    torch.cuda.synchronize()


# the reference's cases for the padded layout (diopi_configs.py:9770-9852): (q shape, key/value heads, is_causal, softmax_scale)
FLASH_CASES = [
    ((1, 64, 64, 128), 64, True, 0.0883), ((1, 256, 16, 128), 16, False, None), ((1, 64, 32, 128), 32, True, 0.125), ((1, 16, 8, 64), 8, True, 0.125),
    ((2, 64, 64, 128), 8, True, 0.0883), ((1, 256, 32, 128), 8, False, None), ((8, 32, 32, 128), 8, True, 0.125),
]


@pytest.mark.parametrize("case", range(len(FLASH_CASES)))
def test_flash_attention_reference_cases(case):
    shape, hkv, causal, scale = FLASH_CASES[case]
    g = gen(900 + case)
    for dt in (torch.float16, torch.bfloat16):
        q = torch.randn(*shape, generator=g).to(dt).to(DEV)
        k, v = (torch.randn(shape[0], shape[1], hkv, shape[3], generator=g).to(dt).to(DEV) for _ in range(2))
        before = snapshot(q, k, v)
        out = F.flash_attention(q, k, v, None, 0, scale, causal, -1, -1)
        lse = F.GLOBAL_STATE["flash_attention_softmax_lse"]
        assert_unmodified(before, q, k, v)
        sc = float(np.float32(scale if scale else 1.0 / math.sqrt(shape[3])))
        exact, lse64 = O.flash_attention(q.cpu(), k.cpu(), v.cpu(), None, 0, sc, causal, exact=True, return_lse=True)
        assert_close(out, exact, **TOL[dt], what=f"padded case {case} {dt}: out vs float64")
        faithful = O.flash_attention(q.cpu(), k.cpu(), v.cpu(), None, 0, sc, causal)
        assert_close(out, faithful, **TOL[dt], what=f"padded case {case} {dt}: out vs the reference's composition", mismatch_ratio=1e-3)
        assert_close(lse, lse64.float(), rtol=1e-4, atol=2e-3, what=f"padded case {case} {dt}: softmax_lse")
    with pytest.raises(rt.FunctionNotImplementedError):
        F.flash_attention(q, k, v, None, 0.5, scale, causal, -1, -1)


def test_multihead_attention_older_names():
    # the reference's cases for the deprecated names (diopi_configs.py, multihead_attention / multihead_attention_varlen):
    # the same statement (multi_head_attention_inside) as the flash-attention operators, so the same oracle serves
    g = gen(950)
    q, k, v = (torch.randn(2, 128, 8, 128, generator=g).half().to(DEV) for _ in range(3))
    for causal, scale in ((True, None), (False, 0.1)):
        out = F.multihead_attention(q, k, v, 0, causal, False, scale)
        lse = F.GLOBAL_STATE["multihead_attention_softmax_lse"]
        exact, lse64 = O.flash_attention(q.cpu(), k.cpu(), v.cpu(), None, 0, scale, causal, exact=True, return_lse=True)
        assert_close(out, exact, **TOL[torch.float16], what="multihead_attention")
        assert_close(lse, lse64.float(), rtol=1e-4, atol=2e-3, what="multihead_attention softmax_lse")
    cu = torch.tensor([0, 37, 37, 200, 256], dtype=torch.int64, device=DEV)
    qp, kp, vp = (t.reshape(256, 8, 128) for t in (q, k, v))
    out = F.multihead_attention_varlen(qp, kp, vp, cu, 163, 0, True, False, None)
    lse = F.GLOBAL_STATE["multihead_attention_varlen_softmax_lse"]
    exact, lse64 = O.flash_attention_varlen(qp.cpu(), kp.cpu(), vp.cpu(), cu.cpu(), cu.cpu(), None, 163, 163, 0, None, True, exact=True, return_lse=True)
    assert_close(out, exact, **TOL[torch.float16], what="multihead_attention_varlen")
    assert_close(lse, lse64.float(), rtol=1e-4, atol=2e-3, what="multihead_attention_varlen softmax_lse")
    with pytest.raises(rt.FunctionNotImplementedError):
        F.multihead_attention(q, k, v, 0.1, True, False, None)
    with pytest.raises(rt.FunctionNotImplementedError):
        F.multihead_attention_varlen(qp, kp, vp, cu, 163, 0, True, True, None)


# ----------------------------------------------------------------------------- prompt flash attention and paged attention
def test_prompt_flash_attention_reference_case_and_long_prompts():
    # the reference's case (diopi_configs.py:9383-9423): 2 sequences of 2 rows, 32 heads of 128, fp16, its boolean mask
    g = gen(960)
    q, k, v = ((torch.randn(4, 4096, generator=g) * 0.5).half().to(DEV) for _ in range(3))
    mask = torch.tensor([[[False, True], [False, False]]] * 2, device=DEV)
    out = F.prompt_flash_attention(q, k, v, mask, [2, 2], 2, 32, 32, 128)
    assert out.shape == (4, 4096)
    ref = O.prompt_flash_attention(q.cpu(), k.cpu(), v.cpu(), mask.cpu(), [2, 2], 2, 32, 32, 128)
    assert_close(out, ref, **TOL[torch.float16], what="prompt_flash_attention, reference case", mismatch_ratio=1e-3)
    assert torch.equal(out[0].cpu(), v[0].cpu()) and torch.equal(out[2].cpu(), v[2].cpu())  # a first row is its own value row
    # prompts long enough for the matrix-core kernel, fewer key/value heads, bf16 and fp32
    for dtype, bs, L, H, Hkv, D in ((torch.float16, 3, 300, 8, 2, 128), (torch.bfloat16, 2, 257, 4, 4, 128), (torch.float32, 2, 40, 4, 2, 64)):
        q = (torch.randn(bs * L, H * D, generator=g) * 0.5).to(dtype).to(DEV)
        k = (torch.randn(bs * L, Hkv * D, generator=g) * 0.5).to(dtype).to(DEV)
        v = (torch.randn(bs * L, Hkv * D, generator=g) * 0.5).to(dtype).to(DEV)
        out = F.prompt_flash_attention(q, k, v, None, [L, L - 1, 1][:bs], L, H, Hkv, D)
        exact = O.prompt_flash_attention(q.cpu(), k.cpu(), v.cpu(), None, [L] * bs, L, H, Hkv, D, exact=True)
        assert_close(out, exact, **TOL[dtype], what=f"prompt_flash_attention {dtype}")
    with pytest.raises(rt.DiopiException):
        F.prompt_flash_attention(q, k, v, None, [40, 40, 40], 40, 4, 2, 64)  # rows do not match batch * max_input_len
    with pytest.raises(rt.DiopiException):
        F.prompt_flash_attention(q, k, v, None, [40, 40], 40, 4, 3, 64)  # heads not a multiple of key/value heads
    assert F.prompt_flash_attention(q[:0], k[:0], v[:0], None, [], 40, 4, 2, 64).numel() == 0


def test_paged_attention_reference_case_and_block_tables():
    # the reference's case (diopi_configs.py:9425-9468): one sequence of 5 tokens, blocks [0, 1] of 128 rows, 1026 cache rows
    g = gen(970)
    H, D = 32, 128
    q = (torch.randn(1, H * D, generator=g) * 0.5).half().to(DEV)
    k = (torch.randn(1026, H * D, generator=g) * 0.5).half().to(DEV)
    v = (torch.randn(1026, H * D, generator=g) * 0.5).half().to(DEV)
    table = torch.tensor([[0, 1]], dtype=torch.int32, device=DEV)
    mask = torch.zeros(1, 1, 5, dtype=torch.bool, device=DEV)
    out = F.paged_attention(q, k, v, mask, [5], H, H, D, table, 128)
    ref = O.paged_attention(q.cpu(), k.cpu(), v.cpu(), mask.cpu(), [5], H, H, D, table.cpu(), 128)
    assert_close(out, ref, **TOL[torch.float16], what="paged_attention, reference case", mismatch_ratio=1e-3)

    # a decode batch over a shuffled block pool: ragged lengths (one empty), grouped heads, int64 table, more sequences
    # than one launch of the table kernel carries
    for dtype, B, Hq, Hkv, bsz, maxlen in ((torch.float16, 70, 8, 2, 16, 700), (torch.bfloat16, 5, 4, 4, 128, 1500), (torch.float32, 3, 4, 2, 8, 50)):
        D = 128 if dtype != torch.float32 else 64
        nblk = (maxlen + bsz - 1) // bsz
        lens = torch.randint(1, maxlen + 1, (B,), generator=g).tolist()
        lens[1] = 0
        lens[0] = maxlen
        pool = B * nblk + 3
        perm = torch.randperm(pool, generator=g)[:B * nblk].view(B, nblk)
        table = perm.to(torch.int64 if dtype == torch.float16 else torch.int32).to(DEV)
        q = (torch.randn(B, Hq * D, generator=g) * 0.5).to(dtype).to(DEV)
        k = (torch.randn(pool * bsz, Hkv * D, generator=g) * 0.5).to(dtype).to(DEV)
        v = (torch.randn(pool * bsz, Hkv * D, generator=g) * 0.5).to(dtype).to(DEV)
        out = F.paged_attention(q, k, v, None, lens, Hq, Hkv, D, table, bsz)
        exact = O.paged_attention(q.cpu(), k.cpu(), v.cpu(), None, lens, Hq, Hkv, D, table.cpu(), bsz, exact=True)
        keep = [i for i in range(B) if lens[i] > 0]
        assert_close(out[keep], exact[keep], **TOL[dtype], what=f"paged_attention {dtype}")
    with pytest.raises(rt.DiopiException):
        F.paged_attention(q, k, v, None, [9, 9, 9], Hq, Hkv, D, table[:, :1], bsz)  # 9 tokens do not fit one block of 8
    with pytest.raises(rt.DiopiException):
        F.paged_attention(q, k, v, None, [9, 9], Hq, Hkv, D, table, bsz)  # batch mismatch
    zero = F.paged_attention(q, k, v, None, [0, 0, 0], Hq, Hkv, D, table, bsz)
    assert float(zero.abs().max()) == 0.0


def test_prompt_flash_attention_full_size_matches_context_attention():
    # 8 prompts of 2048 rows, 32 heads of 128 (the prefill benchmark's head geometry): the padded-batch operator and
    # the lightllm operator on the same rows cut into equal sequences are two entries over one kernel
    g = gen(975)
    bs, L, H, D = 8, 2048, 32, 128
    q, k, v = ((torch.randn(bs * L, H * D, generator=g) * 0.5).half().to(DEV) for _ in range(3))
    out = F.prompt_flash_attention(q, k, v, None, [L] * bs, L, H, H, D)
    want = torch.zeros(bs * L, H, D, dtype=torch.float16, device=DEV)
    start = torch.arange(0, bs * L, L, dtype=torch.int32, device=DEV)
    F.context_attention(q.view(-1, H, D), k.view(-1, H, D), v.view(-1, H, D), want, start, torch.full((bs,), L, dtype=torch.int32, device=DEV), L)
    assert_close(out.view(-1, H, D), want, rtol=2e-3, atol=2e-4, what="prompt_flash_attention vs context_attention at full size")
    # size-independent properties: the first row of a sequence is its value row; rows of sampled (sequence, head) pairs against float64
    assert torch.equal(out[3 * L].cpu(), v[3 * L].cpu())
    for b, h in ((0, 0), (5, 17)):
        rows = slice(b * L, b * L + 300)
        cols = slice(h * D, (h + 1) * D)
        exact = O.prompt_flash_attention(q[rows, cols].cpu(), k[rows, cols].cpu(), v[rows, cols].cpu(), None, [300], 300, 1, 1, D, exact=True)
        assert_close(out[rows, cols], exact, **TOL[torch.float16], what="prompt_flash_attention, sampled rows vs float64")


def test_paged_attention_full_size_equals_the_two_decode_operators():
    # benchmark size (64 sequences of 512..2048 tokens, 32 heads of 128, 1024 blocks of 128 rows): the block table expanded
    # on the host into the row table of the lightllm operators must give the same bits, since the same kernels run
    g = gen(980)
    B, H, D, bsz, nblk = 64, 32, 128, 128, 16
    lens = torch.randint(512, 2049, (B,), generator=g)
    table = torch.randperm(B * nblk, generator=g).view(B, nblk).int()
    q = (torch.randn(B, H * D, generator=g) * 0.5).half().to(DEV)
    k = (torch.randn(B * nblk * bsz, H * D, generator=g) * 0.5).half().to(DEV)
    v = (torch.randn(B * nblk * bsz, H * D, generator=g) * 0.5).half().to(DEV)
    out = F.paged_attention(q, k, v, None, lens.tolist(), H, H, D, table.to(DEV), bsz)
    maxlen = int(lens.max())
    b_loc = torch.zeros(B, maxlen, dtype=torch.int32)
    for i in range(B):
        L = int(lens[i])
        b_loc[i, maxlen - L:] = O.paged_rows(table, i, L, bsz).int()
    start = (torch.cumsum(lens, 0) - lens).int()
    logits = torch.zeros(H, int(lens.sum()), dtype=torch.float16, device=DEV)
    F.token_attention(q.view(B, H, D), k.view(-1, H, D), logits, b_loc.to(DEV), start.to(DEV), lens.int().to(DEV), maxlen)
    want = torch.zeros(B, H, D, dtype=torch.float16, device=DEV)
    F.token_softmax_reducev(logits, v.view(-1, H, D), want, b_loc.to(DEV), start.to(DEV), lens.int().to(DEV), maxlen, 0)
    assert_bit_equal(out.view(B, H, D), want, "paged attention vs token attention + softmax-reduce-v on the expanded table")
    # and a sampled sequence against the float64 oracle
    i = 7
    exact = O.paged_attention(q[i:i + 1].cpu(), k.cpu(), v.cpu(), None, [int(lens[i])], H, H, D, table[i:i + 1], bsz, exact=True)
    assert_close(out[i:i + 1], exact, **TOL[torch.float16], what="paged attention, sampled sequence vs float64")


# ----------------------------------------------------------------------------- base pointers that are not 16-byte aligned
def _off(t: torch.Tensor) -> torch.Tensor:
    """The same values in a dense device tensor whose first element sits one element past an aligned allocation."""
    flat = torch.empty(t.numel() + 1, dtype=t.dtype, device=DEV)
    view = flat[1:].view(t.shape)
    view.copy_(t)
    assert view.is_contiguous() and view.data_ptr() % 16 != 0
    return view


def test_unaligned_base_pointers_take_the_slow_paths_and_stay_correct():
    # a framework may hand over dense views that start in the middle of an allocation: every operator must either
    # use narrower accesses or its general kernel, never a wrong fast path
    g = gen(990)
    dt = torch.float16
    tol = TOL[dt]
    # RMSNorm forward and backward
    x, wgt, go = (torch.randn(64, 512, generator=g) * 0.5).to(dt), torch.randn(512, generator=g).to(dt), (torch.randn(64, 512, generator=g) * 0.5).to(dt)
    xd, wd, god = _off(x), _off(wgt), _off(go)
    out = F.rms_norm(xd, (512,), wd, None, 1e-6)
    inv = F.GLOBAL_STATE["rms_norm_inv_rms"]
    r_out, r_inv = O.rms_norm(x, (512,), wgt, None, 1e-6, exact=True)
    assert_close(out, r_out, what="rms_norm, unaligned", **tol)
    grads = F.rms_norm_backward([god], xd, wd, None, (512,), 1e-6, inv_rms=inv)
    r_gi, r_gw, _ = O.rms_norm_backward(go, x, wgt, inv.cpu(), (512,), exact=True)
    assert_close(grads["input"], r_gi, what="rms_norm_backward grad_input, unaligned", **tol)
    assert_close(grads["weight"], r_gw, rtol=2e-2, atol=2e-2, what="rms_norm_backward grad_weight, unaligned")
    # rotary, both forms
    T, H, D = 33, 4, 128
    q, k = (torch.randn(T, H, D, generator=g) * 0.5).to(dt), (torch.randn(T, H, D, generator=g) * 0.5).to(dt)
    ang = torch.rand(T, 1, D // 2, generator=g) * 6.28
    cos, sin = ang.cos().to(dt), ang.sin().to(dt)
    rot = F.rotary_emb(_off(q), _off(cos), _off(sin), False, False)
    assert_close(rot, O.rotary_emb(q, cos, sin, False, exact=True), what="rotary_emb, unaligned", **tol)
    cos2, sin2 = torch.cat((cos, cos), -1).reshape(T, D), torch.cat((sin, sin), -1).reshape(T, D)
    q2, k2 = _off(q.reshape(T, H * D)), _off(k.reshape(T, H * D))
    rq, rk = O.rotary_emb_v2(q.reshape(T, H * D).clone(), k.reshape(T, H * D).clone(), cos2, sin2, D, exact=True)
    F.rotary_emb_v2(q2, k2, _off(cos2), _off(sin2), D)
    assert_close(q2, rq, what="rotary_emb_v2 query, unaligned", **tol)
    assert_close(k2, rk, what="rotary_emb_v2 key, unaligned", **tol)
    # scatter into the cache
    cache = (torch.randn(96, H, D, generator=g)).to(dt)
    dest = torch.randperm(96, generator=g)[:T].int()
    cd = _off(cache)
    F.destindex_copy_kv(_off(q), dest.to(DEV), cd)
    assert_bit_equal(cd, O.destindex_copy_kv(q, dest, cache.clone()), "destindex_copy_kv, unaligned")
    # decode
    B, L = 3, 40
    lens = torch.tensor([40, 17, 1], dtype=torch.int32)
    b_loc = torch.stack([torch.randperm(96, generator=g)[:L] for _ in range(B)]).int()
    start = (torch.cumsum(lens, 0) - lens).int()
    qd = (torch.randn(B, H, D, generator=g) * 0.5).to(dt)
    vc = (torch.randn(96, H, D, generator=g) * 0.5).to(dt)
    logits = _off(torch.zeros(H, int(lens.sum()), dtype=dt))
    F.token_attention(_off(qd), cd, logits, b_loc.to(DEV), start.to(DEV), lens.to(DEV), L)
    ref_logits = torch.zeros(H, int(lens.sum()), dtype=torch.float64)
    O.token_attention(qd, cd.cpu(), ref_logits, b_loc, start, lens, L, exact=True)
    assert_close(logits, ref_logits, what="token_attention, unaligned", **tol)
    dec = _off(torch.zeros(B, H, D, dtype=dt))
    F.token_softmax_reducev(logits, _off(vc), dec, b_loc.to(DEV), start.to(DEV), lens.to(DEV), L, 0)
    ref_dec = torch.zeros(B, H, D, dtype=torch.float64)
    O.token_softmax_reducev(logits.cpu(), vc, ref_dec, b_loc, start, lens, L, 0, exact=True)
    assert_close(dec, ref_dec, what="token_softmax_reducev, unaligned", **tol)
    # prefill, both interfaces
    Ls = torch.tensor([150, 70], dtype=torch.int32)
    st = torch.tensor([0, 150], dtype=torch.int32)
    pq, pk, pv = ((torch.randn(220, H, D, generator=g) * 0.5).to(dt) for _ in range(3))
    po = _off(torch.zeros(220, H, D, dtype=dt))
    F.context_attention(_off(pq), _off(pk), _off(pv), po, st.to(DEV), Ls.to(DEV), 150)
    ref = torch.zeros(220, H, D, dtype=torch.float64)
    O.context_attention(pq, pk, pv, ref, st, Ls, 150, exact=True)
    assert_close(po, ref, what="context_attention, unaligned", **tol)
    cu = torch.tensor([0, 150, 220], dtype=torch.int32)
    fa = F.flash_attention_varlen(_off(pq), _off(pk), _off(pv), cu.to(DEV), cu.to(DEV), None, 150, 150, 0, None, True)
    assert_close(fa, ref, what="flash_attention_varlen, unaligned", **tol)


# ----------------------------------------------------------------------------- two host threads, two contexts, two streams
def test_two_threads_with_their_own_contexts_and_streams():
    # the operators that take scratch from their context (RMSNormBackward partial rows, decode partials, the prefill tile
    # plan) called from two host threads at once, each on its own stream: results must equal the single-threaded ones
    import threading

    def workload(seed):
        g = gen(seed)
        x = (torch.randn(512, 1024, generator=g) * 0.5).to(DEV)
        w = torch.randn(1024, generator=g).to(DEV)
        go = (torch.randn(512, 1024, generator=g) * 0.5).to(DEV)
        wd = W.cfg3(DEV, seed=seed, scale=1 / 8)
        wp = W.cfg4(DEV, seed=seed, scale=1 / 4)
        return dict(x=x, w=w, go=go, wd=wd, wp=wp)

    state_lock = threading.Lock()  # the wrapper keeps inv_rms in a process-wide dict, like the reference's Python layer

    def run(data, ctx):
        with state_lock:
            out = F.rms_norm(data["x"], (1024,), data["w"], None, 1e-6, ctx=ctx)
            inv = F.GLOBAL_STATE["rms_norm_inv_rms"]
        grads = F.rms_norm_backward([data["go"]], data["x"], data["w"], None, (1024,), 1e-6, ctx=ctx, inv_rms=inv)
        wd = data["wd"]
        logits = torch.zeros(wd["H"], wd["total_len"], dtype=torch.float16, device=DEV)
        F.token_attention(wd["q"], wd["k_cache"], logits, wd["b_loc"], wd["b_start_loc"], wd["b_seq_len"], wd["max_input_len"], ctx=ctx)
        dec = torch.zeros_like(wd["q"])
        F.token_softmax_reducev(logits, wd["v_cache"], dec, wd["b_loc"], wd["b_start_loc"], wd["b_seq_len"], wd["max_input_len"], 0, ctx=ctx)
        wp = data["wp"]
        pre = torch.zeros_like(wp["q"])
        F.context_attention(wp["q"], wp["k"], wp["v"], pre, wp["b_start_loc"], wp["b_seq_len"], wp["max_input_len"], ctx=ctx)
        return [out, grads["input"], grads["weight"], logits, dec, pre]

    datas = [workload(1001), workload(1002)]
    single = []
    for d in datas:
        ctx = rt.Context(own_stream=False)
        single.append([t.clone() for t in run(d, ctx)])
        torch.cuda.synchronize()
    results = [None, None]
    errors = []

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            ctx = rt.Context(stream=stream)
            with torch.cuda.stream(stream):
                for _ in range(10):
                    results[i] = run(datas[i], ctx)
            stream.synchronize()
        except Exception as e:  # surfaced in the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    torch.cuda.synchronize()
    names = ["rms_norm", "grad_input", "grad_weight", "logits", "decode out", "prefill out"]
    for i in range(2):
        for name, got, want in zip(names, results[i], single[i]):
            if name == "grad_weight":  # partial rows are folded in an order that depends on nothing but the launch shape
                assert_close(got, want, rtol=1e-6, atol=1e-6, what=f"thread {i}: {name}")
            else:
                assert_bit_equal(got, want, f"thread {i}: {name}")


# ----------------------------------------------------------------------------- a decode step recorded in a HIP graph
def test_decode_step_in_a_hip_graph_replays_like_eager():
    # serving loops record the decode step once and replay it: scatter of the new K/V rows, score rows, softmax and
    # product with V.  Every launch goes to the context's stream and the scratch comes from the context's pool, so the
    # step must be capturable after one eager run, and every replay must give what the eager call gives on the same inputs.
    w = W.cfg3(DEV, seed=77, scale=1 / 8)
    H, total, mil = w["H"], w["total_len"], w["max_input_len"]
    stream = torch.cuda.Stream()
    ctx = rt.Context(stream=stream)
    logits = torch.zeros(H, total, dtype=torch.float16, device=DEV)
    out = torch.zeros_like(w["q"])

    def step():
        F.destindex_copy_kv(w["new_k"], w["dest_loc"], w["k_cache"], ctx=ctx)
        F.destindex_copy_kv(w["new_v"], w["dest_loc"], w["v_cache"], ctx=ctx)
        F.token_attention(w["q"], w["k_cache"], logits, w["b_loc"], w["b_start_loc"], w["b_seq_len"], mil, ctx=ctx)
        F.token_softmax_reducev(logits, w["v_cache"], out, w["b_loc"], w["b_start_loc"], w["b_seq_len"], mil, 0, ctx=ctx)

    with torch.cuda.stream(stream):
        step()  # eager once: one-time initialisation and the scratch pool's first allocation happen here
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        step()
    g = gen(78)
    for replay in range(3):
        # new inputs in place (the graph holds the addresses), eager work and a synchronisation between the replays
        w["q"].copy_((torch.randn(w["q"].shape, generator=g) * 0.25).half())
        w["new_k"].copy_((torch.randn(w["new_k"].shape, generator=g) * 0.25).half())
        w["new_v"].copy_((torch.randn(w["new_v"].shape, generator=g) * 0.25).half())
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got_logits, got_out = logits.clone(), out.clone()
        logits.zero_()
        out.zero_()
        with torch.cuda.stream(stream):
            step()
        stream.synchronize()
        assert_bit_equal(got_logits, logits, f"replay {replay}: score rows")
        assert_bit_equal(got_out, out, f"replay {replay}: decode output")
        ref = torch.zeros(w["q"].shape, dtype=torch.float64)
        O.token_softmax_reducev(logits.cpu(), w["v_cache"].cpu(), ref, w["b_loc"].cpu(), w["b_start_loc"].cpu(), w["b_seq_len"].cpu(), mil, 0, exact=True)
        assert_close(got_out, ref, what=f"replay {replay}: decode output vs float64", **TOL[torch.float16])


# ----------------------------------------------------------------------------- tensors past 2^31 elements
def test_tensors_with_more_than_two_to_the_31_elements():
    """64-bit addressing: every large tensor here holds 2^31 + 20480 elements (4 GiB of bf16).  Results are compared
    with the oracle on the first, middle and last rows and a random sample, which is where a 32-bit offset would wrap.
    Covers both normalisations and the backward pass, rotary, the cache scatter, the two decode operators and the prefill operator."""
    dt = torch.bfloat16
    rows, H, D = 2 ** 19 + 5, 32, 128
    n2 = H * D
    assert rows * n2 > 2 ** 31
    g = gen(900)
    x = torch.empty(rows, n2, dtype=dt, device=DEV).normal_()
    res = torch.empty(rows, n2, dtype=dt, device=DEV).normal_()
    out = torch.empty(rows, n2, dtype=dt, device=DEV)
    wt = (torch.rand(n2, generator=g) + 0.5).to(dt).to(DEV)
    pick = torch.cat((torch.tensor([0, 1, rows // 2, rows - 2, rows - 1]), torch.randint(0, rows, (27,), generator=g))).to(DEV)
    xs, rs = x[pick].cpu(), res[pick].cpu()

    say("past 2^31: rms_norm")
    o = F.rms_norm(x, (n2,), wt, None, 1e-6)
    want, want_inv = O.rms_norm(xs, (n2,), wt.cpu(), None, 1e-6)
    assert_close(o[pick], want, what="rms_norm past 2^31", **TOL[dt])
    inv_big = F.GLOBAL_STATE["rms_norm_inv_rms"]
    assert_close(inv_big[pick], want_inv, rtol=1e-5, atol=0, what="inv_rms past 2^31")
    del o

    say("past 2^31: rms_norm_backward")
    grads = F.rms_norm_backward([res.view(rows, n2)], x, wt, None, (n2,), 1e-6, inv_rms=inv_big)
    w_gi, _, _ = O.rms_norm_backward(rs, xs, wt.cpu(), inv_big[pick].cpu(), (n2,))
    assert_close(grads["input"][pick], w_gi, what="grad_input past 2^31", **TOL[dt])
    # grad_weight sums half a million rows: second opinion from float64 column sums formed on the device in slabs
    col = torch.zeros(n2, dtype=torch.float64, device=DEV)
    for lo in range(0, rows, 65536):
        hi = min(rows, lo + 65536)
        col += (res[lo:hi].double() * x[lo:hi].double() * inv_big[lo:hi].double()[:, None]).sum(0)
    assert_close(grads["weight"], col.cpu(), rtol=1e-2, atol=1e-2 * math.sqrt(rows), what="grad_weight past 2^31")
    del grads, col

    say("past 2^31: rotary")
    cos = torch.randn(rows, 1, D // 2, generator=g).to(dt).to(DEV)
    sin = torch.randn(rows, 1, D // 2, generator=g).to(dt).to(DEV)
    ro = F.rotary_emb(x.view(rows, H, D), cos, sin, False, False)
    assert_close(ro[pick], O.rotary_emb(xs.view(-1, H, D), cos[pick].cpu(), sin[pick].cpu(), False), what="rotary past 2^31", **TOL[dt])
    del ro

    say("past 2^31: fused residual addition + normalisation, in place")
    out.copy_(x)
    F.fused_add_root_mean_square_norm_inp(out, res, None, wt, 1e-6)
    w_out, w_res = O.fused_add_root_mean_square_norm_inp(xs, rs, None, wt.cpu(), 1e-6)
    assert_bit_equal(res[pick], w_res, "fused norm past 2^31: residual")
    assert_close(out[pick], w_out, what="fused norm past 2^31", **TOL[dt])

    say("past 2^31: destindex_copy_kv")
    cache = out.view(rows, H, D)
    dest = torch.tensor([rows - 1, 0, rows - 3, rows // 2 + 1, 7, rows - 2], dtype=torch.int64, device=DEV)
    newk = torch.randn(6, H, D, generator=g).to(dt).to(DEV)
    others = pick[~torch.isin(pick, dest)]
    untouched = cache[others].clone()
    F.destindex_copy_kv(newk, dest, cache)
    assert_bit_equal(cache[dest], newk, "destindex past 2^31: scattered rows")
    assert_bit_equal(cache[others], untouched, "destindex past 2^31: other rows")

    say("past 2^31: decode over slots at the top of the cache")
    kc, vc = x.view(rows, H, D), res.view(rows, H, D)
    lens = [300, 77]
    maxlen = 320
    b_loc = torch.zeros(2, maxlen, dtype=torch.int32)
    top = torch.randperm(4096, generator=g)[: sum(lens)]
    used = rows - 1 - top  # distinct slots among the last 4096 rows
    b_loc[0, maxlen - lens[0]:] = used[: lens[0]].int()
    b_loc[1, maxlen - lens[1]:] = used[lens[0]:].int()
    b_seq = torch.tensor(lens, dtype=torch.int32)
    b_start = torch.tensor([0, lens[0]], dtype=torch.int32)
    q = torch.randn(2, H, D, generator=g).to(dt)
    logits = torch.zeros(H, sum(lens), dtype=dt, device=DEV)
    F.token_attention(q.to(DEV), kc, logits, b_loc.to(DEV), b_start.to(DEV), b_seq.to(DEV), maxlen)
    o2 = torch.zeros(2, H, D, dtype=dt, device=DEV)
    F.token_softmax_reducev(logits, vc, o2, b_loc.to(DEV), b_start.to(DEV), b_seq.to(DEV), maxlen, 0)
    # the oracle sees a compact cache that holds only the used rows, through a row table renumbered to match
    order = used.sort().values
    small_k, small_v = kc[order.to(DEV)].cpu(), vc[order.to(DEV)].cpu()
    remap = torch.zeros_like(b_loc)
    live = torch.zeros_like(b_loc, dtype=torch.bool)
    live[0, maxlen - lens[0]:] = True
    live[1, maxlen - lens[1]:] = True
    remap[live] = torch.searchsorted(order, b_loc[live].long()).int()
    want_logits = O.token_attention(q, small_k, torch.zeros(H, sum(lens), dtype=dt), remap, b_start, b_seq, maxlen)
    assert_close(logits, want_logits, what="token_attention past 2^31", **TOL[dt])
    want_o = O.token_softmax_reducev(logits.cpu(), small_v, torch.zeros(2, H, D, dtype=dt), remap, b_start, b_seq, maxlen, 0)
    assert_close(o2, want_o, what="token_softmax_reducev past 2^31", **TOL[dt])

    say("past 2^31: prefill over sequences at both ends and in the middle of the token axis")
    starts, plens = [0, rows // 2, rows - 300], [200, 257, 300]
    qv, kv, vv = x.view(rows, H, D), res.view(rows, H, D), out.view(rows, H, D)
    ctx_out = torch.full((rows, H, D), 7.0, dtype=dt, device=DEV)
    F.context_attention(qv, kv, vv, ctx_out, torch.tensor(starts, dtype=torch.int32, device=DEV), torch.tensor(plens, dtype=torch.int32, device=DEV),
                        max(plens))
    for st, ln in zip(starts, plens):
        sl = slice(st, st + ln)
        # against the float64 evaluation: the kernel keeps its scores in fp32, and with unit-variance bf16 inputs the
        # reference's rounding of the scores to bf16 alone moves single outputs by more than the bar
        want_c = O.context_attention(qv[sl].cpu(), kv[sl].cpu(), vv[sl].cpu(), torch.zeros(ln, H, D, dtype=torch.float64), torch.tensor([0]),
                                     torch.tensor([ln]), exact=True)
        assert_close(ctx_out[sl], want_c, what=f"context_attention past 2^31, rows {st}..{st + ln}", **TOL[dt])
    outside = torch.tensor([200, 201, rows // 2 - 1, rows // 2 + 257, rows - 301, 12345], device=DEV)
    assert bool((ctx_out[outside] == 7.0).all()), "rows outside every sequence were written"


# ----------------------------------------------------------------------------- the reference harness's device hooks
def test_harness_hooks_drive_an_operator_without_torch_on_the_device():
    """The way diopi_test reaches the device (conform_test.h:28-43; litert.cpp:370-376): memory from device_malloc,
    copies and synchronisation on a stream from device_make_stream, the operator enqueued on that stream."""
    import ctypes as C
    rtl, impl = rt.libs().rt, rt.libs().impl
    vp = C.c_void_p

    assert rtl.initLibrary() == 0
    stream = vp()
    assert rtl.device_make_stream(C.byref(stream)) == 0 and stream.value

    # byte round trip host -> device -> device -> host, odd size
    rng = np.random.default_rng(5)
    src = rng.integers(0, 256, size=1_000_003, dtype=np.uint8)
    back = np.zeros_like(src)
    a, b = rtl.device_malloc(src.nbytes), rtl.device_malloc(src.nbytes)
    assert a and b
    assert rtl.device_memcpy_h2d_async(stream, a, src.ctypes.data, src.nbytes) == 0
    assert rtl.device_memcpy_d2d_async(stream, b, a, src.nbytes) == 0
    assert rtl.device_memcpy_d2h_async(stream, back.ctypes.data, b, src.nbytes) == 0
    assert rtl.device_synchronize_stream(stream) == 0
    assert np.array_equal(src, back)
    assert rtl.device_memcpy_d2d_async(stream, b, a, 0) == 0  # empty copies are legal
    rtl.device_free(a)
    rtl.device_free(b)

    # RMSNorm at the reference's case shape (diopi_configs.py:9153), every buffer owned by the hooks
    n1, n2, eps = 12, 32, 1e-6
    x = rng.standard_normal((n1, n2)).astype(np.float32)
    w = rng.uniform(0.5, 1.5, n2).astype(np.float32)
    out, inv = np.zeros_like(x), np.zeros(n1, np.float32)
    dx, dw, dout, dinv = (rtl.device_malloc(t.nbytes) for t in (x, w, out, inv))
    assert rtl.device_memcpy_h2d_async(stream, dx, x.ctypes.data, x.nbytes) == 0
    assert rtl.device_memcpy_h2d_async(stream, dw, w.ctypes.data, w.nbytes) == 0
    ctx = rtl.diopirtContextCreate(stream)

    def wrap(ptr, *shape):
        dims = (C.c_int64 * len(shape))(*shape)
        return rtl.diopirtTensorWrap(ptr, dims, None, len(shape), int(rt.Dtype.float32), int(rt.Device.AIChip))

    tx, tw, tout, tinv = wrap(dx, n1, n2), wrap(dw, n2), wrap(dout, n1, n2), wrap(dinv, n1)
    ret = impl.diopiRMSNorm(ctx, tout, tinv, tx, rt.Sizes([n2]).c, tw, None, eps)
    assert ret == 0, rt.get_last_error_string()
    assert rtl.device_memcpy_d2h_async(stream, out.ctypes.data, dout, out.nbytes) == 0
    assert rtl.device_memcpy_d2h_async(stream, inv.ctypes.data, dinv, inv.nbytes) == 0
    assert rtl.device_synchronize_stream(stream) == 0
    want_out, want_inv = O.rms_norm(torch.from_numpy(x), (n2,), torch.from_numpy(w), None, eps)
    assert_close(torch.from_numpy(out), want_out, what="RMSNorm through the harness hooks", **TOL[torch.float32])
    assert_close(torch.from_numpy(inv), want_inv, what="inv_rms through the harness hooks", **TOL[torch.float32])

    # the generator-state hook hands out 808 host bytes owned by the context
    state = rtl.diopirtTensorWrap(None, (C.c_int64 * 1)(0), None, 1, int(rt.Dtype.uint8), int(rt.Device.Host))
    assert rtl.buildGeneratorState(ctx, state) == 0
    numel, dtype, where = C.c_int64(), C.c_int(), C.c_int()
    assert rtl.diopiGetTensorNumel(state, C.byref(numel)) == 0 and numel.value == 808
    assert rtl.diopiGetTensorDtype(state, C.byref(dtype)) == 0 and dtype.value == int(rt.Dtype.uint8)
    assert rtl.diopiGetTensorDevice(state, C.byref(where)) == 0 and where.value == int(rt.Device.Host)

    for t in (tx, tw, tout, tinv, state):
        rtl.diopirtTensorDestroy(t)
    rtl.diopirtContextDestroy(ctx)
    for ptr in (dx, dw, dout, dinv):
        rtl.device_free(ptr)
    assert rtl.device_destroy_stream(stream) == 0
    assert rtl.finalizeLibrary() == 0


class _HookDevice:
    """A caller in the manner of the reference's test runtime (litert.cpp:358-380): every device buffer comes from
    device_malloc, every transfer is an asynchronous copy on a stream from device_make_stream, the operators are enqueued
    on that stream through a context made for it, and the host waits with device_synchronize_stream.  No torch on the device."""

    NP_DTYPES = {np.dtype(np.float16): rt.Dtype.float16, np.dtype(np.float32): rt.Dtype.float32, np.dtype(np.float64): rt.Dtype.float64,
                 np.dtype(np.int32): rt.Dtype.int32, np.dtype(np.int64): rt.Dtype.int64}

    def __init__(self):
        import ctypes as C
        self.C = C
        self.rtl, self.impl = rt.libs().rt, rt.libs().impl
        assert self.rtl.initLibrary() == 0
        self.stream = C.c_void_p()
        assert self.rtl.device_make_stream(C.byref(self.stream)) == 0 and self.stream.value
        self.ctx = self.rtl.diopirtContextCreate(self.stream)
        self.buffers, self.handles = [], []

    def tensor(self, array):
        """Device copy of a numpy array, wrapped in a tensor handle."""
        array = np.ascontiguousarray(array)
        ptr = self.rtl.device_malloc(max(array.nbytes, 1))
        assert ptr
        self.buffers.append(ptr)
        if array.nbytes:
            assert self.rtl.device_memcpy_h2d_async(self.stream, ptr, array.ctypes.data, array.nbytes) == 0
            assert self.rtl.device_synchronize_stream(self.stream) == 0  # the host array may go away after this call
        dims = (self.C.c_int64 * max(array.ndim, 1))(*array.shape)
        h = self.rtl.diopirtTensorWrap(ptr, dims, None, array.ndim, int(self.NP_DTYPES[array.dtype]), int(rt.Device.AIChip))
        assert h
        self.handles.append(h)
        return h, ptr

    def fetch(self, ptr, like):
        host = np.empty_like(like)
        if host.nbytes:
            assert self.rtl.device_memcpy_d2h_async(self.stream, host.ctypes.data, ptr, host.nbytes) == 0
        assert self.rtl.device_synchronize_stream(self.stream) == 0
        return host

    def call(self, name, *args):
        ret = getattr(self.impl, name)(self.ctx, *args)
        assert ret == 0, f"{name}: {ret}: {rt.get_last_error_string()}"

    def close(self):
        for h in self.handles:
            self.rtl.diopirtTensorDestroy(h)
        self.rtl.diopirtContextDestroy(self.ctx)
        for ptr in self.buffers:
            self.rtl.device_free(ptr)
        assert self.rtl.device_destroy_stream(self.stream) == 0
        assert self.rtl.finalizeLibrary() == 0


def test_harness_hooks_drive_the_six_hot_path_operators(golden):
    """rms_norm, rotary_emb, destindex_copy_kv, token_attention, token_softmax_reducev and context_attention on the
    reference's own case shapes (diopi_configs.py:9053-9105, 9137-9263, 9314-9381, 9517-9610), driven the way diopi_test
    drives a backend: memory, copies, stream and synchronisation through the conform_test.h hooks only, results checked
    against the oracle on the host."""
    dev = _HookDevice()
    rng = np.random.default_rng(17)
    try:
        for name in ("float32", "float16"):
            npdt, dt = np.dtype(name), TORCH_DTYPES[name]
            tol = TOL[dt]
            rnd = lambda *shape: rng.standard_normal(shape).astype(npdt)  # noqa: E731

            # ---- rms_norm (with the backward pass on the fp32 cases)
            for case in golden["rms_norm"]["cases"]:
                shape, ns, eps = case["input"], case["normalized_shape"], case["eps"]
                x, w = rnd(*shape), rng.uniform(0.5, 1.5, ns).astype(npdt)
                lead = shape[: len(shape) - len(ns)]
                out, inv = np.zeros_like(x), np.zeros(lead, np.float32)
                (hx, _), (hw, _), (ho, po), (hi, pi) = dev.tensor(x), dev.tensor(w), dev.tensor(out), dev.tensor(inv)
                dev.call("diopiRMSNorm", ho, hi, hx, rt.Sizes(ns).c, hw, None, eps)
                got_out, got_inv = dev.fetch(po, out), dev.fetch(pi, inv)
                want_out, want_inv = O.rms_norm(torch.from_numpy(x), tuple(ns), torch.from_numpy(w), None, eps)
                assert_close(torch.from_numpy(got_out), want_out, what=f"hooks: rms_norm {shape} {name}", **tol)
                assert_close(torch.from_numpy(got_inv), want_inv, what=f"hooks: inv_rms {shape} {name}", **TOL[torch.float32])
                if name == "float32":
                    go = rnd(*shape)
                    gi, gw = np.zeros_like(x), np.zeros_like(w)
                    (hgo, _), (hgi, pgi), (hgw, pgw) = dev.tensor(go), dev.tensor(gi), dev.tensor(gw)
                    dev.call("diopiRMSNormBackward", hgi, hgw, None, hgo, hx, hw, None, hi, rt.Sizes(ns).c, eps)
                    want_gi, want_gw, _ = O.rms_norm_backward(torch.from_numpy(go), torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(got_inv),
                                                              tuple(ns), exact=True)
                    assert_close(torch.from_numpy(dev.fetch(pgi, gi)), want_gi, what=f"hooks: rms_norm grad_input {shape}", rtol=1e-5, atol=1e-5)
                    assert_close(torch.from_numpy(dev.fetch(pgw, gw)), want_gw, what=f"hooks: rms_norm grad_weight {shape}", rtol=1e-4, atol=1e-4)

            # ---- rotary_emb (the interleaved cases answer diopiNoImplement, as the reference's own implementation does)
            for case in golden["rotary_emb"]["cases"]:
                x, cos, sin = rnd(*case["input"]), rnd(*case["cos"]), rnd(*case["cos"])
                out = np.zeros_like(x)
                (hx, _), (hc, _), (hs, _), (ho, po) = dev.tensor(x), dev.tensor(cos), dev.tensor(sin), dev.tensor(out)
                ret = dev.impl.diopiRotaryEmbedding(dev.ctx, ho, hx, hc, hs, bool(case["conj"]), bool(case["interleaved"]))
                if case["interleaved"]:
                    assert ret == int(rt.diopiError.diopi_no_implement)
                    continue
                assert ret == 0, rt.get_last_error_string()
                want = O.rotary_emb(torch.from_numpy(x), torch.from_numpy(cos), torch.from_numpy(sin), case["conj"])
                assert_close(torch.from_numpy(dev.fetch(po, out)), want, what=f"hooks: rotary_emb {case['input']} {name}", **tol)

            # ---- destindex_copy_kv: bit for bit
            for case in golden["destindex_copy_kv"]["cases"]:
                k, cache = rnd(*case["k_shape"]), rnd(*case["out_shape"])
                dest = np.asarray(case["dest_loc"], np.int32)
                (hk, _), (hd, _), (hc, pc) = dev.tensor(k), dev.tensor(dest), dev.tensor(cache)
                dev.call("diopiDestIndexCopyKV", hc, hk, hd)
                want = cache.copy()
                want[dest] = k
                assert dev.fetch(pc, cache).tobytes() == want.tobytes(), f"hooks: destindex_copy_kv {case['k_shape']} {name}"

            # ---- token_attention, then token_softmax_reducev on its logits
            fx = golden["token_attention"]
            q, kc, vc = rnd(*fx["q_shape"]), rnd(*fx["k_shape"]), rnd(*fx["k_shape"])
            b_loc, b_start, b_len = (np.asarray(fx[key], np.int32) for key in ("b_loc", "b_start_loc", "b_seq_len"))
            logits = np.full(fx["out_shape"], -7.0, npdt)
            (hq, _), (hk, _), (hv, _), (hl, pl) = dev.tensor(q), dev.tensor(kc), dev.tensor(vc), dev.tensor(logits)
            (hloc, _), (hst, _), (hln, _) = dev.tensor(b_loc), dev.tensor(b_start), dev.tensor(b_len)
            dev.call("diopiTokenAttentionInference", hl, hq, hk, hloc, hst, hln, fx["max_input_len"])
            got_l = dev.fetch(pl, logits)
            want_l = O.token_attention(torch.from_numpy(q), torch.from_numpy(kc), torch.full(fx["out_shape"], -7.0, dtype=dt), torch.from_numpy(b_loc),
                                       torch.from_numpy(b_start), torch.from_numpy(b_len), fx["max_input_len"])
            assert_close(torch.from_numpy(got_l), want_l, what=f"hooks: token_attention {name}", **tol)
            out = np.zeros(golden["token_softmax_reducev"]["out_shape"], npdt)
            ho, po = dev.tensor(out)
            dev.call("diopiTokenSoftmaxReduceVInference", ho, hl, hv, hloc, hst, hln, fx["max_input_len"], golden["token_softmax_reducev"]["other_kv_index"])
            want_o = O.token_softmax_reducev(torch.from_numpy(got_l), torch.from_numpy(vc), torch.zeros(out.shape, dtype=dt), torch.from_numpy(b_loc),
                                             torch.from_numpy(b_start), torch.from_numpy(b_len), fx["max_input_len"], 0)
            assert_close(torch.from_numpy(dev.fetch(po, out)), want_o, what=f"hooks: token_softmax_reducev {name}", **tol)

            # ---- context_attention
            for case in golden["context_attention"]["cases"]:
                q, k, v = (0.5 * rnd(*case["shape"]) for _ in range(3))
                b_start, b_len = np.asarray(case["b_start_loc"], np.int32), np.asarray(case["b_seq_len"], np.int32)
                out = np.full(case["shape"], 77.0, npdt)
                (hq, _), (hk, _), (hv, _), (ho, po) = dev.tensor(q), dev.tensor(k), dev.tensor(v), dev.tensor(out)
                (hst, _), (hln, _) = dev.tensor(b_start), dev.tensor(b_len)
                dev.call("diopiContextAttentionInference", ho, hq, hk, hv, hst, hln, case["max_input_len"])
                want = O.context_attention(torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v), torch.full(case["shape"], 77.0, dtype=dt),
                                           torch.from_numpy(b_start), torch.from_numpy(b_len), case["max_input_len"])
                assert_close(torch.from_numpy(dev.fetch(po, out)), want, what=f"hooks: context_attention {case['shape']} {name}", **tol)
            say("hooks:", name, "six operators on the reference's case shapes")
    finally:
        dev.close()


def test_c_host_runs_operators_through_the_c_abi():
    """The plain-C host of tests/golden/c_client.c: RMSNorm against a double-precision loop and DestIndexCopyKV against
    a byte-exact scatter, both written in C, with device memory and the stream from the harness hooks."""
    import os
    import subprocess
    client = os.path.join(os.path.dirname(rt.IMPL_LIB_PATH), "diopi_c_client")
    assert os.path.isfile(client), "the C host is built with the libraries"
    res = subprocess.run([client], capture_output=True, text=True, timeout=120)
    say(res.stdout)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "diopiRMSNorm fp32" in res.stdout and "bytes equal" in res.stdout and res.stdout.strip().endswith("c client ok")


# ----------------------------------------------------------------------------- error behaviour on a GPU box
def _strided_view(t):
    big = torch.zeros(*t.shape[:-1], t.shape[-1] * 2, dtype=t.dtype, device=t.device)
    view = big[..., ::2]
    view.copy_(t)
    return view


def test_every_operator_refuses_strided_views_instead_of_reading_them_as_dense():
    # impl/torch follows any stride through ATen; these kernels address rows by shape alone, so a view that is not densely
    # packed must come back as an error from every entry point and every tensor argument (the adaptor's `contiguous: True`
    # makes the copies).  The one exception is by design: diopiRotaryEmbedding follows the strides of cos and sin.
    g = gen(1234)
    B, H, D, T = 2, 4, 128, 6
    lens = [4, 2]

    def R(*shape):
        return torch.randn(*shape, generator=g).half().to(DEV)

    def I(values, dt=torch.int32):
        return torch.tensor(values, dtype=dt, device=DEV)

    loc = [[0, 1, 2, 3], [0, 0, 4, 5]]
    cases = {
        "rms_norm": (lambda x, w: F.rms_norm(x, (256,), w, None, 1e-6), [R(5, 256), R(256)]),
        "rms_norm_backward": (lambda go, x, w: F.rms_norm_backward([go], x, w, None, (256,), 1e-6, inv_rms=torch.ones(5, 1, device=DEV)), [R(5, 256), R(5, 256), R(256)]),
        "root_mean_square_norm_inp": (lambda x, w: F.root_mean_square_norm_inp(x, w, 1e-6), [R(5, 256), R(256)]),
        "fused_add_root_mean_square_norm_inp": (lambda x, r, b, w: F.fused_add_root_mean_square_norm_inp(x, r, b, w, 1e-6), [R(5, 256), R(5, 256), R(256), R(256)]),
        "rotary_emb": (lambda x: F.rotary_emb(x, R(T, 1, D // 2), R(T, 1, D // 2), False, False), [R(T, H, D)]),
        "rotary_emb_v2": (lambda q, k, c, s: F.rotary_emb_v2(q, k, c, s, D), [R(T, H * D), R(T, H * D), R(T, 1, D), R(T, 1, D)]),
        "apply_penalty": (lambda lg, p, f, ids, cnt, cum: F.apply_penalty(lg, p, f, ids, cnt, cum, 3),
                          [R(2, 50), R(2), R(2), I([1, 2, 3, 4]), I([1, 1, 2, 2]), I([0, 3, 4])]),
        "apply_penalty_v2": (lambda lg, p, f, r, ids, cnt: F.apply_penalty_v2(lg, p, f, r, ids, cnt), [R(2, 50), R(4), R(4), R(4), I([1, 2, 53, 54]), I([1, 1, 2, 2])]),
        "destindex_copy_kv": (lambda k, dst, out: F.destindex_copy_kv(k, dst, out), [R(3, H, D), I([0, 5, 2]), R(8, H, D)]),
        "token_attention": (lambda q, k, out, bl, bs, bq: F.token_attention(q, k, out, bl, bs, bq, 4), [R(B, H, D), R(16, H, D), R(H, 6), I(loc), I([0, 4]), I(lens)]),
        "token_softmax_reducev": (lambda lg, v, out, bl, bs, bq: F.token_softmax_reducev(lg, v, out, bl, bs, bq, 4, 0),
                                  [R(H, 6), R(16, H, D), R(B, H, D), I(loc), I([0, 4]), I(lens)]),
        "context_attention": (lambda q, k, v, out, bs, bq: F.context_attention(q, k, v, out, bs, bq, 4),
                              [R(T, H, D), R(T, H, D), R(T, H, D), R(T, H, D), I([0, 4]), I(lens)]),
        "context_attention_no_alloc": (lambda q, k, v, out, bs, bq: F.context_attention_no_alloc(q, k, v, out, bs, bq, 4),
                                       [R(T, H, D), R(T, H, D), R(T, H, D), R(T, H, D), I([0, 4]), I(lens)]),
        "flash_attention_varlen": (lambda q, k, v, cu: F.flash_attention_varlen(q, k, v, cu, cu, None, 4, 4, 0, None, True),
                                   [R(T, H, D), R(T, H, D), R(T, H, D), I([0, 4, 6])]),
        "flash_attention": (lambda q, k, v: F.flash_attention(q, k, v, None, 0, None, True), [R(2, 3, H, D), R(2, 3, H, D), R(2, 3, H, D)]),
        "multihead_attention": (lambda q, k, v: F.multihead_attention(q, k, v, 0, True, False, None), [R(2, 3, H, D), R(2, 3, H, D), R(2, 3, H, D)]),
        "multihead_attention_varlen": (lambda q, k, v, cu: F.multihead_attention_varlen(q, k, v, cu, 4, 0, True, False, None),
                                       [R(T, H, D), R(T, H, D), R(T, H, D), I([0, 4, 6], torch.int64)]),
        "prompt_flash_attention": (lambda q, k, v: F.prompt_flash_attention(q, k, v, None, [3, 3], 3, H, H, D), [R(T, H * D), R(T, H * D), R(T, H * D)]),
        "paged_attention": (lambda q, k, v, bt: F.paged_attention(q, k, v, None, lens, H, H, D, bt, 4), [R(B, H * D), R(16, H * D), R(16, H * D), I([[0, 1], [2, 3]])]),
    }
    for name, (call, tensors) in cases.items():
        call(*[t.clone() for t in tensors])  # the dense call is valid
        for i in range(len(tensors)):
            args = [t.clone() for t in tensors]
            args[i] = _strided_view(args[i])
            assert not args[i].is_contiguous()
            with pytest.raises(rt.DiopiException, match="contiguous"):
                call(*args)
    # the exception: strided cos / sin tables give the result of the dense ones
    x, cos, sin = R(T, H, D), R(T, 1, D // 2), R(T, 1, D // 2)
    assert_bit_equal(F.rotary_emb(x, _strided_view(cos), _strided_view(sin), False, False).cpu(), F.rotary_emb(x, cos, sin, False, False).cpu(),
                     "rotary_emb follows the strides of cos and sin")
    torch.cuda.synchronize()


def test_errors_do_not_launch():
    x = torch.randn(4, 8, device=DEV)
    w = torch.ones(8, device=DEV)
    before = rt.get_last_error_string()
    with pytest.raises(rt.DiopiException):
        F.rms_norm(x, (7,), w, None, 1e-6)  # normalized_shape does not match
    assert rt.get_last_error_string() != before
    with pytest.raises(rt.DiopiException):
        F.rms_norm(x.t(), (4,), torch.ones(4, device=DEV), None, 1e-6)  # non-contiguous input is rejected, not converted
    with pytest.raises(rt.DiopiException):
        F.destindex_copy_kv(x.half(), torch.zeros(4, dtype=torch.int32, device=DEV), x)  # dtype mismatch
    torch.cuda.synchronize()
