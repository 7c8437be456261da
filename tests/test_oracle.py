"""Pins the CPU oracle (oracle/ref_ops.py) against what the reference's own fixtures and the
mathematics fix, so that a dropped term, a wrong sign/index or a transposed operand fails here.
Runs on the CPU; no GPU, no product code."""
import math

import numpy as np
import pytest
import torch

from oracle import ref_ops as O
from tests.conftest import TORCH_DTYPES
from tests.helpers import assert_bit_equal, assert_close


def rng(seed):
    return torch.Generator().manual_seed(seed)


# ----------------------------------------------------------------------------- rms_norm
def test_rms_norm_constant_rows_closed_form():
    # x == c  =>  inv_rms = 1/sqrt(c^2 + eps), out = w * c * inv_rms
    c, eps = 3.0, 1e-2
    x = torch.full((7, 16), c, dtype=torch.float64)
    w = torch.linspace(0.5, 1.5, 16, dtype=torch.float64)
    out, inv = O.rms_norm(x, (16,), w, None, eps)
    assert_close(inv, torch.full((7,), 1 / math.sqrt(c * c + eps), dtype=torch.float64), 1e-14, 0, "inv_rms")
    assert_close(out, (w * c / math.sqrt(c * c + eps)).expand(7, 16), 1e-14, 0, "out")


def test_rms_norm_sign_rows_and_scale_invariance():
    g = rng(0)
    x = (torch.randint(0, 2, (5, 32), generator=g) * 2 - 1).double()
    out, inv = O.rms_norm(x, (32,), torch.ones(32, dtype=torch.float64), None, 1e-6)
    assert_close(out, x / math.sqrt(1 + 1e-6), 1e-14, 0, "+-1 rows")
    # eps = 0: out(a*x) == out(x)
    y = torch.randn(4, 24, generator=g, dtype=torch.float64)
    w = torch.rand(24, generator=g, dtype=torch.float64) + 0.5
    o1, _ = O.rms_norm(y, (24,), w, None, 0.0)
    o2, _ = O.rms_norm(y * 7.5, (24,), w, None, 0.0)
    assert_close(o1, o2, 1e-13, 0, "scale invariance")


def test_rms_norm_energy_identity_and_bias_and_multidim():
    g = rng(1)
    x = torch.randn(3, 2, 7, 8, generator=g, dtype=torch.float64)
    w = torch.rand(7, 8, generator=g, dtype=torch.float64) + 0.5
    b = torch.randn(7, 8, generator=g, dtype=torch.float64)
    eps = 1e-2
    out, inv = O.rms_norm(x, (7, 8), w, None, eps)
    ms = (x * x).mean(dim=(-1, -2))
    # sum((out/w)^2) = n2 * ms / (ms + eps)
    assert_close(((out / w) ** 2).sum(dim=(-1, -2)), 56 * ms / (ms + eps), 1e-12, 0, "energy identity")
    assert tuple(inv.shape) == (3, 2)
    out_b, _ = O.rms_norm(x, (7, 8), w, b, eps)
    assert_close(out_b - out, b.expand_as(out), 1e-12, 1e-14, "bias is added after the scaling")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_rms_norm_modes_agree_and_match_python_twin(dtype):
    # the reference's Python statement (customized_test.py:392-403): weight * (x * rsqrt(mean(x^2) + eps))
    g = rng(2)
    x = torch.randn(35, 125, 32, generator=g).to(dtype)
    w = (torch.rand(32, generator=g) + 0.5).to(dtype)
    out, inv = O.rms_norm(x, (32,), w, None, 1e-6)
    twin = (w.float() * (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6))).to(dtype)
    exact, inv64 = O.rms_norm(x, (32,), w, None, 1e-6, exact=True)
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    assert_close(out, twin, tol, tol, "kernel statement vs python statement")
    assert_close(out, exact, tol, tol, "dtype-faithful vs float64")
    assert inv.dtype == torch.float32 and out.dtype == dtype


# ----------------------------------------------------------------------------- in-place RMS normalisations (lmdeploy set)
def test_inplace_norms_reduce_to_rms_norm_and_to_each_other():
    g = rng(40)
    x = torch.randn(6, 48, generator=g, dtype=torch.float64)
    r = torch.randn(6, 48, generator=g, dtype=torch.float64)
    b = torch.randn(48, generator=g, dtype=torch.float64)
    w = torch.rand(48, generator=g, dtype=torch.float64) + 0.5
    eps = 1e-5
    want, _ = O.rms_norm(x, (48,), w, None, eps, exact=True)  # pinned by the tests above
    assert_close(O.root_mean_square_norm_inp(x, w, eps, exact=True), want, 1e-13, 0, "plain form vs rms_norm")
    out, res = O.fused_add_root_mean_square_norm_inp(x, torch.zeros_like(x), None, w, eps, exact=True)
    assert_close(out, want, 1e-13, 0, "zero residual, no bias vs rms_norm")
    assert_bit_equal(res, x, "zero residual, no bias: the new residual is the input")
    # the new residual is the sum of its three terms, and the output is the plain form applied to it
    out, res = O.fused_add_root_mean_square_norm_inp(x, r, b, w, eps, exact=True)
    assert_close(res, x + r + b, 1e-14, 0, "new residual")
    assert_close(out, O.root_mean_square_norm_inp(x + r + b, w, eps, exact=True), 1e-13, 0, "fused = add, then normalise")
    # a dropped bias or residual term must show
    assert (out - O.fused_add_root_mean_square_norm_inp(x, r, None, w, eps, exact=True)[0]).abs().max() > 1e-3
    assert (out - O.fused_add_root_mean_square_norm_inp(x, torch.zeros_like(r), b, w, eps, exact=True)[0]).abs().max() > 1e-3


def test_inplace_norms_closed_forms():
    # constant rows: s = cr + cx + cb, out = scale * s / sqrt(s^2 + eps)
    cx, cr, cb, eps = 1.5, -0.25, 2.0, 1e-2
    n = 32
    w = torch.linspace(0.5, 1.5, n, dtype=torch.float64)
    x = torch.full((3, n), cx, dtype=torch.float64)
    r = torch.full((3, n), cr, dtype=torch.float64)
    b = torch.full((n,), cb, dtype=torch.float64)
    s = cx + cr + cb
    out, res = O.fused_add_root_mean_square_norm_inp(x, r, b, w, eps, exact=True)
    assert_close(res, torch.full((3, n), s, dtype=torch.float64), 1e-15, 0, "constant rows: residual")
    assert_close(out, (w * s / math.sqrt(s * s + eps)).expand(3, n), 1e-14, 0, "constant rows: output")
    # energy identity: sum((out/scale)^2) = n * ms / (ms + eps)
    g = rng(41)
    y = torch.randn(5, 64, generator=g, dtype=torch.float64) * 3
    w = torch.rand(64, generator=g, dtype=torch.float64) + 0.5
    o = O.root_mean_square_norm_inp(y, w, eps, exact=True)
    ms = (y * y).mean(-1)
    assert_close(((o / w) ** 2).sum(-1), 64 * ms / (ms + eps), 1e-12, 0, "energy identity")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_inplace_norms_dtype_mode_is_close_to_exact_and_stores_a_rounded_residual(dtype):
    g = rng(42)
    x = torch.randn(9, 256, generator=g).to(dtype)
    r = torch.randn(9, 256, generator=g).to(dtype)
    b = torch.randn(256, generator=g).to(dtype)
    w = (torch.rand(256, generator=g) + 0.5).to(dtype)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    out, res = O.fused_add_root_mean_square_norm_inp(x, r, b, w, 1e-6)
    eo, er = O.fused_add_root_mean_square_norm_inp(x, r, b, w, 1e-6, exact=True)
    assert out.dtype == dtype and res.dtype == dtype
    if dtype == torch.float32:
        assert_close(res, er, 2e-7, 1e-6, "the stored residual is the fp32 sum")  # absolute: the terms cancel
    else:  # sums of three 16-bit values are exact in fp32 here, so one rounding is left
        assert_bit_equal(res, er.to(dtype), "the stored residual is the exact sum rounded once")
    assert_close(out, eo, tol, tol, "fused, dtype mode vs float64")
    assert_close(O.root_mean_square_norm_inp(x, w, 1e-6), O.root_mean_square_norm_inp(x, w, 1e-6, exact=True), tol, tol, "plain, dtype mode vs float64")


def test_rms_norm_backward_matches_float64_autograd():
    g = rng(3)
    for shape, ns in [((5, 5), (5,)), ((16, 64, 64), (64, 64)), ((3, 2, 16, 7, 8), (7, 8))]:
        x = torch.randn(*shape, generator=g, dtype=torch.float64, requires_grad=True)
        w = (torch.rand(*ns, generator=g, dtype=torch.float64) + 0.5).requires_grad_()
        b = torch.randn(*ns, generator=g, dtype=torch.float64, requires_grad=True)
        go = torch.randn(*shape, generator=g, dtype=torch.float64)
        eps = 1e-4
        dims = tuple(range(-len(ns), 0))
        y = w * (x * torch.rsqrt((x * x).mean(dims, keepdim=True) + eps)) + b  # textbook RMSNorm
        gx, gw, gb = torch.autograd.grad(y, (x, w, b), go)
        _, inv = O.rms_norm(x.detach(), ns, w.detach(), None, eps)
        ox, ow, ob = O.rms_norm_backward(go, x.detach(), w.detach(), inv, ns, with_bias=True)
        assert_close(ox, gx, 1e-10, 1e-12, "grad_input")
        assert_close(ow, gw, 1e-10, 1e-12, "grad_weight")
        assert_close(ob, gb, 1e-10, 1e-12, "grad_bias")


def test_rms_norm_backward_orthogonality_identity():
    # sum_l x_l * grad_input_l = eps * inv_rms^3 * sum_l g_l x_l   (zero for eps = 0)
    g = rng(4)
    x = torch.randn(9, 40, generator=g, dtype=torch.float64)
    w = torch.rand(40, generator=g, dtype=torch.float64) + 0.5
    go = torch.randn(9, 40, generator=g, dtype=torch.float64)
    for eps in (0.0, 1e-2):
        _, inv = O.rms_norm(x, (40,), w, None, eps)
        gx, _, _ = O.rms_norm_backward(go, x, w, inv, (40,))
        lhs = (x * gx).sum(-1)
        rhs = eps * inv ** 3 * (go * w * x).sum(-1)
        assert_close(lhs, rhs, 1e-9, 1e-12, f"identity eps={eps}")


# ----------------------------------------------------------------------------- rotary
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32, torch.float64])
def test_rotary_position_zero_is_identity_bitwise(dtype):
    g = rng(5)
    x = torch.randn(1, 9, 4, 32, generator=g).to(dtype)
    cos = torch.ones(9, 1, 16, dtype=dtype)
    sin = torch.zeros(9, 1, 16, dtype=dtype)
    for conj in (False, True):
        assert_bit_equal(O.rotary_emb(x, cos, sin, conj), x, "rotation by angle 0")


def test_rotary_norm_preserved_and_conj_inverts_and_quarter_turn():
    g = rng(6)
    x = torch.randn(3, 100, 8, 64, generator=g, dtype=torch.float64)
    ang = torch.rand(100, 1, 32, generator=g, dtype=torch.float64) * 6.28
    cos, sin = ang.cos(), ang.sin()
    y = O.rotary_emb(x, cos, sin, False, exact=True)
    x1, x2 = x.chunk(2, -1)
    y1, y2 = y.chunk(2, -1)
    assert_close(y1 ** 2 + y2 ** 2, x1 ** 2 + x2 ** 2, 1e-12, 1e-14, "pairwise norm")
    assert_close(O.rotary_emb(y, cos, sin, True, exact=True), x, 1e-12, 1e-14, "conj undoes the rotation")
    # a quarter turn (c=0, s=1) maps (x1, x2) -> (-x2, x1); with conj -> (x2, -x1): pins signs and operand order
    q = O.rotary_emb(x, torch.zeros_like(cos), torch.ones_like(sin), False, exact=True)
    assert_close(q, torch.cat((-x2, x1), -1), 0, 0, "quarter turn")
    qc = O.rotary_emb(x, torch.zeros_like(cos), torch.ones_like(sin), True, exact=True)
    assert_close(qc, torch.cat((x2, -x1), -1), 0, 0, "quarter turn, conj")


def test_rotary_reference_shapes_broadcast(golden):
    g = rng(7)
    for case in golden["rotary_emb"]["cases"] + golden["rotary_emb"]["empty_cases"]:
        x = torch.randn(*case["input"], generator=g)
        cos = torch.randn(*case["cos"], generator=g)
        sin = torch.randn(*case["cos"], generator=g)
        if case["interleaved"]:
            with pytest.raises(NotImplementedError):
                O.rotary_emb(x, cos, sin, case["conj"], True)
            continue
        out = O.rotary_emb(x, cos, sin, case["conj"])
        assert out.shape == x.shape
        if x.numel():
            # spot check one element with explicit index arithmetic (right-aligned broadcast)
            half = x.shape[-1] // 2
            idx = tuple(s - 1 for s in x.shape[:-1])
            cidx = tuple(min(i, s - 1) for i, s in zip(idx[len(idx) - (cos.dim() - 1):], cos.shape[:-1])) if cos.dim() > 1 else ()
            c, s_ = float(cos[cidx + (0,)]), float(sin[cidx + (0,)])
            a, b = float(x[idx + (0,)]), float(x[idx + (half,)])
            want = a * c + b * s_ if case["conj"] else a * c - b * s_
            assert abs(float(out[idx + (0,)]) - want) < 1e-5


def test_rotary_v2_identity_tables_and_agreement_with_rotary_emb():
    g = rng(8)
    T, Hq, Hk, dim = 7, 3, 2, 16
    for dtype in (torch.float16, torch.bfloat16, torch.float32, torch.float64):
        q = torch.randn(T, Hq * dim, generator=g).to(dtype)
        k = torch.randn(T, Hk * dim, generator=g).to(dtype)
        q2, k2 = O.rotary_emb_v2(q, k, torch.ones(T, 1, dim, dtype=dtype), torch.zeros(T, 1, dim, dtype=dtype), dim)
        assert_bit_equal(q2, q, "cos = 1, sin = 0 leaves query alone")
        assert_bit_equal(k2, k, "cos = 1, sin = 0 leaves key alone")
    # tables with duplicated halves: the operator is rotary_emb (conj = False) on the [T, heads, dim] view
    q = torch.randn(T, Hq * dim, generator=g, dtype=torch.float64)
    k = torch.randn(T, Hk * dim, generator=g, dtype=torch.float64)
    ang = torch.rand(T, 1, dim // 2, generator=g, dtype=torch.float64) * 6.28
    cos, sin = torch.cat((ang.cos(), ang.cos()), -1), torch.cat((ang.sin(), ang.sin()), -1)
    q2, k2 = O.rotary_emb_v2(q, k, cos, sin, dim, exact=True)
    assert_close(q2.reshape(T, Hq, dim), O.rotary_emb(q.reshape(T, Hq, dim), ang.cos(), ang.sin(), False, exact=True), 1e-13, 1e-14, "query vs rotary_emb")
    assert_close(k2.reshape(T, Hk, dim), O.rotary_emb(k.reshape(T, Hk, dim), ang.cos(), ang.sin(), False, exact=True), 1e-13, 1e-14, "key vs rotary_emb")


def test_rotary_v2_python_loops_with_unequal_table_halves():
    g = rng(9)
    T, H, dim = 4, 2, 8
    q = torch.randn(T, H * dim, generator=g, dtype=torch.float64)
    k = torch.randn(T, dim, generator=g, dtype=torch.float64)
    cos = torch.randn(T, 1, dim, generator=g, dtype=torch.float64)  # not a rotation: the two halves are unrelated numbers
    sin = torch.randn(T, 1, dim, generator=g, dtype=torch.float64)
    q2, k2 = O.rotary_emb_v2(q, k, cos, sin, dim, exact=True)
    for x, y, heads in ((q, q2, H), (k, k2, 1)):
        for t in range(T):
            for h in range(heads):
                for d in range(dim):
                    partner = x[t, h * dim + d + dim // 2] * -1.0 if d < dim // 2 else x[t, h * dim + d - dim // 2]
                    want = x[t, h * dim + d] * cos[t, 0, d] + partner * sin[t, 0, d]
                    assert abs(float(y[t, h * dim + d]) - float(want)) < 1e-13, (t, h, d)


# the reference's value fixtures for the penalty operators (diopi_configs.py:9265-9312 and 9468-9515)
PENALTY_LOGITS = [[0.1, 0.5, 0.4, 0.3, 0.5], [0.2, 0.4, 0.0, 0.0, 0.0], [0.3, 0.4, 0.5, 0.3, 0.0]]
PENALTY_COUNTS = [3, 3, 2, 2, 1, 3, 3, 3, 3, 2, 2]


def test_apply_penalty_reference_fixture_worked_by_hand():
    from fractions import Fraction as Fr
    logits = torch.tensor(PENALTY_LOGITS, dtype=torch.float64)
    pres, freq = [Fr(1, 10), Fr(8, 10), Fr(1)], [Fr(3, 10), Fr(5, 10), Fr(4, 10)]
    ids = [0, 1, 2, 3, 4, 0, 1, 0, 1, 2, 3]
    cum = [0, 5, 7, 11]
    # exact decimal arithmetic, entry by entry, independent of the oracle's tensor expressions
    want = [[Fr(str(v)) for v in row] for row in PENALTY_LOGITS]
    for i in range(3):
        for j in range(cum[i], cum[i + 1]):
            want[i][ids[j]] = want[i][ids[j]] - PENALTY_COUNTS[j] * freq[i] - pres[i]
    assert want[0][0] == Fr(-9, 10) and want[1][1] == Fr(-19, 10) and want[2][3] == Fr(-15, 10) and want[1][2] == 0 and want[2][4] == 0
    got = O.apply_penalty(logits.clone(), torch.tensor([0.1, 0.8, 1.0], dtype=torch.float64), torch.tensor([0.3, 0.5, 0.4], dtype=torch.float64),
                          torch.tensor(ids, dtype=torch.int32), torch.tensor(PENALTY_COUNTS, dtype=torch.int32), torch.tensor(cum, dtype=torch.int32), 5)
    assert_close(got, torch.tensor([[float(v) for v in row] for row in want], dtype=torch.float64), 1e-14, 1e-15, "fixture")
    # entries no sequence lists keep their bits, also in fp16
    l16 = torch.tensor(PENALTY_LOGITS, dtype=torch.float16)
    g16 = O.apply_penalty(l16.clone(), torch.tensor([0.1, 0.8, 1.0]).half(), torch.tensor([0.3, 0.5, 0.4]).half(), torch.tensor(ids, dtype=torch.int32),
                          torch.tensor(PENALTY_COUNTS, dtype=torch.int32), torch.tensor(cum, dtype=torch.int32), 5)
    assert_bit_equal(g16[1, 2:], l16[1, 2:], "untouched entries of sequence 1")
    assert_bit_equal(g16[2, 4:], l16[2, 4:], "untouched entry of sequence 2")
    assert_close(g16.double(), got, 2e-3, 2e-3, "fp16 follows the float64 result")


def test_apply_penalty_v2_reference_fixture_worked_by_hand():
    from fractions import Fraction as Fr
    pen = [Fr(1, 10)] * 4 + [Fr(8, 10)] * 4 + [Fr(1)] * 3
    ids = [0, 1, 2, 3, 4, 5, 6, 8, 9, 10, 11]
    flat = [Fr(str(v)) for row in PENALTY_LOGITS for v in row]
    want = list(flat)
    for j, idx in enumerate(ids):
        x = flat[idx]
        x = x / pen[j] if x > 0 else x * pen[j]
        want[idx] = x - PENALTY_COUNTS[j] * pen[j] - pen[j]
    assert want[0] == Fr(1) - Fr(3, 10) - Fr(1, 10) and want[7] == flat[7] and want[12] == flat[12]  # 7 and 12..14 are not listed
    p = torch.tensor([float(v) for v in pen], dtype=torch.float64)
    got = O.apply_penalty_v2(torch.tensor(PENALTY_LOGITS, dtype=torch.float64), p, p, p, torch.tensor(ids, dtype=torch.int32),
                             torch.tensor(PENALTY_COUNTS, dtype=torch.int32))
    assert_close(got.view(-1), torch.tensor([float(v) for v in want], dtype=torch.float64), 1e-13, 1e-15, "fixture v2")
    # a negative logit is multiplied, not divided
    neg = O.apply_penalty_v2(torch.tensor([[-2.0, 3.0]], dtype=torch.float64), torch.zeros(2, dtype=torch.float64), torch.zeros(2, dtype=torch.float64),
                             torch.tensor([4.0, 4.0], dtype=torch.float64), torch.tensor([0, 1]), torch.tensor([0, 0]))
    assert_close(neg, torch.tensor([[-8.0, 0.75]], dtype=torch.float64), 0, 0, "sign rule")


def test_rotary_fp64_is_computed_in_fp32():
    # rotary.cu:30-43 narrows every operand with static_cast<float>, also for double tensors
    x = torch.tensor([1.0 + 2 ** -40, 3.0], dtype=torch.float64)
    out = O.rotary_emb(x, torch.ones(1, dtype=torch.float64), torch.zeros(1, dtype=torch.float64), False)
    assert float(out[0]) == 1.0


# ----------------------------------------------------------------------------- destindex_copy_kv
def test_destindex_copy_kv_reference_fixtures(golden):
    g = rng(8)
    for case in golden["destindex_copy_kv"]["cases"]:
        dt = TORCH_DTYPES[case["dtype"]]
        k = torch.randn(*case["k_shape"], generator=g).to(dt)
        out = torch.randn(*case["out_shape"], generator=g).to(dt)
        before = out.clone()
        dest = torch.tensor(case["dest_loc"], dtype=torch.int32)
        O.destindex_copy_kv(k, dest, out)
        touched = set(case["dest_loc"])
        for t, d in enumerate(case["dest_loc"]):
            assert_bit_equal(out[d], k[t], f"row {d}")
        for r in range(out.shape[0]):
            if r not in touched:
                assert_bit_equal(out[r], before[r], f"untouched row {r}")


def test_destindex_copy_kv_is_raw_bytes():
    # NaN payloads and negative zeros survive: the copy never goes through arithmetic
    k = torch.tensor([[0x7E01, 0x8000, 0xFC00, 0x0001]], dtype=torch.int32).to(torch.int16).view(torch.float16).reshape(1, 1, 4)
    out = torch.zeros(3, 1, 4, dtype=torch.float16)
    O.destindex_copy_kv(k, torch.tensor([2]), out)
    assert_bit_equal(out[2:3], k)


# ----------------------------------------------------------------------------- token_attention
def test_token_attention_window_fixture(golden):
    fx = golden["token_attention"]
    b_loc = torch.tensor(fx["b_loc"], dtype=torch.int32)
    # independent statement of the window: the last L_i of the first max_input_len entries of row i
    for i, (L, want) in enumerate(zip(fx["b_seq_len"], fx["expected_slots"])):
        row = fx["b_loc"][i][: fx["max_input_len"]]
        assert row[len(row) - L:] == want
        assert O._window(b_loc, i, L, fx["max_input_len"]).tolist() == want
    # k[slot] = slot everywhere, q = ones  =>  out[h, start+t] = slot * D / sqrt(D)
    D = 128
    k = torch.arange(100, dtype=torch.float64).reshape(100, 1, 1).expand(100, 32, D).contiguous()
    q = torch.ones(3, 32, D, dtype=torch.float64)
    out = torch.full((32, 13), -7.0, dtype=torch.float64)
    O.token_attention(q, k, out, b_loc, torch.tensor(fx["b_start_loc"]), torch.tensor(fx["b_seq_len"]), fx["max_input_len"], exact=True)
    flat = [s for w in fx["expected_slots"] for s in w]
    assert_close(out, (torch.tensor(flat, dtype=torch.float64) * D / math.sqrt(D)).expand(32, 13), 1e-14, 0, "slot pattern")


def _brute_token_attention(q, k, b_loc, b_start, b_len, max_len, cols):
    B, H, D = q.shape
    G = H // k.shape[1]
    out = np.full((H, cols), np.nan)
    qn, kn = q.double().numpy(), k.double().numpy()
    for i in range(B):
        L = int(b_len[i])
        for t in range(L):
            slot = int(b_loc[i, max_len - L + t])
            for h in range(H):
                out[h, int(b_start[i]) + t] = float(np.dot(qn[i, h], kn[slot, h // G])) / math.sqrt(D)
    return torch.from_numpy(out)


@pytest.mark.parametrize("G", [1, 4])
def test_token_attention_brute_force_and_closed_forms(G):
    g = rng(9)
    B, Hkv, D, slots, N = 3, 2, 16, 40, 11
    H = Hkv * G
    q = torch.randn(B, H, D, generator=g, dtype=torch.float64)
    k = torch.randn(slots, Hkv, D, generator=g, dtype=torch.float64)
    b_len = torch.tensor([1, 7, 4])
    b_start = torch.tensor([0, 1, 8])
    max_len = 7
    b_loc = torch.stack([torch.randperm(slots, generator=g)[:N] for _ in range(B)]).int()
    out = torch.full((H, 12), float("nan"), dtype=torch.float64)
    O.token_attention(q, k, out, b_loc, b_start, b_len, max_len, exact=True)
    want = _brute_token_attention(q, k, b_loc, b_start, b_len, max_len, 12)
    assert_close(out, want, 1e-13, 1e-14, "brute force")
    # L = 1: a single dot product
    s0 = int(b_loc[0, max_len - 1])
    assert abs(float(out[0, 0]) - float(q[0, 0] @ k[s0, 0]) / math.sqrt(D)) < 1e-13
    # k = q  =>  |q|^2 / sqrt(D)
    kk = torch.zeros_like(k)
    kk[5] = q[0, ::G]
    loc = torch.full((1, 3), 5, dtype=torch.int32)
    o2 = torch.zeros(H, 1, dtype=torch.float64)
    O.token_attention(q[:1], kk, o2, loc, torch.tensor([0]), torch.tensor([1]), 3, exact=True)
    assert abs(float(o2[0, 0]) - float((q[0, 0] ** 2).sum()) / math.sqrt(D)) < 1e-12


# ----------------------------------------------------------------------------- token_softmax_reducev
def test_softmax_reducev_closed_forms(golden):
    fx = golden["token_attention"]
    g = rng(10)
    b_loc = torch.tensor(fx["b_loc"], dtype=torch.int32)
    b_start, b_len = torch.tensor(fx["b_start_loc"]), torch.tensor(fx["b_seq_len"])
    v = torch.randn(100, 32, 128, generator=g, dtype=torch.float64)
    # constant logits => the mean of the gathered rows
    out = torch.zeros(3, 32, 128, dtype=torch.float64)
    O.token_softmax_reducev(torch.full((32, 13), 0.25, dtype=torch.float64), v, out, b_loc, b_start, b_len, 5, 10, exact=True)
    for i, slots in enumerate(fx["expected_slots"]):
        assert_close(out[i], v[slots].mean(0), 1e-13, 1e-14, f"mean of rows, sequence {i}")
    # one dominant logit => that row
    logits = torch.zeros(32, 13, dtype=torch.float64)
    logits[:, 6] = 800.0  # column 6 = sequence 1, token 2 -> slot 5
    O.token_softmax_reducev(logits, v, out, b_loc, b_start, b_len, 5, 10, exact=True)
    assert_close(out[1], v[5], 1e-13, 0, "dominant logit")
    # L = 1 => exactly the row, bit for bit, in 16-bit too
    v16 = v.half()
    o16 = torch.zeros(1, 32, 128, dtype=torch.float16)
    O.token_softmax_reducev(torch.randn(32, 1, generator=g).half(), v16, o16, torch.tensor([[9, 9, 42]], dtype=torch.int32), torch.tensor([0]),
                            torch.tensor([1]), 3, 0)
    assert_bit_equal(o16[0], v16[42], "L = 1")


@pytest.mark.parametrize("G", [1, 2])
def test_softmax_reducev_brute_force(G):
    g = rng(11)
    B, Hkv, D, slots = 2, 3, 8, 30
    H = Hkv * G
    b_len, b_start, max_len = torch.tensor([5, 3]), torch.tensor([0, 5]), 6
    b_loc = torch.stack([torch.randperm(slots, generator=g)[:9] for _ in range(B)]).int()
    logits = torch.randn(H, 8, generator=g, dtype=torch.float64)
    v = torch.randn(slots, Hkv, D, generator=g, dtype=torch.float64)
    out = torch.zeros(B, H, D, dtype=torch.float64)
    O.token_softmax_reducev(logits, v, out, b_loc, b_start, b_len, max_len, 0, exact=True)
    for i in range(B):
        L, s = int(b_len[i]), int(b_start[i])
        for h in range(H):
            x = logits[h, s:s + L].numpy()
            p = np.exp(x - x.max())
            p /= p.sum()
            acc = np.zeros(D)
            for t in range(L):
                acc += p[t] * v[int(b_loc[i, max_len - L + t]), h // G].numpy()
            assert np.allclose(out[i, h].numpy(), acc, rtol=1e-13, atol=1e-14)


def test_softmax_reducev_sequence_without_tokens_gives_zeros():
    """functions_lightllm.cpp:98-104 assigns out[i] for every i: with L = 0 the product has an empty inner dimension,
    whose value is zero whatever the row held before; the neighbours are unaffected."""
    g = rng(12)
    v = torch.randn(20, 2, 8, generator=g).half()
    b_loc = torch.stack([torch.randperm(20, generator=g)[:6] for _ in range(3)]).int()
    logits = torch.randn(2, 7, generator=g).half()
    for exact in (False, True):
        out = torch.full((3, 2, 8), 9.0, dtype=torch.float64 if exact else torch.float16)
        O.token_softmax_reducev(logits, v, out, b_loc, torch.tensor([0, 4, 4]), torch.tensor([4, 0, 3]), 5, 0, exact=exact)
        assert bool((out[1] == 0).all()), "an empty sequence must produce zeros"
        assert bool((out[0] != 9.0).all()) and bool((out[2] != 9.0).all())


# ----------------------------------------------------------------------------- context_attention
def _brute_context(q, k, v, start, L):
    H, D = q.shape[1], q.shape[2]
    out = np.zeros((L, H, D))
    qn, kn, vn = (t.double().numpy() for t in (q, k, v))
    for r in range(L):
        for h in range(H):
            s = np.array([np.dot(qn[start + r, h], kn[start + j, h]) for j in range(r + 1)]) / math.sqrt(D)
            p = np.exp(s - s.max())
            p /= p.sum()
            out[r, h] = sum(p[j] * vn[start + j, h] for j in range(r + 1))
    return torch.from_numpy(out)


def test_context_attention_reference_fixtures(golden):
    g = rng(12)
    for case in golden["context_attention"]["cases"][:3]:
        T, H, D = case["shape"]
        H = 4  # the head count does not interact with the segment logic; keep the brute force quick
        q, k, v = (torch.randn(T, H, D, generator=g, dtype=torch.float64) for _ in range(3))
        out = torch.full((T, H, D), 123.0, dtype=torch.float64)
        bs, bl = torch.tensor(case["b_start_loc"]), torch.tensor(case["b_seq_len"])
        O.context_attention(q, k, v, out, bs, bl, case["max_input_len"], exact=True)
        covered = torch.zeros(T, dtype=torch.bool)
        for s, L in zip(case["b_start_loc"], case["b_seq_len"]):
            assert_close(out[s:s + L], _brute_context(q, k, v, s, L), 1e-12, 1e-13, f"segment at {s}")
            assert_bit_equal(out[s], v[s], "first token of a sequence returns its own v row")
            covered[s:s + L] = True
        assert bool((out[~covered] == 123.0).all()), "rows outside every sequence are untouched"
    # the last fixture leaves rows 192..255 untouched (64+64+128 rows used out of 256: starts 0, 64, 128)
    last = golden["context_attention"]["cases"][3]
    assert last["b_start_loc"][-1] + last["b_seq_len"][-1] == 256


def test_context_attention_constant_v_and_decode_cross_check():
    g = rng(13)
    T, H, D = 24, 2, 16
    q, k = (torch.randn(T, H, D, generator=g, dtype=torch.float64) for _ in range(2))
    v = torch.randn(1, H, D, generator=g, dtype=torch.float64).expand(T, H, D).contiguous()
    out = torch.zeros(T, H, D, dtype=torch.float64)
    O.context_attention(q, k, v, out, torch.tensor([0, 10]), torch.tensor([10, 14]), exact=True)
    assert_close(out, v, 1e-13, 1e-14, "constant V")
    # last row of a sequence == decode attention of that row over the same K/V
    v = torch.randn(T, H, D, generator=g, dtype=torch.float64)
    O.context_attention(q, k, v, out, torch.tensor([0, 10]), torch.tensor([10, 14]), exact=True)
    b_loc = torch.arange(10, 24, dtype=torch.int32).reshape(1, 14)
    logits = torch.zeros(H, 14, dtype=torch.float64)
    O.token_attention(q[23:24], k, logits, b_loc, torch.tensor([0]), torch.tensor([14]), 14, exact=True)
    dec = torch.zeros(1, H, D, dtype=torch.float64)
    O.token_softmax_reducev(logits, v, dec, b_loc, torch.tensor([0]), torch.tensor([14]), 14, 0, exact=True)
    assert_close(dec[0], out[23], 1e-12, 1e-13, "prefill last row vs decode")


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_context_attention_dtype_faithful_close_to_exact(dtype):
    g = rng(14)
    T, H, D = 48, 3, 32
    q, k, v = ((torch.randn(T, H, D, generator=g) * 0.5).to(dtype) for _ in range(3))
    bs, bl = torch.tensor([0, 16]), torch.tensor([16, 32])
    out = torch.zeros(T, H, D, dtype=dtype)
    O.context_attention(q, k, v, out, bs, bl)
    ex = torch.zeros(T, H, D, dtype=torch.float64)
    O.context_attention(q, k, v, ex, bs, bl, exact=True)
    tol = 1e-2 if dtype == torch.float16 else 1e-5
    assert_close(out, ex, tol, tol, "reference composition vs float64")


def test_flash_attention_varlen_causal_mha_is_context_attention():
    g = rng(71)
    cu = torch.tensor([0, 16, 48, 64], dtype=torch.int32)  # diopi_configs.py:9866, second case
    q, k, v = (torch.randn(64, 4, 128, generator=g, dtype=torch.float64) for _ in range(3))
    got = O.flash_attention_varlen(q, k, v, cu, cu, None, 32, 32, 0, None, True, -1, -1, exact=True)
    want = torch.zeros_like(q)
    O.context_attention(q, k, v, want, cu[:-1], cu[1:] - cu[:-1], 32, exact=True)
    assert_close(got, want, 1e-12, 1e-12, "causal varlen attention vs the lightllm prefill statement")
    # first token of every sequence: its own value row
    for b in (0, 16, 48):
        assert_close(got[b], v[b], 1e-14, 1e-15, "first token")


def test_flash_attention_varlen_identical_keys_closed_form():
    g = rng(72)
    n, hq, hkv, d, scale = 9, 4, 2, 16, 0.3
    q = torch.randn(n, hq, d, generator=g, dtype=torch.float64)
    key = torch.randn(hkv, d, generator=g, dtype=torch.float64)
    k = key.expand(n, hkv, d).contiguous()
    v = torch.randn(n, hkv, d, generator=g, dtype=torch.float64)
    cu = torch.tensor([0, n])
    for causal in (True, False):
        out, lse = O.flash_attention_varlen(q, k, v, cu, cu, None, n, n, 0, scale, causal, exact=True, return_lse=True)
        for t in range(n):
            cnt = t + 1 if causal else n
            for h in range(hq):
                assert_close(out[t, h], v[:cnt, h // 2].mean(0), 1e-13, 1e-13, "uniform weights -> mean of the visible values")
                want = scale * float(q[t, h] @ key[h // 2]) + math.log(cnt)
                assert abs(float(lse[0, h, t]) - want) < 1e-12


def test_flash_attention_varlen_python_loops():
    g = rng(73)
    cu = [0, 2, 7, 19]  # ragged, as in diopi_configs.py:9866 (fifth case)
    hq, hkv, d, scale = 4, 2, 8, 0.125
    q = torch.randn(19, hq, d, generator=g, dtype=torch.float64)
    k = torch.randn(19, hkv, d, generator=g, dtype=torch.float64)
    v = torch.randn(19, hkv, d, generator=g, dtype=torch.float64)
    for causal in (False, True):
        out, lse = O.flash_attention_varlen(q, k, v, torch.tensor(cu), torch.tensor(cu), None, 12, 12, 0, scale, causal, exact=True, return_lse=True)
        for i in range(3):
            b, e = cu[i], cu[i + 1]
            for t in range(b, e):
                last = t if causal else e - 1
                for h in range(hq):
                    w = [math.exp(scale * sum(float(q[t, h, x]) * float(k[j, h // 2, x]) for x in range(d))) for j in range(b, last + 1)]
                    tot = sum(w)
                    for x in range(d):
                        want = sum(w[j - b] * float(v[j, h // 2, x]) for j in range(b, last + 1)) / tot
                        assert abs(float(out[t, h, x]) - want) < 1e-12
                    assert abs(float(lse[i, h, t - b]) - math.log(tot)) < 1e-12
        assert float(lse[0, :, 2:].abs().max()) == 0.0  # past the end of a short sequence


def test_flash_attention_varlen_dtype_faithful_stays_near_exact():
    g = rng(74)
    cu = torch.tensor([0, 32, 64, 128, 256], dtype=torch.int32)  # diopi_configs.py:9866, third case (full attention)
    q, k, v = (torch.randn(256, 16, 128, generator=g).half() for _ in range(3))
    kk, vv = k[:, :2].contiguous(), v[:, :2].contiguous()  # the grouped case of 9929: 2 key/value heads
    a = O.flash_attention_varlen(q, kk, vv, cu, cu, None, 128, 128, 0, None, False)
    b = O.flash_attention_varlen(q, kk, vv, cu, cu, None, 128, 128, 0, None, False, exact=True)
    assert_close(a.double(), b.double(), 1e-2, 1e-2, "fp16 composition vs float64")


def test_flash_attention_agrees_with_varlen_and_loops():
    g = rng(75)
    b, t, hq, hkv, d, scale = 3, 5, 4, 2, 8, 0.2
    q = torch.randn(b, t, hq, d, generator=g, dtype=torch.float64)
    k = torch.randn(b, t, hkv, d, generator=g, dtype=torch.float64)
    v = torch.randn(b, t, hkv, d, generator=g, dtype=torch.float64)
    cu = torch.arange(0, (b + 1) * t, t)
    for causal in (True, False):
        out, lse = O.flash_attention(q, k, v, None, 0, scale, causal, exact=True, return_lse=True)
        o2, l2 = O.flash_attention_varlen(q.reshape(b * t, hq, d), k.reshape(b * t, hkv, d), v.reshape(b * t, hkv, d), cu, cu, None, t, t, 0, scale, causal,
                                          exact=True, return_lse=True)
        assert_close(out.reshape(b * t, hq, d), o2, 1e-12, 1e-12, "padded vs variable-length restatement")
        assert_close(lse, l2, 1e-12, 1e-12, "log-sum-exp")
        for bi in range(b):
            for ti in range(t):
                last = ti if causal else t - 1
                for h in range(hq):
                    w = [math.exp(scale * float(q[bi, ti, h] @ k[bi, j, h // 2])) for j in range(last + 1)]
                    want = sum(w[j] * v[bi, j, h // 2] for j in range(last + 1)) / sum(w)
                    assert_close(out[bi, ti, h], want, 1e-12, 1e-12, "loops")
                    assert abs(float(lse[bi, h, ti]) - math.log(sum(w))) < 1e-12


def test_prompt_flash_attention_is_context_attention_on_equal_sequences():
    g = rng(81)
    bs, L, H, D = 3, 7, 4, 16
    q, k, v = (torch.randn(bs * L, H * D, generator=g, dtype=torch.float64) for _ in range(3))
    got = O.prompt_flash_attention(q, k, v, None, [L] * bs, L, H, H, D, exact=True)
    want = torch.zeros(bs * L, H, D, dtype=torch.float64)
    O.context_attention(q.view(-1, H, D), k.view(-1, H, D), v.view(-1, H, D), want, torch.arange(0, bs * L, L), torch.full((bs,), L), L, exact=True)
    assert_close(got.view(-1, H, D), want, 1e-12, 1e-12, "padded prompt attention vs the lightllm prefill statement")
    for b in range(bs):  # the first row of a sequence sees only itself
        assert_close(got[b * L], v[b * L], 1e-14, 1e-15, "first row")
    # the dtype-faithful composition on the reference's case shape (diopi_configs.py:9383-9423) stays near the float64 value
    q16, k16, v16 = ((torch.randn(4, 4096, generator=g) * 0.5).half() for _ in range(3))
    mask = torch.tensor([[[False, True], [False, False]]] * 2)
    a = O.prompt_flash_attention(q16, k16, v16, mask, [2, 2], 2, 32, 32, 128)
    b = O.prompt_flash_attention(q16, k16, v16, mask, [2, 2], 2, 32, 32, 128, exact=True)
    assert a.shape == (4, 4096) and a.dtype == torch.float16
    assert_close(a.double(), b.double(), 1e-2, 1e-2, "fp16 composition vs float64")


def test_prompt_flash_attention_python_loops_with_fewer_kv_heads():
    g = rng(82)
    bs, L, H, Hkv, D = 2, 5, 4, 2, 8
    q = torch.randn(bs * L, H * D, generator=g, dtype=torch.float64)
    k = torch.randn(bs * L, Hkv * D, generator=g, dtype=torch.float64)
    v = torch.randn(bs * L, Hkv * D, generator=g, dtype=torch.float64)
    got = O.prompt_flash_attention(q, k, v, None, [L, 3], L, H, Hkv, D, exact=True)  # a shorter actual length changes nothing
    for b in range(bs):
        for t in range(L):
            for h in range(H):
                hk = h // (H // Hkv)
                qv = q[b * L + t, h * D:(h + 1) * D]
                w = [math.exp(float(qv @ k[b * L + j, hk * D:(hk + 1) * D]) / math.sqrt(D)) for j in range(t + 1)]
                want = sum(w[j] * v[b * L + j, hk * D:(hk + 1) * D] for j in range(t + 1)) / sum(w)
                assert_close(got[b * L + t, h * D:(h + 1) * D], want, 1e-12, 1e-12, "loops")
    # one key/value head: the statement's own broadcast (customized_test.py:775) gives the same numbers
    k1, v1 = k[:, :D].contiguous(), v[:, :D].contiguous()
    got1 = O.prompt_flash_attention(q, k1, v1, None, [L, L], L, H, 1, D, exact=True)
    xq = q.view(bs, L, H, D).transpose(1, 2)
    sc = torch.matmul(xq, k1.view(bs, L, 1, D).transpose(1, 2).transpose(2, 3)) / math.sqrt(D)
    sc = sc.masked_fill(torch.triu(torch.ones(L, L, dtype=torch.bool), 1), float("-inf")).softmax(-1)
    want1 = torch.matmul(sc, v1.view(bs, L, 1, D).transpose(1, 2)).transpose(1, 2).reshape(bs * L, H * D)
    assert_close(got1, want1, 1e-12, 1e-12, "broadcast single key/value head")


def test_paged_attention_reference_case_and_block_tables():
    g = rng(83)
    # diopi_configs.py:9425-9468: one sequence of 5 tokens, 32 heads of 128, 1026 cache rows, blocks [0, 1] of 128 rows:
    # the statement (customized_test.py:797-819) reads rows 0..4
    H, D = 32, 128
    q = (torch.randn(1, H * D, generator=g) * 0.5).half()
    k = (torch.randn(1026, H * D, generator=g) * 0.5).half()
    v = (torch.randn(1026, H * D, generator=g) * 0.5).half()
    table = torch.tensor([[0, 1]], dtype=torch.int32)
    mask = torch.zeros(1, 1, 5, dtype=torch.bool)
    got = O.paged_attention(q, k, v, mask, [5], H, H, D, table, 128)
    assert O.paged_rows(table, 0, 5, 128).tolist() == [0, 1, 2, 3, 4]
    kk = k[:5].view(1, 5, H, D).transpose(1, 2)
    logics = (torch.matmul(q.view(1, 1, H, D).transpose(1, 2)[0], kk.transpose(2, 3)) / math.sqrt(D)).reshape(H, 5)
    want = torch.matmul(logics.softmax(-1).reshape(1, H, 1, 5), v[:5].view(1, 5, H, D).transpose(1, 2)).view(1, H * D)
    assert torch.equal(got, want), "the statement's own arithmetic on rows 0..4"
    ex = O.paged_attention(q, k, v, mask, [5], H, H, D, table, 128, exact=True)
    assert_close(got.double(), ex.double(), 1e-2, 1e-2, "fp16 composition vs float64")

    # shuffled block tables, several sequences, grouped heads: explicit loops in float64
    B, H, Hkv, D, bsz = 3, 4, 2, 8, 4
    lens = [6, 0, 9]
    table = torch.tensor([[5, 2, 7], [1, 1, 1], [0, 6, 3]], dtype=torch.int64)
    q = torch.randn(B, H * D, generator=g, dtype=torch.float64)
    k = torch.randn(8 * bsz, Hkv * D, generator=g, dtype=torch.float64)
    v = torch.randn(8 * bsz, Hkv * D, generator=g, dtype=torch.float64)
    got = O.paged_attention(q, k, v, None, lens, H, Hkv, D, table, bsz, exact=True)
    assert O.paged_rows(table, 0, 6, bsz).tolist() == [20, 21, 22, 23, 8, 9]
    assert float(got[1].abs().max()) == 0.0
    for i in (0, 2):
        rows = [int(table[i, t // bsz]) * bsz + t % bsz for t in range(lens[i])]
        for h in range(H):
            hk = h // 2
            w = [math.exp(float(q[i, h * D:(h + 1) * D] @ k[r, hk * D:(hk + 1) * D]) / math.sqrt(D)) for r in rows]
            want = sum(wj * v[r, hk * D:(hk + 1) * D] for wj, r in zip(w, rows)) / sum(w)
            assert_close(got[i, h * D:(h + 1) * D], want, 1e-12, 1e-12, "loops")

    # the same numbers from the two lightllm decode statements on the expanded row table
    maxlen = max(lens)
    b_loc = torch.zeros(B, maxlen, dtype=torch.int64)
    for i in range(B):
        if lens[i]:
            b_loc[i, maxlen - lens[i]:] = O.paged_rows(table, i, lens[i], bsz)
    start = torch.tensor([0, 6, 6])
    blen = torch.tensor(lens)
    logits = torch.zeros(H, sum(lens), dtype=torch.float64)
    O.token_attention(q.view(B, H, D), k.view(-1, Hkv, D), logits, b_loc, start, blen, maxlen, exact=True)
    out = torch.zeros(B, H, D, dtype=torch.float64)
    O.token_softmax_reducev(logits, v.view(-1, Hkv, D), out, b_loc, start, blen, maxlen, 0, exact=True)
    assert_close(got.view(B, H, D), out, 1e-12, 1e-12, "paged attention vs token_attention + token_softmax_reducev")


# ----------------------------------------------------------------------------- fused decoder attention (lmdeploy set)
def _fused_inputs(seed, B, H, Hkv, D, S, layers=2, dtype=torch.float64, bias=True):
    g = rng(seed)
    hid, N = H * D, (H + 2 * Hkv) * D
    x = torch.randn(B, hid, generator=g).to(dtype)
    w = (torch.randn(hid, N, generator=g) / math.sqrt(hid)).to(dtype)
    b = torch.randn(N, generator=g).to(dtype) if bias else None
    kc = torch.randn(layers, B, Hkv, S, D, generator=g).to(dtype)
    vc = torch.randn(layers, B, Hkv, S, D, generator=g).to(dtype)
    return x, w, b, kc, vc


def test_fused_decoder_attention_python_loops():
    """Every step of the header's prose written out with explicit loops in float64 (functions_lmdeploy.h:104-135)."""
    B, H, Hkv, D, S = 3, 4, 2, 8, 6
    x, w, b, kc, vc = _fused_inputs(40, B, H, Hkv, D, S)
    seq = torch.tensor([0, 3, 9])          # the last one has wrapped around the 6-row cache
    pad = torch.tensor([0, 1, 2])
    fin = torch.tensor([False, False, False])
    step, layer, theta = 12, 1, 10000.0
    kc2, vc2 = kc.clone(), vc.clone()
    got = O.fused_decoder_attention_inp(x, w, b, kc2, vc2, fin, pad, seq, step, layer, H, Hkv, D, S, D, theta, exact=True)
    G = H // Hkv
    for bi in range(B):
        qkv = [sum(float(x[bi, i]) * float(w[i, n]) for i in range(H * D)) + float(b[n]) for n in range((H + 2 * Hkv) * D)]
        pos = step - 1 - int(pad[bi])
        heads = [qkv[h * D:(h + 1) * D] for h in range(H + 2 * Hkv)]
        for h in range(H + Hkv):           # q and k heads rotate, v heads do not
            r = list(heads[h])
            for j in range(D // 2):
                ang = pos * theta ** (-2.0 * j / D)
                r[j] = heads[h][j] * math.cos(ang) - heads[h][j + D // 2] * math.sin(ang)
                r[j + D // 2] = heads[h][j] * math.sin(ang) + heads[h][j + D // 2] * math.cos(ang)
            heads[h] = r
        L = int(seq[bi])
        slot = L % S
        for hk in range(Hkv):
            assert_close(kc2[layer, bi, hk, slot], torch.tensor(heads[H + hk], dtype=torch.float64), 1e-12, 1e-12, "cached k row")
            assert_close(vc2[layer, bi, hk, slot], torch.tensor(heads[H + Hkv + hk], dtype=torch.float64), 1e-12, 1e-12, "cached v row")
        toks = [t % S for t in range(max(0, L + 1 - S), L + 1)]
        for h in range(H):
            hk = h // G
            sc = [sum(heads[h][d] * float(kc2[layer, bi, hk, t, d]) for d in range(D)) / math.sqrt(D) for t in toks]
            m = max(sc)
            e = [math.exp(s_ - m) for s_ in sc]
            den = sum(e) + 1e-6
            for d in range(D):
                want = sum(e[i] / den * float(vc2[layer, bi, hk, t, d]) for i, t in enumerate(toks))
                assert abs(float(got[bi, h * D + d]) - want) < 1e-10, (bi, h, d)
    # every other cache row and the other layer are untouched
    keep = torch.ones_like(kc, dtype=torch.bool)
    for bi in range(B):
        keep[layer, bi, :, int(seq[bi]) % S] = False
    assert torch.equal(kc2[keep], kc[keep]) and torch.equal(vc2[keep], vc[keep])


def test_fused_decoder_attention_reduces_to_the_decode_pair():
    """An identity projection at rotary position 0 leaves q, k, v equal to slices of the input: the result must then be
    token_attention + token_softmax_reducev (both pinned above) on the cache rows, for the dtype-faithful mode too."""
    B, H, D, S = 2, 2, 8, 16
    Hkv = H
    for dt in (torch.float64, torch.float16):
        g = rng(41)
        hid = 3 * H * D
        x = torch.randn(B, hid, generator=g).to(dt)
        w = torch.eye(hid).to(dt)          # q = x[:, :HD], k = x[:, HD:2HD], v = x[:, 2HD:]
        kc = torch.randn(1, B, Hkv, S, D, generator=g).to(dt)
        vc = torch.randn(1, B, Hkv, S, D, generator=g).to(dt)
        seq = torch.tensor([4, 7])
        kc2, vc2 = kc.clone(), vc.clone()
        got = O.fused_decoder_attention_inp(x, w, None, kc2, vc2, None, None, seq, 1, 0, H, Hkv, D, S, D, 10000.0, exact=dt == torch.float64)
        for bi in range(B):
            n = int(seq[bi]) + 1
            assert_bit_equal(kc2[0, bi, :, n - 1], x[bi, H * D:2 * H * D].view(Hkv, D), "position 0 and identity weights: k row is the input slice")
            loc = torch.arange(n, dtype=torch.int32).reshape(1, n)
            krows, vrows = kc2[0, bi].transpose(0, 1).contiguous(), vc2[0, bi].transpose(0, 1).contiguous()
            lg = torch.zeros(H, n, dtype=dt)
            O.token_attention(x[bi, :H * D].view(1, H, D), krows, lg, loc, torch.tensor([0]), torch.tensor([n]), n, exact=dt == torch.float64)
            o = torch.zeros(1, H, D, dtype=dt)
            O.token_softmax_reducev(lg, vrows, o, loc, torch.tensor([0]), torch.tensor([n]), n, 0, exact=dt == torch.float64)
            # the eps of the fused form moves the probabilities by at most 1e-6 relative
            tol = dict(rtol=2e-6, atol=1e-9) if dt == torch.float64 else dict(rtol=1e-2, atol=1e-2)
            assert_close(got[bi, :H * D].view(H, D), o[0], what=f"fused vs decode pair {dt}", **tol)
            assert_bit_equal(got[bi, H * D:].to(dt), x[bi, H * D:], "columns past H*D keep their values")


def test_fused_decoder_attention_first_token_and_finished_rows():
    """With nothing cached the output is the projected v row itself (softmax over one token, up to the eps); a finished row
    keeps its hidden state and its cache rows."""
    B, H, Hkv, D, S = 2, 4, 1, 8, 4
    x, w, b, kc, vc = _fused_inputs(42, B, H, Hkv, D, S, layers=1)
    kc2, vc2 = kc.clone(), vc.clone()
    got = O.fused_decoder_attention_inp(x, w, b, kc2, vc2, torch.tensor([False, True]), None, torch.tensor([0, 2]), 1, 0, H, Hkv, D, S, D, 10000.0, exact=True)
    v_row = (x[0] @ w + b)[(H + Hkv) * D:]
    for h in range(H):
        assert_close(got[0, h * D:(h + 1) * D], v_row / (1 + 1e-6), 1e-12, 1e-12, "one token: its v row")
    assert torch.equal(got[1], x[1]) and torch.equal(kc2[0, 1], kc[0, 1]) and torch.equal(vc2[0, 1], vc[0, 1])
