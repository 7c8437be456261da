"""Comparison helpers shared by the parity tests.

`assert_close` is the reference harness's criterion (check_result.py:138-149 of the reference:
|dev - ref| <= atol + rtol * |ref|, with at most a small fraction of elements allowed to miss),
made strict here: no element may miss unless `mismatch_ratio` says otherwise.
"""
import numpy as np
import torch

# The bars this build is held to: bit-exact for index work; fp32 rtol 1e-5; 16-bit atol = rtol = 1e-2.
# atol for fp32 is the reference harness's own default (global_settings.py:4-15).
TOL = {
    torch.float64: dict(rtol=1e-9, atol=1e-9),
    torch.float32: dict(rtol=1e-5, atol=1e-5),
    torch.float16: dict(rtol=1e-2, atol=1e-2),
    torch.bfloat16: dict(rtol=1e-2, atol=1e-2),
}


def report(dev: torch.Tensor, ref: torch.Tensor):
    d = dev.detach().double().cpu()
    r = ref.detach().double().cpu()
    diff = (d - r).abs()
    max_abs = float(diff.max()) if diff.numel() else 0.0
    denom = r.abs().clamp_min(1e-30)
    max_rel = float((diff / denom).max()) if diff.numel() else 0.0
    return max_abs, max_rel


def assert_close(dev: torch.Tensor, ref: torch.Tensor, rtol: float, atol: float, what: str = "", mismatch_ratio: float = 0.0):
    assert tuple(dev.shape) == tuple(ref.shape), f"{what}: shape {tuple(dev.shape)} vs {tuple(ref.shape)}"
    d = dev.detach().double().cpu().numpy()
    r = ref.detach().double().cpu().numpy()
    ok = np.isclose(d, r, rtol=rtol, atol=atol, equal_nan=True)
    bad = ok.size - int(ok.sum())
    if bad > mismatch_ratio * ok.size:
        max_abs, max_rel = report(dev, ref)
        idx = np.argwhere(~ok)[:5]
        raise AssertionError(f"{what}: {bad}/{ok.size} elements outside rtol={rtol} atol={atol}; max_abs={max_abs:.3e} max_rel={max_rel:.3e}; "
                             f"first misses at {idx.tolist()}: dev={d[tuple(idx[0])]} ref={r[tuple(idx[0])]}")


def assert_bit_equal(dev: torch.Tensor, ref: torch.Tensor, what: str = ""):
    assert dev.dtype == ref.dtype and tuple(dev.shape) == tuple(ref.shape), what
    a = dev.detach().cpu().contiguous().view(torch.uint8)
    b = ref.detach().cpu().contiguous().view(torch.uint8)
    assert torch.equal(a, b), f"{what}: tensors differ bitwise ({int((a != b).sum())} bytes)"
