"""The measurement probes of bench.py (diopi_amd/lib/libdiopi_probes.so): the library loads and refuses bad arguments without a
device; on the device the gather probe writes exactly the bytes its description says and the matrix-rate probe reports clocks."""
import ctypes
import os

import numpy as np
import pytest
import torch

from diopi_amd import runtime as rt

LIB = os.path.join(os.path.dirname(rt.IMPL_LIB_PATH), "libdiopi_probes.so")


def _lib():
    lib = ctypes.CDLL(LIB)
    lib.diopiProbeTokenGather.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                          ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                          ctypes.c_int]
    lib.diopiProbeCopy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int]
    lib.diopiProbeMatrixRate.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 4
    return lib


def test_probe_library_loads_and_refuses_bad_arguments():
    lib = _lib()
    for name in ("diopiProbeTokenGather", "diopiProbeCopy", "diopiProbeMatrixRate"):
        assert hasattr(lib, name)
    # every refusal comes before the first device call
    assert lib.diopiProbeCopy(None, None, None, 24, 4) == 1            # not a multiple of 16 bytes
    assert lib.diopiProbeCopy(None, None, None, 0, 4) == 1
    assert lib.diopiProbeMatrixRate(None, None, None, 4, 3, 10, 0) == 1  # 4 or 8 waves
    assert lib.diopiProbeMatrixRate(None, None, None, 0, 4, 10, 0) == 1
    ok = dict(mode=3, row=2048, mil=64, batch=2, maxlen=64, stride=4096, pieces=4, bpt=128, tile=128, split=2)

    def gather(**kw):
        a = dict(ok, **kw)
        return lib.diopiProbeTokenGather(None, a["mode"], None, a["row"], None, a["mil"], None, None, a["batch"], a["maxlen"], None, a["stride"], a["pieces"],
                                         a["bpt"], a["tile"], a["split"])

    assert gather(mode=0) == 1 and gather(mode=8) == 1 and gather(mode=4) == 1 and gather(mode=16) == 1
    assert gather(row=2000) == 1                # a part of a row is 16 bytes times a power of two
    assert gather(split=3) == 1
    assert gather(pieces=3) == 1                # the bytes of a token divide evenly over the pieces
    assert gather(stride=4100) == 1
    assert gather(tile=100, pieces=128) == 1    # a piece of a tile is whole 16-byte packets
    assert gather(batch=0) == 1


@pytest.mark.gpu
def test_gather_probe_writes_the_bytes_of_its_tiles_and_nothing_else():
    lib = _lib()
    dev = "cuda"
    slots, row_bytes, mil = 4096, 2048, 700
    lengths = [5, 300, 700, 129]
    B = len(lengths)
    g = torch.Generator().manual_seed(7)
    cache = torch.randint(0, 255, (slots, row_bytes), dtype=torch.uint8, generator=g).to(dev)
    loc = torch.stack([torch.randperm(slots, generator=g)[:mil] for _ in range(B)]).int().to(dev)
    start = torch.tensor(np.concatenate(([0], np.cumsum(lengths)[:-1])), dtype=torch.int32, device=dev)
    length = torch.tensor(lengths, dtype=torch.int32, device=dev)
    total = sum(lengths)
    heads, e, tile = 32, 2, 128
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for pieces, split in ((heads, 1), (heads, 2), (2 * heads, 4), (4, 1), (1, 2)):
        per_token = heads * e // pieces
        stride = (total * per_token + 15) // 16 * 16 + 64
        out = torch.zeros(pieces * stride, dtype=torch.uint8, device=dev)
        for mode in (2, 3, 7, 15):
            out.zero_()
            assert lib.diopiProbeTokenGather(stream, mode, cache.data_ptr(), row_bytes, loc.data_ptr(), mil, start.data_ptr(), length.data_ptr(), B, max(lengths),
                                             out.data_ptr(), stride, pieces, heads * e, tile, split) == 0
            torch.cuda.synchronize()
            got = out.cpu().numpy().reshape(pieces, stride)
            want = np.zeros((pieces, stride), dtype=bool)
            for i, L in enumerate(lengths):
                for t0 in range(0, L, tile):
                    n = min(tile, L - t0)
                    first = ((int(start[i]) + t0) * per_token) // 16 * 16
                    want[:, first: first + (n * per_token) // 16 * 16] = True
            # every packet the probe stores holds (acc, acc + 1, acc + 2, acc + 3) with acc >= the thread index: never four zero words
            words = got.view(np.uint32).reshape(pieces, -1, 4)
            written = (words != 0).any(axis=2)
            wantp = want.reshape(pieces, -1, 16).all(axis=2)
            assert (written[~wantp] == False).all(), (pieces, split, mode)  # noqa: E712
            assert written[wantp].all(), (pieces, split, mode)
        # reads only: the output is left alone
        out.zero_()
        assert lib.diopiProbeTokenGather(stream, 1, cache.data_ptr(), row_bytes, loc.data_ptr(), mil, start.data_ptr(), length.data_ptr(), B, max(lengths),
                                         out.data_ptr(), stride, pieces, heads * e, tile, split) == 0
        torch.cuda.synchronize()
        assert int(out.count_nonzero()) == 0


@pytest.mark.gpu
def test_copy_and_matrix_rate_probes():
    lib = _lib()
    dev = "cuda"
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    n = 16 * (4096 * 3 + 5)   # whole groups of four packets and a tail
    src = torch.randint(0, 255, (n,), dtype=torch.uint8, device=dev)
    dst = torch.zeros_like(src)
    assert lib.diopiProbeCopy(stream, dst.data_ptr(), src.data_ptr(), n, 7) == 0
    torch.cuda.synchronize()
    assert torch.equal(src, dst)
    for waves in (4, 8):
        for bf16 in (0, 1):
            clocks = torch.zeros(3 * waves * 2, dtype=torch.int64, device=dev)
            sink = torch.zeros(4, dtype=torch.float32, device=dev)
            assert lib.diopiProbeMatrixRate(stream, clocks.data_ptr(), sink.data_ptr(), 3, waves, 50, bf16) == 0
            torch.cuda.synchronize()
            c = clocks.cpu().view(-1, 2)
            # 800 products of 32 matrix-pipe clocks each (16 when two waves share a SIMD and overlap perfectly)
            assert (c[:, 0] >= 50 * 16 * 16).all() and (c[:, 1] > 0).all()
            assert float(sink.abs().sum()) == 0.0


@pytest.mark.gpu
@pytest.mark.timeout(600)
def test_bench_probe_modes_run_and_print_json():
    """`bench.py --probe ...` end to end in a child process: every line it prints is JSON and the expected entries are there."""
    import json
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for mode, extra, needle in (("matrix-rate", [], "v_mfma_f32_32x32x16_f16"), ("token-attention-floor", ["--only", "cfg3"], "gather + logits-sized write"),
                                ("sustained-clock", ["--probe-seconds", "3.5"], "all-zero tensors")):
        r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--probe", mode, "--steps", "5", "--warmup", "2", "--warm-seconds", "0"] + extra,
                           cwd=root, capture_output=True, text=True, timeout=500)
        assert r.returncode == 0, r.stderr[-2000:]
        lines = [json.loads(ln) for ln in r.stdout.splitlines() if ln.strip()]
        assert lines and lines[0]["probe"] == mode
        assert any(needle in str(ln.get("what", "")) for ln in lines), lines
        for ln in lines[1:]:
            assert ln.get("us", ln.get("ms", ln.get("ms_per_call", 0))) > 0
        if mode == "sustained-clock" and lines[0]["readings_total"] > 0:
            # where the board's tool answers at all: every reading taken under load is a plausible shader clock, never more than a
            # step above the device's maximum (a phase may go without a reading when the tool is slow: the test runs them for 3.5 s)
            seen = [ln for ln in lines[1:] if ln["readings"] >= 1]
            assert all(100 < ln["sclk_MHz_median"] <= lines[0]["device_max_clock_MHz"] + 50 for ln in seen), lines
