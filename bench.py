#!/usr/bin/env python3
"""Benchmark of the gfx950 DIOPI LLaMA-inference operators on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only cfg3] [--no-cpu]

A "step" is one pass of the decode hot path at the configured decode shape (fp16, batch 64,
32 heads x 128, KV cache [131072, 32, 128], lengths ~U(512, 2048)): two diopiDestIndexCopyKV calls
(new K rows, new V rows), diopiTokenAttentionInference and diopiTokenSoftmaxReduceVInference.
`value` is decode tokens/s (batch / step time).  The same JSON line carries, under "ops", the
achieved HBM GB/s (or TFLOP/s) and roofline fraction of every operator at every configured shape,
each next to the CPU restatement of the reference timed on this box's host cores.

Timing: inputs resident in HBM; W untimed warm-up steps; K timed steps bracketed by HIP events on the
stream the kernels are launched on (and a device synchronisation on both sides).  Operators whose
working set is near the 256 MB last-level cache rotate over three buffer sets.
Algorithmic bytes / flops are the formulas in diopi_amd/workloads.py.
"""
import argparse
import ctypes
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2500.0    # dense fp16 / bf16
WARM_SECONDS = 0.3          # untimed load before every timed region (clock ramp)
# HBM bytes per launch of the two decode kernels at the seeded cfg3 workload, measured with `rocprofv3 --pmc FETCH_SIZE`
# and `--pmc WRITE_SIZE` (one counter per run).  The counters cannot be read from inside this script: the readings, the
# scale of each counter (what it reads for a plain copy of known size) and the commands are kept in the file below,
# which is rewritten whenever the decode kernels change; a line `<kernel> total_cached_tokens=<n> hbm_bytes=<b>` per kernel.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "decode_kernels_cfg3_hbm_traffic.txt")


def measured_traffic(kernel, total_tokens):
    """HBM bytes per launch of `kernel` from the tracked counter summary, or None when it has no line for this workload."""
    try:
        with open(TRAFFIC_FILE) as f:
            for ln in f:
                parts = ln.split()
                if len(parts) >= 3 and parts[0] == kernel and parts[1] == f"total_cached_tokens={total_tokens}" and parts[2].startswith("hbm_bytes="):
                    return int(parts[2].split("=", 1)[1])
    except OSError:
        pass
    return None


def token_attention_floor(args, torch, rt, W, impl, ctx, check):
    """What the memory system charges for diopiTokenAttentionInference's access pattern at the cfg5 shape (cfg3 with --only cfg3),
    without arithmetic.

    Times, on the operator's own inputs and stream: the operator; a gather of the same cache rows through the same b_loc
    windows (256-token tiles, one work-group each); the gather plus a write of the logits' volume cut into pieces of 256
    bytes to 32 KiB per tile (512 bytes, one run per head, is the layout the interface prescribes); the writes alone; and a
    plain copy of the same number of bytes.  Prints one JSON line per measurement."""
    lib = ctypes.CDLL(os.path.join(os.path.dirname(rt.IMPL_LIB_PATH), "libdiopi_probes.so"))
    lib.diopiProbeTokenGather.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                          ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
    lib.diopiProbeCopy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int]
    dev = "cuda:0"
    which = "cfg3" if "cfg3" in args.only else "cfg5"
    w = W.cfg3(dev, seed=3) if which == "cfg3" else W.cfg5(dev, seed=5)
    B, H, Hkv, D, total, mil = w["B"], w["H"], w["Hkv"], w["D"], w["total_len"], w["max_input_len"]
    e = 2
    row_bytes = Hkv * D * e
    tile = 256
    logits = torch.zeros(H, total, dtype=w["dtype"], device=dev)
    h = {k: rt.Tensor(w[k]) for k in ("k_cache", "q", "b_loc", "b_seq_len", "b_start_loc")}
    h["logits"] = rt.Tensor(logits)
    assert w["b_loc"].dtype == torch.int32 and w["b_seq_len"].dtype == torch.int32 and w["b_start_loc"].dtype == torch.int32
    stream = ctypes.c_void_p(ctx.torch_stream.cuda_stream)
    max_len = int(w["b_seq_len"].max())
    read_bytes = total * row_bytes
    write_bytes = total * H * e
    out = torch.zeros(write_bytes + 65536, dtype=torch.uint8, device=dev)
    src = torch.zeros(read_bytes, dtype=torch.uint8, device=dev)
    dst = torch.zeros(read_bytes, dtype=torch.uint8, device=dev)

    def timed(fn, steps=args.steps, warmup=args.warmup):
        for _ in range(warmup):
            fn()
        ctx.synchronize()
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < args.warm_seconds:
            for _ in range(8):
                fn()
            ctx.synchronize()
        e0, e1 = rt.Event(), rt.Event()
        e0.record(ctx)
        for _ in range(steps):
            fn()
        e1.record(ctx)
        ms = e0.elapsed_ms(e1)
        ctx.synchronize()
        return ms / steps * 1e3

    def say(**kw):
        print(json.dumps(kw), flush=True)

    def gather(mode, pieces, split, tile=tile):
        per_piece = (total * H * e // pieces + 15) // 16 * 16
        r = lib.diopiProbeTokenGather(stream, mode, w["k_cache"].data_ptr(), row_bytes, w["b_loc"].data_ptr(), mil, w["b_start_loc"].data_ptr(),
                                      w["b_seq_len"].data_ptr(), B, max_len, out.data_ptr(), per_piece, pieces, H * e, tile, split)
        assert r == 0, "diopiProbeTokenGather refused its arguments"

    say(probe="token-attention-floor", workload="%s %s [B=%d, H=%d, Hkv=%d, D=%d]" % (which, str(w["dtype"])[6:], B, H, Hkv, D), tokens=total, read_MB=round(read_bytes / 1e6, 1),
        logits_MB=round(write_bytes / 1e6, 1), tile_tokens=tile, steps=args.steps)
    us = timed(lambda: check(impl.diopiTokenAttentionInference(ctx.handle, h["logits"].handle, h["q"].handle, h["k_cache"].handle, h["b_loc"].handle,
                                                               h["b_start_loc"].handle, h["b_seq_len"].handle, mil), "diopiTokenAttentionInference"))
    say(what="diopiTokenAttentionInference", us=round(us, 1), GBs=round((read_bytes + write_bytes) / us / 1e3, 1))
    # the read side alone, for each way of sharing a row between work-groups and each cache policy; the best one carries the writes
    best = None
    for split in (1, 2, 4, 8, 16, 32):
        if row_bytes // split > 4096 or row_bytes // split < 256:
            continue
        for nt in (0, 4):
            for tt in (128, 256):
                us = timed(lambda: gather(1 + nt, H, split, tt))
                us_few = timed(lambda: gather(1 + nt + 8, H, split, tt))
                say(what="gather only", row_bytes_per_work_group=row_bytes // split, non_temporal=bool(nt), tile_tokens=tt, us=round(us, 1),
                    GBs=round(read_bytes / us / 1e3, 1), us_two_loads_in_flight=round(us_few, 1))
                if tt == tile and (best is None or us < best[0]):
                    best = (us, split, nt)
    _, split, nt = best
    for pieces in (2 * H, H, H // 2, H // 4, H // 16, 1):
        piece_bytes = tile * H * e // pieces
        us_both = timed(lambda: gather(3 + nt, pieces, split))
        us_few = timed(lambda: gather(3 + nt + 8, pieces, split))
        us_wr = timed(lambda: gather(2, pieces, split))
        say(what="gather + logits-sized write", row_bytes_per_work_group=row_bytes // split, non_temporal=bool(nt), piece_bytes=piece_bytes,
            interface_layout=(pieces == H), us=round(us_both, 1), GBs=round((read_bytes + write_bytes) / us_both / 1e3, 1),
            us_two_loads_in_flight=round(us_few, 1), write_only_us=round(us_wr, 1))
    wgs = 8 * int(rt.libs().rt.diopirtDeviceComputeUnits(0))
    us = timed(lambda: lib.diopiProbeCopy(stream, dst.data_ptr(), src.data_ptr(), read_bytes, wgs))
    say(what="plain copy of the read volume", us=round(us, 1), GBs=round(2 * read_bytes / us / 1e3, 1))


def matrix_rate(args, torch, rt, W, impl, ctx, check):
    """The rate and the clock a loop of nothing but v_mfma_f32_32x32x16 products sustains on every compute unit (operands in
    registers, finite non-trivial values), and diopiContextAttentionInference at cfg4 in the same process: the published
    2.5 PFLOP/s is 1024 flop per clock and SIMD at 2.4 GHz; under a sustained matrix load the part runs slower."""
    lib = ctypes.CDLL(os.path.join(os.path.dirname(rt.IMPL_LIB_PATH), "libdiopi_probes.so"))
    lib.diopiProbeMatrixRate.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 4
    dev = "cuda:0"
    cus = int(rt.libs().rt.diopirtDeviceComputeUnits(0))
    stream = ctypes.c_void_p(ctx.torch_stream.cuda_stream)
    sink = torch.zeros(4, dtype=torch.float32, device=dev)
    iters = 40000  # 640 000 products per wave: about 10 ms

    def say(**kw):
        print(json.dumps(kw), flush=True)

    say(probe="matrix-rate", compute_units=cus, products_per_wave=16 * iters, flop_per_product=32768)
    for name, bf16 in (("f16", 0), ("bf16", 1)):
        for waves in (4, 8):
            clocks = torch.zeros(cus * waves * 2, dtype=torch.int64, device=dev)
            for _ in range(3):  # the first launches bring the part to its sustained state
                assert lib.diopiProbeMatrixRate(stream, clocks.data_ptr(), sink.data_ptr(), cus, waves, iters, bf16) == 0
            ctx.synchronize()
            e0, e1 = rt.Event(), rt.Event()
            e0.record(ctx)
            assert lib.diopiProbeMatrixRate(stream, clocks.data_ptr(), sink.data_ptr(), cus, waves, iters, bf16) == 0
            e1.record(ctx)
            ms = e0.elapsed_ms(e1)
            ctx.synchronize()
            c = clocks.cpu().view(-1, 2).double()
            flop = cus * waves * iters * 16 * 32768.0
            ghz = float((c[:, 0] / c[:, 1]).mean()) * 0.1
            # pipe share: 32 clocks per product and SIMD over the shader clocks the slowest wave of a SIMD needed
            per_simd = waves // 4
            pipe = per_simd * iters * 16 * 32.0 / float(c[:, 0].max())
            say(what="v_mfma_f32_32x32x16_" + name, waves_per_simd=per_simd, ms=round(ms, 3), TFLOPs=round(flop / ms / 1e9, 1),
                shader_GHz=round(ghz, 3), matrix_pipe_busy=round(pipe, 3))
    w4 = W.cfg4(dev, seed=4)
    flops = W.context_attention_flops(w4["seq_len_host"], w4["H"], w4["D"])
    for name, dt in (("f16", torch.float16), ("bf16", torch.bfloat16)):
        q, k, v = (w4[x].to(dt) for x in ("q", "k", "v"))
        out = torch.zeros_like(q)
        h = {n_: rt.Tensor(t) for n_, t in (("q", q), ("k", k), ("v", v), ("out", out), ("start", w4["b_start_loc"]), ("len", w4["b_seq_len"]))}

        def call():
            check(impl.diopiContextAttentionInference(ctx.handle, h["out"].handle, h["q"].handle, h["k"].handle, h["v"].handle, h["start"].handle,
                                                      h["len"].handle, w4["max_input_len"]), "diopiContextAttentionInference")
            ctx.clear_tensors()

        for _ in range(args.warmup + 200):
            call()
        ctx.synchronize()
        e0, e1 = rt.Event(), rt.Event()
        e0.record(ctx)
        for _ in range(args.steps):
            call()
        e1.record(ctx)
        ms = e0.elapsed_ms(e1) / args.steps
        ctx.synchronize()
        say(what="diopiContextAttentionInference cfg4 " + name, ms=round(ms, 4), TFLOPs=round(flops / ms / 1e9, 1))


# Child process of the sustained-clock probe: reads the board's shader clock (and power, where the tool reports it) twice a
# second with rocm-smi and prints "unix_time MHz watts" lines until its standard input closes.  Started before the parent
# touches the GPU; it never opens the device itself.
CLOCK_SAMPLER = r"""
import re, select, subprocess, sys, time
while not select.select([sys.stdin], [], [], 0.5)[0]:
    try:
        txt = subprocess.run(["rocm-smi", "--showclocks", "--showpower"], capture_output=True, text=True, timeout=10).stdout
    except Exception:
        continue
    clk = re.search(r"sclk clock level: \d+: \((\d+)Mhz\)", txt)
    pw = re.search(r"Power \(W\): ([0-9.]+)", txt)
    if clk:
        print(time.time(), clk.group(1), pw.group(1) if pw else "nan", flush=True)
"""


def sustained_clock(args, torch, rt, W, impl, ctx, check, sampler):
    """What shader clock the board holds while one operator runs back to back (--probe-seconds each, 7 by default): the prefill operator at
    cfg4 on fp16 tensors, on bf16 tensors and on all-zero tensors, and the two decode operators at cfg3.  The readings come
    from rocm-smi in a child process; a JSON line per workload with the median of the readings taken after the first 2 s."""
    from diopi_amd.runtime import Tensor
    dev = "cuda:0"
    phases = []

    def run(name, call, seconds=args.probe_seconds):
        for _ in range(20):
            call()
        ctx.synchronize()
        t0 = time.time()
        n = 0
        while time.time() - t0 < seconds:
            for _ in range(200):
                call()
            ctx.synchronize()
            n += 200
        t1 = time.time()
        phases.append((name, t0, t1, (t1 - t0) / n * 1e3))

    w4 = W.cfg4(dev, seed=4)
    flops = W.context_attention_flops(w4["seq_len_host"], w4["H"], w4["D"])
    hs, hl = Tensor(w4["b_start_loc"]), Tensor(w4["b_seq_len"])
    for name, make in (("diopiContextAttentionInference cfg4 fp16", lambda t: t), ("diopiContextAttentionInference cfg4 tokens in bf16", lambda t: t.to(torch.bfloat16)),
                       ("diopiContextAttentionInference cfg4 shape, all-zero tensors", torch.zeros_like)):
        q, k, v = (make(w4[n]) for n in ("q", "k", "v"))
        o = torch.zeros_like(q)
        h = {n: Tensor(t) for n, t in dict(q=q, k=k, v=v, o=o).items()}

        def prefill():
            check(impl.diopiContextAttentionInference(ctx.handle, h["o"].handle, h["q"].handle, h["k"].handle, h["v"].handle, hs.handle, hl.handle,
                                                      w4["max_input_len"]), "diopiContextAttentionInference")
            ctx.clear_tensors()

        run(name, prefill)
    del w4, q, k, v, o, h
    torch.cuda.empty_cache()
    w3 = W.cfg3(dev, seed=3)
    logits = torch.zeros(w3["H"], w3["total_len"], dtype=w3["dtype"], device=dev)
    out = torch.zeros_like(w3["q"])
    h3 = {n: Tensor(w3[n]) for n in ("k_cache", "v_cache", "q", "b_loc", "b_seq_len", "b_start_loc")}
    hlg, hout = Tensor(logits), Tensor(out)

    def decode():
        check(impl.diopiTokenAttentionInference(ctx.handle, hlg.handle, h3["q"].handle, h3["k_cache"].handle, h3["b_loc"].handle, h3["b_start_loc"].handle,
                                                h3["b_seq_len"].handle, w3["max_input_len"]), "diopiTokenAttentionInference")
        check(impl.diopiTokenSoftmaxReduceVInference(ctx.handle, hout.handle, hlg.handle, h3["v_cache"].handle, h3["b_loc"].handle, h3["b_start_loc"].handle,
                                                     h3["b_seq_len"].handle, w3["max_input_len"], 0), "diopiTokenSoftmaxReduceVInference")
        ctx.clear_tensors()

    run("diopiTokenAttentionInference + diopiTokenSoftmaxReduceVInference cfg3", decode)
    sampler.stdin.close()
    readings = []
    for ln in sampler.stdout:
        parts = ln.split()
        if len(parts) == 3:
            readings.append((float(parts[0]), float(parts[1]), float(parts[2])))
    sampler.wait(timeout=30)
    nominal = int(rt.libs().rt.diopirtDeviceClockKHz(0)) / 1000.0
    print(json.dumps(dict(probe="sustained-clock", source="rocm-smi --showclocks --showpower, two readings a second from a child process",
                          device_max_clock_MHz=nominal, readings_total=len(readings))), flush=True)
    for name, t0, t1, ms in phases:
        mine = sorted(r for r in readings if t0 + 2.0 <= r[0] <= t1)
        clk = sorted(r[1] for r in mine)
        pw = sorted(r[2] for r in mine if r[2] == r[2])
        e = dict(what=name, ms_per_call=round(ms, 4), readings=len(clk), sclk_MHz_median=clk[len(clk) // 2] if clk else None,
                 sclk_MHz_min=clk[0] if clk else None, sclk_MHz_max=clk[-1] if clk else None, power_W_median=pw[len(pw) // 2] if pw else None)
        if "ContextAttention" in name:
            e["TFLOPs"] = round(flops / ms / 1e9, 1)
            if clk:
                e["fraction_of_max_clock"] = round(clk[len(clk) // 2] / nominal, 3)
        print(json.dumps(e), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-diagnostic", action="store_true", help="skip the entries marked diagnostic (counter runs: they launch the same kernels on other data)")
    ap.add_argument("--only", type=str, default="", help="comma-separated subset of cfg1,cfg2,penalty,cfg3,cfg4,cfg5")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--probe", type=str, default="", help="instead of the benchmark, run a probe: token-attention-floor (the memory cost of TokenAttention's access pattern at cfg5) "
                    "matrix-rate (what a loop of nothing but matrix products sustains, beside the prefill kernel at cfg4) or sustained-clock (the shader clock the board "
                    "holds under the prefill and decode operators, read with rocm-smi)")
    ap.add_argument("--probe-seconds", type=float, default=7.0, help="sustained-clock: how long each workload runs (the first 2 s of readings are dropped)")
    ap.add_argument("--warm-seconds", type=float, default=WARM_SECONDS, help="untimed load before every timed region, on top of --warmup")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the headline CPU baseline sample")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every operator here is a single-device kernel and nothing in this build "
              "uses a second GPU (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    sampler = None
    if args.probe == "sustained-clock":  # the reader of the board's clock starts before this process touches the GPU
        import subprocess
        sampler = subprocess.Popen([sys.executable, "-c", CLOCK_SAMPLER], stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)

    import torch

    from diopi_amd import runtime as rt
    from diopi_amd import workloads as W
    from diopi_amd.runtime import Sizes, Tensor

    if not torch.cuda.is_available() or rt.device_count() < 1:
        print("bench.py needs a GPU: the operators have no CPU path", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)
    dev = "cuda:0"
    impl = rt.libs().impl
    ctx = rt.Context()
    K, Wm = args.steps, args.warmup
    only = set(x for x in args.only.split(",") if x)
    cores = torch.get_num_threads()
    # the first processor's identification as /proc/cpuinfo gives it: model name plus the numeric family / model / stepping
    cpu_model = "unknown"
    try:
        ident = {}
        with open("/proc/cpuinfo") as f:
            for ln in f:
                if ":" not in ln:
                    if ident:
                        break
                    continue
                key, val = (x.strip() for x in ln.split(":", 1))
                if key in ("vendor_id", "model name", "cpu family", "model", "stepping", "cpu MHz"):
                    ident[key] = val
        if ident:
            cpu_model = "{} ({}, family {} model {} stepping {}, {} MHz)".format(
                ident.get("model name", "?"), ident.get("vendor_id", "?"), ident.get("cpu family", "?"), ident.get("model", "?"),
                ident.get("stepping", "?"), ident.get("cpu MHz", "?"))
    except OSError:
        pass

    def check(ret, what):
        rt.check_returncode(ret, what)

    if args.probe:
        if args.probe == "token-attention-floor":
            token_attention_floor(args, torch, rt, W, impl, ctx, check)
        elif args.probe == "matrix-rate":
            matrix_rate(args, torch, rt, W, impl, ctx, check)
        elif args.probe == "sustained-clock":
            sustained_clock(args, torch, rt, W, impl, ctx, check, sampler)
        else:
            print("unknown probe %r (known: token-attention-floor, matrix-rate, sustained-clock)" % args.probe, file=sys.stderr)
            sys.exit(2)
        return

    class Timing(float):
        """Average milliseconds per step of one timed region, with the median and minimum over its blocks."""
        median = minimum = None

    def timed(step_fn, steps=K, warmup=Wm):
        """Average milliseconds per call of step_fn(i), events on the context's stream."""
        for i in range(warmup):
            step_fn(i)
        ctx.synchronize()
        # the GPU only reaches its sustained clocks after a few hundred milliseconds of load: keep warming up (untimed)
        # until that much time has passed, so that the K timed steps do not include the ramp
        t_warm = time.perf_counter()
        i = warmup
        while time.perf_counter() - t_warm < args.warm_seconds:
            for _ in range(8):
                step_fn(i)
                i += 1
            ctx.synchronize()
        torch.cuda.synchronize()
        # one event before the K steps, one after each block of about a tenth of them: the K steps are timed as one
        # region (the average), and the blocks give a median and a minimum without an event behind every launch
        nblocks = max(1, min(10, steps // 5))
        bounds = [round(b * steps / nblocks) for b in range(nblocks + 1)]
        events = [rt.Event() for _ in range(nblocks + 1)]
        events[0].record(ctx)
        for b in range(nblocks):
            for i in range(bounds[b], bounds[b + 1]):
                step_fn(i)
            events[b + 1].record(ctx)
        ms = events[0].elapsed_ms(events[-1])
        per_block = sorted(events[b].elapsed_ms(events[b + 1]) / (bounds[b + 1] - bounds[b]) for b in range(nblocks))
        ctx.synchronize()
        torch.cuda.synchronize()
        t = Timing(ms / steps)
        t.median, t.minimum = per_block[len(per_block) // 2], per_block[0]
        return t

    def cpu_time(fn, budget_s=3.0, min_reps=1, max_reps=5):
        """Median seconds of fn() on the host after one warm-up, bounded by a time budget."""
        fn()
        ts = []
        t_all = time.perf_counter()
        while len(ts) < max_reps and (len(ts) < min_reps or time.perf_counter() - t_all < budget_s):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        ts.sort()
        return ts[len(ts) // 2]

    ops = []
    # the matrix peak the published figure corresponds to, worked out from what the device reports: compute units x 4 SIMDs
    # x 1024 flop per clock and SIMD (v_mfma_f32_32x32x16: 32768 flop in 32 clocks) x the maximum shader clock
    props = torch.cuda.get_device_properties(0)
    clock_khz, cus = int(rt.libs().rt.diopirtDeviceClockKHz(0)), int(rt.libs().rt.diopirtDeviceComputeUnits(0))
    device_peak = {"name": props.name, "compute_units": cus, "max_clock_MHz": clock_khz / 1000.0,
                   "mfma_f16_TFLOPs_from_device": round(cus * 4 * 1024 * clock_khz * 1e3 / 1e12, 1)}

    def record(name, cfg, ms, work, bound, dtype, cpu=None, note=None):
        e = dict(op=name, config=cfg, dtype=dtype, ms=round(ms, 5), bound=bound)
        if getattr(ms, "median", None) is not None:
            e.update(ms_median=round(ms.median, 5), ms_min=round(ms.minimum, 5))
        if bound == "hbm":
            ach = work / (ms * 1e-3) / 1e9
            e.update(bytes=int(work), achieved_GBs=round(ach, 1), frac=round(ach / HBM_PEAK_GBS, 4))
        else:
            ach = work / (ms * 1e-3) / 1e12
            e.update(flops=int(work), achieved_TFLOPs=round(ach, 2), frac=round(ach / MFMA_PEAK_TFLOPS, 4))
        if cpu is not None:
            e["cpu"] = cpu
        if note:
            e["note"] = note
        ops.append(e)
        print("# " + json.dumps(e), file=sys.stderr, flush=True)
        return e

    from oracle import ref_ops as O  # the CPU baseline leg only

    # ------------------------------------------------------------------ cfg1: RMSNorm fwd + bwd, fp32
    if not only or "cfg1" in only:
        sets = [W.cfg1(dev, seed=1 + s) for s in range(3)]
        n1, n2 = sets[0]["n1"], sets[0]["n2"]
        ns = Sizes((n2,))
        hs = []
        for s in sets:
            s["out"] = torch.empty_like(s["x"])
            s["inv"] = torch.empty(n1, dtype=torch.float32, device=dev)
            s["gi"] = torch.empty_like(s["x"])
            s["gw"] = torch.empty_like(s["weight"])
            hs.append({k: Tensor(s[k]) for k in ("x", "weight", "grad_out", "out", "inv", "gi", "gw")})

        def fwd(i):
            h = hs[i % 3]
            check(impl.diopiRMSNorm(ctx.handle, h["out"].handle, h["inv"].handle, h["x"].handle, ns.c, h["weight"].handle, None, 1e-6), "diopiRMSNorm")

        def bwd(i):
            h = hs[i % 3]
            check(impl.diopiRMSNormBackward(ctx.handle, h["gi"].handle, h["gw"].handle, None, h["grad_out"].handle, h["x"].handle, h["weight"].handle, None,
                                            h["inv"].handle, ns.c, 1e-6), "diopiRMSNormBackward")
            ctx.clear_tensors()

        ms_f = timed(fwd)
        ms_b = timed(bwd)
        cpu_f = cpu_b = None
        if not args.no_cpu:
            xc, wc, gc = sets[0]["x"].cpu(), sets[0]["weight"].cpu(), sets[0]["grad_out"].cpu()
            ic = sets[0]["inv"].cpu()
            t = cpu_time(lambda: O.rms_norm(xc, (n2,), wc, None, 1e-6))
            cpu_f = dict(seconds=round(t, 4), GBs=round(W.rmsnorm_fwd_bytes(n1, n2, 4) / t / 1e9, 2), cores=cores, sample="full shape")
            t = cpu_time(lambda: O.rms_norm_backward(gc, xc, wc, ic, (n2,)))
            cpu_b = dict(seconds=round(t, 4), GBs=round(W.rmsnorm_bwd_bytes(n1, n2, 4) / t / 1e9, 2), cores=cores, sample="full shape")
        record("diopiRMSNorm", "cfg1 fp32 [8192,4096]", ms_f, W.rmsnorm_fwd_bytes(n1, n2, 4), "hbm", "f32", cpu_f)
        record("diopiRMSNormBackward", "cfg1 fp32 [8192,4096]", ms_b, W.rmsnorm_bwd_bytes(n1, n2, 4), "hbm", "f32", cpu_b)
        del sets, hs
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ cfg2: bf16 prologue
    if not only or "cfg2" in only:
        sets = [W.cfg2(dev, seed=2 + s) for s in range(3)]
        T, H, D, n2 = sets[0]["T"], sets[0]["H"], sets[0]["D"], sets[0]["n2"]
        ns = Sizes((n2,))
        hs = []
        for s in sets:
            s["out"] = torch.empty_like(s["x"])
            s["inv"] = torch.empty(T, dtype=torch.float32, device=dev)
            s["qo"] = torch.empty_like(s["q"])
            s["ko"] = torch.empty_like(s["k"])
            # full-width tables for the fused in-place operator (same angles in both halves)
            s["cos2"] = torch.cat((s["cos"], s["cos"]), -1).contiguous()
            s["sin2"] = torch.cat((s["sin"], s["sin"]), -1).contiguous()
            # hidden state and residual of the fused in-place normalisation (they keep accumulating: same work every step)
            s["hid"] = s["x"].clone()
            s["res"] = torch.zeros_like(s["x"])
            hs.append({k: Tensor(s[k]) for k in ("x", "weight", "out", "inv", "q", "k", "cos", "sin", "qo", "ko", "cos2", "sin2", "hid", "res")})

        def norm(i):
            h = hs[i % 3]
            check(impl.diopiRMSNorm(ctx.handle, h["out"].handle, h["inv"].handle, h["x"].handle, ns.c, h["weight"].handle, None, 1e-6), "diopiRMSNorm")

        def rot(i):
            h = hs[i % 3]
            check(impl.diopiRotaryEmbedding(ctx.handle, h["qo"].handle, h["q"].handle, h["cos"].handle, h["sin"].handle, False, False), "diopiRotaryEmbedding")
            check(impl.diopiRotaryEmbedding(ctx.handle, h["ko"].handle, h["k"].handle, h["cos"].handle, h["sin"].handle, False, False), "diopiRotaryEmbedding")

        def rot2(i):
            # in place: the buffers keep rotating by the same angles, which does not change the work
            h = hs[i % 3]
            check(impl.diopiRotaryEmbeddingV2(ctx.handle, h["qo"].handle, h["ko"].handle, h["cos2"].handle, h["sin2"].handle, D), "diopiRotaryEmbeddingV2")

        def addnorm(i):
            h = hs[i % 3]
            check(impl.diopiFusedAddRootMeanSquareNormInp(ctx.handle, h["hid"].handle, h["res"].handle, None, h["weight"].handle, 1e-6),
                  "diopiFusedAddRootMeanSquareNormInp")

        ms_n = timed(norm)
        ms_r = timed(rot)
        ms_r2 = timed(rot2)
        ms_an = timed(addnorm)
        cpu_n = cpu_r = None
        if not args.no_cpu:
            xc, wc = sets[0]["x"].cpu(), sets[0]["weight"].cpu()
            t = cpu_time(lambda: O.rms_norm(xc, (n2,), wc, None, 1e-6))
            cpu_n = dict(seconds=round(t, 4), GBs=round(W.rmsnorm_fwd_bytes(T, n2, 2) / t / 1e9, 2), cores=cores, sample="full shape")
            qc, cc, sc = sets[0]["q"].cpu(), sets[0]["cos"].cpu(), sets[0]["sin"].cpu()
            t = cpu_time(lambda: O.rotary_emb(qc, cc, sc, False))
            cpu_r = dict(seconds=round(2 * t, 4), GBs=round(W.rotary_bytes(T, H, D, 2) / t / 1e9, 2), cores=cores, sample="q call timed, k call assumed equal")
        record("diopiRMSNorm", "cfg2 bf16 [16384,4096]", ms_n, W.rmsnorm_fwd_bytes(T, n2, 2), "hbm", "bf16", cpu_n)
        record("diopiRotaryEmbedding x2 (q,k)", "cfg2 bf16 [16384,32,128]", ms_r, 2 * W.rotary_bytes(T, H, D, 2), "hbm", "bf16", cpu_r)
        record("diopiRotaryEmbeddingV2 (q,k in place, one launch)", "cfg2 bf16 [16384,32,128] x2", ms_r2, 2 * 2 * T * H * D * 2 + 2 * T * D * 2, "hbm", "bf16",
               None, note="widening beyond the seven hot-path operators; bytes = read+write of q and k, full-width cos/sin once")
        record("diopiFusedAddRootMeanSquareNormInp (residual add + RMSNorm, in place)", "cfg2 bf16 [16384,4096] x2", ms_an, 4 * T * n2 * 2 + n2 * 2, "hbm",
               "bf16", None, note="widening beyond the seven hot-path operators; bytes = read+write of the hidden state and of the residual, scale once")
        del sets, hs
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ sampling penalties on the step's logits
    if not only or "penalty" in only:
        import numpy as np
        Bp, Vp, Lp = 64, 32000, 1024  # 64 sequences, LLaMA vocabulary, 1024 distinct generated ids each
        rng = np.random.Generator(np.random.PCG64(17))
        ids = torch.from_numpy(np.concatenate([rng.permutation(Vp)[:Lp] for _ in range(Bp)]).astype(np.int32)).to(dev)
        cnt = torch.from_numpy(rng.integers(1, 20, size=Bp * Lp).astype(np.int32)).to(dev)
        cum = torch.arange(0, (Bp + 1) * Lp, Lp, dtype=torch.int32, device=dev)
        lg = torch.randn(Bp, Vp, device=dev).half()
        pres, freq = torch.rand(Bp, device=dev).half(), torch.rand(Bp, device=dev).half()
        hp = {k: Tensor(v) for k, v in dict(lg=lg, pres=pres, freq=freq, ids=ids, cnt=cnt, cum=cum).items()}

        def pen(i):
            check(impl.diopiApplyPenalty(ctx.handle, hp["lg"].handle, hp["pres"].handle, hp["freq"].handle, hp["ids"].handle, hp["cnt"].handle,
                                         hp["cum"].handle, Lp), "diopiApplyPenalty")

        ms_p = timed(pen)
        record("diopiApplyPenalty", "fp16 logits [64,32000], 1024 ids per sequence", ms_p, Bp * Lp * (4 + 4 + 2 + 2), "hbm", "f16", None,
               note="widening beyond the seven hot-path operators; a 65536-element scatter, bound by launch and memory latency, not bandwidth; "
                    "bytes = id + count + logit read + logit write per listed token")
        del hp, lg, ids, cnt
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ decode configurations
    def decode(w, tag, dtype_name):
        e = 2
        B, H, Hkv, D, total = w["B"], w["H"], w["Hkv"], w["D"], w["total_len"]
        logits = torch.zeros(H, total, dtype=w["dtype"], device=dev)
        out = torch.zeros_like(w["q"])
        h = {k: Tensor(w[k]) for k in ("k_cache", "v_cache", "q", "new_k", "new_v", "dest_loc", "b_loc", "b_seq_len", "b_start_loc")}
        h["logits"], h["out"] = Tensor(logits), Tensor(out)
        mil = w["max_input_len"]

        def copy_kv(i):
            check(impl.diopiDestIndexCopyKV(ctx.handle, h["k_cache"].handle, h["new_k"].handle, h["dest_loc"].handle), "diopiDestIndexCopyKV")
            check(impl.diopiDestIndexCopyKV(ctx.handle, h["v_cache"].handle, h["new_v"].handle, h["dest_loc"].handle), "diopiDestIndexCopyKV")

        def att(i):
            check(impl.diopiTokenAttentionInference(ctx.handle, h["logits"].handle, h["q"].handle, h["k_cache"].handle, h["b_loc"].handle,
                                                    h["b_start_loc"].handle, h["b_seq_len"].handle, mil), "diopiTokenAttentionInference")

        def redv(i):
            check(impl.diopiTokenSoftmaxReduceVInference(ctx.handle, h["out"].handle, h["logits"].handle, h["v_cache"].handle, h["b_loc"].handle,
                                                         h["b_start_loc"].handle, h["b_seq_len"].handle, mil, 0), "diopiTokenSoftmaxReduceVInference")
            ctx.clear_tensors()

        def step(i):
            copy_kv(i)
            att(i)
            redv(i)

        ms_copy = timed(copy_kv)
        ms_att = timed(att)
        ms_red = timed(redv)
        ms_step = timed(step)
        # the same four launches recorded once in a HIP graph and replayed, the way a serving loop runs its decode step
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=ctx.torch_stream):
            step(0)

        def replay(i):
            with torch.cuda.stream(ctx.torch_stream):
                graph.replay()

        ms_graph = timed(replay)
        del graph
        b_att = W.token_attention_bytes(total, B, H, Hkv, D, e)
        b_red = W.softmax_reducev_bytes(total, B, H, Hkv, D, e)
        b_copy = 2 * W.destindex_bytes(B, Hkv, D, e)
        cpu = None
        if not args.no_cpu:
            # bounded sample: the first sequences of the batch through the reference's per-sequence composition; one
            # untimed warm-up pass over the first sequence sizes the sample so that a warm-up pass and three timed
            # passes over it fit the budget; the median of the three is reported
            qc, blc, bsc, bln = w["q"].cpu(), w["b_loc"].cpu(), w["b_start_loc"].cpu(), w["b_seq_len"].cpu()
            budget = args.cpu_seconds if tag == "cfg3" else 4.0

            def prepare(n):
                sel = slice(n, n + 1)
                used = torch.unique(blc[sel].long())
                remap = torch.zeros(int(used.max()) + 1, dtype=torch.int32)
                remap[used] = torch.arange(used.numel(), dtype=torch.int32)
                return dict(sel=sel, ks=w["k_cache"][used.to(dev)].cpu(), vs=w["v_cache"][used.to(dev)].cpu(), loc=remap[blc[sel].long()],
                            lg=torch.zeros(H, total, dtype=w["dtype"]), oc=torch.zeros(1, H, D, dtype=w["dtype"]))

            def run(p):
                t0 = time.perf_counter()
                O.token_attention(qc[p["sel"]], p["ks"], p["lg"], p["loc"], bsc[p["sel"]], bln[p["sel"]], mil)
                O.token_softmax_reducev(p["lg"], p["vs"], p["oc"], p["loc"], bsc[p["sel"]], bln[p["sel"]], mil, 0)
                return time.perf_counter() - t0

            first = prepare(0)
            run(first)                      # warm-up: threads, allocator, code paths
            per_tok = run(first) / max(1, int(bln[0]))
            nseq, tok = 1, int(bln[0])
            while nseq < B and per_tok * (tok + int(bln[nseq])) * 4 < budget:
                tok += int(bln[nseq])
                nseq += 1
            sample = [first] + [prepare(n) for n in range(1, nseq)]
            for p_ in sample[1:]:
                run(p_)                     # warm-up pass over the rest of the sample
            reps = sorted(sum(run(p_) for p_ in sample) for _ in range(3))
            spent = reps[1]
            frac_tok = tok / total
            cpu = dict(seconds_sample=round(spent, 3), seconds_all_reps=[round(x, 3) for x in reps], sequences=nseq,
                       tokens_per_s=round(nseq / spent, 2), GBs=round((b_att + b_red) * frac_tok / spent / 1e9, 3), cores=cores,
                       sample=f"first {nseq} of {B} sequences ({tok} of {total} cached tokens), attention only, cache rows pre-gathered; "
                              f"one warm-up pass, median of 3 timed passes")
            del sample, first
        record("diopiDestIndexCopyKV x2 (K,V)", f"{tag} {B} tokens", ms_copy, b_copy, "hbm", dtype_name,
               note="launch-bound at this size: 1 MiB of traffic per call")
        record("diopiTokenAttentionInference", tag, ms_att, b_att, "hbm", dtype_name)
        record("diopiTokenSoftmaxReduceVInference", tag, ms_red, b_red, "hbm", dtype_name)
        e_step = record("decode step (copy K,V + attention)", tag, ms_step, b_copy + b_att + b_red, "hbm", dtype_name, cpu)
        e_step["tokens_per_s"] = round(B / (ms_step * 1e-3), 1)
        e_step["attention_only_tokens_per_s"] = round(B / ((ms_att + ms_red) * 1e-3), 1)
        e_graph = record("decode step replayed from a HIP graph (the same four launches, recorded once)", tag, ms_graph, b_copy + b_att + b_red, "hbm", dtype_name,
                         None, note="not the headline: the headline times the four calls through the C ABI")
        e_graph["tokens_per_s"] = round(B / (ms_graph * 1e-3), 1)
        return dict(ms_step=ms_step, ms_att=ms_att, ms_red=ms_red, b_att=b_att, b_red=b_red, B=B, total=total, cpu=cpu)

    head = None
    if not only or "cfg3" in only:
        w3 = W.cfg3(dev, seed=3)
        head = decode(w3, "cfg3", "f16")
        # DestIndexCopyKV away from the launch-bound regime: a full permutation of 65536 rows of 8 KiB
        Tn = 65536
        src = w3["k_cache"][:Tn].clone()
        perm = torch.randperm(Tn, device=dev).int() + Tn
        hsrc, hperm, hcache = Tensor(src), Tensor(perm), Tensor(w3["k_cache"])
        ms = timed(lambda i: check(impl.diopiDestIndexCopyKV(ctx.handle, hcache.handle, hsrc.handle, hperm.handle), "diopiDestIndexCopyKV"))
        record("diopiDestIndexCopyKV", f"sweep: {Tn} tokens x 8 KiB", ms, W.destindex_bytes(Tn, 32, 128, 2), "hbm", "f16")
        # the same decode step through the paged-attention interface: the cache as 1024 blocks of 128 rows, each sequence
        # on 16 blocks drawn from a random permutation, its cfg3 length; both decode kernels plus the table expansion
        B3, H3, D3 = w3["B"], w3["H"], w3["D"]
        lens3 = [int(x) for x in w3["b_seq_len"].cpu()]
        table = torch.randperm(1024, device=dev).int().view(B3, 16)
        q2, k2, v2 = w3["q"].view(B3, H3 * D3), w3["k_cache"].view(-1, H3 * D3), w3["v_cache"].view(-1, H3 * D3)
        o2 = torch.zeros_like(q2)
        hp = {k: Tensor(v) for k, v in dict(q=q2, k=k2, v=v2, o=o2, t=table).items()}
        sz = rt.Sizes(lens3)

        def paged(i):
            check(impl.diopiPagedAttention(ctx.handle, hp["o"].handle, hp["q"].handle, hp["k"].handle, hp["v"].handle, None, sz.c, H3, H3, D3,
                                           hp["t"].handle, 128), "diopiPagedAttention")
            ctx.clear_tensors()

        ms_pg = timed(paged)
        e_pg = record("diopiPagedAttention (blocks of 128 rows)", f"cfg3 lengths fp16 B={B3}", ms_pg, head["b_att"] + head["b_red"], "hbm", "f16", None,
                      note="widening beyond the seven hot-path operators; block table -> row table, then the two decode kernels")
        e_pg["tokens_per_s"] = round(B3 / (ms_pg * 1e-3), 1)
        del src, perm, hsrc, hperm, hcache, hp, q2, k2, v2, o2, table
        torch.cuda.empty_cache()
        # the same decode step behind the fused lmdeploy interface: QKV projection of [64, 4096] hidden states, bias, rotary,
        # cache insertion and attention over contiguous per-sequence caches [1, 64, 32, 2048, 128] with the cfg3 lengths
        # (one token fewer cached, so that the window of every row is its cfg3 length); no logits tensor exists
        hid, S3 = H3 * D3, 2048
        N3 = 3 * H3 * D3
        g3 = torch.Generator(device=dev)
        g3.manual_seed(33)
        xs = [(torch.randn(B3, hid, device=dev, generator=g3) * 0.5).to(torch.float16) for _ in range(3)]
        wq = (torch.randn(hid, N3, device=dev, generator=g3) / math.sqrt(hid)).to(torch.float16)
        bq = torch.randn(N3, device=dev, generator=g3).to(torch.float16)
        kcs = w3["k_cache"].view(1, B3, S3, H3, D3).permute(0, 1, 3, 2, 4).contiguous()
        vcs = w3["v_cache"].view(1, B3, S3, H3, D3).permute(0, 1, 3, 2, 4).contiguous()
        cached = (w3["b_seq_len"] - 1).to(torch.int32)
        hfz = {k: Tensor(v) for k, v in dict(w=wq, b=bq, k=kcs, v=vcs, s=cached).items()}
        hxs = [Tensor(x) for x in xs]
        size = ctypes.c_int64(-1)
        check(impl.diopiFusedDecoderAttentionInp(ctx.handle, hxs[0].handle, hfz["w"].handle, hfz["b"].handle, None, ctypes.byref(size), 0, hfz["k"].handle,
                                                 hfz["v"].handle, None, None, hfz["s"].handle, 2048, 0, H3, H3, D3, S3, D3, 10000.0), "size query")
        wsp = torch.empty(int(size.value), dtype=torch.int8, device=dev)
        hwsp = Tensor(wsp)

        def fused(i):
            check(impl.diopiFusedDecoderAttentionInp(ctx.handle, hxs[i % 3].handle, hfz["w"].handle, hfz["b"].handle, hwsp.handle, ctypes.byref(size), 0,
                                                     hfz["k"].handle, hfz["v"].handle, None, None, hfz["s"].handle, 2048, 0, H3, H3, D3, S3, D3, 10000.0),
                  "diopiFusedDecoderAttentionInp")

        ms_fz = timed(fused)
        kv_rows = int(w3["b_seq_len"].sum())
        b_proj = hid * N3 * 2 + N3 * 2 + B3 * hid * 2 + B3 * N3 * 2            # weights, bias, hidden states in, q / new k / new v out
        b_attn = kv_rows * 2 * H3 * D3 * 2 + B3 * H3 * D3 * 2 * 2 + 4 * B3    # one K and one V row per cached token, q in, output, lengths
        e_fz = record("diopiFusedDecoderAttentionInp (projection + rotary + cache insert + attention)", f"cfg3 lengths fp16 B={B3} hidden={hid}", ms_fz,
                      b_proj + b_attn, "hbm", "f16", None,
                      note="widening (lmdeploy set): the decode step without a logits tensor; bytes = projection weights once + one K and one V row "
                           "per cached token; compare its attention share with TokenAttention + TokenSoftmaxReduceV above, which move the same rows "
                           "plus the logits twice")
        e_fz["tokens_per_s"] = round(B3 / (ms_fz * 1e-3), 1)
        e_fz["projection_bytes"], e_fz["attention_bytes"] = int(b_proj), int(b_attn)
        del w3, xs, wq, bq, kcs, vcs, hfz, hxs, wsp, hwsp
        torch.cuda.empty_cache()

    if not only or "cfg5" in only:
        w5 = W.cfg5(dev, seed=5)
        decode(w5, "cfg5", "bf16")
        del w5
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ cfg4: prefill
    if not only or "cfg4" in only:
        w4 = W.cfg4(dev, seed=4)
        out = torch.zeros_like(w4["q"])
        h = {k: Tensor(w4[k]) for k in ("q", "k", "v", "b_start_loc", "b_seq_len")}
        h["out"] = Tensor(out)
        flops = W.context_attention_flops(w4["seq_len_host"], w4["H"], w4["D"])

        def pre(i):
            check(impl.diopiContextAttentionInference(ctx.handle, h["out"].handle, h["q"].handle, h["k"].handle, h["v"].handle, h["b_start_loc"].handle,
                                                      h["b_seq_len"].handle, w4["max_input_len"]), "diopiContextAttentionInference")
            ctx.clear_tensors()  # the tile plan goes back to the context's pool

        ms = timed(pre)
        cpu = None
        if not args.no_cpu:
            # the reference materialises [H, L, L] scores and ATen's fp16 matmul on the host is slow: time the first
            # 256 rows of the shortest sequence only and scale by flops
            i = int(w4["seq_len_host"].argmin())
            s, L = int(w4["b_start_loc"][i]), min(256, int(w4["seq_len_host"][i]))
            qc, kc, vc = (w4[k][s:s + L].cpu() for k in ("q", "k", "v"))
            oc = torch.zeros_like(qc)
            t0 = time.perf_counter()
            O.context_attention(qc, kc, vc, oc, torch.tensor([0]), torch.tensor([L]), L)
            t = time.perf_counter() - t0
            f1 = W.context_attention_flops([L], w4["H"], w4["D"])
            cpu = dict(seconds_sample=round(t, 3), TFLOPs=round(f1 / t / 1e12, 4), cores=cores,
                       sample=f"first {L} rows of the shortest sequence; extrapolated by flops to the full configuration: {t * flops / f1:.1f} s")
        record("diopiContextAttentionInference", f"cfg4 fp16 B=8 T={w4['T']}", ms, flops, "mfma", "f16", cpu)

        # the same tokens through the flash-attention interface: cumulative lengths, 32 query heads over 8 key/value
        # heads, log-sum-exp output (same flop count: every query head still meets every visible key)
        cu = torch.cat((w4["b_start_loc"], w4["b_start_loc"][-1:] + w4["b_seq_len"][-1:])).to(torch.int32)
        k8, v8 = w4["k"][:, :8].contiguous(), w4["v"][:, :8].contiguous()
        lse = torch.zeros(w4["B"], w4["H"], w4["max_input_len"], dtype=torch.float32, device=dev)
        hf = {k: Tensor(v) for k, v in dict(cu=cu, k8=k8, v8=v8, lse=lse).items()}
        scale = 1.0 / math.sqrt(w4["D"])

        def fav(i):
            check(impl.diopiFlashAttentionVarLen(ctx.handle, h["out"].handle, hf["lse"].handle, None, h["q"].handle, hf["k8"].handle, hf["v8"].handle,
                                                 hf["cu"].handle, hf["cu"].handle, None, w4["max_input_len"], w4["max_input_len"], 0.0, scale, True, -1, -1),
                  "diopiFlashAttentionVarLen")
            ctx.clear_tensors()

        ms_f = timed(fav)
        record("diopiFlashAttentionVarLen (causal, 32 heads over 8 kv heads, lse)", f"cfg4 tokens fp16 B=8 T={w4['T']}", ms_f, flops, "mfma", "f16", None,
               note="widening beyond the seven hot-path operators; the prefill kernel in its general form")
        # the lightllm operator once more with bf16 tensors (same tokens, same flop count)
        qb, kb, vb = (w4[k].to(torch.bfloat16) for k in ("q", "k", "v"))
        ob = torch.zeros_like(qb)
        hb = {k: Tensor(v) for k, v in dict(q=qb, k=kb, v=vb, o=ob).items()}

        def pre_bf16(i):
            check(impl.diopiContextAttentionInference(ctx.handle, hb["o"].handle, hb["q"].handle, hb["k"].handle, hb["v"].handle, h["b_start_loc"].handle,
                                                      h["b_seq_len"].handle, w4["max_input_len"]), "diopiContextAttentionInference")
            ctx.clear_tensors()

        ms_b = timed(pre_bf16)
        record("diopiContextAttentionInference", f"cfg4 tokens in bf16 B=8 T={w4['T']}", ms_b, flops, "mfma", "bf16", None)
        # diagnostic, not a result: the fp16 kernel once more on all-zero tensors of the same shape.  The instruction stream is
        # the same; what differs is the data-dependent switching in the matrix pipes, and with it the clock the power limit allows
        if not args.no_diagnostic:
            qz, kz, vz = (torch.zeros_like(w4[k]) for k in ("q", "k", "v"))
            hz = {k: Tensor(v) for k, v in dict(q=qz, k=kz, v=vz).items()}

            def pre_zero(i):
                check(impl.diopiContextAttentionInference(ctx.handle, h["out"].handle, hz["q"].handle, hz["k"].handle, hz["v"].handle,
                                                          h["b_start_loc"].handle, h["b_seq_len"].handle, w4["max_input_len"]), "diopiContextAttentionInference")
                ctx.clear_tensors()

            ms_z = timed(pre_zero)
            record("diopiContextAttentionInference", f"cfg4 shape, all-zero q/k/v (diagnostic) B=8 T={w4['T']}", ms_z, flops, "mfma", "f16", None,
                   note="not a result: same instruction stream as the cfg4 entry without data-dependent switching; the gap to the cfg4 entry is clock")
            del hz, qz, kz, vz
        del w4, hf, k8, v8, lse, hb, qb, kb, vb, ob
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ the JSON line
    line = {
        "metric": "decode-attn tokens/s at bs=64 (per-op achieved HBM GB/s and % of peak under 'ops')",
        "value": None, "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": Wm, "ms_per_step": None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "cfg3 decode step fp16: 2x DestIndexCopyKV [64,32,128] -> cache [131072,32,128], TokenAttention + "
                               "TokenSoftmaxReduceV, batch 64, 32 heads x 128, b_loc [64,2048], seq_len ~U(512,2048)"},
        "roofline": None, "cpu_baseline": None, "ops": ops,
        "host": {"cpu_model": cpu_model, "threads_used": cores},
        "peaks": {"hbm_GBs": HBM_PEAK_GBS, "mfma_f16_TFLOPs": MFMA_PEAK_TFLOPS, "device": device_peak},
    }
    if head is not None:
        line["value"] = round(head["B"] / (head["ms_step"] * 1e-3), 1)
        line["ms_per_step"] = round(head["ms_step"], 5)
        line["config"]["total_cached_tokens"] = head["total"]
        # dominant kernel of the step: the slower of the two attention halves
        if head["ms_att"] >= head["ms_red"]:
            kname, kms, kbytes = "tokenAttStaged (diopiTokenAttentionInference)", head["ms_att"], head["b_att"]
        else:
            kname, kms, kbytes = "softmaxReduceVWave+Merge (diopiTokenSoftmaxReduceVInference)", head["ms_red"], head["b_red"]
        traffic = measured_traffic(kname.split(" ")[0], head["total"])
        ach = kbytes / (kms * 1e-3) / 1e9
        line["roofline"] = {"bound": "hbm", "kernel": kname, "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                            "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": traffic, "algorithmic_bytes": int(kbytes), "ms": round(kms, 5),
                            "traffic_over_algorithmic": round(traffic / kbytes, 4) if traffic else None}
        if head["cpu"] is not None:
            c = head["cpu"]
            line["cpu_baseline"] = {"value": c["tokens_per_s"], "unit": "tokens/s", "cores": c["cores"], "kind": "port", "sample": c["sample"],
                                    "cpu_model": cpu_model}
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
