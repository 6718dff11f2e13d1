#!/usr/bin/env python3
"""Benchmark of the MI355X GEMM / fused-attention hot path (one GPU).

``python bench.py --gpus 1 --steps K --warmup W`` prints ONE JSON line.  A "step" is one pass of the
hot path over one batch of synthetic input; the headline workload is the configuration the metric's
target is quoted on: the fp16 GEMM M = N = K = 8192 with fp32 accumulation (fp16 output).  The other
configurations of the metric (fp32 / fp16 projection GEMMs, fp32 and fp16 / bf16 causal prefill
attention, bf16 decode attention and its projection GEMM) are timed the same way and reported under
``others`` with their own roofline objects.

Inputs are resident in HBM before the timed region; the timed region is bracketed by
``torch.cuda.synchronize()`` and by HIP events recorded on the stream the kernels are launched on
(torch's current stream, whose handle is what the C ABI receives).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "GEMM & fused-attn TFLOP/s (% MFMA peak), decode-attn GB/s, 1x MI355X"
# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch), each scaled by what the
# same counter reads for a 1 GiB device copy; the runs and factors are in profiles/ (one summary per kernel).  None = not
# measured yet.
TRAFFIC_BYTES = {
    # profiles/hbm_traffic_pmc_mi355x.md: FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 (KiB -> bytes), last three dispatches of each kernel
    "gemm_f16_8192": int((786920 * 2.0 + 131340) * 1024),
    "gemm_bf16_8192": int((787044 * 2.0 + 131400) * 1024),
    "gemm_f16_proj": int((17114 * 2.0 + 24584) * 1024),
    "gemm_f16_proj_f32out": int((17048 * 2.0 + 49165) * 1024),
    "gemm_f32_proj": int((43104 * 2.0 + 49152) * 1024),
    "gemm_f32_1024": int((12318 * 2.0 + 4096) * 1024),
    "decode_bf16": int((1048770 * 2.0 + 512) * 1024),
    "attn_f16_prefill": int((144204 * 2.0 + 132098) * 1024),
    "attn_bf16_prefill": int((144033 * 2.0 + 132102) * 1024),
    "attn_f32_prefill": int((22634 * 2.0 + 12480) * 1024),
    # two launches each: the skinny kernel, then the pass that sums its K ranges
    "gemm_bf16_decode_proj": int(((17442 + 2071) * 2.0 + 4096 + 256) * 1024),
    "gemm_bf16_decode_qkv": int(((50203 + 3863) * 2.0 + 7680 + 768) * 1024),
    "gemm_bf16_decode_qkv_rope": int(((50203 + 3864) * 2.0 + 7680 + 768) * 1024),
    # profiles/grouped_decode_and_fp32_few_row_gemm_mi355x.md (kernel + its merge / summing pass; the summing pass of the 16-row product
    # reads its 16 ranges of 16 x 4096 fp32 partials back: 4 MiB, 2049 KiB on the counter)
    "decode_bf16_gqa": int(((262418 + 1108) * 2.0 + 1040 + 512) * 1024),
    "decode_f32_gqa": int(((525392 + 1108) * 2.0 + 2176 + 512) * 1024),
    "gemm_f32_m16": int(((33819 + 2049) * 2.0 + 4096 + 256) * 1024),
    "attn_f16_prefill_d256": int((135459 * 2.0 + 131620) * 1024),
    "attn_bf16_prefill_d256": int((135583 * 2.0 + 131635) * 1024),
}
# MI355X published dense peaks
PEAK_TFLOPS = {"f16": 2500.0, "bf16": 2500.0, "f32": 157.3}
PEAK_HBM_GBS = 8000.0
# the untimed warm-up of every configuration lasts at least this long, whatever --warmup says (outside the timed region)
MIN_WARM_MS = 60.0


def _sclk_mhz():
    """Engine clock the driver reports right now (MHz), or None: the line of pp_dpm_sclk marked with '*'."""
    import glob
    for path in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")):
        try:
            for line in open(path):
                if "*" in line:
                    return int(line.split(":")[1].strip().lower().split("mhz")[0])
        except (OSError, ValueError, IndexError):
            continue
    return None


def _power_uw():
    """Board power the driver reports right now (microwatts), and the cap, or (None, None): hwmon power1_average where the driver has
    it, else power1_input."""
    import glob
    for d in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*")):
        for name in ("power1_average", "power1_input"):
            try:
                val = int(open(os.path.join(d, name)).read())
            except (OSError, ValueError):
                continue
            try:
                cap = int(open(os.path.join(d, "power1_cap")).read())
            except (OSError, ValueError):
                cap = None
            return val, cap
    return None, None


def _load_trace(torch, fn, steps, min_ms=80.0):
    """Board power and engine clock sampled WHILE the workload runs: a third pass (it never touches the timed figures) that keeps
    `steps`-long batches of the step queued for at least `min_ms` while a thread reads the driver's files every millisecond or so.
    Returns {"power_w": {...}, "sclk_mhz": {...}} or None where the driver offers neither file."""
    import threading
    if _power_uw()[0] is None and _sclk_mhz() is None:
        return None
    stop = threading.Event()
    pw, ck = [], []

    def sample():
        while not stop.is_set():
            p, _ = _power_uw()
            c = _sclk_mhz()
            if p is not None:
                pw.append(p / 1e6)
            if c is not None:
                ck.append(c)
            time.sleep(0.001)

    th = threading.Thread(target=sample, daemon=True)
    t0 = time.perf_counter()
    n = 0
    for _ in range(steps):          # the queue is filled before the first sample is taken
        fn()
    th.start()
    while (time.perf_counter() - t0) * 1e3 < min_ms:
        for _ in range(steps):
            fn()
        n += steps
        # (no synchronisation between the batches beyond what keeps the queue bounded: the device stays busy throughout)
        if n % (8 * steps) == 0:
            torch.cuda.synchronize()
    stop.set()
    th.join()
    torch.cuda.synchronize()
    out = {}
    if pw:
        out["power_w"] = {"mean": round(sum(pw) / len(pw), 1), "max": round(max(pw), 1), "samples": len(pw),
                          "cap": None if _power_uw()[1] is None else round(_power_uw()[1] / 1e6, 1)}
    if ck:
        out["sclk_mhz"] = {"mean": round(sum(ck) / len(ck), 1), "min": min(ck), "max": max(ck), "samples": len(ck)}
    return out or None


def _events_time(torch, fn, steps, warmup, min_warm_ms=MIN_WARM_MS):
    """`warmup` untimed steps, continued until `min_warm_ms` of wall time has passed (a launch sequence needs some tens of
    milliseconds of its own load before the clock management of the device settles), then exactly `steps` timed steps.
    Returns the mean over the timed region (one event pair around the `steps` launches, on the launch stream), the wall-clock
    mean, and the median / 95th percentile / spread of single steps from a second pass with one event pair per step."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t_warm = time.perf_counter()
    while (time.perf_counter() - t_warm) * 1e3 < min_warm_ms:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
    clk0 = _sclk_mhz()
    # pass 1: exactly `steps` launches back to back between ONE pair of events -- the figure every throughput is computed from
    # (an event between two launches costs a few microseconds of its own, which matters for the 10-30 us configurations)
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    clk_load = _sclk_mhz()          # launches are asynchronous: for steps of a millisecond the device is still in the timed region here
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ms = start.elapsed_time(end) / steps
    clk1 = _sclk_mhz()
    # pass 2: the same number of steps, each bracketed by its own pair of events, for the spread (median, 95th percentile)
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    evs[0].record()
    for i in range(steps):
        fn()
        evs[i + 1].record()
    torch.cuda.synchronize()
    per = sorted(evs[i].elapsed_time(evs[i + 1]) for i in range(steps))
    stats = {"median_ms": round(per[len(per) // 2], 5), "p95_ms": round(per[min(len(per) - 1, int(math.ceil(0.95 * len(per))) - 1)], 5),
             "min_ms": round(per[0], 5), "max_ms": round(per[-1], 5), "sclk_mhz_before_after": [clk0, clk1], "sclk_mhz_while_queued": clk_load,
             "note": "single steps timed in a second pass with one event pair each (includes the events' own cost)"}
    trace = _load_trace(torch, fn, steps)
    if trace:
        stats["under_load"] = trace        # board power (W) and engine clock (MHz) sampled in a third pass with the step kept queued
    return ms, wall_ms, stats


def _summarize_profile(directory, last):
    """Reads what rocprofv3 wrote under `directory` (CSV output) and prints, per kernel, the figures of its LAST `last` dispatches
    only: the timed region of a configuration is what it launches last, its warm-up launches come before.  Kernel-trace files give
    the duration (us), counter-collection files the counter values (per dispatch).  Needs no GPU."""
    import collections
    import csv
    import glob
    for f in sorted(glob.glob(os.path.join(directory, "**", "*kernel_trace.csv"), recursive=True)):
        per = collections.defaultdict(list)
        for row in csv.DictReader(open(f)):
            per[row["Kernel_Name"]].append((int(row["Start_Timestamp"]), int(row["End_Timestamp"])))
        print("# %s: duration in us over the last %d dispatches of each kernel" % (os.path.relpath(f, directory), last))
        for name, v in sorted(per.items(), key=lambda kv: -sum(e - s for s, e in kv[1])):
            v.sort()
            tail = [(e - s) / 1e3 for s, e in v[-last:]]
            print("%-130s calls=%d last=%d avg=%.2f min=%.2f max=%.2f (all calls avg %.2f)" % (
                name[:130], len(v), len(tail), sum(tail) / len(tail), min(tail), max(tail), sum((e - s) / 1e3 for s, e in v) / len(v)))
    for f in sorted(glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True)):
        per = collections.defaultdict(lambda: collections.defaultdict(list))
        for row in csv.DictReader(open(f)):
            per[row["Kernel_Name"]][row["Counter_Name"]].append(float(row["Counter_Value"]))
        print("# %s: counter value per dispatch, mean over the last %d dispatches of each kernel" % (os.path.relpath(f, directory), last))
        for name, cs in per.items():
            print("%-130s %s" % (name[:130], "  ".join("%s=%.6g (n=%d)" % (c, sum(v[-last:]) / len(v[-last:]), len(v)) for c, v in sorted(cs.items()))))
    return 0


def _roof_flops(kind, flops, ms, traffic=None):
    ach = flops / (ms * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": round(ach, 3), "peak": PEAK_TFLOPS[kind], "unit": "TFLOP/s",
            "frac": round(ach / PEAK_TFLOPS[kind], 4), "traffic": traffic}


def _roof_bytes(nbytes, ms, traffic=None):
    ach = nbytes / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(ach, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": round(ach / PEAK_HBM_GBS, 4), "traffic": traffic}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--only", default="", help="comma list of workloads to time besides the headline (default: all)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three 1 GiB device copies (a plain copy kernel of known size) so that FETCH_SIZE / "
                         "WRITE_SIZE counters collected over this command can be scaled")
    ap.add_argument("--diagnostic-data", choices=["zeros", "ones"], default=None,
                    help="NOT the metric: fill every operand with one value instead of seeded Gaussians.  The instruction stream is the "
                         "same, the switching activity in the data paths is minimal; the difference to the default run is what the "
                         "board's power management costs at this load")
    ap.add_argument("--clock-probe", type=float, default=0.0, metavar="SECONDS",
                    help="NOT the metric: keep the headline GEMM (then the bf16 causal prefill) queued for SECONDS each and sample the "
                         "engine clock the driver reports meanwhile; prints one JSON line with the median clock and the rate")
    ap.add_argument("--summarize-profile", default=None, metavar="DIR",
                    help="NOT a run: print per-kernel durations and counter values from the CSV files rocprofv3 wrote under DIR, over the "
                         "last --last dispatches of each kernel (the timed region; warm-up launches come first)")
    ap.add_argument("--last", type=int, default=20, help="dispatches per kernel that --summarize-profile looks at")
    args = ap.parse_args()
    if args.summarize_profile:
        return _summarize_profile(args.summarize_profile, max(1, args.last))
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (the path shards without "
              "communication over (batch, head) and over row slabs of C)" % args.gpus, file=sys.stderr)
        return 2

    import torch
    from aidotnet.tensors_amd import Mi355Backend

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    be = Mi355Backend(synchronous=False)       # launches are asynchronous inside the timed region
    W = be.WrapTensor
    steps, warmup = args.steps, args.warmup
    g = torch.Generator(device="cuda")
    g.manual_seed(20250)
    dts = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}

    def randn(*shape, std=1.0, kind="f32"):
        if args.diagnostic_data is not None:
            return torch.full(shape, 0.0 if args.diagnostic_data == "zeros" else 1.0, device="cuda", dtype=dts[kind])
        return (std * torch.randn(*shape, device="cuda", generator=g)).to(dts[kind])

    if args.clock_probe > 0:
        def sustained(fn, flops):
            for _ in range(20):
                fn()
            torch.cuda.synchronize()
            clocks, calls, t0 = [], 0, time.perf_counter()
            while time.perf_counter() - t0 < args.clock_probe:
                for _ in range(100):
                    fn()
                calls += 100
                c = _sclk_mhz()                 # read while the hundred launches above are still queued
                if c:
                    clocks.append(c)
                torch.cuda.synchronize()
            el = time.perf_counter() - t0
            clocks.sort()
            return {"sclk_mhz_median": clocks[len(clocks) // 2] if clocks else None, "sclk_mhz_min": clocks[0] if clocks else None,
                    "sclk_mhz_max": clocks[-1] if clocks else None, "us_per_call_wall": round(el / calls * 1e6, 2),
                    "tflops_wall": round(flops * calls / el / 1e12, 1)}
        n = 8192
        a = randn(n, n, kind="f16"); b = randn(n, n, std=0.02, kind="f16"); c = torch.empty(n, n, device="cuda", dtype=torch.float16)
        A, B, C = W(a), W(b), W(c)
        probe = {"data": args.diagnostic_data or "gaussian", "seconds_each": args.clock_probe,
                 "gemm_f16_8192": sustained(lambda: be.Hgemm(A, B, C, n, n, n), 2.0 * n * n * n)}
        Bn, H, S, D = 4, 32, 2048, 128
        q = randn(Bn, H, S, D, kind="bf16"); k = randn(Bn, H, S, D, kind="bf16"); v = randn(Bn, H, S, D, kind="bf16")
        o = torch.empty(Bn, H, S, D, device="cuda"); lse = torch.empty(Bn, H, S, device="cuda")
        probe["attn_bf16_prefill"] = sustained(
            lambda: be.FlashAttentionHalf("bf16", W(q), W(k), W(v), W(o), W(lse), Bn, H, S, S, D, 1.0 / math.sqrt(D), True),
            4.0 * Bn * H * D * (S * (S + 1) / 2))
        print(json.dumps(probe))
        return 0

    # ------------------------------------------------------------------ headline: fp16 GEMM 8192^3
    n = 8192
    a = randn(n, n, kind="f16")
    b = randn(n, n, std=0.02, kind="f16")
    c = torch.empty(n, n, device="cuda", dtype=torch.float16)
    A, B, C = W(a), W(b), W(c)
    ms, wall_ms, stats = _events_time(torch, lambda: be.Hgemm(A, B, C, n, n, n), steps, warmup)
    flops = 2.0 * n * n * n
    value = flops / (ms * 1e-3) / 1e12
    out = {
        "metric": METRIC, "value": round(value, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic" if args.diagnostic_data is None else "DIAGNOSTIC all-%s operands (not the metric)" % args.diagnostic_data,
        "config": {"workload": "fp16 GEMM C=A*B, M=N=K=8192, fp32 accumulate, fp16 out (A~N(0,1), B~N(0,0.02^2), seeded)",
                   "wall_ms_per_step": round(wall_ms, 5), "min_warmup_ms": MIN_WARM_MS},
        "step_stats": stats,
        "roofline": _roof_flops("f16", flops, ms, TRAFFIC_BYTES.get("gemm_f16_8192")),
    }
    del a, b, c

    # ------------------------------------------------------------------ the metric's other configurations
    others = []
    only = set(x for x in args.only.split(",") if x)

    def want(name, extra=False):
        # extra workloads (shapes beside the listed configurations) run only when --only names them
        return name in only if (only or extra) else True

    def add(name, kind, workload, ms, roof, stats):
        others.append({"name": name, "dtype": kind, "workload": workload, "ms_per_step": round(ms, 5), "roofline": roof,
                       "step_stats": stats})

    def uniform(*shape, kind="f32"):
        if args.diagnostic_data is not None:
            return randn(*shape, kind=kind)
        return (2.0 * torch.rand(*shape, device="cuda", generator=g) - 1.0).to(dts[kind])

    def gemm_case(name, kind, M, N, K, out32=False, hbm=False, rotate=1, wstd=0.02, uniform_inputs=False, extra=False, packed=False, rope=None):
        if not want(name, extra):
            return
        # rotate > 1: cycle through that many distinct weight matrices so the timed loop reads HBM, not the
        # 256 MB last-level cache
        # uniform_inputs: A and B i.i.d. uniform[-1, 1] (the 1024^3 configuration); otherwise N(0,1) activations and N(0, wstd^2) weights
        a_ = uniform(M, K, kind=kind) if uniform_inputs else randn(M, K, kind=kind)
        bs = [uniform(K, N, kind=kind) if uniform_inputs else randn(K, N, std=wstd, kind=kind) for _ in range(rotate)]
        c_ = torch.empty(M, N, device="cuda", dtype=torch.float32 if (kind == "f32" or out32) else dts[kind])
        A_, C_ = W(a_), W(c_)
        Bs = [W(x) for x in bs]
        if packed:
            # the weights packed once, outside the timed region (what a resident model does); the product reads the packed form
            Bs = [be.PackB(kind, Bx, K, N) for Bx in Bs]
            fn1 = lambda Bx: be.GemmPackedB(kind, A_, Bx, None, C_, M, N, K, outputIsFp32=(kind == "f32" or out32))
        elif kind == "f32":
            fn1 = lambda Bx: be.Gemm(A_, Bx, C_, M, N, K)
        elif kind == "f16":
            fn1 = (lambda Bx: be.GemmFp16In32fOut(A_, Bx, C_, M, N, K)) if out32 else (lambda Bx: be.Hgemm(A_, Bx, C_, M, N, K))
        else:
            fn1 = (lambda Bx: be.GemmBf16In32fOut(A_, Bx, C_, M, N, K)) if out32 else (lambda Bx: be.Bf16Gemm(A_, Bx, C_, M, N, K))
        if rope is not None:
            # rope = (head_dim, rotated columns, position): the product with the interleaved rotary embedding in its summing pass
            hd, rcols, pos = rope
            half = hd // 2
            ang = torch.arange(pos + 1, device="cuda", dtype=torch.float32)[:, None] * (10000.0 ** (-torch.arange(half, device="cuda") * 2.0 / hd))[None, :]
            cs_, sn_ = W(torch.cos(ang).contiguous()), W(torch.sin(ang).contiguous())
            fn1 = lambda Bx: be.GemmRope(kind, A_, Bx, C_, M, N, K, cs_, sn_, hd, rcols, 1, pos)
        it = [0]

        def fn():
            fn1(Bs[it[0] % rotate]); it[0] += 1
        ms_, _, st_ = _events_time(torch, fn, steps, warmup)
        fl = 2.0 * M * N * K
        if hbm:
            eb = a_.element_size()
            nbytes = (M * K + K * N) * eb + M * N * c_.element_size()
            roof = _roof_bytes(nbytes, ms_, TRAFFIC_BYTES.get(name))
            roof["tflops"] = round(fl / (ms_ * 1e-3) / 1e12, 3)
            roof["note"] = "%d weight matrices rotated to defeat the last-level cache" % rotate
        else:
            roof = _roof_flops(kind, fl, ms_, TRAFFIC_BYTES.get(name))
        add(name, kind, "GEMM M=%d N=%d K=%d%s%s%s" % (M, N, K, " fp32 out" if out32 and kind != "f32" else "", " (pre-packed B)" if packed else "",
                                                      " + interleaved RoPE over the first %d columns (head dim %d) in the same call" % (rope[1], rope[0]) if rope else ""),
            ms_, roof, st_)

    def attn_case(name, kind, Bn, H, S, D, extra=False):
        if not want(name, extra):
            return
        q = randn(Bn, H, S, D, kind=kind); k = randn(Bn, H, S, D, kind=kind); v = randn(Bn, H, S, D, kind=kind)
        o = torch.empty(Bn, H, S, D, device="cuda"); lse = torch.empty(Bn, H, S, device="cuda")
        sc = 1.0 / math.sqrt(D)
        if kind == "f32":
            fn = lambda: be.FlashAttentionV2(W(q), W(k), W(v), W(o), W(lse), Bn, H, S, S, D, sc, True)
        else:
            fn = lambda: be.FlashAttentionHalf(kind, W(q), W(k), W(v), W(o), W(lse), Bn, H, S, S, D, sc, True)
        ms_, _, st_ = _events_time(torch, fn, steps, warmup)
        exact = 4.0 * Bn * H * D * (S * (S + 1) / 2)
        roof = _roof_flops(kind, exact, ms_, TRAFFIC_BYTES.get(name))
        roof["tflops_full_matrix_convention"] = round(4.0 * Bn * H * S * S * D / (ms_ * 1e-3) / 1e12, 3)
        add(name, kind, "causal attention B=%d H=%d S=%d d=%d (fp32 softmax/accumulate, fp32 O + LSE)" % (Bn, H, S, D), ms_, roof, st_)

    def decode_case(name, kind, Bn, H, S, D, Hkv=0, rotate=1, extra=False):
        if not want(name, extra):
            return
        # Hkv: K/V heads of a grouped-query cache (0 = one per query head); rotate: distinct caches cycled through so that a cache
        # smaller than the 256 MB last-level cache is still read from HBM
        kvh = Hkv or H
        q = randn(Bn, H, 1, D, kind=kind)
        ks_ = [randn(Bn, kvh, S, D, kind=kind) for _ in range(rotate)]
        vs_ = [randn(Bn, kvh, S, D, kind=kind) for _ in range(rotate)]
        o = torch.empty(Bn, H, 1, D, device="cuda")
        sc = 1.0 / math.sqrt(D)
        it = [0]

        def fn():
            j = it[0] % rotate; it[0] += 1
            be.DecodeAttention(kind, W(q), W(ks_[j]), W(vs_[j]), W(o), Bn, H, S, D, sc, numKVHeads=kvh)
        ms_, _, st_ = _events_time(torch, fn, steps, warmup)
        nbytes = 2.0 * Bn * kvh * S * D * q.element_size()
        add(name, kind, "decode attention B=%d H=%d%s q_len=1 KV=%d d=%d, contiguous KV cache" % (Bn, H, " Hkv=%d" % kvh if Hkv else "", S, D), ms_,
            _roof_bytes(nbytes, ms_, TRAFFIC_BYTES.get(name)), st_)

    gemm_case("gemm_f32_1024", "f32", 1024, 1024, 1024, uniform_inputs=True)
    gemm_case("gemm_f32_proj", "f32", 4096, 3072, 768)
    gemm_case("gemm_f16_proj", "f16", 4096, 3072, 768)
    gemm_case("gemm_f16_proj_f32out", "f16", 4096, 3072, 768, out32=True)
    gemm_case("gemm_bf16_8192", "bf16", 8192, 8192, 8192)
    attn_case("attn_f32_prefill", "f32", 8, 12, 512, 64)
    attn_case("attn_f16_prefill", "f16", 4, 32, 2048, 128)
    attn_case("attn_bf16_prefill", "bf16", 4, 32, 2048, 128)
    decode_case("decode_bf16", "bf16", 32, 32, 4096, 128)
    gemm_case("gemm_bf16_decode_proj", "bf16", 32, 4096, 4096, hbm=True, rotate=12)
    # the decode step's concatenated [Wq|Wk|Wv] projection (SimdGemm.SgemmConcatenatedProjections), plain and with Q and K rotated in the same call
    gemm_case("gemm_bf16_decode_qkv", "bf16", 32, 12288, 4096, hbm=True, rotate=4)
    gemm_case("gemm_bf16_decode_qkv_rope", "bf16", 32, 12288, 4096, hbm=True, rotate=4, rope=(128, 8192, 4095))
    # shapes beside the listed configurations (run with --only NAME[,NAME...]): grouped-query decode, fp32 products with few rows,
    # a causal fp32 attention grid of several rounds
    decode_case("decode_bf16_gqa", "bf16", 32, 32, 4096, 128, Hkv=8, rotate=2, extra=True)
    decode_case("decode_f32_gqa", "f32", 32, 32, 4096, 128, Hkv=8, extra=True)
    gemm_case("gemm_f32_m16", "f32", 16, 4096, 4096, hbm=True, rotate=6, extra=True)
    gemm_case("gemm_f32_m128", "f32", 128, 4096, 4096, extra=True)
    # an output projection onto a vocabulary of odd width (rows of B off the 16-byte grid), plain and with the weight packed once
    gemm_case("gemm_bf16_vocab50257", "bf16", 64, 50257, 768, hbm=True, rotate=6, extra=True)
    gemm_case("gemm_bf16_vocab50257_packed", "bf16", 64, 50257, 768, hbm=True, rotate=6, extra=True, packed=True)
    attn_case("attn_f32_prefill_b32", "f32", 32, 12, 512, 64, extra=True)
    attn_case("attn_f16_prefill_d256", "f16", 2, 32, 2048, 256, extra=True)
    attn_case("attn_bf16_prefill_d256", "bf16", 2, 32, 2048, 256, extra=True)
    out["others"] = others

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_(generator=g)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ------------------------------------------------------------------ CPU baseline (bounded sample, about 20 s of host time)
    if not args.no_cpu:
        try:
            import numpy as np
            import oracle      # test infrastructure: used here only as the reported CPU baseline
            threads = min(oracle.max_threads(), os.cpu_count() or 1)
            rng = np.random.default_rng(0)

            def median_time(fn, reps):
                ts = []
                for _ in range(reps):
                    t0 = time.perf_counter(); fn(); ts.append(time.perf_counter() - t0)
                return sorted(ts)[len(ts) // 2]

            # headline workload, all host threads: the whole 8192^3 product, fp32 path on fp16-rounded inputs
            ah = rng.standard_normal((n, n)).astype(np.float16).astype(np.float32)
            bh = (0.02 * rng.standard_normal((n, n))).astype(np.float16).astype(np.float32)
            oracle.sgemm(ah[:256], bh, 256, n, n, threads=threads)    # warm-up
            tsec = median_time(lambda: oracle.sgemm(ah, bh, n, n, n, threads=threads), 5)
            # the same product on ONE thread, on a 256-row slab
            rows1 = 256
            oracle.sgemm(ah[:64], bh, 64, n, n, threads=1)
            t1 = median_time(lambda: oracle.sgemm(ah[:rows1], bh, rows1, n, n, threads=1), 3)
            # causal fp32 attention B8 H12 S512 d64 (the reference's per-(batch, head) loop of two SGEMMs around a softmax)
            Bn, Hn, Sn, Dn = 8, 12, 512, 64
            qa, ka, va = (rng.standard_normal((Bn, Hn, Sn, Dn)).astype(np.float32) for _ in range(3))
            oracle.attention_f32(qa, ka, va, 1.0 / math.sqrt(Dn), True, threads=threads)
            ta = median_time(lambda: oracle.attention_f32(qa, ka, va, 1.0 / math.sqrt(Dn), True, threads=threads), 5)
            ta1 = median_time(lambda: oracle.attention_f32(qa[:1], ka[:1], va[:1], 1.0 / math.sqrt(Dn), True, threads=1), 3)
            attn_flops = 4.0 * Bn * Hn * Dn * (Sn * (Sn + 1) / 2)
            out["cpu_baseline"] = {
                "value": round(2.0 * n * n * n / tsec / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": "C restatement of the reference SimdGemm (6x16 AVX2 FMA tile, Kc=512, 2-D tile parallelism) on the whole "
                          "8192 x 8192 x 8192 product (fp32 path on fp16-rounded inputs), median of 5, %.2f s each" % tsec,
                "one_thread": {"value": round(2.0 * rows1 * n * n / t1 / 1e12, 5), "unit": "TFLOP/s", "cores": 1,
                               "sample": "%d-row slab of the same product, median of 3, %.2f s each" % (rows1, t1)},
                "attention_f32_causal_B8_H12_S512_d64": {
                    "value": round(attn_flops / ta / 1e12, 5), "unit": "TFLOP/s (causal-exact FLOPs)", "cores": threads,
                    "ms": round(ta * 1e3, 3),
                    "one_thread_value": round(attn_flops / Bn / ta1 / 1e12, 5),
                    "sample": "C restatement of CpuEngine.FlashAttentionFloat (explicit K^T, two sequential SGEMMs per head around a "
                              "scalar-expf softmax, parallel over batch x head), median of 5; one thread: batch 0 only, median of 3"},
            }
        except Exception as ex:     # the baseline is a reported extra, never the product path
            out["cpu_baseline"] = {"value": None, "unit": "TFLOP/s", "cores": 0, "kind": "port", "sample": "failed: %r" % (ex,)}

    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
