#!/usr/bin/env python3
"""Benchmark of the FP8 blockwise-scaled GEMM on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config Cx] [--all] [--no-cpu]

A step is one GEMM of the headline shape (M=6144, N=4608, K=7168) on synthetic inputs that are
already resident in HBM (seeded N(0,1) fp32, quantised to e4m3fn with amax/448 block scales).
`value` comes from K back-to-back launches between two HIP events on the launch stream, issued by
the library's own launch loop with no host gap after a clock-settling phase (`settle_launches`, about
0.4 s of the same launch, whatever --warmup says: the shader clock and the board power need tens of
milliseconds of load to reach their steady state) and W warm-up launches. The first K launches of
the process after only W warm-up launches are reported beside it (`cold_clock_burst`). The line also
carries the min / median of individually timed launches, a run with operands rotated out of the
Infinity Cache, the roofline fraction, the CPU baseline, the correctness gate against the oracle and,
without --config, `all_configs`: time, roofline fraction and correctness gate of all five
configurations. With --config Cx only that configuration is run (this is the form the rocprofv3
summaries under profiles/ are taken with). --all adds quantisers, the grouped form, operand-bit
variations and the register-only MFMA ceiling. Prints ONE JSON line on stdout; tables go to stderr.
"""
import glob
import hashlib
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0      # MI355X published dense fp8 MFMA peak
PEAK_HBM_GBS = 8000.0         # MI355X published HBM3E bandwidth

CONFIGS = {
    "C1": (1024, 1536, 7168, 8135),
    "C2": (6144, 4608, 7168, 65436),
    "C3": (6144, 7168, 2048, 76547),
    "C4": (6144, 7168, 256, 764243),
    "C5": (1024, 576, 7168, 12346),
}
# measured only when named with --config (not part of the default run): a shape whose last round of 256x256 tiles is
# a quarter full, the automatic plan of which is the persistent schedule with a last round of half tiles
EXTRA_CONFIGS = {
    "H1": (8192, 4608, 7168, 4321),
}
RTOL, ATOL, ATOL_REFERENCE = 2e-2, 1e-2, 1e-3
SETTLE_SECONDS = 0.4
KERNEL_SOURCES = ("fp8_gemm_kernels.h", "fp8_gemm_persistent.h", "fp8_gemm_skinny.h", "gemm_launcher.hip")


def kernel_source_sha():
    """Short hash of the GEMM kernel sources: a traffic figure in profiles/ belongs to the kernels it was measured on."""
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "radeonflow_kernels_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:12]


def measured_traffic(config, cfg):
    """HBM-side bytes per GEMM, summed over every kernel the plan launches (a split-K plan: the partial-sum kernel and
    the reduction), from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summaries under profiles/ (lines
    '@traffic config=C2 plan=0,1,2 fetch_kib=... write_kib=... fetch_factor=... write_factor=... source_sha=...').
    Returns (bytes, note), or (None, why) when there is no summary for this configuration and plan or when the kernel
    sources have changed since it was taken."""
    plan = "%d,%d,%d" % (cfg.variant, cfg.split_k, cfg.stream_k)
    why = "no rocprofv3 traffic summary for %s under profiles/" % config
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.txt"))):
        for line in open(path):
            if not line.startswith("@traffic"):
                continue
            kv = dict(x.split("=", 1) for x in line.split()[1:])
            if kv.get("config") != config:
                continue
            if kv.get("plan") != plan:
                why = "%s was taken with plan %s, this run uses %s" % (os.path.basename(path), kv.get("plan"), plan)
                continue
            if kv.get("source_sha") != kernel_source_sha():
                why = "%s was taken on other kernel sources (%s, now %s)" % (os.path.basename(path), kv.get("source_sha"),
                                                                            kernel_source_sha())
                continue
            fetch = float(kv["fetch_kib"]) * float(kv["fetch_factor"]) * 1024
            write = float(kv["write_kib"]) * float(kv["write_factor"]) * 1024
            return fetch + write, "fetch %.1f MB + write %.1f MB per GEMM (all its kernels), profiles/%s" % (
                fetch / 1e6, write / 1e6, os.path.basename(path))
    return None, why


def algorithmic_bytes(m, n, k):
    qk, qn = k // 128, (n + 127) // 128
    return m * k + n * k + 2 * m * n + 4 * m * qk + 4 * qn * qk


def to_gpu(data):
    a, b, sa, sb, c = data

    def colmajor(t):
        return t.T.contiguous().cuda().T
    return colmajor(a), colmajor(b), colmajor(sa), colmajor(sb), torch.zeros(c.shape, dtype=torch.bfloat16, device="cuda")


def settled_us(rfk, g, steps, warmup, settle_seconds=SETTLE_SECONDS):
    """Average microseconds per GEMM over `steps` launches, after a settling phase of about `settle_seconds` of the same
    launch plus `warmup` launches. Everything is enqueued back to back by one call of the library's launch loop
    (rf_fp8_gemm_time: HIP events on the launch stream around the last `steps` launches), so there is no host gap
    between settling and timing. Returns (us, settle_launches)."""
    est = rfk.fp8_mm_time(*g, warmup=1, iters=3)
    settle = max(1, int(settle_seconds * 1e6 / max(est, 1.0)))
    torch.cuda.synchronize()
    us = rfk.fp8_mm_time(*g, warmup=settle + warmup, iters=steps)
    torch.cuda.synchronize()
    return us, settle


def time_gemm(rfk, sets, steps, warmup, stream):
    """Average microseconds per GEMM over `steps` back-to-back launches from Python, HIP events on the launch stream.
    `sets` is a list of operand tuples used in rotation (one tuple: operands stay warm in L2 / Infinity Cache)."""
    with torch.cuda.stream(stream):
        for i in range(warmup):
            rfk.fp8_mm(*sets[i % len(sets)])
        stream.synchronize()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(steps):
            rfk.fp8_mm(*sets[i % len(sets)])
        e1.record(stream)
        stream.synchronize()
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / steps


def cold_operands_us(rfk, g, m, n, k, steps, warmup, stream):
    """Microseconds per GEMM with operands that are not in the 256 MB Infinity Cache: enough copies of the operand set
    in rotation that a set is evicted before its turn comes again. Returns (us, copies, bytes of all copies)."""
    set_bytes = algorithmic_bytes(m, n, k)
    ncopies = max(3, int(2 * 256e6 / set_bytes) + 1)
    sets = [g] + [tuple(t.clone() for t in g) for _ in range(ncopies - 1)]
    us = time_gemm(rfk, sets, max(steps, 2 * ncopies), max(warmup, 2 * ncopies), stream)
    del sets
    return us, ncopies, ncopies * set_bytes


def roofline_of_work(flop, nbytes, us):
    """The same for any launch given its algorithmic FLOP and bytes (the grouped form: every expert's weights, every
    row of A and of C once)."""
    tflops, gbs = flop / us / 1e6, nbytes / us / 1e3
    if flop / (PEAK_FP8_TFLOPS * 1e12) >= nbytes / (PEAK_HBM_GBS * 1e9):
        return {"bound": "mfma", "achieved": round(tflops, 2), "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                "frac": round(tflops / PEAK_FP8_TFLOPS, 4), "algorithmic_flop": flop, "algorithmic_bytes": nbytes}
    return {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": round(gbs / PEAK_HBM_GBS, 4), "algorithmic_flop": flop, "algorithmic_bytes": nbytes}


def roofline_of(m, n, k, us):
    """The roofline that bounds the shape (the larger of flop / fp8 peak and algorithmic bytes / HBM peak) and the
    fraction of it a launch of `us` microseconds reaches."""
    flop, nbytes = 2.0 * m * n * k, algorithmic_bytes(m, n, k)
    tflops, gbs = flop / us / 1e6, nbytes / us / 1e3
    if flop / (PEAK_FP8_TFLOPS * 1e12) >= nbytes / (PEAK_HBM_GBS * 1e9):
        return {"bound": "mfma", "achieved": round(tflops, 2), "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                "frac": round(tflops / PEAK_FP8_TFLOPS, 4)}
    return {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": round(gbs / PEAK_HBM_GBS, 4)}


def clock_under_load(rfk, g, seconds, us_per_launch):
    """Shader clock and board power while the GEMM runs back to back for `seconds`, read from the amdgpu driver's
    sysfs files (pp_dpm_sclk, hwmon power1_input / power1_average) by a polling thread; the launches are issued by
    the library's own timing loop, which does not hold the interpreter lock. None where the files cannot be read."""
    import glob
    import threading
    cards = [c for c in sorted(glob.glob("/sys/class/drm/card*/device")) if os.path.exists(c + "/pp_dpm_sclk")]
    if not cards:
        return None

    def sample():
        best = None
        for card in cards:
            try:
                cur = [l for l in open(card + "/pp_dpm_sclk").read().splitlines() if l.rstrip().endswith("*")]
                mhz = float(cur[0].split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
                watts = None
                for f in glob.glob(card + "/hwmon/hwmon*/power1_input") + glob.glob(card + "/hwmon/hwmon*/power1_average"):
                    watts = float(open(f).read()) / 1e6
                    break
            except (OSError, ValueError, IndexError):
                continue
            if best is None or mhz > best[0]:
                best = (mhz, watts)
        return best

    got, done = [], threading.Event()

    def poll():
        while not done.is_set():
            v = sample()
            if v:
                got.append(v)
            time.sleep(0.02)

    t = threading.Thread(target=poll)
    t.start()
    try:
        us = rfk.fp8_mm_time(*g, warmup=20, iters=max(50, int(seconds * 1e6 / us_per_launch)))
    finally:
        done.set()
        t.join()
    got = got[len(got) // 3:]            # the clock needs tens of milliseconds to settle
    if not got:
        return None
    watts = [w for _, w in got if w is not None]
    mhz = sum(v for v, _ in got) / len(got)
    return {"sclk_mhz": round(mhz, 1), "power_w": round(sum(watts) / len(watts), 1) if watts else None,
            "us_per_gemm": round(us, 2), "samples": len(got),
            "fp8_peak_at_this_clock_tflops": round(PEAK_FP8_TFLOPS * mhz / 2400.0, 1),
            "source": "sysfs pp_dpm_sclk and hwmon power, mean over the last two thirds of %.1f s of back-to-back launches" % seconds}


def per_launch_us(rfk, g, launches, stream):
    """Each launch bracketed by its own pair of HIP events (clocks already warm): list of microseconds."""
    with torch.cuda.stream(stream):
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(launches)]
        for a, b in ev:
            a.record(stream)
            rfk.fp8_mm(*g)
            b.record(stream)
        stream.synchronize()
    return [a.elapsed_time(b) * 1e3 for a, b in ev]


def parity_report(rfk, cref, rk, data, g, stream, expect=None, truth_rows=64):
    """Kernel output against the oracle (dequantise, fp32 matmul, bf16) at the graded tolerance and at the reference
    harness's atol, plus the largest error against an fp64 evaluation on a sample of rows."""
    a, b, sa, sb, c = data
    m, n = c.shape
    if expect is None:
        expect = rk.ref_kernel((a, b, sa, sb, torch.zeros((m, n), dtype=torch.bfloat16)))
    with torch.cuda.stream(stream):
        g[4].zero_()
        rfk.fp8_mm(*g)
        stream.synchronize()
    got = g[4].cpu()
    gb, eb = got.view(torch.uint16).numpy(), expect.view(torch.uint16).numpy()
    bad, mx, _ = cref.allclose(gb, eb, RTOL, ATOL)
    bad_ref, _, _ = cref.allclose(gb, eb, RTOL, ATOL_REFERENCE)
    rows = np.unique(np.linspace(0, m - 1, min(truth_rows, m)).astype(np.int64))
    truth = cref.ref_gemm_f64(*rk.raw_layouts(data), rows=rows)
    err64 = float(np.max(np.abs(got.float().numpy()[rows].astype(np.float64) - truth)))
    return {"rtol": RTOL, "atol": ATOL, "mismatches": bad, "max_abs_err": round(mx, 5),
            "mismatches_at_reference_atol_1e-3": bad_ref, "max_abs_err_vs_fp64_on_%d_rows" % len(rows): round(err64, 5),
            "elements": int(m * n), "pass": bad == 0}


def measure_config(rfk, cref, rk, name, steps, warmup, stream, with_cpu, settle_seconds, keep=False, cold_too=True):
    """One configuration: inputs, settled launch time, roofline fraction, correctness gate. Returns the record (and
    the inputs with keep=True)."""
    m, n, k, seed = {**CONFIGS, **EXTRA_CONFIGS}[name]
    t0 = time.time()
    data = rk.generate_input_blockquant(m, n, k, seed)
    g = to_gpu(data)
    gen_s = time.time() - t0
    cold = rfk.fp8_mm_time(*g, warmup=warmup, iters=steps) if keep else None     # the process's first launches
    us, settle = settled_us(rfk, g, steps, warmup, settle_seconds)
    cfg = rfk.select_config(m, n, k)
    schedule = {0: "gemm_fp8_blockscale_tile", 1: "gemm_fp8_blockscale_streamk", 2: "gemm_fp8_blockscale_persistent",
                3: "gemm_fp8_blockscale_persistent with a last round of half tiles", 4: "gemm_fp8_blockscale_skinny"}
    launches = 1 if cfg.split_k == 1 else 2
    rec = {"shape": [m, n, k], "us_per_gemm": round(us, 2), "settle_launches": settle,
           "tflops": round(2.0 * m * n * k / us / 1e6, 1), "gbs_algorithmic": round(algorithmic_bytes(m, n, k) / us / 1e3, 1),
           "roofline": roofline_of(m, n, k, us),
           "plan": {"variant": cfg.variant, "split_k": cfg.split_k, "group_m": cfg.group_m, "stream_k": cfg.stream_k},
           "kernel": "%s (variant %d, split_k %d)%s" % (schedule.get(cfg.stream_k, "?"), cfg.variant, cfg.split_k,
                                                         " + reduce_splitk_bf16" if launches == 2 else ""),
           "kernel_launches_per_gemm": launches}
    traffic, note = measured_traffic(name, cfg)
    rec["roofline"]["traffic"] = traffic
    rec["roofline"]["traffic_note"] = note
    if cold_too:
        us_cold, ncopies, nbytes = cold_operands_us(rfk, g, m, n, k, max(steps, 50), max(warmup, 50), stream)
        rec["cold_operands"] = {"us_per_gemm": round(us_cold, 2), "frac": roofline_of(m, n, k, us_cold)["frac"],
                                "note": "%d operand sets in rotation (%.0f MB > 256 MB Infinity Cache), launches from Python"
                                        % (ncopies, nbytes / 1e6)}
    expect = cpu_s = None
    if with_cpu:
        a, b, sa, sb, c = data
        if keep:
            # CPU baseline = the oracle's torch restatement of the reference path (dequantise, fp32 matmul, bf16) on
            # the host cores, whole workload, best of 3 after a small warm-up
            rk.ref_kernel((a[:128], b, sa[:128], sb, torch.zeros((128, n), dtype=torch.bfloat16)))
            cpu_s = float("inf")
            for _ in range(3):
                t0 = time.perf_counter()
                expect = rk.ref_kernel((a, b, sa, sb, torch.zeros((m, n), dtype=torch.bfloat16)))
                cpu_s = min(cpu_s, time.perf_counter() - t0)
        par = parity_report(rfk, cref, rk, data, g, stream, expect)
        rec["parity"] = par if keep else {"mismatches": par["mismatches"],
                                          "mismatches_at_reference_atol_1e-3": par["mismatches_at_reference_atol_1e-3"],
                                          "max_abs_err": par["max_abs_err"], "elements": par["elements"], "pass": par["pass"]}
    if keep:
        return rec, data, g, gen_s, cold, cpu_s
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=200, help="untimed launches directly before the timed ones")
    ap.add_argument("--config", default=None, choices=sorted(CONFIGS) + sorted(EXTRA_CONFIGS),
                    help="run only this configuration (default: C2 as the headline plus all_configs)")
    ap.add_argument("--all", action="store_true", help="also quantisers, grouped form, operand bits, MFMA ceiling")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and the parity gate")
    ap.add_argument("--settle", type=float, default=SETTLE_SECONDS, help="seconds of launches before the timed region")
    ap.add_argument("--no-clock", action="store_true", help="skip the 0.6 s clock and power read-out (shorter profiler traces)")
    ap.add_argument("--timed-only", action="store_true",
                    help="with --config: stop after the settled, timed launches (for profiler runs: the last --steps "
                         "launches of the trace are then exactly the timed region)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (output tiles are independent: "
              "several GPUs would each take a range of rows or columns, with no exchange)" % args.gpus, file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2

    import radeonflow_kernels_amd as rfk
    rfk.lib()        # fails loudly if libgemm.so is missing
    from oracle import cref, ref_kernel as rk      # checker + CPU baseline only

    prop = torch.cuda.get_device_properties(0)
    clock_mhz = getattr(prop, "clock_rate", 2400000) / 1e3
    derived_peak = prop.multi_processor_count * clock_mhz * 1e6 * 8192 / 1e12
    stream = torch.cuda.Stream()

    headline = args.config or "C2"
    m, n, k, seed = {**CONFIGS, **EXTRA_CONFIGS}[headline]
    if args.timed_only:
        if not args.config:
            print("bench.py: --timed-only needs --config", file=sys.stderr)
            return 2
        mm, nn, kk, seed_ = {**CONFIGS, **EXTRA_CONFIGS}[args.config]
        gg = to_gpu(rk.generate_input_blockquant(mm, nn, kk, seed_))
        us_, settle_ = settled_us(rfk, gg, args.steps, args.warmup, args.settle)
        cfg_ = rfk.select_config(mm, nn, kk)
        print(json.dumps({"config": args.config, "us_per_gemm": round(us_, 2), "steps": args.steps, "warmup": args.warmup,
                          "settle_launches": settle_, "roofline": roofline_of(mm, nn, kk, us_),
                          "plan": {"variant": cfg_.variant, "split_k": cfg_.split_k, "group_m": cfg_.group_m,
                                   "stream_k": cfg_.stream_k}}))
        return 0
    rec, data, g, gen_s, us_burst, cpu_s = measure_config(rfk, cref, rk, headline, args.steps, args.warmup, stream,
                                                          not args.no_cpu, args.settle, keep=True, cold_too=False)
    us = rec["us_per_gemm"]
    flop = 2.0 * m * n * k
    tflops = flop / us / 1e6
    with torch.cuda.stream(stream):
        rfk.fp8_mm_time(*g, warmup=rec["settle_launches"] // 2, iters=1)      # the clock falls back within milliseconds
    samples = sorted(per_launch_us(rfk, g, max(20, min(args.steps, 200)), stream))
    us_cold, ncopies, cold_bytes = cold_operands_us(rfk, g, m, n, k, max(args.steps, 50), max(args.warmup, 50), stream)
    rec["cold_operands"] = {"us_per_gemm": round(us_cold, 2), "frac": roofline_of(m, n, k, us_cold)["frac"],
                            "note": "%d operand sets in rotation (%.0f MB > 256 MB Infinity Cache), launches from Python"
                                    % (ncopies, cold_bytes / 1e6)}
    roofline = dict(rec["roofline"])
    roofline["kernel"] = rec["kernel"]
    roofline["avg_launch_us"] = round(us, 2)
    roofline["algorithmic_flop_per_launch"] = flop
    roofline["algorithmic_bytes_per_launch"] = algorithmic_bytes(m, n, k)

    out = {
        "metric": "TFLOP/s per blockscaled fp8 GEMM (M=%d,N=%d,K=%d)" % (m, n, k),
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "settle_launches": rec["settle_launches"],
        "ms_per_step": round(us / 1e3, 5), "us_per_gemm": round(us, 2),
        "us_min": round(samples[0], 2), "us_median": round(samples[len(samples) // 2], 2),
        "cold_clock_burst": {"us_per_gemm": round(us_burst, 2), "tflops": round(flop / us_burst / 1e6, 2),
                             "note": "the first %d launches of the process after %d warm-up launches: shader clock and "
                                     "board power have not reached their state under load" % (args.steps, args.warmup)},
        "cold_operands": {"us_per_gemm": round(us_cold, 2), "tflops": round(flop / us_cold / 1e6, 2),
                          "pct_fp8_mfma_peak": round(100 * flop / us_cold / 1e6 / PEAK_FP8_TFLOPS, 2),
                          "note": "%d operand sets in rotation (%.0f MB > 256 MB Infinity Cache)"
                                  % (ncopies, cold_bytes / 1e6)},
        "pct_fp8_mfma_peak": round(100 * tflops / PEAK_FP8_TFLOPS, 2),
        "achieved_hbm_gbs_algorithmic": rec["gbs_algorithmic"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3fn",
        "data": "synthetic (seeded N(0,1) fp32 -> e4m3fn, amax/448 block scales), random inputs resident in HBM",
        "config": {"workload": "%s: blockscaled fp8 GEMM M=%d N=%d K=%d, a[K][M] b[K][N] fp8, fp32 scales, bf16 C"
                               % (headline, m, n, k),
                   "plan": rec["plan"],
                   "device": prop.name, "compute_units": prop.multi_processor_count, "clock_mhz": clock_mhz,
                   "derived_fp8_peak_tflops": round(derived_peak, 1), "input_generation_s": round(gen_s, 2),
                   "kernel_source_sha": kernel_source_sha()},
        "roofline": roofline,
    }

    if not args.no_clock:
        with torch.cuda.stream(stream):
            out["clock_under_load"] = clock_under_load(rfk, g, 0.6, us)

    if not args.no_cpu:
        out["cpu_baseline"] = {"value": round(flop / cpu_s / 1e12, 4), "unit": "TFLOP/s",
                               "cores": torch.get_num_threads(), "kind": "port", "seconds": round(cpu_s, 2),
                               "host_cpu_count": os.cpu_count(),
                               "sample": "whole %s workload, best of 3 runs (dequantise + fp32 matmul + bf16 cast), torch CPU" % headline}
        out["parity"] = rec["parity"]

    if args.config is None:
        # all five configurations: settled time, roofline fraction and the same correctness gate
        print("%-3s %-16s %9s %9s %9s %6s %6s %9s %9s  %s" % ("cfg", "shape", "us", "us cold", "TFLOP/s", "bound", "frac",
              "bad@1e-2", "bad@1e-3", "plan"), file=sys.stderr)
        out["all_configs"] = {}
        for name in sorted(CONFIGS):
            if name == headline:
                r = {x: rec[x] for x in rec if x != "parity"}
                if "parity" in rec:
                    r["parity"] = {x: rec["parity"][x] for x in ("mismatches", "mismatches_at_reference_atol_1e-3",
                                                                  "max_abs_err", "elements", "pass")}
            else:
                r = measure_config(rfk, cref, rk, name, args.steps, args.warmup, stream, not args.no_cpu,
                                   min(args.settle, 0.25))
            out["all_configs"][name] = r
            par = r.get("parity")
            print("%-3s %-16s %9.2f %9.2f %9.1f %6s %6.3f %9s %9s  %r" % (
                name, "%dx%dx%d" % tuple(r["shape"]), r["us_per_gemm"], r["cold_operands"]["us_per_gemm"], r["tflops"],
                r["roofline"]["bound"],
                r["roofline"]["frac"], par["mismatches"] if par else "-",
                par["mismatches_at_reference_atol_1e-3"] if par else "-", r["plan"]), file=sys.stderr)

    if args.all:
        # the block quantisers that produce the operands (HBM-bound: source read once, fp8 + scales written once)
        out["quantisers"] = {}
        for label, fn, rows in (("quantize_a", rfk.quantize_a, m), ("quantize_b", rfk.quantize_b, n)):
            for dt in (torch.float32, torch.bfloat16):
                src = torch.randn((rows, k), device="cuda", dtype=dt)
                with torch.cuda.stream(stream):
                    for _ in range(10):
                        fn(src)
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(stream)
                    for _ in range(20):
                        fn(src)
                    e1.record(stream)
                    stream.synchronize()
                u = e0.elapsed_time(e1) * 1e3 / 20
                nbytes = rows * k * (src.element_size() + 1) + 4 * (k // 128) * (rows if label == "quantize_a" else (rows + 127) // 128)
                key = "%s_%s_%dx%d" % (label, "f32" if dt == torch.float32 else "bf16", rows, k)
                out["quantisers"][key] = {"us": round(u, 2), "gbs": round(nbytes / u / 1e3, 1),
                                          "pct_hbm_peak": round(100 * nbytes / u / 1e3 / PEAK_HBM_GBS, 2)}
                print("%-34s %8.2f us %8.1f GB/s (%.1f %% of 8 TB/s; includes the allocation of the outputs by torch)"
                      % (key, u, nbytes / u / 1e3, 100 * nbytes / u / 1e3 / PEAK_HBM_GBS), file=sys.stderr)
                del src
        # grouped form (expert GEMMs after sorting tokens by expert): 32 groups of uneven size, N=4096, K=7168
        rng = np.random.default_rng(1)
        cuts = np.sort(rng.choice(np.arange(1, 8192 // 16), 31, replace=False)) * 16
        offs = [0] + [int(x) for x in cuts] + [8192]
        gm, gn, gk, gg = 8192, 4096, 7168, 32
        fp8 = torch.float8_e4m3fn
        ga = torch.randint(0, 120, (gk, gm), dtype=torch.uint8, device="cuda").view(fp8).T
        gb = torch.randint(0, 120, (gg, gk, gn), dtype=torch.uint8, device="cuda").view(fp8).permute(0, 2, 1)
        gsa = (torch.rand((gk // 128, gm), device="cuda") * 1e-2).T
        gsb = (torch.rand((gg, gk // 128, gn // 128), device="cuda") * 1e-2).permute(0, 2, 1)
        gc = torch.empty((gm, gn), dtype=torch.bfloat16, device="cuda")
        # the same groups with 0..15 rows fewer each (token counts are not multiples of 16): the same tiles, but A has
        # to be staged with every group padded to a multiple of 16 first
        sizes16 = [b_ - a_ for a_, b_ in zip(offs, offs[1:])]
        sizes_any = [max(1, sz - int(r)) for sz, r in zip(sizes16, rng.integers(0, 16, len(sizes16)))]
        offs_any = [0] + [int(x) for x in np.cumsum(sizes_any)]
        gm_any = offs_any[-1]
        ga_any = torch.randint(0, 120, (gk, gm_any), dtype=torch.uint8, device="cuda").view(fp8).T
        gsa_any = (torch.rand((gk // 128, gm_any), device="cuda") * 1e-2).T
        gc_any = torch.empty((gm_any, gn), dtype=torch.bfloat16, device="cuda")
        for key, offs_, ops_ in (("grouped", offs, (ga, gb, gsa, gsb, gc)),
                                 ("grouped_any_sizes", offs_any, (ga_any, gb, gsa_any, gsb, gc_any))):
            gm_ = offs_[-1]
            with torch.cuda.stream(stream):
                for _ in range(max(args.warmup // 4 + 5, 600)):       # ~0.2 s of the same launch: the clock has settled
                    rfk.fp8_mm_grouped(*ops_, offs_)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(50):
                    rfk.fp8_mm_grouped(*ops_, offs_)
                e1.record(stream)
                stream.synchronize()
            u = e0.elapsed_time(e1) * 1e3 / 50
            tf = 2.0 * gm_ * gn * gk / u / 1e6
            sizes = [b - a for a, b in zip(offs_, offs_[1:])]
            # every expert's weights are read once: with 256 rows per expert on average they are most of the bytes
            gbytes = gm_ * gk + gg * gn * gk + 2 * gm_ * gn + 4 * (gk // 128) * (gm_ + gg * (gn // 128))
            out[key] = {"workload": "32 groups, %d rows in total (%d..%d per group), N=%d K=%d" % (
                            gm_, min(sizes), max(sizes), gn, gk),
                        "us": round(u, 2), "tflops": round(tf, 1), "pct_fp8_mfma_peak": round(100 * tf / PEAK_FP8_TFLOPS, 2),
                        "algorithmic_mb": round(gbytes / 1e6, 1), "gbs": round(gbytes / u / 1e3, 1),
                        "pct_hbm_peak": round(100 * gbytes / u / 1e3 / PEAK_HBM_GBS, 2),
                        "roofline": roofline_of_work(2.0 * gm_ * gn * gk, gbytes, u)}
            print("%s %s: %.2f us  %.1f TFLOP/s (%.1f %% of the fp8 peak), %.0f GB/s algorithmic (%.1f %% of 8 TB/s)" % (
                  key, out[key]["workload"], u, tf, 100 * tf / PEAK_FP8_TFLOPS, gbytes / u / 1e3,
                  100 * gbytes / u / 1e3 / PEAK_HBM_GBS), file=sys.stderr)
        # arbitrary sizes again, with the activations quantised straight into the padded layout (quantize_a_grouped):
        # no staging copy at all
        xg = torch.randn((gm_any, gk), device="cuda", dtype=torch.bfloat16)
        with torch.cuda.stream(stream):
            a_pad, sa_pad = rfk.quantize_a_grouped(xg, offs_any)
            for _ in range(max(args.warmup // 4 + 5, 600)):
                rfk.fp8_mm_grouped_padded(a_pad, gb, sa_pad, gsb, gc_any, offs_any)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(50):
                rfk.fp8_mm_grouped_padded(a_pad, gb, sa_pad, gsb, gc_any, offs_any)
            e1.record(stream)
            stream.synchronize()
            u = e0.elapsed_time(e1) * 1e3 / 50
            e0.record(stream)
            for _ in range(20):
                rfk.quantize_a_grouped(xg, offs_any)
            e1.record(stream)
            stream.synchronize()
            uq = e0.elapsed_time(e1) * 1e3 / 20
        tf = 2.0 * gm_any * gn * gk / u / 1e6
        out["grouped_any_sizes_padded_layout"] = {
            "workload": out["grouped_any_sizes"]["workload"] + ", activations written by quantize_a_grouped",
            "us": round(u, 2), "tflops": round(tf, 1), "pct_fp8_mfma_peak": round(100 * tf / PEAK_FP8_TFLOPS, 2),
            "quantize_a_grouped_bf16_us": round(uq, 2),
            "roofline": roofline_of_work(2.0 * gm_any * gn * gk,
                                         gm_any * gk + gg * gn * gk + 2 * gm_any * gn + 4 * (gk // 128) * (gm_any + gg * (gn // 128)), u)}
        print("grouped_any_sizes_padded_layout: %.2f us  %.1f TFLOP/s (quantize_a_grouped bf16 -> padded layout: %.2f us, "
              "includes the allocation of its outputs by torch)" % (u, tf, uq), file=sys.stderr)
        del xg, a_pad, sa_pad, ga_any, gsa_any, gc_any
        # the reference's 18 benchmark shapes (scripts/problems/gemm/task.yml:66-84 of the reference tree; its contest
        # ranks by their geometric mean), random fp8 bytes and scales resident in HBM, automatic plan
        ref_shapes = [(1024, 1536, 7168), (1024, 3072, 1536), (1024, 576, 7168), (1024, 7168, 256), (1024, 7168, 2048),
                      (1024, 4608, 7168), (1024, 7168, 2304), (1024, 512, 7168), (1024, 4096, 512), (6144, 1536, 7168),
                      (6144, 3072, 1536), (6144, 576, 7168), (6144, 7168, 256), (6144, 7168, 2048), (6144, 4608, 7168),
                      (6144, 7168, 2304), (6144, 512, 7168), (6144, 4096, 512)]
        out["reference_benchmark_shapes"] = {}
        log_sum = 0.0
        for (bm_, bn_, bk_) in ref_shapes:
            qk_, qn_ = bk_ // 128, (bn_ + 127) // 128
            ops = (torch.randint(0, 120, (bk_, bm_), dtype=torch.uint8, device="cuda").view(fp8).T,
                   torch.randint(0, 120, (bk_, bn_), dtype=torch.uint8, device="cuda").view(fp8).T,
                   (torch.rand((qk_, bm_), device="cuda") * 1e-2).T, (torch.rand((qk_, qn_), device="cuda") * 1e-2).T,
                   torch.empty((bm_, bn_), dtype=torch.bfloat16, device="cuda"))
            with torch.cuda.stream(stream):
                u, _ = settled_us(rfk, ops, 50, 20, 0.1)
            log_sum += np.log(u)
            out["reference_benchmark_shapes"]["%dx%dx%d" % (bm_, bn_, bk_)] = round(u, 2)
            del ops
        out["reference_benchmark_shapes"]["geometric_mean_us"] = round(float(np.exp(log_sum / len(ref_shapes))), 2)
        print("the reference's 18 benchmark shapes: %r" % (out["reference_benchmark_shapes"],), file=sys.stderr)
        # the same launch with other operand bits (same shapes, scales and plan): the chip's clock under load depends
        # on how many bits toggle, so the time does too
        out["operand_bits"] = {"quantised_normal_us": round(us, 2)}
        for label in ("zeros", "random_bytes"):
            ops = []
            for t in g[:2]:
                x = torch.empty_like(t)
                u8 = x.view(torch.uint8)
                if label == "zeros":
                    u8.zero_()
                else:
                    u8.random_(0, 256)
                    u8[(u8 & 0x7F) == 0x7F] = 0           # no NaN codes
                ops.append(x)
            u = time_gemm(rfk, [(ops[0], ops[1]) + tuple(g[2:])], args.steps, args.warmup, stream)
            out["operand_bits"][label + "_us"] = round(u, 2)
            del ops
        print("C2 launch time by operand bits: %r" % (out["operand_bits"],), file=sys.stderr)
        # Calibration only (nothing of the product runs through it): what the vendor's library reaches on the headline
        # shape for a plain fp8 GEMM WITHOUT block scales (torch._scaled_mm: K-contiguous operands, one scale per tensor
        # or per row, so no fold per K block), on the same box in the same run. It says what "per cent of the published
        # peak" means for any fp8 GEMM under this chip's power limit.
        try:
            xm = torch.randn((m, k), device="cuda")
            wm = torch.randn((n, k), device="cuda")
            cal = {}
            for label, sx_, sw_ in (("per_tensor_scales", (xm.abs().amax() / 448).float(), (wm.abs().amax() / 448).float()),
                                    ("per_row_scales", (xm.abs().amax(dim=1, keepdim=True) / 448).float(),
                                     (wm.abs().amax(dim=1, keepdim=True) / 448).float())):
                a8_, b8_ = (xm / sx_).to(fp8), (wm / sw_).to(fp8)
                sb_ = sw_.t() if sw_.dim() == 2 else sw_
                fn_ = lambda: torch._scaled_mm(a8_, b8_.t(), scale_a=sx_, scale_b=sb_, out_dtype=torch.bfloat16)  # noqa: E731
                with torch.cuda.stream(stream):
                    for _ in range(2500):
                        fn_()
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(stream)
                    for _ in range(100):
                        fn_()
                    e1.record(stream)
                    stream.synchronize()
                u = e0.elapsed_time(e1) * 1e3 / 100
                cal[label] = {"us": round(u, 2), "tflops": round(flop / u / 1e6, 1),
                              "pct_fp8_mfma_peak": round(100 * flop / u / 1e6 / PEAK_FP8_TFLOPS, 2)}
            cal["note"] = ("torch._scaled_mm (the vendor's GEMM library) on %dx%dx%d, fp8 e4m3fn -> bf16, no block scales: "
                           "calibration of the target only, not a code path of this library" % (m, n, k))
            out["calibration_vendor_fp8_gemm_without_block_scales"] = cal
            print("calibration, vendor library, plain fp8 GEMM without block scales: %r" % (cal,), file=sys.stderr)
            del xm, wm
        except Exception as e:      # an installation without that routine or format: the calibration is simply absent
            print("calibration with torch._scaled_mm not available: %s" % str(e)[:200], file=sys.stderr)
        # what the chip sustains on the same MFMA instruction from registers alone (clock under its power limit);
        # run as a child process once the GEMM work above is done
        probe = os.path.join(ROOT, "bench_probes", "mfma_ceiling")
        if os.path.exists(probe):
            import subprocess
            torch.cuda.synchronize()
            r = subprocess.run([probe, "0.3"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)
            if r.returncode == 0:
                out["mfma_ceiling"] = json.loads(r.stdout.strip().splitlines()[-1])
                out["mfma_ceiling"]["gemm_pct_of_normal_ceiling"] = round(100 * out["value"] / out["mfma_ceiling"]["normal"], 2)
                out["mfma_ceiling"]["gemm_pct_of_ceiling_with_folds_and_lds_reads"] = round(
                    100 * out["value"] / out["mfma_ceiling"]["normal_with_folds_and_lds_reads"], 2)
                print("register-only MFMA ceiling: %r" % (out["mfma_ceiling"],), file=sys.stderr)
            else:
                print("mfma_ceiling failed: %s" % r.stderr.strip(), file=sys.stderr)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
