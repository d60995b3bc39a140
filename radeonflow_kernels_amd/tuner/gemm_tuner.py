"""Brute-force plan sweep on one MI355X.

The reference tuner (tuner/gemm_tuner.py:317-534, tuner/gemm_batch.py:196-200) renders a C++ template per
configuration, compiles it for gfx942, runs each binary and pastes the winner into the launcher as a
DISPATCH_GEMM(...) line. Here nothing is recompiled: every kernel variant is already in libgemm.so and a plan
(variant, split_k, group_m) is passed to rf_fp8_gemm_ex at run time, so a sweep is a loop of timed launches.

  python -m radeonflow_kernels_amd.tuner.gemm_tuner --M 6144 --N 4608 --K 7168        one shape
  python -m radeonflow_kernels_amd.tuner.gemm_tuner --all [--extended] --emit          every known shape (and M = 16 ...
                                                                                       8192 for each of their (N, K)),
                                                                                       then rewrite csrc/tuned_plans.inc
  python -m radeonflow_kernels_amd.tuner.gemm_tuner --M .. --N .. --K .. --emit-file my.plans
                                                  append the winner to a plan file: rf_gemm_load_plans(path) or the
                                                  environment variable RF_GEMM_PLANS uses it without a rebuild
Results go to stdout and, with --out DIR, to DIR/gemm_<M>x<N>x<K>.json (all candidates, best first).
"""
import argparse
import json
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
PLANS_INC = os.path.join(os.path.dirname(HERE), "csrc", "tuned_plans.inc")

# the five benchmark configurations, then the reference's benchmark and test shapes
# (scripts/problems/gemm/task.yml:53-84 of the reference tree)
SHAPES = [
    (1024, 1536, 7168), (6144, 4608, 7168), (6144, 7168, 2048), (6144, 7168, 256), (1024, 576, 7168),
    (1024, 3072, 1536), (1024, 7168, 256), (1024, 7168, 2048), (1024, 4608, 7168), (1024, 7168, 2304),
    (1024, 512, 7168), (1024, 4096, 512), (6144, 1536, 7168), (6144, 3072, 1536), (6144, 576, 7168),
    (6144, 7168, 2304), (6144, 512, 7168), (6144, 4096, 512),
    (64, 64, 128), (64, 1536, 7168), (64, 3072, 1536), (64, 576, 7168), (96, 7168, 256), (96, 7168, 2048),
    (96, 4608, 7168), (128, 7168, 2304), (128, 512, 7168), (512, 4096, 512), (512, 1536, 7168),
]
# token counts a server sees, over the (N, K) pairs of the shapes above (--extended)
EXTENDED_M = (16, 32, 48, 64, 96, 128, 192, 256, 384, 512, 768, 1024, 1536, 2048, 3072, 4096, 6144, 8192)
EXTENDED = [(m, n, k) for (n, k) in sorted({(n, k) for _, n, k in SHAPES if (n, k) != (64, 128)}) for m in EXTENDED_M
            if (m, n, k) not in SHAPES]
SPLITS = (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 16)
GROUPS = (4, 8, 16)


def _inputs(m, n, k):
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(m * 7 + n * 3 + k)
    a = torch.randint(0, 120, (k, m), dtype=torch.uint8, device=dev, generator=g).view(torch.float8_e4m3fn).T
    b = torch.randint(0, 120, (k, n), dtype=torch.uint8, device=dev, generator=g).view(torch.float8_e4m3fn).T
    sa = (torch.rand((k // 128, m), device=dev, generator=g) * 0.01 + 0.001).T
    sb = (torch.rand((k // 128, (n + 127) // 128), device=dev, generator=g) * 0.01 + 0.001).T
    c = torch.zeros((m, n), dtype=torch.bfloat16, device=dev)
    return a, b, sa, sb, c


def _time(rfk, args, cfg, iters):
    # timed inside the library: a Python call costs more than the GPU time of the small shapes
    return rfk.fp8_mm_time(*args, config=cfg, warmup=3, iters=iters)


def tune_shape(rfk, m, n, k, log=print):
    """Times every usable plan; returns a list of dicts sorted by time."""
    args = _inputs(m, n, k)
    default = rfk.select_config(m, n, k)
    if default.variant < 0:
        log("%dx%dx%d: bounds-checked kernel only (M or N not a multiple of 16)" % (m, n, k))
        return []
    flop = 2.0 * m * n * k
    # clocks ramp up over tens of milliseconds of load: warm up with the default plan before comparing
    t_est = _time(rfk, args, None, 20)
    _time(rfk, args, None, max(20, int(60e3 / max(t_est, 1.0))))
    iters = max(20, min(400, int(20e3 / max(t_est, 1.0))))
    rfk.fp8_mm(*args)
    torch.cuda.synchronize()
    ref = args[4].clone()
    out = []
    ncu = torch.cuda.get_device_properties(0).multi_processor_count
    for v in rfk.variants():
        tiles = -(-m // v["block_m"]) * -(-n // v["block_n"])
        # schedules: 0 = one workgroup per tile (with K splits), 1 = stream-K, 2 = persistent whole tiles,
        # 3 = persistent with a last round of half tiles, 4 = skinny K (K = 128 ... 512; listed under variant 0)
        for split, sk in [(sp, 0) for sp in SPLITS] + [(1, 1), (1, 2), (1, 3), (1, 4)]:
            if split > k // 128 or (sk == 1 and (tiles < ncu or not v["stream_k"])):
                continue
            if sk == 0 and not rfk.plan_can_run(v, split, k):
                continue
            if sk in (2, 3) and (not v["persistent"] or m < v["block_m"] or m % 16 or n % v["block_n"] or (k // 128) % 2):
                continue
            if sk == 4 and (v["variant"] != 0 or k > 512 or m % 16 or n % 64):
                continue
            if sk == 3:
                left = tiles % ncu
                if v["variant"] != 0 or tiles < ncu or left == 0 or (left + 7) // 8 * 8 + left > ncu:
                    continue
            for gm in (GROUPS if sk != 4 else GROUPS[1:2]):          # the skinny-K schedule has no tile order to group
                cfg = rfk.GemmConfig(v["variant"], split, gm, sk)
                args[4].zero_()
                us = _time(rfk, args, cfg, iters)
                # every plan must reproduce the default plan's output up to split-K reassociation
                err = (args[4].float() - ref.float()).abs().max().item()
                scale = ref.float().abs().max().item() + 1e-30
                out.append(dict(variant=v["variant"], block_m=v["block_m"], block_n=v["block_n"], split_k=split,
                                group_m=gm, stream_k=sk, us=round(us, 2), tflops=round(flop / us / 1e6, 1),
                                max_abs_dev_vs_default=err, ok=bool(err <= 2e-2 * scale)))
    out = [o for o in out if o["ok"]]
    out.sort(key=lambda o: o["us"])
    return out


def best_for_table(cands):
    """The winner that goes into a plan table or plan file: the fastest candidate that is not a stream-K plan. Whether
    stream-K can run depends on the compute-unit count of the device (it needs at least one tile per unit), so a table
    that may be read on another device does not carry it; it stays available through an explicit rf_gemm_config."""
    for c in cands:
        if c["stream_k"] != 1:
            return c
    return None


def emit_plans(results, path=PLANS_INC):
    lines = ["// Generated by radeonflow_kernels_amd/tuner/gemm_tuner.py --all [--extended] --emit on one MI355X; do not edit by hand.",
             "// {M, N, K, variant, split_k, group_m, stream_k},   best time, TFLOP/s"]
    for (m, n, k), cands in results.items():
        b = best_for_table(cands)
        if b is None:
            continue
        lines.append("{%d, %d, %d, %d, %d, %d, %d},   // %.2f us, %.1f TFLOP/s" % (
            m, n, k, b["variant"], b["split_k"], b["group_m"], b["stream_k"], b["us"], b["tflops"]))
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--M", type=int)
    ap.add_argument("--N", type=int)
    ap.add_argument("--K", type=int)
    ap.add_argument("--all", action="store_true")
    ap.add_argument("--extended", action="store_true", help="with --all: also M = 16 ... 8192 for every (N, K) of the list")
    ap.add_argument("--emit", nargs="?", const=PLANS_INC, default=None, metavar="PATH",
                    help="rewrite csrc/tuned_plans.inc, or PATH if given (rebuild libgemm.so afterwards)")
    ap.add_argument("--emit-file", default=None, help="append the best plan of every tuned shape to this plan file")
    ap.add_argument("--out", default=None)
    ap.add_argument("--part", default=None, metavar="I/N", help="with --all: only every N-th shape, starting at the I-th (a sweep in N runs)")
    a = ap.parse_args()
    sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
    import radeonflow_kernels_amd as rfk
    rfk.lib()
    shapes = (SHAPES + (EXTENDED if a.extended else [])) if a.all else [(a.M, a.N, a.K)]
    if a.part:
        i, n_parts = (int(x) for x in a.part.split("/"))
        shapes = shapes[i::n_parts]
    results = {}
    for (m, n, k) in shapes:
        cands = tune_shape(rfk, m, n, k)
        results[(m, n, k)] = cands
        if cands:
            b, w = cands[0], cands[-1]
            d = rfk.select_config(m, n, k)
            print("%5d x %5d x %5d: best %8.2f us (%7.1f TFLOP/s) variant %d split %d group %d stream_k %d | slowest "
                  "%.2f us | default plan (%d,%d,%d,%d)" % (m, n, k, b["us"], b["tflops"], b["variant"], b["split_k"],
                                                         b["group_m"], b["stream_k"], w["us"], d.variant, d.split_k,
                                                         d.group_m, d.stream_k), flush=True)
        if a.out and cands:
            os.makedirs(a.out, exist_ok=True)
            with open(os.path.join(a.out, "gemm_%dx%dx%d.json" % (m, n, k)), "w") as f:
                json.dump(cands, f, indent=1)
    if a.emit:
        emit_plans(results, a.emit)
        print("wrote", a.emit)
    if a.emit_file:
        with open(a.emit_file, "a") as f:
            for (m, n, k), cands in results.items():
                b = best_for_table(cands)
                if b is not None:
                    f.write("%d %d %d %d %d %d %d   # %.2f us, %.1f TFLOP/s\n" % (
                        m, n, k, b["variant"], b["split_k"], b["group_m"], b["stream_k"], b["us"], b["tflops"]))
        print("appended to", a.emit_file)


if __name__ == "__main__":
    main()
