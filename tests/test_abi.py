"""CPU-only checks of the C ABI: libgemm.so loads, exports what include/rf_gemm.h declares, and rejects bad
arguments before touching a device."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "rf_gemm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(run|rf_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from radeonflow_kernels_amd import gemm
    lib = ctypes.CDLL(gemm.LIB_PATH)
    names = _declared_functions()
    assert "run" in names and "rf_fp8_gemm" in names and len(names) >= 10
    for n in names:
        assert hasattr(lib, n), "libgemm.so does not export %s" % n
    assert sorted(gemm.EXPORTS) == names


def _declared_parameter_counts():
    text = open(os.path.join(ROOT, "include", "rf_gemm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for name, params in re.findall(r"\b(run|rf_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        params = params.strip()
        out[name] = 0 if params in ("", "void") else params.count(",") + 1
    return out


def test_python_binding_declares_as_many_arguments_as_the_header():
    """A ctypes prototype with the wrong number or kind of arguments silently truncates 64-bit device pointers to
    32 bits: every entry point the mirror calls with pointers must carry argtypes of the header's length, and
    every pointer parameter must be a pointer type."""
    from radeonflow_kernels_amd import gemm
    L = gemm.lib()
    counts = _declared_parameter_counts()
    with_pointers = [n for n in counts if n not in ("rf_gemm_num_variants", "rf_gemm_destroy", "rf_gemm_last_error",
                                                    "rf_gemm_clear_plans")]
    for name in with_pointers:
        at = getattr(L, name).argtypes
        assert at is not None, "%s has no ctypes prototype" % name
        assert len(at) == counts[name], "%s: %d argtypes, header declares %d" % (name, len(at), counts[name])
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "rf_gemm.h")).read(), flags=re.S)
    for name, params in re.findall(r"\b(run|rf_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        if name not in with_pointers:
            continue
        for decl, ct in zip(params.split(","), getattr(L, name).argtypes):
            is_ptr = "*" in decl or "hipStream_t" in decl
            ct_ptr = ct is ctypes.c_void_p or ct is ctypes.c_char_p or hasattr(ct, "contents")
            assert is_ptr == ct_ptr, "%s: parameter '%s' bound as %r" % (name, decl.strip(), ct)


def test_perf_metrics_layout_matches_the_reference_struct():
    from radeonflow_kernels_amd.gemm import PerfMetrics, PerfMetricEntry, GemmConfig
    assert ctypes.sizeof(PerfMetricEntry) == 28
    assert ctypes.sizeof(PerfMetrics) == 4 + 20 * 28 == 564
    assert PerfMetrics.entries.offset == 4
    assert PerfMetricEntry.time.offset == 20 and PerfMetricEntry.gflops.offset == 24
    assert ctypes.sizeof(GemmConfig) == 16


def test_status_codes_without_a_device():
    from radeonflow_kernels_amd import gemm
    L = gemm.lib()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    assert L.rf_fp8_gemm(p, p, p, p, p, 16, 16, 100, None) == 1          # K not a multiple of 128
    assert b"K=100" in L.rf_gemm_last_error()
    assert L.rf_fp8_gemm(p, p, p, p, p, 16, 16, 0, None) == 1
    assert L.rf_fp8_gemm(p, p, p, p, p, -1, 16, 128, None) == 1
    assert L.rf_fp8_gemm(None, p, p, p, p, 16, 16, 128, None) == 2        # null pointer
    assert L.rf_gemm_num_variants() >= 1
    info = [ctypes.c_int() for _ in range(5)]
    assert L.rf_gemm_variant_info(0, *[ctypes.byref(x) for x in info]) == 0
    assert info[0].value % 16 == 0 and info[4].value <= 160 * 1024        # fits the 160 KiB LDS of a gfx950 CU
    assert L.rf_gemm_variant_info(999, *[ctypes.byref(x) for x in info]) == 4


def test_run_aborts_on_an_unsupported_shape_like_the_reference_launcher():
    code = ("import ctypes,sys; sys.path.insert(0,%r); from radeonflow_kernels_amd import gemm; L=gemm.lib(); "
            "b=ctypes.create_string_buffer(64); p=ctypes.addressof(b); L.run(p,p,p,p,p,64,64,100,None,None)" % ROOT)
    r = subprocess.run([sys.executable, "-c", code], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert r.returncode == -6                                              # SIGABRT
    assert "Unsupported shape M=64, K=100, N=64" in r.stdout


def test_python_mirror_rejects_cpu_tensors_and_wrong_layouts():
    import pytest
    import torch
    import radeonflow_kernels_amd as rfk
    a = torch.zeros((16, 128), dtype=torch.uint8).view(torch.float8_e4m3fn)
    with pytest.raises(ValueError):
        rfk.fp8_mm(a, a, torch.zeros(16, 1), torch.zeros(1, 1), torch.zeros((16, 16), dtype=torch.bfloat16))


def test_plan_files_parse_without_a_device(tmp_path):
    """rf_gemm_load_plans only reads and validates the file (plans are matched against shapes at launch): the tuner's
    line format, the brace format of csrc/tuned_plans.inc, comments; a bad line fails the whole file and names it."""
    from radeonflow_kernels_amd import gemm
    L = gemm.lib()
    good = tmp_path / "plans.txt"
    good.write_text("# shape            variant split group schedule\n"
                    "6144 4608 7168 0 1 16 2\n"
                    "{1024, 1536, 7168, 3, 4, 8, 0},   // 24.2 us\n"
                    "\n"
                    "  512 512 256 1 2 4 0   # trailing comment\n")
    try:
        assert gemm.load_plans(str(good)) == 3
        inc = os.path.join(ROOT, "radeonflow_kernels_amd", "csrc", "tuned_plans.inc")
        assert gemm.load_plans(inc) == sum(1 for l in open(inc) if l.startswith("{"))
        n = ctypes.c_int(-1)
        for text, line in (("512 512 256 1 2 4\n", 1),                       # six fields
                           ("512 512 256 1 2 4 0\n512 512 200 1 1 4 0\n", 2),   # K not a multiple of 128
                           ("512 512 256 99 1 4 0\n", 1),                    # no such variant
                           ("512 512 256 0 2 4 2\n", 1),                     # persistent schedule with a K split
                           ("512 512 256 0 1 4 0 7\n", 1)):                  # eight fields
            bad = tmp_path / "bad.txt"
            bad.write_text(text)
            assert L.rf_gemm_load_plans(str(bad).encode(), ctypes.byref(n)) == 4
            assert ("bad.txt:%d" % line).encode() in L.rf_gemm_last_error()
            assert n.value == -1
        assert L.rf_gemm_load_plans(str(tmp_path / "missing.txt").encode(), None) == 4
        assert L.rf_gemm_load_plans(None, None) == 2
    finally:
        gemm.clear_plans()


def test_compiled_in_plan_table_only_holds_plans_its_shapes_can_run():
    """Every line of csrc/tuned_plans.inc names an existing variant, a split that leaves every part at least one K
    block, and the persistent schedules only where the shape allows them (a plan that cannot run is skipped at lookup,
    so a bad line would silently fall back to the cost model)."""
    from radeonflow_kernels_amd import gemm
    L = gemm.lib()
    inc = os.path.join(ROOT, "radeonflow_kernels_amd", "csrc", "tuned_plans.inc")
    plans = [tuple(int(x) for x in re.findall(r"-?\d+", l.split("}")[0])) for l in open(inc) if l.startswith("{")]
    assert len(plans) >= 29 and len(set(p[:3] for p in plans)) == len(plans)        # one plan per shape
    for m, n, k, variant, split, group, schedule in plans:
        bm, bn = ctypes.c_int(), ctypes.c_int()
        assert L.rf_gemm_variant_info(variant, ctypes.byref(bm), ctypes.byref(bn), None, None, None) == 0
        assert m % 16 == 0 and n % 16 == 0 and k % 128 == 0 and 1 <= split <= k // 128 and group >= 1
        assert schedule in (0, 2, 3, 4), "the stream-K schedule is never tabled"
        if schedule == 4:
            assert variant == 0 and split == 1 and k in (128, 256, 384, 512) and n % 64 == 0
        if schedule in (2, 3):
            assert L.rf_gemm_variant_has_persistent(variant) == 1 and split == 1
            assert m >= bm.value and n % bn.value == 0 and (k // 128) % 2 == 0
        if schedule == 3:
            # measured on 256 compute units: whole rounds first, then a last round that is at most half full (on a
            # device with another count the plan is checked again at lookup and skipped if it does not fit)
            tiles = -(-m // 256) * (n // 256)
            left = tiles % 256
            assert variant == 0 and tiles >= 256 and 0 < left and (left + 7) // 8 * 8 + left <= 256


def test_tuner_never_writes_a_stream_k_winner_into_a_table_or_plan_file(tmp_path):
    """Stream-K needs one tile per compute unit of the device it runs on, so tables and plan files carry the fastest
    plan of another schedule instead."""
    from radeonflow_kernels_amd.tuner import gemm_tuner as t
    cand = lambda sk, us: dict(variant=0, split_k=1, group_m=4, stream_k=sk, us=us, tflops=1.0)
    assert t.best_for_table([cand(1, 10.0), cand(2, 11.0), cand(0, 12.0)])["stream_k"] == 2
    assert t.best_for_table([cand(1, 10.0)]) is None and t.best_for_table([]) is None
    out = tmp_path / "plans.inc"
    t.emit_plans({(512, 512, 256): [cand(1, 10.0), cand(0, 12.0)], (256, 256, 256): [cand(1, 9.0)]}, str(out))
    lines = [l for l in out.read_text().splitlines() if l.startswith("{")]
    assert len(lines) == 1 and lines[0].startswith("{512, 512, 256, 0, 1, 4, 0}")


def test_planner_arithmetic_on_the_host_for_any_compute_unit_count(tmp_path):
    """rf_gemm_plan_for needs no device. With 256 compute units a tabled shape gets its tabled plan; with any other count
    the table (measured on 256) is left aside and the cost model counts rounds for the count given: every plan names an
    existing variant and a split that leaves each part a K block, the persistent schedules only where the shape allows
    them, the half-tile schedule only when the last round of 256 x 256 tiles on that many units is at most half full,
    never stream-K, and the skinny-K schedule for up to four K blocks with a large C whatever the count. A loaded plan
    file still wins on every count."""
    import radeonflow_kernels_amd as rfk
    inc = os.path.join(ROOT, "radeonflow_kernels_amd", "csrc", "tuned_plans.inc")
    table = {p[:3]: p[3:] for p in (tuple(int(x) for x in re.findall(r"-?\d+", l.split("}")[0])) for l in open(inc)
                                     if l.startswith("{"))}
    for shape in ((6144, 4608, 7168), (1024, 1536, 7168), (1024, 576, 7168), (6144, 7168, 256)):
        c = rfk.plan_for(*shape, 256)
        assert (c.variant, c.split_k, c.group_m, c.stream_k) == table[shape]
    nv = rfk.lib().rf_gemm_num_variants()
    for ncu in (8, 64, 104, 128, 228, 304):
        for (m, n, k) in list(table)[::7] + [(8192, 4608, 7168), (4096, 4096, 4096), (640, 640, 640), (48, 48, 128)]:
            c = rfk.plan_for(m, n, k, ncu)
            assert 0 <= c.variant < nv and 1 <= c.split_k <= k // 128 and c.stream_k in (0, 2, 3, 4), (ncu, m, n, k, c)
            bm, bn = ctypes.c_int(), ctypes.c_int()
            assert rfk.lib().rf_gemm_variant_info(c.variant, ctypes.byref(bm), ctypes.byref(bn), None, None, None) == 0
            if c.stream_k in (2, 3):
                assert c.split_k == 1 and m >= bm.value and n % bn.value == 0 and (k // 128) % 2 == 0
            if c.stream_k == 3:
                tiles = -(-m // 256) * (n // 256)
                left = tiles % ncu
                assert c.variant == 0 and tiles >= ncu and 0 < left and (left + 7) // 8 * 8 + left <= ncu
            if c.stream_k == 4:
                assert k in (128, 256, 384, 512) and m % 16 == 0 and n % 64 == 0
        assert rfk.plan_for(6144, 7168, 256, ncu).stream_k == 4
        assert rfk.plan_for(2048, 2048, 256, ncu).stream_k != 4            # below six million outputs
        assert rfk.plan_for(4096, 4096, 512, ncu).stream_k == 4            # three or four K blocks: from two million on
        assert rfk.plan_for(6144, 7168, 384, ncu).stream_k == 4
        assert rfk.plan_for(6144, 7168, 512, ncu).stream_k != 4            # K = 512: up to sixteen strips only
        assert rfk.plan_for(512, 2048, 512, ncu).stream_k != 4
        assert rfk.plan_for(4096, 4096, 640, ncu).stream_k != 4
    # fewer units, more rounds: 2048 x 2048 x 7168 is 64 tiles of 256 x 256: no K split is worth it on 8 units
    assert rfk.plan_for(2048, 2048, 7168, 8).split_k == 1
    # ragged shapes are planned at their padded size
    c, d = rfk.plan_for(1000, 1530, 1024, 128), rfk.plan_for(1008, 1536, 1024, 128)
    assert (c.variant, c.split_k, c.stream_k) == (d.variant, d.split_k, d.stream_k)
    plans = tmp_path / "p.plans"
    plans.write_text("4096 4096 4096 1 2 4 0\n")
    try:
        assert rfk.load_plans(str(plans)) == 1
        for ncu in (64, 256):
            c = rfk.plan_for(4096, 4096, 4096, ncu)
            assert (c.variant, c.split_k, c.group_m, c.stream_k) == (1, 2, 4, 0)
    finally:
        rfk.clear_plans()
    cfg = rfk.GemmConfig()
    assert rfk.lib().rf_gemm_plan_for(16, 16, 100, 256, ctypes.byref(cfg)) == 1
    assert rfk.lib().rf_gemm_plan_for(16, 16, 128, 0, ctypes.byref(cfg)) == 1
    assert rfk.lib().rf_gemm_plan_for(16, 16, 128, 256, None) == 2


def test_grouped_variant_choice_on_the_host():
    """rf_grouped_variant_for needs no device. The queue form (5) is taken where its last tiles of 64..256 rows save at
    least 7 % of the rows the other 256-wide forms compute and it has 1.5 items per compute unit (2.5 below K = 4096);
    groups the other forms fit as well, or too few items, keep those forms; tiny problems take the form with the most
    workgroups; bad arguments are refused."""
    import numpy as np
    import radeonflow_kernels_amd as rfk

    def offs(sizes):
        return [0] + [int(x) for x in np.cumsum(sizes)]

    rng = np.random.default_rng(1)
    cuts = np.sort(rng.choice(np.arange(1, 8192 // 16), 31, replace=False)) * 16
    uneven = [0] + [int(x) for x in cuts] + [8192]                       # 32 groups of 16..816 rows
    assert rfk.grouped_variant_for(uneven, 4096, 7168) == 5
    assert rfk.grouped_variant_for(uneven, 4096, 7168, num_cu=304) == 5
    assert rfk.grouped_variant_for(offs([256] * 32), 4096, 7168) in (0, 4)      # nothing to save
    assert rfk.grouped_variant_for(offs([128] * 64), 4096, 7168) == 1
    assert rfk.grouped_variant_for(offs([384] * 20), 4096, 7168) in (1, 4)
    small = offs([int(x) * 16 for x in np.random.default_rng(5).integers(1, 25, 16)])    # 16 groups of 16..384 rows
    assert rfk.grouped_variant_for(small, 2048, 7168) != 5              # 170 items for 256 units
    assert rfk.grouped_variant_for(small, 7168, 7168) == 5              # the same groups, 3.5 times the column tiles
    assert rfk.grouped_variant_for(uneven, 4096, 2048) == 5             # 816 items: 3.2 per unit
    assert rfk.grouped_variant_for(uneven, 2048, 2048) != 5             # 408 items: 1.6 per unit, short items
    assert rfk.grouped_variant_for(offs([64] * 8), 1024, 512) == 3      # no form fills the units: the most workgroups
    for bad in (([0, 16, 8], 256, 256), ([1, 16], 256, 256), ([0, 16], 256, 100), ([0, 16], 0, 256)):
        with pytest.raises(RuntimeError):
            rfk.grouped_variant_for(*bad)
