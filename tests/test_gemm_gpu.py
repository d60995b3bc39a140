"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle."""
import ctypes
import os

import numpy as np
import pytest
import torch

from oracle import cref, ref_kernel as rk
from helpers import (ATOL, ATOL_REFERENCE, CONFIGS, RTOL, assert_close_to_oracle, assert_few_mismatches_at_reference_atol,
                     bf16_bits, exact_problem, oracle_bf16, to_gpu)

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def rfk():
    import radeonflow_kernels_amd as r
    assert torch.cuda.is_available(), "these tests need the GPU"
    r.lib()   # raises if libgemm.so has not been built: no fallback exists
    return r


def _run(rfk, data, config=None, canary=0):
    if canary:
        g, buf = to_gpu(data, canary_elems=canary)
    else:
        g, buf = to_gpu(data), None
    rfk.fp8_mm(*g, config=config)
    torch.cuda.synchronize()
    if buf is not None:
        tail = buf[g[4].numel():].float().cpu().numpy()
        assert np.all(tail == -7.0), "store past the end of C"
    return g[4]


GOLDEN = sorted(f for f in os.listdir(os.path.join(os.path.dirname(__file__), "golden")) if f.endswith(".npz"))


@pytest.mark.parametrize("name", GOLDEN)
def test_golden_fixtures(rfk, name):
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", name))
    a = torch.from_numpy(z["a"]).view(torch.float8_e4m3fn).T
    b = torch.from_numpy(z["b"]).view(torch.float8_e4m3fn).T
    sa = torch.from_numpy(z["a_scale"]).T
    sb = torch.from_numpy(z["b_scale"]).T
    c = torch.zeros((a.shape[0], b.shape[0]), dtype=torch.bfloat16)
    out = _run(rfk, (a, b, sa, sb, c), canary=4096)
    assert_close_to_oracle(out, z["c_bf16"], RTOL, ATOL_REFERENCE, name)


@pytest.mark.parametrize("gen", ["blockquant", "reference_style"])
@pytest.mark.parametrize("m,n,k", [(256, 384, 512), (512, 576, 1024), (272, 144, 256), (16, 16, 128), (128, 7168, 256)])
def test_every_variant_and_split(rfk, gen, m, n, k):
    f = rk.generate_input_blockquant if gen == "blockquant" else rk.generate_input_reference_style
    data = f(m, n, k, seed=m + n + k)
    exp = oracle_bf16(data)
    for v in rfk.variants():
        for split in (1, 2, 3):
            if not rfk.plan_can_run(v, split, k):
                continue
            cfg = rfk.GemmConfig(v["variant"], split, 4, 0)
            out = _run(rfk, data, config=cfg, canary=1024)
            assert_close_to_oracle(out, exp, RTOL, ATOL, "variant %r split %d" % (v, split))
            assert_few_mismatches_at_reference_atol(out, exp, "variant %r split %d" % (v, split))


@pytest.mark.parametrize("m,n", [(1024, 1536), (640, 576), (768, 2304), (2048, 384), (1040, 208)])
def test_split_k_grid_reaches_every_tile_and_split_once(rfk, m, n):
    """Every variant with 2 to 16 K splits (counts that divide the 16 K blocks and counts that leave the last split
    short), on tile grids that do and do not divide by the number of XCDs: bit-exact on data whose sums are exact in
    any order, after a launch of another problem with the same plan (partial sums of a tile or split nobody computed
    would be that problem's)."""
    k = 2048
    data = exact_problem(m, n, k, seed=m + n)
    exp = oracle_bf16(data)
    other = to_gpu(exact_problem(m, n, k, seed=m + n + 1))
    for v in rfk.variants():
        for split in (2, 3, 4, 5, 8, 16):
            if not rfk.plan_can_run(v, split, k):
                continue
            cfg = rfk.GemmConfig(v["variant"], split, 3, 0)
            rfk.fp8_mm(*other, config=cfg)                  # fills the workspace with another problem's sums
            out = _run(rfk, data, config=cfg, canary=1024)
            assert np.array_equal(bf16_bits(out), exp), "variant %r split %d" % (v, split)


@pytest.mark.parametrize("m,n,k", [(256, 384, 512), (512, 576, 1024), (272, 144, 256), (16, 16, 128), (1024, 1536, 7168),
                                   (48, 80, 7168), (33, 47, 384)])
def test_bit_exact_on_exactly_representable_data(rfk, m, n, k):
    """Small-integer fp8 values and power-of-two scales: every product, partial sum and fold is exact in
    fp32 in any order, so the HIP path and the oracle must agree bit for bit. Catches any wrong index,
    scale, K coverage or store address without being blurred by rounding."""
    data = exact_problem(m, n, k, seed=m * 31 + n)
    exp = oracle_bf16(data)
    a, b, sa, sb = rk.raw_layouts(data)
    assert np.array_equal(exp, cref.ref_gemm_blockfold(a, b, sa, sb)[1])      # exact on the CPU in both orders
    tiled = m % 16 == 0 and n % 16 == 0
    plans = [None]
    if tiled:
        plans += [rfk.GemmConfig(v["variant"], s, gm, 0) for v in rfk.variants() for s, gm in ((1, 1), (2, 8), (3, 3))
                  if rfk.plan_can_run(v, s, k)]
    for cfg in plans:
        out = _run(rfk, data, config=cfg, canary=1024)
        assert np.array_equal(bf16_bits(out), exp), "plan %r" % (cfg,)


@pytest.mark.parametrize("m,n,k", [(2048, 2048, 512), (1536, 3072, 384), (4096, 4608, 1024), (6144, 4608, 256),
                                   (1040, 2064, 640)])
def test_stream_k_bit_exact_and_counters_self_reset(rfk, m, n, k):
    """Persistent stream-K grid on shapes with at least as many tiles as CUs: equal shares of the work line cut
    tiles at arbitrary K blocks, the last arriver sums the partials. Exact data makes any summation order give
    the same bits. Run twice: the arrival counters must be back at zero after the first launch."""
    data = exact_problem(m, n, k, seed=m + 3 * n + k)
    exp = oracle_bf16(data)
    ncu = torch.cuda.get_device_properties(0).multi_processor_count
    tried = 0
    for v in rfk.variants():
        tiles = -(-m // v["block_m"]) * -(-n // v["block_n"])
        if tiles < ncu or not v["stream_k"]:
            continue
        for gm in (1, 8):
            cfg = rfk.GemmConfig(v["variant"], 1, gm, 1)
            for rep in range(2):
                out = _run(rfk, data, config=cfg, canary=1024)
                assert np.array_equal(bf16_bits(out), exp), "plan %r rep %d" % (cfg, rep)
            tried += 1
    assert tried > 0


@pytest.mark.parametrize("m,n,k", [(512, 512, 256), (2048, 2048, 512), (2560, 1920, 256), (6144, 4608, 256),
                                   (4096, 2048, 1024), (1024, 1536, 7168)])
def test_persistent_schedule_bit_exact(rfk, m, n, k):
    """One pipeline running across the tiles of a workgroup (1, 2 or 3 tiles each, uneven counts included): exact
    data, so every tile must equal the oracle bit for bit whatever was prefetched or left in registers by the
    previous tile. Twice in a row on the same buffers."""
    data = exact_problem(m, n, k, seed=5 * m + n + k)
    exp = oracle_bf16(data)
    tried = 0
    for v in rfk.variants():
        if not v["persistent"] or m % v["block_m"] or n % v["block_n"]:
            continue
        for gm in (1, 8):
            cfg = rfk.GemmConfig(v["variant"], 1, gm, 2)
            for rep in range(2):
                out = _run(rfk, data, config=cfg, canary=1024)
                assert np.array_equal(bf16_bits(out), exp), "plan %r rep %d" % (cfg, rep)
            tried += 1
    assert tried > 0


@pytest.mark.parametrize("m,n,k", [(272, 512, 256), (624, 768, 512), (1008, 1024, 256), (2000, 512, 768)])
def test_persistent_schedule_with_a_last_row_of_tiles_that_overlaps_the_one_before(rfk, m, n, k):
    """M is a multiple of 16 but not of the tile height: the last row of tiles starts at M - BM and shares rows with
    its neighbour. Exact data against the oracle, bit for bit, twice; then data with rounding in it against the
    one-workgroup-per-tile kernel of the same variant, bit for bit as well and the same on every launch: a row's result
    does not depend on where in a tile the row sits, so both tiles that compute a shared row store the same value."""
    data = exact_problem(m, n, k, seed=3 * m + n + k)
    exp = oracle_bf16(data)
    noisy = rk.generate_input_blockquant(m, n, k, seed=m + k)
    tried = 0
    for v in rfk.variants():
        if not v["persistent"] or m < v["block_m"] or m % v["block_m"] == 0 or n % v["block_n"]:
            continue
        cfg = rfk.GemmConfig(v["variant"], 1, 8, 2)
        for rep in range(2):
            out = _run(rfk, data, config=cfg, canary=1024)
            assert np.array_equal(bf16_bits(out), exp), "plan %r rep %d" % (cfg, rep)
        tiles = bf16_bits(_run(rfk, noisy, config=rfk.GemmConfig(v["variant"], 1, 8, 0), canary=1024)).copy()
        for rep in range(3):
            out = _run(rfk, noisy, config=cfg, canary=1024)
            assert np.array_equal(bf16_bits(out), tiles), "plan %r rep %d differs from the tile kernel" % (cfg, rep)
        tried += 1
    assert tried > 0


def test_ragged_m_under_a_persistent_plan_writes_c_in_place(rfk, tmp_path):
    """M = 1001: A and a_scale are staged with 1008 rows; with a persistent plan for the padded shape the kernel writes
    the 1001 true rows straight into C (the last tile's stores are masked by row) and nothing behind them."""
    m, n, k = 1001, 1024, 512
    path = tmp_path / "p.plans"
    path.write_text("1008 %d %d 0 1 8 2\n" % (n, k))
    data = exact_problem(m, n, k, seed=77)
    try:
        assert rfk.load_plans(str(path)) == 1
        got = rfk.select_config(1008, n, k)
        assert (got.variant, got.stream_k) == (0, 2)
        for rep in range(2):
            out = _run(rfk, data, canary=2048)
            assert np.array_equal(bf16_bits(out), oracle_bf16(data)), "rep %d" % rep
    finally:
        rfk.clear_plans()


@pytest.mark.parametrize("m,k,schedule", [(6000, 512, 2), (6001, 512, 2), (6000, 256, 4), (6001, 256, 4)])
def test_large_m_that_is_not_a_tile_multiple_runs_a_whole_tile_plan_automatically(rfk, m, k, schedule):
    """6000 and 6001 rows with C4's N: the automatic plan is the persistent schedule at K = 512 and the skinny-K schedule
    at K = 256 (for 6001 on the shape padded to 6016 rows, with C written in place: both schedules mask the padding
    rows in their stores); exact data, bit for bit, canary behind the last true row intact."""
    n = 7168
    assert rfk.select_config(m, n, k).stream_k == schedule
    data = exact_problem(m, n, k, seed=m)
    out = _run(rfk, data, canary=8192)
    assert np.array_equal(bf16_bits(out), oracle_bf16(data))


@pytest.mark.parametrize("m,n,k", [(4608, 4096, 256), (4352, 4096, 512), (4592, 4096, 256), (2320, 8192, 256),
                                   (8192, 4608, 256)])
def test_persistent_schedule_with_a_last_round_of_half_tiles(rfk, m, n, k):
    """More tiles than CUs and a last round that is at most half full (32, 16, 32, 64 and 64 left-over tiles on 256
    CUs; 4592 and 2320 rows also end on a tile row that overlaps the one before): the left-over tiles are computed as
    upper and lower halves by two workgroups each. Exact data against the oracle, bit for bit, twice; then data with
    rounding in it against the one-workgroup-per-tile kernel, bit for bit and the same on every launch."""
    if torch.cuda.get_device_properties(0).multi_processor_count != 256:
        pytest.skip("left-over counts are worked out for 256 compute units")
    data = exact_problem(m, n, k, seed=m + 3 * n + k)
    exp = oracle_bf16(data)
    for gm in (1, 8):
        cfg = rfk.GemmConfig(0, 1, gm, 3)
        for rep in range(2):
            out = _run(rfk, data, config=cfg, canary=1024)
            assert np.array_equal(bf16_bits(out), exp), "plan %r rep %d" % (cfg, rep)
    noisy = rk.generate_input_blockquant(m, n, k, seed=m + k)
    tiles = bf16_bits(_run(rfk, noisy, config=rfk.GemmConfig(0, 1, 8, 0), canary=1024)).copy()
    for rep in range(3):
        out = _run(rfk, noisy, config=rfk.GemmConfig(0, 1, 8, 3), canary=1024)
        assert np.array_equal(bf16_bits(out), tiles), "rep %d differs from the tile kernel" % rep


def test_half_tile_schedule_under_a_ragged_m_writes_c_in_place(rfk, tmp_path):
    """4593 rows: the operands are staged with 4608 rows and the plan of the padded shape, here the half-tile
    schedule, stores only the true rows (the lower half tiles of the last tile row are masked by row)."""
    m, n, k = 4593, 4096, 256
    path = tmp_path / "p.plans"
    path.write_text("4608 %d %d 0 1 8 3\n" % (n, k))
    data = exact_problem(m, n, k, seed=78)
    try:
        assert rfk.load_plans(str(path)) == 1
        got = rfk.select_config(4608, n, k)
        if got.stream_k != 3:
            pytest.skip("the half-tile schedule does not fit this device's CU count")
        for rep in range(2):
            out = _run(rfk, data, canary=8192)
            assert np.array_equal(bf16_bits(out), oracle_bf16(data)), "rep %d" % rep
    finally:
        rfk.clear_plans()


def test_half_tile_schedule_rejects_shapes_it_does_not_fit(rfk):
    for m, n, k, variant in [(2048, 2048, 256, 0),      # fewer tiles than CUs
                             (8192, 2048, 256, 0),      # 256 tiles: no last round
                             (6144, 4608, 256, 0),      # 432 tiles: last round more than half full
                             (4608, 4096, 384, 0),      # three K blocks
                             (4608, 4096, 256, 3)]:     # not the 256 x 256 tile
        data = exact_problem(m, n, k, seed=1)
        with pytest.raises(RuntimeError):
            _run(rfk, data, config=rfk.GemmConfig(variant, 1, 8, 3))


@pytest.mark.parametrize("m,n,k", [(128, 256, 256), (16, 64, 128), (272, 320, 256), (1040, 448, 128), (2048, 2048, 256),
                                   (6000, 7168, 256), (96, 7168, 256), (400, 1216, 256),
                                   (64, 256, 512), (16, 64, 384), (272, 320, 512), (1040, 448, 384), (4096, 4096, 512),
                                   (6000, 4096, 384), (80, 7168, 512), (400, 1216, 512)])
def test_skinny_k_schedule_bit_exact(rfk, m, n, k):
    """K = 128 ... 512 under the skinny-K schedule (the B operand of a 256-column strip in registers, A streamed in
    items of 128 rows, 64 rows from three K blocks on, C stored m-tile by m-tile): strips that end in a partial
    64-column wave tile, a last item with fewer rows, one to many items and strips per workgroup. Exact data against
    the oracle, bit for bit, twice
    on the same buffers with the canary intact; then data with rounding in it against the one-workgroup-per-tile
    kernel, bit for bit as well (same MFMA, same folds in the same K order)."""
    cfg = rfk.GemmConfig(0, 1, 8, 4)
    data = exact_problem(m, n, k, seed=m + n + k)
    exp = oracle_bf16(data)
    for rep in range(2):
        out = _run(rfk, data, config=cfg, canary=1024)
        assert np.array_equal(bf16_bits(out), exp), "rep %d" % rep
    noisy = rk.generate_input_blockquant(m, n, k, seed=m + k)
    ref = bf16_bits(_run(rfk, noisy, config=rfk.GemmConfig(1, 1, 8, 0))).copy()
    out = _run(rfk, noisy, config=cfg, canary=1024)
    assert np.array_equal(bf16_bits(out), ref)
    assert_close_to_oracle(out, oracle_bf16(noisy), RTOL, ATOL, "skinny K")


@pytest.mark.parametrize("m,n,k", [(64, 128, 256), (1024, 1536, 7168), (208, 576, 1024), (64, 1536, 7168), (1024, 512, 512),
                                   (208, 576, 768), (512, 3072, 1536), (128, 128, 384)])
def test_k_split_inside_the_workgroup_equals_the_two_launch_form(rfk, m, n, k):
    """Variants whose wave groups split K inside one workgroup (partial sums added through LDS in part order) against
    the same tile with split_k = the number of groups (fp32 partial sums through memory + the reduction kernel): the
    same bits on data with rounding in it, the oracle's bits on exact data, twice on the same buffers, canary intact;
    and K block counts their groups do not divide are refused."""
    tried = 0
    for v in rfk.variants():
        if v["k_groups"] < 2:
            continue
        twin = [w for w in rfk.variants() if w["k_groups"] == 1 and (w["block_m"], w["block_n"], w["waves_m"], w["waves_n"])
                == (v["block_m"], v["block_n"], v["waves_m"], v["waves_n"]) and w["lds_bytes"] * v["k_groups"] <= v["lds_bytes"]
                and w["lds_bytes"] * v["k_groups"] > v["lds_bytes"] - 4096]
        assert len(twin) == 1, "the one-group variant with the same tile and stage count"
        cfg, cfg2 = rfk.GemmConfig(v["variant"], 1, 8, 0), rfk.GemmConfig(twin[0]["variant"], v["k_groups"], 8, 0)
        if (k // 128) % v["k_groups"] != 0:
            with pytest.raises(RuntimeError):                   # K blocks the groups do not divide: refused
                _run(rfk, exact_problem(m, n, k, seed=1), config=cfg)
            tried += 1
            continue
        data = exact_problem(m, n, k, seed=m + n + k)
        exp = oracle_bf16(data)
        for rep in range(2):
            assert np.array_equal(bf16_bits(_run(rfk, data, config=cfg, canary=1024)), exp), "rep %d" % rep
        noisy = rk.generate_input_blockquant(m, n, k, seed=m + k)
        ref = bf16_bits(_run(rfk, noisy, config=cfg2)).copy()
        out = _run(rfk, noisy, config=cfg, canary=1024)
        assert np.array_equal(bf16_bits(out), ref)
        assert_close_to_oracle(out, oracle_bf16(noisy), RTOL, ATOL, "K split inside the workgroup")
        for bad in (rfk.GemmConfig(v["variant"], 2, 8, 0), rfk.GemmConfig(v["variant"], 1, 8, 2)):
            with pytest.raises(RuntimeError):
                _run(rfk, data, config=bad)
        tried += 1
    assert tried > 0


def test_skinny_k_schedule_rejects_shapes_it_does_not_fit(rfk):
    for (m, n, k, variant) in ((256, 256, 640, 0), (256, 256, 1024, 0), (40, 256, 256, 0), (256, 96, 256, 0), (256, 256, 256, 1)):
        data = exact_problem(m, n, k, seed=1)
        with pytest.raises(RuntimeError):
            _run(rfk, data, config=rfk.GemmConfig(variant, 1, 8, 4))


def test_persistent_schedule_rejects_ragged_shapes(rfk):
    data = exact_problem(272, 144, 256, seed=1)
    with pytest.raises(RuntimeError):
        _run(rfk, data, config=rfk.GemmConfig(0, 1, 1, 2))
    data = exact_problem(256, 256, 384, seed=1)           # three K blocks
    with pytest.raises(RuntimeError):
        _run(rfk, data, config=rfk.GemmConfig(0, 1, 1, 2))


@pytest.mark.parametrize("m,n,k", [(3, 130, 256), (1, 1, 128), (17, 64, 384), (5, 257, 128), (100, 72, 256)])
def test_bounds_checked_kernel_on_odd_shapes(rfk, m, n, k):
    data = rk.generate_input_reference_style(m, n, k, seed=7 * m + n)
    cfg = rfk.select_config(m, n, k)
    assert cfg.variant == -1
    out = _run(rfk, data, canary=512)
    assert_close_to_oracle(out, oracle_bf16(data), RTOL, ATOL, "checked kernel")
    assert_few_mismatches_at_reference_atol(out, oracle_bf16(data), "checked kernel")


# the reference's own test shapes and seeds (scripts/problems/gemm/task.yml:53-64), its input style
REFERENCE_TESTS = [(64, 64, 128, 6635), (64, 1536, 7168, 6635), (64, 3072, 1536, 1236), (64, 576, 7168, 542),
                   (96, 7168, 256, 1234), (96, 7168, 2048, 4153), (96, 4608, 7168, 412), (128, 7168, 2304, 624),
                   (128, 512, 7168, 2514), (512, 4096, 512, 543), (512, 1536, 7168, 12341)]


@pytest.mark.parametrize("m,n,k,seed", REFERENCE_TESTS)
def test_reference_test_shapes(rfk, m, n, k, seed):
    data = rk.generate_input_reference_style(m, n, k, seed)
    out = _run(rfk, data, canary=1024)
    exp = oracle_bf16(data)
    assert_close_to_oracle(out, exp, RTOL, ATOL, "reference test shape")
    assert_few_mismatches_at_reference_atol(out, exp, "reference test shape")
    assert rk.check_implementation(data, out.cpu(), rtol=RTOL, atol=ATOL) == ""


@pytest.mark.parametrize("name", ["C1", "C4", "C5"])
def test_benchmark_configs_full_oracle(rfk, name):
    m, n, k, seed = CONFIGS[name]
    data = rk.generate_input_blockquant(m, n, k, seed)
    out = _run(rfk, data, canary=1024)
    exp = oracle_bf16(data)
    mx = assert_close_to_oracle(out, exp, RTOL, ATOL, name)
    bad = assert_few_mismatches_at_reference_atol(out, exp, name)
    print("%s: max abs err %.4g, mismatches at atol 1e-3: %d of %d" % (name, mx, bad, m * n))


@pytest.mark.parametrize("name", ["C2", "C3"])
def test_benchmark_configs_full_size_sampled_rows_and_properties(rfk, name):
    m, n, k, seed = CONFIGS[name]
    data = rk.generate_input_blockquant(m, n, k, seed)
    g = to_gpu(data)
    rfk.fp8_mm(*g)
    torch.cuda.synchronize()
    base = g[4].clone()
    # (1) sampled rows against the oracle (dequantise, fp32 accumulate over full K) and the fp64 truth
    rng = np.random.default_rng(seed)
    rows = np.unique(np.concatenate([[0, 1, 255, 256, m - 1], rng.integers(0, m, 43)])).astype(np.int32)
    a, b, sa, sb = rk.raw_layouts(data)
    _, exp16 = cref.ref_gemm_f32(a, b, sa, sb, rows=rows)
    got = base[torch.from_numpy(rows).long().cuda()]
    assert_close_to_oracle(got, exp16, RTOL, ATOL, name + " sampled rows")
    assert_few_mismatches_at_reference_atol(got, exp16, name + " sampled rows")
    truth = cref.ref_gemm_f64(a, b, sa, sb, rows=rows)
    err = np.abs(cref.bf16_to_f32(bf16_bits(got)).astype(np.float64) - truth)
    assert np.all(err <= 2.0 ** -8 * np.abs(truth) + ATOL), "further than one bf16 rounding + atol from the fp64 truth"
    # (2) doubling a_scale doubles every output exactly (power of two: same roundings)
    g2 = (g[0], g[1], (g[2].T.contiguous() * 2).T, g[3], torch.zeros_like(base))
    rfk.fp8_mm(*g2)
    torch.cuda.synchronize()
    assert torch.equal(g2[4].float(), base.float() * 2)
    # (3) permuting the rows of A (and of a_scale) permutes the rows of C bit for bit
    perm = torch.randperm(m, generator=torch.Generator().manual_seed(seed)).cuda()
    ap = g[0][perm].T.contiguous().T
    sp = g[2][perm].T.contiguous().T
    g3 = (ap, g[1], sp, g[3], torch.zeros_like(base))
    rfk.fp8_mm(*g3)
    torch.cuda.synchronize()
    assert torch.equal(g3[4].view(torch.int16), base[perm].view(torch.int16))
    # (4) zero a_scale gives an all-zero C (every element is written)
    g4 = (g[0], g[1], torch.zeros_like(g[2].T.contiguous()).T, g[3], torch.full_like(base, 3.0))
    rfk.fp8_mm(*g4)
    torch.cuda.synchronize()
    assert torch.count_nonzero(g4[4]) == 0


# the reference's benchmark shapes and seeds (scripts/problems/gemm/task.yml:66-84), its input style (bf16 normals cast
# to fp8, signed normal scales)
REFERENCE_BENCHMARKS = [(1024, 1536, 7168, 8135), (1024, 3072, 1536, 6251), (1024, 576, 7168, 12346),
                        (1024, 7168, 256, 5364), (1024, 7168, 2048, 6132), (1024, 4608, 7168, 7531),
                        (1024, 7168, 2304, 12345), (1024, 512, 7168, 6563), (1024, 4096, 512, 17512),
                        (6144, 1536, 7168, 6543), (6144, 3072, 1536, 234), (6144, 576, 7168, 9863),
                        (6144, 7168, 256, 764243), (6144, 7168, 2048, 76547), (6144, 4608, 7168, 65436),
                        (6144, 7168, 2304, 452345), (6144, 512, 7168, 12341), (6144, 4096, 512, 45245)]


@pytest.mark.parametrize("m,n,k,seed", REFERENCE_BENCHMARKS)
def test_reference_benchmark_shapes_sampled_rows(rfk, m, n, k, seed):
    """Every benchmark shape of the reference under its tabled plan: 48 sampled rows (tile edges among them) against
    the oracle at the graded tolerance, few mismatches at the reference harness's atol, canary intact."""
    data = rk.generate_input_reference_style(m, n, k, seed)
    g, buf = to_gpu(data, canary_elems=1024)
    rfk.fp8_mm(*g)
    torch.cuda.synchronize()
    assert np.all(buf[g[4].numel():].float().cpu().numpy() == -7.0), "store past the end of C"
    rng = np.random.default_rng(seed)
    rows = np.unique(np.concatenate([[0, 1, 127, 128, 255, 256, m - 1], rng.integers(0, m, 41)])).astype(np.int32)
    a, b, sa, sb = rk.raw_layouts(data)
    _, exp16 = cref.ref_gemm_f32(a, b, sa, sb, rows=rows)
    got = g[4][torch.from_numpy(rows).long().cuda()]
    what = "%dx%dx%d" % (m, n, k)
    assert_close_to_oracle(got, exp16, RTOL, ATOL, what)
    assert_few_mismatches_at_reference_atol(got, exp16, what)


def test_run_entry_writes_metrics_from_the_stream_callback(rfk):
    from radeonflow_kernels_amd import gemm
    data = rk.generate_input_blockquant(256, 256, 512, 3)
    g = to_gpu(data)
    t_ms, gflops, count = gemm.run_with_metrics(*g)
    assert count == 0                      # the GEMM launcher leaves `count` alone
    assert t_ms > 0 and gflops > 0
    assert abs(gflops - 2.0 * 256 * 256 * 512 / (t_ms * 1e-3) / 1e9) <= 1e-3 * gflops
    assert_close_to_oracle(g[4], oracle_bf16(data), RTOL, ATOL, "run()")


def test_non_default_stream_and_repeat_calls(rfk):
    data = rk.generate_input_reference_style(256, 512, 1024, 11)
    exp = oracle_bf16(data)
    g = to_gpu(data)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        for _ in range(3):
            g[4].zero_()
            rfk.fp8_mm(*g)
    s.synchronize()
    assert_close_to_oracle(g[4], exp, RTOL, ATOL, "side stream")


def test_status_codes(rfk):
    L = rfk.lib()
    t = torch.zeros(1024, dtype=torch.uint8, device="cuda")
    p = t.data_ptr()
    assert L.rf_fp8_gemm(p, p, p, p, p, 16, 16, 100, None) == 1      # RF_ERR_BAD_SHAPE
    assert L.rf_fp8_gemm(p, p, p, p, p, 0, 16, 128, None) == 1
    assert L.rf_fp8_gemm(None, p, p, p, p, 16, 16, 128, None) == 2   # RF_ERR_NULL_POINTER
    bad = rfk.GemmConfig(99, 1, 1, 0)
    assert L.rf_fp8_gemm_ex(p, p, p, p, p, 16, 16, 128, ctypes.byref(bad), None) == 4
    assert b"unsupported shape" in L.rf_gemm_last_error() or L.rf_gemm_last_error() != b""


def test_plans_loaded_from_a_file_take_precedence_and_can_be_cleared(rfk, tmp_path):
    """A plan file changes what the automatic path launches for its shapes (and only for them); results stay bit-exact;
    a plan that cannot run for its shape is skipped; clearing restores the built-in choice. The environment variable
    form is checked in a fresh process."""
    import subprocess
    import sys
    m, n, k = 512, 768, 512
    before = rfk.select_config(m, n, k)
    other = rfk.select_config(1024, 1536, 7168)
    forced = (1, 2, 4, 0) if (before.variant, before.split_k) != (1, 2) else (3, 1, 4, 0)
    path = tmp_path / "my.plans"
    path.write_text("%d %d %d 0 1 8 2\n" % (m, n, k + 128)                      # persistent with an odd number of K blocks: skipped
                    + "%d %d %d %d %d %d %d\n" % ((m, n, k) + forced))
    try:
        assert rfk.load_plans(str(path)) == 2
        got = rfk.select_config(m, n, k)
        assert (got.variant, got.split_k, got.group_m, got.stream_k) == forced
        odd = rfk.select_config(m, n, k + 128)
        assert odd.stream_k != 2
        again = rfk.select_config(1024, 1536, 7168)
        assert (again.variant, again.split_k, again.stream_k) == (other.variant, other.split_k, other.stream_k)
        data = exact_problem(m, n, k, seed=77)
        assert np.array_equal(bf16_bits(_run(rfk, data, canary=256)), oracle_bf16(data))
    finally:
        rfk.clear_plans()
    after = rfk.select_config(m, n, k)
    assert (after.variant, after.split_k, after.stream_k) == (before.variant, before.split_k, before.stream_k)
    code = ("import radeonflow_kernels_amd as r; c = r.select_config(%d, %d, %d); "
            "print(c.variant, c.split_k, c.group_m, c.stream_k)" % (m, n, k))
    env = dict(os.environ, RF_GEMM_PLANS=str(path))
    out = subprocess.run([sys.executable, "-c", code], env=env, cwd=ROOT, stdout=subprocess.PIPE, text=True, timeout=300)
    assert out.returncode == 0 and tuple(int(x) for x in out.stdout.split()) == forced
    env["RF_GEMM_PLANS"] = str(tmp_path / "missing.plans")
    out = subprocess.run([sys.executable, "-c", code], env=env, cwd=ROOT, stdout=subprocess.PIPE,
                         stderr=subprocess.PIPE, text=True, timeout=300)
    assert out.returncode != 0 and "cannot open plan file" in out.stderr


def _random_shapes(count, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        # tile multiples, multiples of 192, ragged multiples of 16 and the occasional odd size, K from 1 to 20 blocks
        m = int(rng.choice([rng.integers(1, 33) * 128, rng.integers(1, 22) * 192, rng.integers(1, 200) * 16,
                            rng.integers(1, 700)]))
        n = int(rng.choice([rng.integers(1, 33) * 128, rng.integers(1, 22) * 192, rng.integers(1, 200) * 16,
                            rng.integers(1, 700)]))
        k = int(rng.integers(1, 21)) * 128
        out.append((m, n, k))
    return out


@pytest.mark.parametrize("m,n,k", _random_shapes(28, seed=20240607))
def test_automatic_plan_on_random_shapes_is_bit_exact(rfk, m, n, k):
    """Whatever plan the table or the cost model picks for a shape nobody tuned (any tile family, K split, persistent
    schedule, bounds-checked kernel), the result on exactly representable data equals the oracle bit for bit and
    nothing is stored past the end of C."""
    data = exact_problem(m, n, k, seed=m * 31 + n * 7 + k)
    out = _run(rfk, data, canary=512)
    assert np.array_equal(bf16_bits(out), oracle_bf16(data)), "plan %r" % (rfk.select_config(m, n, k),)


@pytest.mark.parametrize("m,n,k", [(100, 4096, 512), (1000, 576, 1024), (257, 1000, 256), (1, 4096, 7168), (7, 2050, 384),
                                   (4097, 130, 256), (1020, 768, 512), (500, 1536, 2048), (2040, 2048, 256)])
def test_ragged_shapes_above_the_size_threshold_run_padded_and_bit_exact(rfk, m, n, k):
    """M or N not a multiple of 16 (or below 16): the operands are staged with padded rows, the tiled kernels run on
    the padded shape; C is written in place when only M is ragged (directly or by the split-K reduction) and comes
    back from a staged copy otherwise (ragged N, or a padded M that takes the persistent schedule). Exact data must match the oracle bit for bit, nothing may be
    stored past the end of C, and the reported plan is a tiled one."""
    assert rfk.select_config(m, n, k).variant >= 0
    data = exact_problem(m, n, k, seed=3 * m + 5 * n + k)
    for rep in range(2):                                           # the staging buffer is reused
        out = _run(rfk, data, canary=777)
        assert np.array_equal(bf16_bits(out), oracle_bf16(data)), "repetition %d" % rep


def test_unaligned_operands_run_padded_and_bit_exact(rfk):
    """Operands that start 1, 2 and 4 bytes off a 16-byte boundary (views into larger buffers)."""
    m, n, k = 256, 384, 512
    data = exact_problem(m, n, k, seed=99)
    a, b, sa, sb, _ = data
    dev, fp8 = torch.device("cuda:0"), torch.float8_e4m3fn

    def shifted(t_km, off):                                       # [rows, K] view, stride (1, rows), storage offset off
        rows = t_km.shape[0]
        flat = torch.zeros(t_km.numel() + 64, dtype=torch.uint8, device=dev)
        flat[off:off + t_km.numel()] = t_km.T.contiguous().view(torch.uint8).reshape(-1).to(dev)
        return flat[off:off + t_km.numel()].view(fp8).view(t_km.shape[1], rows).T

    g = to_gpu(data)
    cbuf = torch.full((m * n + 64,), -7.0, dtype=torch.bfloat16, device=dev)
    c = cbuf[2:2 + m * n].view(m, n)                              # 4 bytes off
    assert c.data_ptr() % 16 == 4
    rfk.fp8_mm(shifted(a, 1), shifted(b, 2), g[2], g[3], c)
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(c), oracle_bf16(data))
    assert float(cbuf[:2].float().abs().max()) == 7.0 and float(cbuf[2 + m * n:].float().abs().min()) == 7.0



def test_library_side_timing_loop(rfk):
    """rf_fp8_gemm_time launches the plan warmup + iters times and reports a plausible average; the result buffer holds
    the GEMM afterwards; bad arguments are refused."""
    m, n, k = 256, 384, 512
    data = exact_problem(m, n, k, seed=4)
    g = to_gpu(data)
    us = rfk.fp8_mm_time(*g, warmup=2, iters=50)
    torch.cuda.synchronize()
    assert 0.5 < us < 200.0
    assert np.array_equal(bf16_bits(g[4]), oracle_bf16(data))
    forced = rfk.fp8_mm_time(*g, config=rfk.GemmConfig(1, 2, 4, 0), warmup=1, iters=10)
    assert 0.5 < forced < 400.0
    with pytest.raises(RuntimeError):
        rfk.fp8_mm_time(*g, iters=0)


def test_hip_graph_replays_match_eager(rfk):
    """Quantiser + GEMM (automatic plan, a split-K plan with its reduction, the persistent schedule) captured into one
    HIP graph: every replay, with new inputs and eager launches in between, gives the bits of the eager run. The
    library allocates nothing during the capture because the eager runs before it have grown the split-K workspace."""
    m, n, k = 512, 512, 1024
    dev = torch.device("cuda:0")
    gen = torch.Generator().manual_seed(5)
    b, sb = rfk.quantize_b(torch.randn((n, k), generator=gen).to(dev))
    xs = [torch.randn((m, k), generator=gen).to(dev) for _ in range(4)]
    plans = [None, rfk.GemmConfig(3, 4, 8, 0), rfk.GemmConfig(0, 1, 4, 2)]

    def step(x, outs):
        a, sa = rfk.quantize_a(x)
        for c, plan in zip(outs, plans):
            rfk.fp8_mm(a, b, sa, sb, c, config=plan)

    def outputs():
        return [torch.zeros((m, n), dtype=torch.bfloat16, device=dev) for _ in plans]

    eager = [outputs() for _ in xs]
    for x, outs in zip(xs, eager):
        step(x, outs)
    torch.cuda.synchronize()
    assert not torch.equal(eager[0][0], eager[1][0])
    x_static, outs_static = xs[0].clone(), outputs()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(x_static, outs_static)
    for i in (1, 2, 3, 0, 2):
        x_static.copy_(xs[i])
        for c in outs_static:
            c.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for c, e, plan in zip(outs_static, eager[i], plans):
            assert torch.equal(c.view(torch.uint16), e.view(torch.uint16)), "replay with input %d, plan %r" % (i, plan)
        again = outputs()                      # the program's own eager work between two replays
        step(xs[(i + 1) % 4], again)
        torch.cuda.synchronize()
        assert torch.equal(again[1].view(torch.uint16), eager[(i + 1) % 4][1].view(torch.uint16))


def test_operand_beyond_2_gib_is_addressed_with_64_bits(rfk):
    """A of more than 2^31 bytes: rows near the end are reached only if every index is computed in 64 bits. Values in
    {0, +-1} and scales in {0.5, 1, 2} keep every sum exact in fp32, so sampled rows must match the oracle bit for bit."""
    m, n, k = 163840, 256, 13312
    assert m * k > 2 ** 31
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(11)
    codes = torch.tensor([0x00, 0x38, 0xB8, 0x38], dtype=torch.uint8, device=dev)
    a8 = codes[torch.randint(0, 4, (k, m), device=dev, generator=gen)]
    b8 = codes[torch.randint(0, 4, (k, n), device=dev, generator=gen)]
    pow2 = torch.tensor([0.5, 1.0, 2.0], device=dev)
    sa = pow2[torch.randint(0, 3, (k // 128, m), device=dev, generator=gen)]
    sb = pow2[torch.randint(0, 3, (k // 128, n // 128), device=dev, generator=gen)]
    c = torch.zeros((m, n), dtype=torch.bfloat16, device=dev)
    fp8 = torch.float8_e4m3fn
    rows = np.unique(np.concatenate([[0, 1, 77, m // 2, m - 17, m - 1],
                                     np.random.default_rng(5).integers(0, m, 26)])).astype(np.int32)
    exp = cref.ref_gemm_blockfold(a8.cpu().numpy(), b8.cpu().numpy(), sa.cpu().numpy(), sb.cpu().numpy(), rows=rows)[1]
    for cfg in (None, rfk.GemmConfig(3, 1, 8, 0), rfk.GemmConfig(0, 2, 4, 0)):
        c.zero_()
        rfk.fp8_mm(a8.view(fp8).T, b8.view(fp8).T, sa.T, sb.T, c, config=cfg)
        torch.cuda.synchronize()
        got = bf16_bits(c[torch.from_numpy(rows.astype(np.int64)).to(dev)])
        assert np.array_equal(got, exp), "plan %r" % (cfg,)


@pytest.mark.parametrize("m,n,k", [(256, 384, 512), (1024, 576, 1024), (100, 130, 256)])
def test_signed_zeros_and_negative_scales(rfk, m, n, k):
    """Rows of -0 and +0 codes and rows with negative scales (the reference draws signed scales,
    tests/gemm/gemm_test.cpp:90-92): sums of signed zeros must come out as the oracle's +0, bit for bit, under every plan."""
    a, b, sa, sb, c = exact_problem(m, n, k, seed=5)
    a8, b8 = a.view(torch.uint8).clone(), b.view(torch.uint8).clone()
    a8[0:m:3, :] = 0x80
    a8[1:m:7, :] = 0x00
    b8[0:n:5, :] = 0x80
    sa = sa.clone()
    sa[2:m:4, :] *= -1.0
    data = (a8.view(torch.float8_e4m3fn), b8.view(torch.float8_e4m3fn), sa, sb, c)
    exp = oracle_bf16(data)
    plans = [None]
    if m % 16 == 0 and n % 16 == 0:
        plans += [rfk.GemmConfig(v["variant"], s, 4, 0) for v in rfk.variants() for s in (1, 2, 4) if rfk.plan_can_run(v, s, k)]
        plans += [rfk.GemmConfig(v["variant"], 1, 4, 2) for v in rfk.variants()
                  if v["persistent"] and m % v["block_m"] == 0 and n % v["block_n"] == 0 and (k // 128) % 2 == 0]
    for cfg in plans:
        out = _run(rfk, data, config=cfg)
        assert np.array_equal(bf16_bits(out), exp), "plan %r" % (cfg,)


@pytest.mark.parametrize("m,n,k", [(256, 384, 512), (1024, 576, 1024), (100, 130, 256)])
def test_nan_codes_poison_their_row_or_column_only(rfk, m, n, k):
    """e4m3fn NaN codes (0x7f, 0xff) in A make the whole output row NaN, in B the whole column, exactly where the oracle
    has NaN (the reference's checker requires NaN positions to match, tests/checker/checker.cpp:10-105); everything else
    stays bit-exact."""
    a, b, sa, sb, c = exact_problem(m, n, k, seed=6)
    a8, b8 = a.view(torch.uint8).clone(), b.view(torch.uint8).clone()
    a8[5, 17] = 0x7F
    a8[m - 1, k - 1] = 0xFF
    b8[3, k // 2] = 0x7F
    data = (a8.view(torch.float8_e4m3fn), b8.view(torch.float8_e4m3fn), sa, sb, c)
    exp = oracle_bf16(data)
    exp_nan = (exp & 0x7FFF) > 0x7F80
    assert exp_nan[5].all() and exp_nan[m - 1].all() and exp_nan[:, 3].all() and exp_nan.sum() == 2 * n + m - 2
    plans = [None]
    if m % 16 == 0 and n % 16 == 0:
        plans += [rfk.GemmConfig(v["variant"], s, 4, 0) for v in rfk.variants() for s in (1, 3) if rfk.plan_can_run(v, s, k)]
        plans += [rfk.GemmConfig(v["variant"], 1, 4, 2) for v in rfk.variants()
                  if v["persistent"] and m % v["block_m"] == 0 and n % v["block_n"] == 0 and (k // 128) % 2 == 0]
    for cfg in plans:
        got = bf16_bits(_run(rfk, data, config=cfg))
        got_nan = (got & 0x7FFF) > 0x7F80
        assert np.array_equal(got_nan, exp_nan), "NaN positions, plan %r" % (cfg,)
        assert np.array_equal(got[~exp_nan], exp[~exp_nan]), "plan %r" % (cfg,)


def _random_operands(m, n, k, seed):
    """fp8 codes 0..119 (finite, positive) and positive scales: rounding everywhere, no structure for a kernel to lean on"""
    gen = torch.Generator(device="cuda").manual_seed(seed)
    fp8 = torch.float8_e4m3fn
    a = torch.randint(0, 120, (k, m), dtype=torch.uint8, device="cuda", generator=gen).view(fp8).T
    b = torch.randint(0, 120, (k, n), dtype=torch.uint8, device="cuda", generator=gen).view(fp8).T
    sa = (torch.rand((k // 128, m), device="cuda", generator=gen) * 1e-2).T
    sb = (torch.rand((k // 128, (n + 127) // 128), device="cuda", generator=gen) * 1e-2).T
    return a, b, sa, sb


def _bits_under(rfk, ops, m, n, cfg):
    c = torch.full((m, n), -3.0, dtype=torch.bfloat16, device="cuda")
    rfk.fp8_mm(*ops, c, config=cfg)
    torch.cuda.synchronize()
    return bf16_bits(c)


def test_skinny_k_schedule_on_random_shapes_equals_the_tile_kernel(rfk):
    """40 seeded random shapes (M a multiple of 16 up to 8300, N a multiple of 64 up to 7600, K = 128 ... 512) with
    rounding in every product: the skinny-K schedule gives the bits of the one-workgroup-per-tile kernel, twice."""
    rng = np.random.default_rng(3)
    for case in range(40):
        m = int(rng.integers(1, 260)) * 16 if rng.random() < 0.7 else int(rng.integers(1, 520)) * 16
        n = int(rng.integers(1, 65)) * 64 if rng.random() < 0.7 else int(rng.integers(1, 120)) * 64
        k = int(rng.choice([128, 256, 384, 512]))
        ops = _random_operands(m, n, k, case)
        ref = _bits_under(rfk, ops, m, n, rfk.GemmConfig(1, 1, 8, 0))
        for rep in range(2):
            assert np.array_equal(_bits_under(rfk, ops, m, n, rfk.GemmConfig(0, 1, 8, 4)), ref), (m, n, k, rep)


def test_k_split_inside_the_workgroup_on_random_shapes_equals_the_two_launch_form(rfk):
    """30 seeded random shapes with an even number of K blocks: every variant that splits K between two wave groups
    gives the bits of its one-group twin with split_k = 2 (partial sums through memory + reduction kernel)."""
    rng = np.random.default_rng(7)
    pairs = [(v["variant"], w["variant"]) for v in rfk.variants() if v["k_groups"] == 2 for w in rfk.variants()
             if w["k_groups"] == 1 and (w["block_m"], w["block_n"], w["waves_m"], w["waves_n"]) ==
             (v["block_m"], v["block_n"], v["waves_m"], v["waves_n"]) and 0 <= v["lds_bytes"] - 2 * w["lds_bytes"] < 4096]
    assert len(pairs) >= 2
    for case in range(30):
        m, n, k = int(rng.integers(1, 130)) * 16, int(rng.integers(1, 200)) * 16, int(rng.integers(1, 30)) * 256
        ops = _random_operands(m, n, k, 100 + case)
        for v, twin in pairs:
            ref = _bits_under(rfk, ops, m, n, rfk.GemmConfig(twin, 2, 8, 0))
            assert np.array_equal(_bits_under(rfk, ops, m, n, rfk.GemmConfig(v, 1, 8, 0)), ref), (v, m, n, k)
