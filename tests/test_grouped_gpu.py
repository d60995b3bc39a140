"""Grouped GEMM (one launch, rows sorted by group, one weight matrix per group) against the oracle applied group
by group. Exact data for bit-for-bit equality, quantised N(0,1) data at the graded tolerance."""
import numpy as np
import pytest
import torch

from oracle import cref, ref_kernel as rk
from helpers import RTOL, ATOL, assert_close_to_oracle, bf16_bits, exact_problem, oracle_bf16

pytestmark = pytest.mark.gpu
CANARY = 2048


@pytest.fixture(scope="module")
def rfk():
    import radeonflow_kernels_amd as m
    m.lib()
    return m


def _grouped_problem(rows, n, k, seed, exact):
    """Per-group problems from the usual generators, glued into the grouped layouts.
    Returns (device tensors a, b, a_scale, b_scale, c, canary buffer), row_offsets, expected bf16 bits [M_total, N]."""
    offs = np.concatenate([[0], np.cumsum(rows)]).astype(np.int64)
    m_total, groups = int(offs[-1]), len(rows)
    qk, qn = k // 128, (n + 127) // 128
    a_km = np.zeros((k, m_total), np.uint8)
    as_qm = np.zeros((qk, m_total), np.float32)
    b_gkn = np.zeros((groups, k, n), np.uint8)
    bs_gqq = np.zeros((groups, qk, qn), np.float32)
    exp = np.zeros((m_total, n), np.uint16)
    for g, r in enumerate(rows):
        mg = max(int(r), 16)            # empty groups still get weights
        data = exact_problem(mg, n, k, seed + g) if exact else rk.generate_input_blockquant(mg, n, k, seed + g)
        a, b, sa, sb = rk.raw_layouts(data)
        b_gkn[g], bs_gqq[g] = b, sb
        if r:
            a_km[:, offs[g]:offs[g + 1]] = a[:, :r]
            as_qm[:, offs[g]:offs[g + 1]] = sa[:, :r]
            sub = (data[0][:r], data[1], data[2][:r], data[3], torch.zeros((int(r), n), dtype=torch.bfloat16))
            exp[offs[g]:offs[g + 1]] = oracle_bf16(sub)
    dev, fp8 = torch.device("cuda:0"), torch.float8_e4m3fn
    a_t = torch.from_numpy(a_km).to(dev).view(fp8).T                       # [M_total, K] stride (1, M_total)
    as_t = torch.from_numpy(as_qm).to(dev).T
    b_t = torch.from_numpy(b_gkn).to(dev).view(fp8).permute(0, 2, 1)       # [G, N, K] stride (K*N, 1, N)
    bs_t = torch.from_numpy(bs_gqq).to(dev).permute(0, 2, 1)
    buf = torch.full((m_total * n + CANARY,), -7.0, dtype=torch.bfloat16, device=dev)
    c = buf[: m_total * n].view(m_total, n)
    c.zero_()
    return (a_t, b_t, as_t, bs_t, c, buf), [int(x) for x in offs], exp


def _check_canary(buf, used):
    assert np.all(buf[used:].float().cpu().numpy() == -7.0), "store past the end of C"


CASES = [([256, 128, 512, 64], 512, 256), ([16, 0, 48, 400, 0, 32], 576, 384), ([1024], 256, 512),
         ([128] * 32, 2048, 256), ([0, 0, 272], 144, 128), ([640, 16, 16, 2048, 112], 7168, 256),
         ([272, 384, 128, 400, 16, 656], 512, 256),      # left-overs of 16, 128, 128, 144, 16 and 144 rows
         ([int(x) * 16 for x in np.random.default_rng(7).integers(0, 40, 24)], 768, 384)]   # 24 groups of 0..624 rows


@pytest.mark.parametrize("rows,n,k", CASES)
def test_grouped_bit_exact_on_exact_data(rfk, rows, n, k):
    g, offs, exp = _grouped_problem(rows, n, k, seed=11 * n + k, exact=True)
    for variant in (-1, 0, 1, 2, 3, 4, 5):
        g[4].zero_()
        rfk.fp8_mm_grouped(*g[:5], offs, variant=variant)
        torch.cuda.synchronize()
        assert np.array_equal(bf16_bits(g[4]), exp), "variant %d" % variant
        _check_canary(g[5], g[4].numel())


@pytest.mark.parametrize("rows,n,k", [([256, 128, 512, 64], 512, 1024), ([48, 400, 32], 576, 7168)])
def test_grouped_quantised_data_within_tolerance(rfk, rows, n, k):
    g, offs, exp = _grouped_problem(rows, n, k, seed=5, exact=False)
    rfk.fp8_mm_grouped(*g[:5], offs)
    torch.cuda.synchronize()
    assert_close_to_oracle(g[4], exp, RTOL, ATOL, "grouped")
    _check_canary(g[5], g[4].numel())


@pytest.mark.parametrize("rows,n,k", [([5, 17, 0, 100], 130, 256), ([33, 64], 72, 128), ([7, 9], 64, 128)])
def test_grouped_ragged_n_or_tiny_problems_take_the_checked_kernel(rfk, rows, n, k):
    g, offs, exp = _grouped_problem(rows, n, k, seed=3, exact=True)
    rfk.fp8_mm_grouped(*g[:5], offs)
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(g[4]), exp)
    _check_canary(g[5], g[4].numel())


RAGGED = [([5, 17, 0, 100, 333, 1], 512, 256), ([1, 1, 1, 1, 300], 256, 384), ([255, 257, 129, 0, 143, 15], 768, 256),
          ([1000], 256, 128), ([int(x) for x in np.random.default_rng(3).integers(0, 300, 40)], 576, 256),
          ([int(x) for x in np.random.default_rng(4).integers(0, 21, 256)], 256, 128)]      # 256 groups of 0..20 rows


@pytest.mark.parametrize("rows,n,k", RAGGED)
def test_grouped_any_group_sizes_bit_exact(rfk, rows, n, k):
    """Group sizes that are not multiples of 16 (what token routing produces): A is staged with padded groups, C is
    written in place, so rows of the next group must survive and nothing may land past the end."""
    g, offs, exp = _grouped_problem(rows, n, k, seed=31 + n, exact=True)
    for variant in (-1, 0, 1, 2, 3, 4, 5):
        g[4].fill_(-3.0)
        rfk.fp8_mm_grouped(*g[:5], offs, variant=variant)
        torch.cuda.synchronize()
        assert np.array_equal(bf16_bits(g[4]), exp), "variant %d" % variant
        _check_canary(g[5], g[4].numel())


def test_grouped_any_group_sizes_quantised_data(rfk):
    rows, n, k = [77, 130, 1, 260, 45], 1024, 1024
    g, offs, exp = _grouped_problem(rows, n, k, seed=8, exact=False)
    rfk.fp8_mm_grouped(*g[:5], offs)
    torch.cuda.synchronize()
    assert_close_to_oracle(g[4], exp, RTOL, ATOL, "grouped, ragged sizes")
    _check_canary(g[5], g[4].numel())


@pytest.mark.parametrize("shift", [1, 2, 3, 7])
def test_grouped_unaligned_a(rfk, shift):
    """A that does not start on a 16-byte boundary (a view into a larger buffer) goes through the same staging copy."""
    rows, n, k = [48, 100, 16], 256, 256
    g, offs, exp = _grouped_problem(rows, n, k, seed=2, exact=True)
    a = g[0]
    m_total = a.shape[0]
    raw = torch.zeros(k * m_total + 64, dtype=torch.uint8, device=a.device)
    raw[shift:shift + k * m_total] = a.T.contiguous().view(torch.uint8).reshape(-1)
    a2 = raw[shift:shift + k * m_total].view(k, m_total).view(torch.float8_e4m3fn).T
    assert a2.data_ptr() % 16 == shift
    rfk.fp8_mm_grouped(a2, *g[1:5], offs)
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(g[4]), exp)


def test_grouped_equals_separate_gemms(rfk):
    """The grouped launch and one plain fp8_mm per group give the same bits (same kernel family, same order)."""
    rows, n, k = [256, 384, 128], 1536, 1024
    g, offs, _ = _grouped_problem(rows, n, k, seed=9, exact=False)
    rfk.fp8_mm_grouped(*g[:5], offs, variant=1)
    torch.cuda.synchronize()
    a, b, sa, sb, c = g[:5]
    for i, r in enumerate(rows):
        lo, hi = offs[i], offs[i + 1]
        ai = a[lo:hi].T.contiguous().T                # standalone [r, K] with stride (1, r)
        si = sa[lo:hi].T.contiguous().T
        ci = torch.zeros((r, n), dtype=torch.bfloat16, device=a.device)
        rfk.fp8_mm(ai, b[i], si, sb[i], ci, config=rfk.GemmConfig(3, 1, 8, 0))      # 128x256 tiles, like variant 1
        torch.cuda.synchronize()
        assert torch.equal(ci.view(torch.uint16), c[lo:hi].view(torch.uint16)), "group %d" % i


def test_grouped_status_codes(rfk):
    import ctypes
    L = rfk.lib()
    offs = (ctypes.c_int32 * 3)(0, 16, 8)
    assert L.rf_fp8_gemm_grouped(None, None, None, None, None, offs, 2, 128, 128, -1, None) == 1      # decreasing offsets
    offs = (ctypes.c_int32 * 2)(0, 0)
    assert L.rf_fp8_gemm_grouped(None, None, None, None, None, offs, 1, 128, 128, -1, None) == 0      # nothing to do
    offs = (ctypes.c_int32 * 2)(0, 16)
    assert L.rf_fp8_gemm_grouped(None, None, None, None, None, offs, 1, 128, 128, -1, None) == 2      # null pointers
    assert L.rf_fp8_gemm_grouped(None, None, None, None, None, offs, 1, 128, 100, -1, None) == 1      # bad K
    assert L.rf_fp8_gemm_grouped(None, None, None, None, None, offs, 300, 128, 128, -1, None) == 1    # too many groups


PADDED_CASES = [([100, 37, 0, 400, 1, 16, 255], 512, 256), ([5] * 40, 256, 384), ([1000], 256, 128),
                ([0, 0, 17], 144, 128), ([int(x) for x in np.random.default_rng(11).integers(0, 300, 48)], 768, 512)]


@pytest.mark.parametrize("kind", ["f32", "bf16"])
@pytest.mark.parametrize("rows,n,k", PADDED_CASES)
def test_grouped_quantiser_writes_the_padded_layout_of_the_oracle_quantiser(rfk, rows, n, k, kind):
    """quantize_a_grouped: every group's rows start at a multiple of 16 and equal, bit for bit, the oracle quantiser's
    rows of the same activations (values with ties, zeros and large magnitudes among them); the padding rows hold zero
    codes with scale 1; nothing is written past the padded matrix."""
    rng = np.random.default_rng(sum(rows) + k)
    offs = [0] + [int(x) for x in np.cumsum(rows)]
    m_total = offs[-1]
    x = (rng.standard_normal((m_total, k)) * rng.choice([1e-3, 1.0, 300.0], (m_total, 1))).astype(np.float32)
    x[rng.random((m_total, k)) < 0.05] = 0.0
    xt = torch.from_numpy(x).cuda()
    if kind == "bf16":
        xt = xt.to(torch.bfloat16)
        x = xt.float().cpu().numpy()
    a_ref, as_ref = cref.quantize_a(x)                          # [K][M_total], [K/128][M_total]
    pad = rfk.grouped_padded_offsets(offs)
    assert pad[0] == 0 and all(p % 16 == 0 for p in pad) and pad[-1] == sum((r + 15) // 16 * 16 for r in rows)
    a, sa = rfk.quantize_a_grouped(xt, offs)
    torch.cuda.synchronize()
    a_np = a.T.contiguous().view(torch.uint8).cpu().numpy()     # [K][M_pad]
    sa_np = sa.T.contiguous().cpu().numpy()
    assert a_np.shape == (k, pad[-1]) and sa_np.shape == (k // 128, pad[-1])
    for g, r in enumerate(rows):
        assert np.array_equal(a_np[:, pad[g]:pad[g] + r], a_ref[:, offs[g]:offs[g + 1]]), "codes of group %d" % g
        assert np.array_equal(sa_np[:, pad[g]:pad[g] + r], as_ref[:, offs[g]:offs[g + 1]]), "scales of group %d" % g
        assert not a_np[:, pad[g] + r:pad[g + 1]].any() and np.all(sa_np[:, pad[g] + r:pad[g + 1]] == 1.0)


@pytest.mark.parametrize("rows,n,k", PADDED_CASES)
def test_grouped_gemm_on_the_padded_layout_equals_the_staged_path(rfk, rows, n, k):
    """Activations quantised straight into the padded layout, then fp8_mm_grouped_padded: the same bits as quantising
    them back to back and letting fp8_mm_grouped stage them, for every tile variant; rows of C outside the groups'
    true rows do not exist and the canary behind C stays intact."""
    rng = np.random.default_rng(sum(rows) + n)
    offs = [0] + [int(x) for x in np.cumsum(rows)]
    m_total, groups = offs[-1], len(rows)
    x = torch.from_numpy(rng.standard_normal((m_total, k)).astype(np.float32)).cuda()
    w = torch.from_numpy(rng.standard_normal((groups * n, k)).astype(np.float32)).cuda()
    b2, sb2 = rfk.quantize_b(w)                                 # [G*N, K] stride (1, G*N): regroup into [G][K][N]
    fp8 = torch.float8_e4m3fn
    b = b2.T.contiguous().view(torch.uint8).view(k, groups, n).permute(1, 0, 2).contiguous().view(fp8).permute(0, 2, 1)
    qn = (n + 127) // 128
    if n % 128 == 0:
        sb = sb2.T.contiguous().view(k // 128, groups, qn).permute(1, 0, 2).contiguous().permute(0, 2, 1)
    else:                                                       # a group's blocks do not line up: one scale everywhere
        sb = torch.full((groups, k // 128, qn), 0.01, device="cuda").permute(0, 2, 1)
    a_flat, sa_flat = rfk.quantize_a(x)
    a_pad, sa_pad = rfk.quantize_a_grouped(x, offs)
    for variant in (-1, 0, 1, 2, 3, 4, 5):
        buf = torch.full((m_total * n + CANARY,), -7.0, dtype=torch.bfloat16, device="cuda")
        c1 = torch.zeros((m_total, n), dtype=torch.bfloat16, device="cuda")
        c2 = buf[: m_total * n].view(m_total, n)
        c2.zero_()
        rfk.fp8_mm_grouped(a_flat, b, sa_flat, sb, c1, offs, variant=variant)
        rfk.fp8_mm_grouped_padded(a_pad, b, sa_pad, sb, c2, offs, variant=variant)
        torch.cuda.synchronize()
        assert torch.equal(c1.view(torch.uint16), c2.view(torch.uint16)), "variant %d" % variant
        assert bool(c1.float().abs().sum() > 0)
        _check_canary(buf, m_total * n)


def test_grouped_queue_form_repeats_two_streams_and_graph_replays(rfk):
    """The queue form (variant 5: resident workgroups that draw tiles from one counter per XCD). Its counters return
    to zero with the last draw of every launch, so launches of different layouts follow each other on one stream
    without a clear in between; two streams have their own counters and may overlap; a launch captured into a HIP graph
    replays to the same bits, with the program's own eager launches between the replays. Layouts: 24 uneven groups
    (whole groups per queue), 5 groups (the line cut by estimated time), 3 tiles in all (fewer than workgroups)."""
    layouts = [([int(x) * 16 for x in np.random.default_rng(9).integers(0, 40, 24)], 768, 384),
               ([272, 16, 640, 0, 128], 512, 256), ([64, 16, 48], 256, 128)]
    probs = [_grouped_problem(rows, n, k, seed=77 + n, exact=True) for rows, n, k in layouts]

    def launch_and_check(i, stream=None):
        g, offs, exp = probs[i]
        g[4].fill_(-5.0)
        with torch.cuda.stream(stream or torch.cuda.current_stream()):
            rfk.fp8_mm_grouped(*g[:5], offs, variant=5)
        return lambda: (np.array_equal(bf16_bits(g[4]), exp), "layout %d" % i)

    for i in (0, 1, 2, 1, 0, 0, 2):                       # one stream, no clear between launches
        check = launch_and_check(i)
        torch.cuda.synchronize()
        ok, what = check()
        assert ok, what
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    for _ in range(4):                                    # two streams at once, each with its own counters
        c1, c2 = launch_and_check(0, s1), launch_and_check(1, s2)
        torch.cuda.synchronize()
        for ok, what in (c1(), c2()):
            assert ok, "two streams, " + what
    g, offs, exp = probs[0]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rfk.fp8_mm_grouped(*g[:5], offs, variant=5)
    for _ in range(3):
        g[4].fill_(-5.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(bf16_bits(g[4]), exp), "graph replay"
        check = launch_and_check(1)                       # eager work between two replays
        torch.cuda.synchronize()
        assert check()[0]


def test_grouped_uneven_groups_take_the_queue_form_automatically(rfk):
    """Uneven groups whose last tiles are much shorter than 128 rows, enough of them for 2.5 items per compute unit: the
    automatic choice is the queue form (rf_grouped_variant_for says so) and gives the bits of every other form (all
    compute a row of C with the same operations in the same order)."""
    rows = [16, 32, 272, 48, 528, 64, 16, 80, 304, 16, 32, 144, 16, 784, 48, 32, 16, 64, 272, 16] * 2
    g, offs, exp = _grouped_problem(rows, 4096, 256, seed=123, exact=True)
    assert rfk.grouped_variant_for(offs, 4096, 256, torch.cuda.get_device_properties(0).multi_processor_count) == 5
    for variant in (-1, 5, 1):
        g[4].zero_()
        rfk.fp8_mm_grouped(*g[:5], offs, variant=variant)
        torch.cuda.synchronize()
        assert np.array_equal(bf16_bits(g[4]), exp), "variant %d" % variant
    _check_canary(g[5], g[4].numel())


def test_grouped_queue_form_on_random_layouts_equals_the_128_row_tiles(rfk):
    """60 seeded random layouts (1 to 256 groups of 0 to 700 rows, half of them with sizes that are not multiples of 16;
    N = 256 ... 4096, K = 128 ... 1024) with rounding in every product: the queue form, the queue form again and the
    automatic choice give the bits of the 128 x 256 tiles, and rows of C outside the groups' rows keep their fill."""
    rng = np.random.default_rng(1)
    fp8 = torch.float8_e4m3fn
    for case in range(60):
        groups = int(rng.choice([1, 2, 3, 5, 8, 13, 16, 17, 31, 64, 100, 200, 256]))
        hi = int(rng.choice([20, 70, 130, 300, 700]))
        sizes = [int(x) for x in rng.integers(0, hi + 1, groups)]
        if rng.random() < 0.5:
            sizes = [s // 16 * 16 for s in sizes]
        if sum(sizes) == 0:
            sizes[0] = 16
        n, k = int(rng.choice([256, 272, 512, 768, 1024, 1536, 2048, 4096])), int(rng.choice([128, 256, 384, 512, 1024]))
        offs = [0] + [int(x) for x in np.cumsum(sizes)]
        gm = offs[-1]
        gen = torch.Generator(device="cuda").manual_seed(case)
        a = torch.randint(0, 120, (k, gm), dtype=torch.uint8, device="cuda", generator=gen).view(fp8).T
        b = torch.randint(0, 120, (groups, k, n), dtype=torch.uint8, device="cuda", generator=gen).view(fp8).permute(0, 2, 1)
        sa = (torch.rand((k // 128, gm), device="cuda", generator=gen) * 1e-2).T
        sb = (torch.rand((groups, k // 128, (n + 127) // 128), device="cuda", generator=gen) * 1e-2).permute(0, 2, 1)
        outs = []
        for variant in (1, 5, 5, -1):
            c = torch.full((gm, n), -3.0, dtype=torch.bfloat16, device="cuda")
            rfk.fp8_mm_grouped(a, b, sa, sb, c, offs, variant=variant)
            torch.cuda.synchronize()
            outs.append(bf16_bits(c))
        for o in outs[1:]:
            assert np.array_equal(outs[0], o), (case, groups, n, k, sizes[:12])
