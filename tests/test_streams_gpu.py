"""GPU tests of the launch path's temporary memory: launches on different streams of one device do not share buffers,
buffer growth never waits for the device, and plans that cannot run are skipped at lookup."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import ref_kernel as rk
from helpers import bf16_bits, exact_problem, oracle_bf16, to_gpu

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rfk():
    import radeonflow_kernels_amd as r
    assert torch.cuda.is_available(), "these tests need the GPU"
    r.lib()
    return r


def _alone(rfk, g):
    g[4].zero_()
    rfk.fp8_mm(*g)
    torch.cuda.synchronize()
    return bf16_bits(g[4]).copy()


def test_split_k_and_ragged_launches_on_three_streams_match_their_single_stream_results(rfk):
    """Two split-K GEMMs of the C1 shape and one ragged-M GEMM (staged through the pad buffer, split along K as well)
    run concurrently on three streams with different data, several launches deep. Each result equals, bit for bit,
    what the same call gives when it has the device to itself."""
    m, n, k = 1024, 1536, 7168
    assert rfk.select_config(m, n, k).split_k > 1, "this test wants a split-K plan for the C1 shape"
    problems = [to_gpu(rk.generate_input_blockquant(m, n, k, seed)) for seed in (101, 202)]
    problems.append(to_gpu(rk.generate_input_blockquant(1000, 1536, 7168, 303)))        # ragged M: staged copy
    alone = [_alone(rfk, g) for g in problems]
    assert not np.array_equal(alone[0], alone[1])
    streams = [torch.cuda.Stream() for _ in problems]
    for g in problems:
        g[4].zero_()
    torch.cuda.synchronize()
    for _ in range(6):                                   # deep queues, so the launches really overlap
        for g, s in zip(problems, streams):
            with torch.cuda.stream(s):
                rfk.fp8_mm(*g)
    torch.cuda.synchronize()
    for i, g in enumerate(problems):
        assert np.array_equal(bf16_bits(g[4]), alone[i]), "problem %d differs when run beside the others" % i


@pytest.mark.timeout(120)
def test_run_with_metrics_then_a_call_that_grows_the_buffers_does_not_wait_for_the_device(rfk):
    """run(metrics) leaves a timing callback pending on the stream; the next call needs a larger split-K workspace and
    a larger staging buffer. Neither may wait for the device while holding a lock the callback needs (the host would
    wait for the device, the device for the callback, the callback for the lock)."""
    from radeonflow_kernels_amd import gemm
    L = rfk.lib()
    L.rf_gemm_destroy()                                  # start from empty buffers
    s = torch.cuda.Stream()
    small = to_gpu(exact_problem(250, 256, 2048, 5))     # ragged, small buffers
    big = to_gpu(exact_problem(1000, 1536, 7168, 6))     # ragged, larger staging copy and split-K workspace
    exp_small, exp_big = oracle_bf16(exact_problem(250, 256, 2048, 5)), oracle_bf16(exact_problem(1000, 1536, 7168, 6))
    pms = [gemm.PerfMetrics() for _ in range(4)]
    ptr = ctypes.c_void_p(s.cuda_stream)
    with torch.cuda.stream(s):
        for i, g in enumerate((small, big, small, big)):
            a, b, sa, sb, c = g
            L.run(a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), c.data_ptr(), a.shape[0], b.shape[0],
                  a.shape[1], ctypes.byref(pms[i]), ptr)     # no synchronisation between the calls
    s.synchronize()
    torch.cuda.synchronize()
    assert all(pm.entries[0].time > 0 for pm in pms)
    assert np.array_equal(bf16_bits(small[4]), exp_small)
    assert np.array_equal(bf16_bits(big[4]), exp_big)


def test_more_streams_than_buffer_sets(rfk):
    """Only launches that need temporary memory take a buffer set, and there are 32 sets per device. 40 streams (made
    with hipStreamCreate: torch hands out 32 distinct ones) run a one-kernel plan each (no set is used, nothing changes
    hands), then 32 of them run a split-K plan (all sets taken), then a 33rd does: the least recently used set changes
    hands without a host wait, and the results stay bit-exact. The same on a stream that is being captured into a graph
    is refused with RF_ERR_BAD_CONFIG, the capture stays valid, and rf_fp8_gemm_static records the same GEMM into it
    instead; the replayed graph gives the same bits."""
    hip = ctypes.CDLL("libamdhip64.so")
    L = rfk.lib()
    L.rf_gemm_destroy()
    direct = exact_problem(256, 256, 256, 31)
    exp_direct = oracle_bf16(direct)
    assert rfk.select_config(256, 256, 256).split_k == 1
    split = exact_problem(128, 512, 7168, 32)
    exp_split = oracle_bf16(split)
    assert rfk.select_config(128, 512, 7168).split_k > 1
    handles = []
    for _ in range(40):
        h = ctypes.c_void_p()
        assert hip.hipStreamCreate(ctypes.byref(h)) == 0
        handles.append(h)
    assert len({h.value for h in handles}) == 40

    def launch(fn, g, h):
        a, b, sa, sb, c = g
        return fn(a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), c.data_ptr(), a.shape[0], b.shape[0],
                  a.shape[1], h)

    try:
        gd = [to_gpu(direct) for _ in handles]
        gs = [to_gpu(split) for _ in range(34)]
        torch.cuda.synchronize()
        for g, h in zip(gd, handles):
            assert launch(L.rf_fp8_gemm, g, h) == 0
        torch.cuda.synchronize()
        assert all(np.array_equal(bf16_bits(g[4]), exp_direct) for g in gd)
        for g, h in zip(gs[:33], handles[:33]):          # the 33rd takes over the first stream's set
            assert launch(L.rf_fp8_gemm, g, h) == 0
        gs[0][4].zero_()
        torch.cuda.synchronize()
        assert launch(L.rf_fp8_gemm, gs[0], handles[0]) == 0     # and the first stream takes over the second's
        torch.cuda.synchronize()
        assert all(np.array_equal(bf16_bits(g[4]), exp_split) for g in gs[:33])
        # a 34th stream that needs temporary memory, under capture: refused, and the capture goes on
        cap, g = handles[35], gs[33]
        graph, graph_exec = ctypes.c_void_p(), ctypes.c_void_p()
        assert hip.hipStreamBeginCapture(cap, 2) == 0            # hipStreamCaptureModeRelaxed
        rc = launch(L.rf_fp8_gemm, g, cap)
        msg = L.rf_gemm_last_error().decode()
        rc_static = launch(L.rf_fp8_gemm_static, g, cap)
        assert hip.hipStreamEndCapture(cap, ctypes.byref(graph)) == 0
        assert rc == 4 and "captured" in msg, (rc, msg)
        assert rc_static == 0
        assert hip.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, 0) == 0
        g[4].zero_()
        torch.cuda.synchronize()
        for _ in range(2):
            assert hip.hipGraphLaunch(graph_exec, cap) == 0
            assert hip.hipStreamSynchronize(cap) == 0
            assert np.array_equal(bf16_bits(g[4]), exp_split)
            g[4].zero_()
            torch.cuda.synchronize()
        hip.hipGraphExecDestroy(graph_exec)
        hip.hipGraphDestroy(graph)
    finally:
        torch.cuda.synchronize()
        L.rf_gemm_destroy()
        for h in handles:
            hip.hipStreamDestroy(h)


def test_stream_k_plan_for_a_shape_with_fewer_tiles_than_compute_units_is_skipped(rfk, tmp_path):
    """A stream-K plan splits each tile between at most two workgroups, which needs at least one tile per compute unit.
    A plan file that asks for it on a smaller shape is ignored for that shape; the result stays bit-exact."""
    sk = [v["variant"] for v in rfk.variants() if v["stream_k"]]
    assert sk, "no variant with a stream-K form"
    m, n, k = 512, 512, 1024                             # 4 tiles of 256 x 256
    before = rfk.select_config(m, n, k)
    path = tmp_path / "sk.plans"
    path.write_text("%d %d %d %d 1 1 1\n" % (m, n, k, sk[0]))
    try:
        assert rfk.load_plans(str(path)) == 1
        got = rfk.select_config(m, n, k)
        assert got.stream_k != 1
        assert (got.variant, got.split_k, got.stream_k) == (before.variant, before.split_k, before.stream_k)
        data = exact_problem(m, n, k, seed=9)
        g = to_gpu(data)
        rfk.fp8_mm(*g)
        rfk.fp8_mm(*g)                                   # a stale arrival counter would show on the second launch
        torch.cuda.synchronize()
        assert np.array_equal(bf16_bits(g[4]), oracle_bf16(data))
        ragged = exact_problem(m - 8, n, k, seed=10)     # the staged path picks its plan by the same rule
        g = to_gpu(ragged)
        rfk.fp8_mm(*g)
        torch.cuda.synchronize()
        assert np.array_equal(bf16_bits(g[4]), oracle_bf16(ragged))
    finally:
        rfk.clear_plans()


def test_small_grouped_problem_takes_the_variant_with_the_most_workgroups(rfk):
    """8 groups of 64 rows, N = 1024: no tile shape gives every compute unit a workgroup, so the automatic choice is
    the one with the most workgroups; its result equals the explicit 128 x 64 variant's bit for bit."""
    from oracle import cref
    rng = np.random.default_rng(4)
    groups, rows, n, k = 8, 64, 1024, 512
    m_total = groups * rows
    fp8 = torch.float8_e4m3fn
    vals = np.array([0, 1, 2, 3, -1, -2, -3], np.float32)
    a = torch.from_numpy(cref.f32_to_e4m3fn(rng.choice(vals, (k, m_total)))).view(fp8).cuda().T
    b = torch.from_numpy(cref.f32_to_e4m3fn(rng.choice(vals, (groups, k, n)))).view(fp8).cuda().transpose(1, 2)
    sa = torch.from_numpy(rng.choice(np.array([0.5, 1, 2], np.float32), (k // 128, m_total))).cuda().T
    sb = torch.from_numpy(rng.choice(np.array([0.5, 1, 2], np.float32), (groups, k // 128, n // 128))).cuda().transpose(1, 2)
    offs = [g * rows for g in range(groups + 1)]
    out = {}
    for variant in (-1, 3):
        c = torch.zeros((m_total, n), dtype=torch.bfloat16, device="cuda")
        rfk.fp8_mm_grouped(a, b, sa, sb, c, offs, variant=variant)
        torch.cuda.synchronize()
        out[variant] = bf16_bits(c)
    assert np.any(out[3] != 0) and np.array_equal(out[-1], out[3])
