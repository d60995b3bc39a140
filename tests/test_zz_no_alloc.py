"""GPU test of rf_fp8_gemm_static, the entry point that allocates nothing: its output equals rf_fp8_gemm's bit for bit
on calls that use the static scratch array in different ways, one after the other."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import ref_kernel as rk
from helpers import RTOL, ATOL, assert_close_to_oracle, bf16_bits, oracle_bf16, to_gpu

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rfk():
    import radeonflow_kernels_amd as r
    assert torch.cuda.is_available(), "these tests need the GPU"
    r.lib()
    return r


def _both(rfk, data):
    g = to_gpu(data)
    rfk.fp8_mm(*g)
    torch.cuda.synchronize()
    want = bf16_bits(g[4]).copy()
    g[4].fill_(-3.0)
    free_before = torch.cuda.mem_get_info()[0]
    rfk.fp8_mm_static(*g)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the amount of free device memory"
    return bf16_bits(g[4]), want


def test_static_entry_matches_the_allocating_entry_on_two_calls_in_a_row(rfk):
    """First the C1 shape (split-K: 25 MB of partial sums in the scratch array), then a smaller ragged shape (staging
    copies and split-K partials at other offsets of the same array, which still holds the first call's data), then a
    shape that needs no scratch memory at all. Every result equals rf_fp8_gemm's bits and the oracle within tolerance."""
    assert rfk.lib().rf_gemm_static_scratch_bytes() == 32 << 20
    m, n, k = 1024, 1536, 7168
    assert rfk.select_config(m, n, k).split_k > 1
    for shape, seed in (((m, n, k), 21), ((250, 576, 2048), 22), ((512, 512, 1024), 23), ((1000, 1536, 7168), 24)):
        data = rk.generate_input_blockquant(*shape, seed)
        got, want = _both(rfk, data)
        assert np.array_equal(got, want), "shape %r differs from rf_fp8_gemm" % (shape,)
        assert_close_to_oracle(torch.from_numpy(got.view(np.int16)).view(torch.bfloat16), oracle_bf16(data), RTOL, ATOL,
                               "static %r" % (shape,))


def test_static_entry_fits_the_plan_to_its_scratch_array(rfk, tmp_path):
    """Shapes whose plan under rf_fp8_gemm needs more than the 32 MiB array still run, and allocate nothing:
    * M = 5001 with K = 7168 (a 36 MB staging copy of A): computed in row ranges that take turns in the array;
    * the same with a ragged N as well (B and C are staged too);
    * a plan file that asks for four K parts of 16.8 MB each: cut down to one part;
    * a stream-K plan from a plan file: replaced by the automatic plan.
    Exact data, so every fitted plan must give the oracle's bits (and rf_fp8_gemm's); then data with rounding in it
    against the oracle within tolerance; the canary behind C stays intact; a small split-K shape afterwards still matches
    rf_fp8_gemm bit for bit (the array holds the earlier calls' data)."""
    from helpers import exact_problem
    L = rfk.lib()

    def static_run(data, canary=4096):
        g, buf = to_gpu(data, canary_elems=canary)
        g[4].fill_(-3.0)
        free_before = torch.cuda.mem_get_info()[0]
        rfk.fp8_mm_static(*g)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the amount of free device memory"
        assert bool((buf[g[4].numel():].float() == -7.0).all()), "store past the end of C"
        return g[4]

    for (m, n, k) in ((5001, 512, 7168), (5001, 500, 7168)):
        assert k * ((m + 15) // 16 * 16) > (32 << 20)
        data = exact_problem(m, n, k, seed=m + n)
        assert np.array_equal(bf16_bits(static_run(data)), oracle_bf16(data)), (m, n, k)
        noisy = rk.generate_input_blockquant(m, n, k, seed=m)
        assert_close_to_oracle(static_run(noisy), oracle_bf16(noisy), RTOL, ATOL, "static, row ranges %r" % ((m, n, k),))
    plans = tmp_path / "big.plans"
    plans.write_text("2048 2048 1024 1 4 8 0\n4096 4096 512 0 1 8 1\n")
    try:
        assert rfk.load_plans(str(plans)) == 2
        for (m, n, k) in ((2048, 2048, 1024), (4096, 4096, 512)):
            got = rfk.select_config(m, n, k)
            assert (got.split_k, got.stream_k) == ((4, 0) if k == 1024 else (1, 1))
            data = exact_problem(m, n, k, seed=k)
            assert np.array_equal(bf16_bits(static_run(data)), oracle_bf16(data)), (m, n, k)
            noisy = rk.generate_input_blockquant(m, n, k, seed=k + 1)
            assert_close_to_oracle(static_run(noisy), oracle_bf16(noisy), RTOL, ATOL, "static, fitted plan %r" % ((m, n, k),))
    finally:
        rfk.clear_plans()
    data = rk.generate_input_blockquant(256, 1536, 7168, 25)
    got, want = _both(rfk, data)
    assert np.array_equal(got, want)
