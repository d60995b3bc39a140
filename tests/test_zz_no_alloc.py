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


def test_static_entry_rejects_shapes_beyond_its_scratch_array(rfk):
    """A ragged M of 6008 with K = 7168 needs a 43 MB staging copy of A: refused with the size in the message, C is
    not touched, and the entry point keeps working afterwards."""
    L = rfk.lib()
    m, n, k = 6008, 512, 7168
    a = torch.zeros((k, m), dtype=torch.uint8, device="cuda")
    b = torch.zeros((k, n), dtype=torch.uint8, device="cuda")
    sa = torch.ones((k // 128, m), dtype=torch.float32, device="cuda")
    sb = torch.ones((k // 128, n // 128), dtype=torch.float32, device="cuda")
    c = torch.full((m, n), -5.0, dtype=torch.bfloat16, device="cuda")
    rc = L.rf_fp8_gemm_static(a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), c.data_ptr(), m, n, k, None)
    torch.cuda.synchronize()
    assert rc == 4
    msg = L.rf_gemm_last_error().decode()
    assert "rf_fp8_gemm_static" in msg and "bytes of scratch memory" in msg and str(32 << 20) in msg
    assert bool((c == -5.0).all())
    assert L.rf_fp8_gemm(a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), c.data_ptr(), m, n, k, None) == 0
    torch.cuda.synchronize()
    assert bool((c == 0).all())
    data = rk.generate_input_blockquant(256, 1536, 7168, 25)
    got, want = _both(rfk, data)
    assert np.array_equal(got, want)
