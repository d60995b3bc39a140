"""Pins the oracle GEMM: brute force, algebraic invariants, layout/index coding, the torch restatement."""
import os

import numpy as np
import pytest
import torch

from oracle import ref_kernel as rk


def _rand_problem(rng, M, N, K, signed_scales=True):
    a = rng.integers(0, 256, (K, M), dtype=np.uint8)
    b = rng.integers(0, 256, (K, N), dtype=np.uint8)
    a[(a & 0x7F) == 0x7F] = 0x38      # no NaN codes
    b[(b & 0x7F) == 0x7F] = 0xB8
    # keep magnitudes modest so that fp32 sums stay well conditioned
    a = (a & 0x80) | np.minimum(a & 0x7F, 0x4F)
    b = (b & 0x80) | np.minimum(b & 0x7F, 0x4F)
    sa = rng.normal(size=(K // 128, M)).astype(np.float32)
    sb = rng.normal(size=(K // 128, (N + 127) // 128)).astype(np.float32)
    if not signed_scales:
        sa, sb = np.abs(sa) + 0.1, np.abs(sb) + 0.1
    return a.astype(np.uint8), b.astype(np.uint8), sa, sb


def _brute_f64(cref, a, b, sa, sb):
    """Independent numpy formulation: dense dequantised matrices, one fp64 matmul."""
    K, M = a.shape
    N = b.shape[1]
    A = cref.e4m3fn_to_f32(a).astype(np.float64).T * np.repeat(sa.astype(np.float64), 128, axis=0).T   # [M][K]
    Bs = np.repeat(np.repeat(sb.astype(np.float64), 128, axis=0), 128, axis=1)[:, :N]                  # [K][N]
    B = cref.e4m3fn_to_f32(b).astype(np.float64) * Bs
    return A @ B


@pytest.mark.parametrize("M,N,K", [(3, 130, 256), (1, 1, 128), (17, 64, 384), (5, 257, 128)])
def test_oracle_vs_bruteforce(cref, M, N, K):
    rng = np.random.default_rng(M * 1000 + N)
    a, b, sa, sb = _rand_problem(rng, M, N, K)
    truth = _brute_f64(cref, a, b, sa, sb)
    o64 = cref.ref_gemm_f64(a, b, sa, sb)
    assert np.allclose(o64, truth, rtol=1e-12, atol=1e-9)
    o32, o16 = cref.ref_gemm_f32(a, b, sa, sb)
    scale = np.abs(truth).max() + 1
    assert np.abs(o32 - truth).max() < 1e-4 * scale          # fp32 accumulation noise only
    f32, f16 = cref.ref_gemm_blockfold(a, b, sa, sb)
    assert np.abs(f32 - truth).max() < 1e-4 * scale
    assert np.array_equal(o16, cref.f32_to_bf16(o32))


def test_unit_scales_reduce_to_plain_integer_gemm(cref):
    rng = np.random.default_rng(5)
    M, N, K = 8, 48, 256
    # small integers are exact in e4m3 and their dot products are exact in fp32
    ints = np.array([0, 1, 2, 3, 4, -1, -2, -3, -4], np.float32)
    A = rng.choice(ints, (M, K)); B = rng.choice(ints, (N, K))
    a = cref.f32_to_e4m3fn(A).T.copy(); b = cref.f32_to_e4m3fn(B).T.copy()
    sa = np.ones((2, M), np.float32); sb = np.ones((2, 1), np.float32)
    o32, _ = cref.ref_gemm_f32(a, b, sa, sb)
    assert np.array_equal(o32, (A.astype(np.int64) @ B.astype(np.int64).T).astype(np.float32))
    f32, _ = cref.ref_gemm_blockfold(a, b, sa, sb)
    assert np.array_equal(f32, o32)


def test_block_linearity_and_removal(cref):
    rng = np.random.default_rng(6)
    M, N, K = 4, 160, 384
    a, b, sa, sb = _rand_problem(rng, M, N, K)
    base = cref.ref_gemm_f64(a, b, sa, sb)
    # zeroing K-block 1's a-scales removes exactly that block's contribution
    sa0 = sa.copy(); sa0[1, :] = 0
    only1 = base - cref.ref_gemm_f64(a, b, sa0, sb)
    sa_only = np.zeros_like(sa); sa_only[1, :] = sa[1, :]
    assert np.allclose(only1, cref.ref_gemm_f64(a, b, sa_only, sb), rtol=1e-10, atol=1e-9)
    # doubling that block's scale adds the contribution once more (power of two: exact in fp32 too)
    sa2 = sa.copy(); sa2[1, :] *= 2
    assert np.allclose(cref.ref_gemm_f64(a, b, sa2, sb), base + only1, rtol=1e-10, atol=1e-9)
    o32, _ = cref.ref_gemm_f32(a, b, sa_only, sb)
    o32x2, _ = cref.ref_gemm_f32(a, b, sa_only * 2, sb)
    assert np.array_equal(o32x2, o32 * 2)
    # negating b_scale of N-block 1 flips only columns 128..159
    sbn = sb.copy(); sbn[:, 1] *= -1
    flipped = cref.ref_gemm_f64(a, b, sa, sbn)
    assert np.allclose(flipped[:, :128], base[:, :128]) and np.allclose(flipped[:, 128:], -base[:, 128:])


def test_one_hot_rows_and_row_permutation(cref):
    rng = np.random.default_rng(7)
    M, N, K = 6, 64, 256
    a, b, sa, sb = _rand_problem(rng, M, N, K, signed_scales=False)
    # row 2 of A = one-hot at k=131 with value 1.0 -> C[2,:] = sa[1,2]*sb[1,0]*B[:,131]
    a[:, 2] = 0; a[131, 2] = 0x38
    o32, _ = cref.ref_gemm_f32(a, b, sa, sb)
    expect = (np.float32(1.0) * sa[1, 2]) * (cref.e4m3fn_to_f32(b[131, :]) * sb[1, 0])
    assert np.array_equal(o32[2], expect.astype(np.float32))
    perm = rng.permutation(M)
    p32, _ = cref.ref_gemm_f32(a[:, perm].copy(), b, sa[:, perm].copy(), sb)
    assert np.array_equal(p32, o32[perm])
    # row subset API returns the same rows
    r32, _ = cref.ref_gemm_f32(a, b, sa, sb, rows=[4, 1])
    assert np.array_equal(r32, o32[[4, 1]])
    assert np.array_equal(cref.ref_gemm_f64(a, b, sa, sb, rows=[5]), cref.ref_gemm_f64(a, b, sa, sb)[[5]])


def test_index_coded_scales_catch_transposed_or_misstrided_reads(cref):
    M, N, K = 7, 300, 384
    QK, QN = 3, 3
    a = np.full((K, M), 0x38, np.uint8)           # all ones
    b = np.full((K, N), 0x38, np.uint8)
    sa = (1 + np.arange(QK)[:, None] + np.arange(M)[None, :] / 8).astype(np.float32)        # exact in fp32
    sb = (1 + 2 * np.arange(QK)[:, None] + np.arange(QN)[None, :] / 4).astype(np.float32)
    o64 = cref.ref_gemm_f64(a, b, sa, sb)
    for m in (0, 3, 6):
        for n in (0, 127, 128, 299):
            expect = sum(128 * float(sa[kb, m]) * float(sb[kb, n // 128]) for kb in range(QK))
            assert o64[m, n] == expect
    o32, _ = cref.ref_gemm_f32(a, b, sa, sb)
    assert np.allclose(o32, o64, rtol=1e-6)


def test_ragged_last_n_block_uses_its_own_scale_column(cref):
    rng = np.random.default_rng(8)
    M, N, K = 4, 576, 128
    a, b, sa, sb = _rand_problem(rng, M, N, K)
    assert sb.shape == (1, 5)
    base = cref.ref_gemm_f64(a, b, sa, sb)
    sb2 = sb.copy(); sb2[0, 4] *= 3
    alt = cref.ref_gemm_f64(a, b, sa, sb2)
    assert np.allclose(alt[:, :512], base[:, :512]) and np.allclose(alt[:, 512:], 3 * base[:, 512:])


@pytest.mark.parametrize("gen", ["blockquant", "reference_style"])
@pytest.mark.parametrize("m,n,k,seed", [(64, 64, 128, 6635), (96, 320, 256, 1234), (128, 576, 384, 542)])
def test_torch_restatement_agrees_with_c_oracle(cref, gen, m, n, k, seed):
    f = rk.generate_input_blockquant if gen == "blockquant" else rk.generate_input_reference_style
    data = f(m, n, k, seed)
    assert data[0].shape == (m, k) and data[0].stride() == (1, m)          # transposed view of [K][M]
    assert data[1].shape == (n, k) and data[1].stride() == (1, n)
    assert data[2].shape == (m, k // 128) and data[3].shape == ((n + 127) // 128, k // 128)
    c = rk.ref_kernel(data)
    a, b, sa, sb = rk.raw_layouts(data)
    o32, o16 = cref.ref_gemm_f32(a, b, sa, sb)
    truth = cref.ref_gemm_f64(a, b, sa, sb)
    c32 = c.to(torch.float32).numpy()
    # both fp32 paths sit within a few bf16 ulps of the fp64 truth and of each other
    tol = 2.0 ** -7 * np.abs(truth) + 1e-4 * np.abs(truth).max()
    assert np.all(np.abs(c32 - truth) <= tol)
    assert np.all(np.abs(cref.bf16_to_f32(o16) - truth) <= tol)
    bad, _, _ = cref.allclose(c.view(torch.uint16).numpy(), o16, rtol=2e-2, atol=1e-3)
    assert bad == 0
    assert rk.check_implementation(data, c) == ""


def test_check_implementation_flags_errors_like_the_reference_rule(cref):
    data = rk.generate_input_blockquant(64, 128, 128, 1)
    c = rk.ref_kernel(data).clone()
    assert rk.check_implementation(data, c) == ""
    bad = c.clone(); bad[3, 5] = bad[3, 5] * 1.05 + 0.01
    assert "Number of mismatched elements: 1" in rk.check_implementation(data, bad)
    nanc = c.clone(); nanc[0, 0] = float("nan")
    assert rk.check_implementation(data, nanc) != ""
    infc = c.clone(); infc[1, 1] = float("inf")
    assert rk.check_implementation(data, infc) != ""
    # C restatement of the rule gives the same counts
    g = bad.view(torch.uint16).numpy(); e = c.view(torch.uint16).numpy()
    assert cref.allclose(g, e, 2e-2, 1e-3)[0] == 1
    assert cref.allclose(nanc.view(torch.uint16).numpy(), e, 2e-2, 1e-3)[0] == 1
    assert cref.allclose(infc.view(torch.uint16).numpy(), e, 2e-2, 1e-3)[0] == 1


def test_golden_fixtures_replay(cref):
    d = os.path.join(os.path.dirname(__file__), "golden")
    for name in sorted(os.listdir(d)):
        if not name.endswith(".npz"):
            continue
        z = np.load(os.path.join(d, name))
        o32, o16 = cref.ref_gemm_f32(z["a"], z["b"], z["a_scale"], z["b_scale"])
        assert np.array_equal(o16, z["c_bf16"]), name
