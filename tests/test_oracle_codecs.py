"""Pins the oracle's number formats against the installed PyTorch CPU library and closed forms."""
import numpy as np
import torch


def test_e4m3fn_decode_exhaustive_vs_torch(cref):
    codes = np.arange(256, dtype=np.uint8)
    mine = cref.e4m3fn_to_f32(codes)
    ref = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(np.isnan(mine), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.array_equal(mine[ok], ref[ok])
    assert np.array_equal(np.signbit(mine[ok]), np.signbit(ref[ok]))


def test_e4m3fn_decode_landmarks(cref):
    d = cref.e4m3fn_to_f32(np.array([0x00, 0x80, 0x01, 0x07, 0x08, 0x38, 0x7E, 0xFE, 0x7F, 0xFF], np.uint8))
    assert d[0] == 0 and not np.signbit(d[0]) and d[1] == 0 and np.signbit(d[1])
    assert d[2] == 2.0 ** -9 and d[3] == 7 * 2.0 ** -9 and d[4] == 2.0 ** -6
    assert d[5] == 1.0 and d[6] == 448.0 and d[7] == -448.0
    assert np.isnan(d[8]) and np.isnan(d[9])


def test_e4m3fn_encode_roundtrip_all_finite_codes(cref):
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], np.uint8)
    vals = cref.e4m3fn_to_f32(codes)
    assert np.array_equal(cref.f32_to_e4m3fn(vals), codes)


def test_e4m3fn_encode_midpoints_round_to_even(cref):
    pos = np.arange(0, 0x7F, dtype=np.uint8)          # 0 .. 448 ascending
    v = cref.e4m3fn_to_f32(pos).astype(np.float64)
    mid = ((v[:-1] + v[1:]) / 2).astype(np.float32)   # exactly representable in fp32
    enc = cref.f32_to_e4m3fn(mid)
    expect = np.where(pos[:-1] % 2 == 0, pos[:-1], pos[1:])
    assert np.array_equal(enc, expect)
    # just below / above the midpoint go down / up
    lo = np.nextafter(mid, np.float32(0)).astype(np.float32)
    hi = np.nextafter(mid, np.float32(1e9)).astype(np.float32)
    assert np.array_equal(cref.f32_to_e4m3fn(lo), pos[:-1])
    assert np.array_equal(cref.f32_to_e4m3fn(hi), pos[1:])
    assert np.array_equal(cref.f32_to_e4m3fn(-mid), expect | 0x80)


def test_e4m3fn_encode_random_vs_torch(cref):
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.uniform(-470, 470, 200000), rng.normal(0, 1, 200000), rng.normal(0, 0.01, 100000),
        np.array([0.0, -0.0, 448, -448, 464, 464.0001, 479.9, 480, 1e9, -1e9, 2.0 ** -10, 2.0 ** -10 * 1.0001,
                  3 * 2.0 ** -10, np.inf, -np.inf, np.nan]),
    ]).astype(np.float32)
    mine = cref.f32_to_e4m3fn(x)
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(mine, ref)


def test_bf16_rne_vs_torch(cref):
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 2 ** 32, 500000, dtype=np.uint64).astype(np.uint32)
    ties = (rng.integers(0, 2 ** 16, 5000, dtype=np.uint64).astype(np.uint32) << 16) | 0x8000
    x = np.concatenate([bits, ties, np.array([0x7F800000, 0xFF800000, 0x7F7FFFFF, 0x00000001], np.uint32)]).view(np.float32)
    mine = cref.f32_to_bf16(x)
    ref = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.uint16).numpy()
    nan = np.isnan(x)
    assert np.array_equal(mine[~nan], ref[~nan])
    assert np.all(np.isnan(cref.bf16_to_f32(mine[nan])))
    # the reference's integer-add rounding agrees wherever the input is not NaN
    fast = cref.f32_to_bf16(x, fast=True)
    assert np.array_equal(fast[~nan], ref[~nan])


def test_bf16_decode(cref):
    h = np.array([0x3F80, 0xBF80, 0x0000, 0x7F80, 0x4049], np.uint16)
    assert np.array_equal(cref.bf16_to_f32(h), np.array([1, -1, 0, np.inf, 3.140625], np.float32))


def _hash64_numpy(seed, i):
    with np.errstate(over="ignore"):
        z = np.uint64(seed) * np.uint64(0x9E3779B97F4A7C15) + i.astype(np.uint64) * np.uint64(0xD1B54A32D192ED03) \
            + np.uint64(0x2545F4914F6CDD1D)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def test_randn_counter_based_and_moments(cref):
    a = cref.randn(1234, 100000)
    b = cref.randn(1234, 1000, offset=500)
    assert np.array_equal(a[500:1500], b)            # element i depends on (seed, i) only
    assert not np.array_equal(a[:1000], cref.randn(1235, 1000))
    assert abs(a.mean()) < 0.02 and abs(a.std() - 1) < 0.02
    assert abs((a ** 3).mean()) < 0.05 and abs((a ** 4).mean() - 3) < 0.15
    # numpy restatement of the same construction (integer hash exact; transcendental part to 1 ulp)
    i = np.arange(4096, dtype=np.uint64)
    h = _hash64_numpy(1234, i)
    assert all(int(h[j]) == cref.hash64(1234, int(j)) for j in (0, 1, 17, 4095))
    u1 = (((h >> np.uint64(40)) & np.uint64(0xFFFFFF)).astype(np.float64) + 1) / 16777216.0
    u2 = ((h >> np.uint64(8)) & np.uint64(0xFFFFFF)).astype(np.float64) / 16777216.0
    z = (np.sqrt(-2 * np.log(u1)) * np.cos(2 * np.pi * u2)).astype(np.float32)
    assert np.allclose(a[:4096], z, rtol=1e-6, atol=1e-7)


def test_randn_golden_prefix(cref):
    import json, os
    g = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "randn_seed8135_first16.json")))
    got = cref.randn(8135, 16)
    assert np.allclose(got, np.array(g["values"], np.float32), rtol=1e-6, atol=1e-7)
    assert [cref.hash64(8135, i) for i in range(4)] == g["hash64_first4"]


def test_quantisers_match_definition(cref):
    rng = np.random.default_rng(3)
    M, N, K = 5, 200, 256
    A = rng.normal(size=(M, K)).astype(np.float32)
    B = rng.normal(size=(N, K)).astype(np.float32)
    A[2, 128:256] = 0                                      # an all-zero block -> scale 1
    a, sa = cref.quantize_a(A)
    b, sb = cref.quantize_b(B)
    assert a.shape == (K, M) and sa.shape == (2, M) and b.shape == (K, N) and sb.shape == (2, 2)
    for m in range(M):
        for kb in range(2):
            blk = A[m, kb * 128:(kb + 1) * 128]
            s = np.float32(np.abs(blk).max()) / np.float32(448) if np.abs(blk).max() > 0 else np.float32(1)
            assert sa[kb, m] == s
            exp = torch.from_numpy(blk / s).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
            assert np.array_equal(a[kb * 128:(kb + 1) * 128, m], exp)
    for nb in range(2):
        for kb in range(2):
            blk = B[nb * 128:min(N, (nb + 1) * 128), kb * 128:(kb + 1) * 128]
            s = np.float32(np.abs(blk).max()) / np.float32(448)
            assert sb[kb, nb] == s
            exp = torch.from_numpy(blk / s).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
            assert np.array_equal(b[kb * 128:(kb + 1) * 128, nb * 128:min(N, (nb + 1) * 128)], exp.T)
    # every non-zero block reaches +-448 exactly
    dec = np.abs(cref.e4m3fn_to_f32(a))
    assert dec[:128, 0].max() == 448
