"""GPU block quantisers against the CPU oracle's quantisers: bytes and scales must agree bit for bit
(integer / byte work; the only float steps are two correctly rounded fp32 divisions)."""
import numpy as np
import pytest
import torch

from oracle import cref, ref_kernel as rk
from helpers import RTOL, ATOL, assert_close_to_oracle, oracle_bf16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rfk():
    import radeonflow_kernels_amd as m
    m.lib()
    return m


def _source(rows, k, seed, kind):
    x = cref.randn(seed, rows * k).reshape(rows, k)
    if kind == "wide":          # many binades, exact zeros, negative zeros, a zero block, a huge value
        x = x * np.exp2(np.floor(cref.randn(seed + 1, rows * k).reshape(rows, k) * 6)).astype(np.float32)
        x[::7, ::5] = 0.0
        x[1::11, 3::13] = -0.0
        x[: min(rows, 3), :128] = 0.0
        x[rows // 2, k // 2] = 3.0e38
        x[rows - 1, k - 1] = 1.0e-41        # fp32 denormal
    if kind == "boundary":      # quotients x/scale within a few fp32 ulps of the midpoints between fp8 codes
        rng = np.random.default_rng(seed)
        amax = np.exp2(rng.integers(-20, 20, (rows, k // 128, 1))).astype(np.float32) * rng.uniform(1, 2, (rows, k // 128, 1)).astype(np.float32)
        codes = np.arange(0, 126, dtype=np.uint8)
        vals = cref.e4m3fn_to_f32(codes)
        mids = ((vals[:-1] + vals[1:]) / 2).astype(np.float32)                   # exact in fp32
        pick = mids[rng.integers(0, len(mids), (rows, k // 128, 128))]
        scale = (amax / np.float32(448.0)).astype(np.float32)
        x = (pick * scale).astype(np.float32)
        x = (x.view(np.int32) + rng.integers(-3, 4, x.shape).astype(np.int32)).view(np.float32)   # +-3 ulp
        x *= rng.choice(np.array([-1.0, 1.0], np.float32), x.shape)
        x[:, :, 0] = amax[:, :, 0]                                             # pin the block maximum
        x = x.reshape(rows, k)
    if kind == "ties":          # bf16-representable sources whose quotients are exact ties or one bf16 step away
        rng = np.random.default_rng(seed)
        e = rng.integers(-12, 12, (rows, k // 128, 1))
        amax = (np.float32(448.0) * np.exp2(e)).astype(np.float32)                # scale = 2^e exactly
        vals = cref.e4m3fn_to_f32(np.arange(0, 127, dtype=np.uint8))
        mids = ((vals[:-1] + vals[1:]) / 2).astype(np.float32)                   # at most 5 significant bits
        x = (mids[rng.integers(0, len(mids), (rows, k // 128, 128))] * np.exp2(e)).astype(np.float32)
        step = rng.integers(-1, 2, x.shape).astype(np.int32) << 16               # -1, 0, +1 bf16 steps
        x = (x.view(np.int32) + step).view(np.float32)
        x *= rng.choice(np.array([-1.0, 1.0], np.float32), x.shape)
        x[:, :, 0] = amax[:, :, 0]
        # every fourth block: a maximum with a full bf16 mantissa, so that the scale is not a power of two and the
        # quotients of small-mantissa values land on and around boundaries by themselves
        odd = (np.float32(1.0) + rng.integers(1, 128, (rows, k // 128)).astype(np.float32) / np.float32(128.0))
        x[:, ::4, 0] = (x[:, ::4, 0] * odd[:, ::4] / np.float32(1.75)).astype(np.float32)
        x = x.reshape(rows, k)
        x = (x.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32)          # bf16-exact
    if kind == "special":       # NaNs of both signs (quiet and signalling patterns), infinities, an all-NaN block
        u = x.view(np.uint32)
        u[0, 5] = 0x7FC00000
        u[0, 77] = 0xFFC00000
        u[min(rows - 1, 2), 3] = 0x7F800001           # signalling pattern, first elements of a lane's run
        u[min(rows - 1, 2), 4] = 0xFF800001
        u[min(rows - 1, 5), k - 1] = 0x7FFFFFFF       # last element of a row
        x[min(rows - 1, 9), 17] = np.inf
        x[min(rows - 1, 12), 130 % k] = -np.inf
        x[min(rows - 1, 12), 131 % k] = np.nan
        x[min(rows - 1, 20), :128] = np.nan
        x[rows - 1, k - 128:] *= np.float32(1e-30)    # a block whose scale is far from 1
    return np.ascontiguousarray(x, dtype=np.float32)


def _codes_equal(got, exp, x):
    """Byte-for-byte, except that inf / inf (an infinite element divided by its block's infinite scale) may give a NaN
    code of either sign: IEEE 754 leaves the sign of a NaN created by an invalid operation open, x86 makes it
    negative, gfx950 positive. got/exp are [K][rows], x is the [rows][K] source."""
    free = np.isinf(x).T & ((np.asarray(exp) & 0x7F) == 0x7F)
    g, e = np.asarray(got).copy(), np.asarray(exp).copy()
    g[free] &= 0x7F
    e[free] &= 0x7F
    return np.array_equal(g, e)


def _unpack(q, s):
    """(fp8 view [rows,K] stride (1,rows), scales view) -> numpy arrays in the launcher's memory layouts."""
    return q.T.contiguous().view(torch.uint8).cpu().numpy(), s.T.contiguous().cpu().numpy()


@pytest.mark.parametrize("kind", ["normal", "wide", "boundary", "special", "ties"])
@pytest.mark.parametrize("rows,k", [(128, 128), (256, 512), (1024, 7168), (576, 1024), (200, 256), (1, 128), (33, 384),
                                    (6144, 256)])
def test_quantize_a_matches_oracle_bit_for_bit(rfk, rows, k, kind):
    x = _source(rows, k, 1000 + rows + k, kind)
    a_ref, as_ref = cref.quantize_a(x)
    q, s = rfk.quantize_a(torch.from_numpy(x).cuda())
    torch.cuda.synchronize()
    assert q.shape == (rows, k) and q.stride() == (1, rows) and s.shape == (rows, k // 128)
    a_gpu, as_gpu = _unpack(q, s)
    assert np.array_equal(as_gpu.view(np.uint32), np.asarray(as_ref).view(np.uint32))
    assert _codes_equal(a_gpu, a_ref, x)


@pytest.mark.parametrize("kind", ["normal", "wide", "boundary", "special", "ties"])
@pytest.mark.parametrize("rows,k", [(128, 128), (256, 512), (1536, 7168), (576, 1024), (200, 256), (1, 128), (33, 384)])
def test_quantize_b_matches_oracle_bit_for_bit(rfk, rows, k, kind):
    w = _source(rows, k, 2000 + rows + k, kind)
    b_ref, bs_ref = cref.quantize_b(w)
    q, s = rfk.quantize_b(torch.from_numpy(w).cuda())
    torch.cuda.synchronize()
    assert s.shape == ((rows + 127) // 128, k // 128)
    b_gpu, bs_gpu = _unpack(q, s)
    assert np.array_equal(bs_gpu.view(np.uint32), np.asarray(bs_ref).view(np.uint32))
    assert _codes_equal(b_gpu, b_ref, w)


@pytest.mark.parametrize("kind", ["normal", "wide", "special", "ties"])
@pytest.mark.parametrize("rows,k", [(256, 512), (200, 256)])
def test_bf16_sources_equal_fp32_sources_of_the_same_values(rfk, rows, k, kind):
    x = torch.from_numpy(_source(rows, k, 77, kind)).bfloat16()
    qa, sa = rfk.quantize_a(x.cuda())
    qa32, sa32 = rfk.quantize_a(x.float().cuda())
    qb, sb = rfk.quantize_b(x.cuda())
    qb32, sb32 = rfk.quantize_b(x.float().cuda())
    torch.cuda.synchronize()
    for got, exp in ((qa, qa32), (qb, qb32)):
        assert torch.equal(got.view(torch.uint8), exp.view(torch.uint8))
    assert torch.equal(sa, sa32) and torch.equal(sb, sb32)


def test_quantise_then_gemm_end_to_end(rfk):
    """fp32 activations and weights quantised on the GPU and multiplied on the GPU, against the oracle GEMM run on
    the oracle's own quantisation of the same sources."""
    m, n, k = 512, 576, 1024
    x = cref.randn(4242, m * k).reshape(m, k)
    w = cref.randn(4243, n * k).reshape(n, k)
    qa, sa = rfk.quantize_a(torch.from_numpy(x).cuda())
    qb, sb = rfk.quantize_b(torch.from_numpy(w).cuda())
    out = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda:0")
    rfk.fp8_mm(qa, qb, sa, sb, out)
    torch.cuda.synchronize()
    a_ref, as_ref = cref.quantize_a(x)
    b_ref, bs_ref = cref.quantize_b(w)

    def views(codes, scales):          # [K][rows] storage -> the [rows, K] views ref_kernel takes
        return torch.from_numpy(np.asarray(codes)).view(torch.float8_e4m3fn).T, torch.from_numpy(np.asarray(scales)).T
    a_t, as_t = views(a_ref, as_ref)
    b_t, bs_t = views(b_ref, bs_ref)
    exp = oracle_bf16((a_t, b_t, as_t, bs_t, torch.zeros((m, n), dtype=torch.bfloat16)))
    assert_close_to_oracle(out, exp, RTOL, ATOL, "quantise + gemm")


def test_cast_matches_the_oracle_encoder_on_a_dense_sweep_of_all_floats(rfk):
    """Every 61st fp32 bit pattern (70 million values: all binades, denormals, infinities, NaNs of both signs) and a
    dense neighbourhood of every boundary between fp8 codes."""
    bits = np.arange(0, 2 ** 32, 61, dtype=np.uint64).astype(np.uint32)
    vals = cref.e4m3fn_to_f32(np.arange(0, 127, dtype=np.uint8))
    mids = np.concatenate([(vals[:-1] + vals[1:]) / 2, [464.0, 448.0, 480.0]]).astype(np.float32)
    near = (mids.view(np.uint32)[:, None].astype(np.int64) + np.arange(-40, 41)[None, :]).astype(np.uint32).ravel()
    bits = np.concatenate([bits, near, near | np.uint32(0x80000000)])
    bits = bits[: bits.size // 4 * 4 + 0]
    x = torch.from_numpy(bits.view(np.float32).copy())
    got = rfk.cast_to_e4m3fn(x.cuda()).view(torch.uint8).cpu().numpy()
    exp = cref.f32_to_e4m3fn(x.numpy())
    bad = np.nonzero(got != exp)[0]
    assert bad.size == 0, "first mismatch: bits %08x got %02x expected %02x" % (bits[bad[0]], got[bad[0]], exp[bad[0]])
    # a tail that is not a multiple of four
    y = torch.from_numpy(bits[:1027].view(np.float32).copy()).cuda()
    assert np.array_equal(rfk.cast_to_e4m3fn(y).view(torch.uint8).cpu().numpy(), exp[:1027])


def test_status_codes(rfk):
    L = rfk.lib()
    x = torch.zeros((128, 128), device="cuda")
    q = torch.empty((128, 128), dtype=torch.uint8, device="cuda")
    s = torch.empty((1, 128), device="cuda")
    assert L.rf_quantize_a_f32(x.data_ptr(), 128, 100, q.data_ptr(), s.data_ptr(), None) == 1     # RF_ERR_BAD_SHAPE
    assert L.rf_quantize_a_f32(None, 128, 128, q.data_ptr(), s.data_ptr(), None) == 2            # RF_ERR_NULL_POINTER
    assert L.rf_quantize_a_f32(x.data_ptr() + 4, 127, 128, q.data_ptr(), s.data_ptr(), None) == 4  # misaligned source


def test_quantize_a_source_beyond_4_gib(rfk):
    """A source of more than 2^32 bytes (and more than 2^31 elements of output index range per K row times rows):
    sampled rows, the last ones included, against the oracle's quantiser run on those rows alone (a row's scales and
    codes depend on nothing but the row)."""
    rows, k = 163840, 7168
    assert rows * k * 4 > 2 ** 32
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn((rows, k), device=dev, generator=gen)
    q, s = rfk.quantize_a(x)
    torch.cuda.synchronize()
    pick = np.unique(np.concatenate([[0, 1, 127, 128, rows // 2, rows - 129, rows - 2, rows - 1],
                                     np.random.default_rng(9).integers(0, rows, 24)]))
    idx = torch.from_numpy(pick).to(dev)
    a_ref, as_ref = cref.quantize_a(np.ascontiguousarray(x[idx].cpu().numpy()))        # [K][len(pick)], [K/128][len(pick)]
    got_codes = q[idx].contiguous().view(torch.uint8).cpu().numpy().T                   # q is [rows, K] stride (1, rows)
    got_scales = s[idx].contiguous().cpu().numpy().T
    assert np.array_equal(got_scales.view(np.uint32), np.asarray(as_ref).view(np.uint32))
    assert np.array_equal(got_codes, np.asarray(a_ref))
