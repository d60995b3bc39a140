"""torch-CPU restatement of the reference problem definition. Test infrastructure only.

Follows scripts/problems/gemm/reference.py of the reference tree:
  generate_input_reference_style  <- reference.py:11-37 (bf16 randn -> fp8, signed randn scales,
                                     transposed views), with this repo's counter-based generator
                                     in place of the CUDA Philox stream (which cannot be replayed
                                     on a CPU) and OCP e4m3fn in place of e4m3fnuz.
  ref_kernel                      <- reference.py:40-85 (expand scales, dequantise, a @ b.T, bf16).
  check_implementation            <- reference.py:87 + scripts/utils.py:31-91 (verbose_allclose).
  generate_input_blockquant       <- the benchmark's synthetic inputs: seeded N(0,1) fp32, amax/448
                                     scales per (row,128-K) for A and per 128x128 block for B.
Tensors use the reference's strides: a, b, a_scale, b_scale are transposed views of
[K][M], [K][N], [QK][M], [QK][QN] storage, c is contiguous [M][N] bf16.
"""
import numpy as np
import torch

from . import cref

BLOCK = 128
FP8 = torch.float8_e4m3fn


def _fp8_from_codes(codes_np):
    return torch.from_numpy(codes_np).view(FP8)


def generate_input_blockquant(m, n, k, seed):
    """Benchmark-style inputs. Returns (a[m,k] fp8, b[n,k] fp8, a_scale[m,qk], b_scale[qn,qk], c[m,n] bf16)."""
    assert k % BLOCK == 0
    A32 = cref.randn(seed, m * k, offset=0).reshape(m, k)
    B32 = cref.randn(seed, n * k, offset=1 << 40).reshape(n, k)
    a_km, as_qm = cref.quantize_a(A32)
    b_kn, bs_qq = cref.quantize_b(B32)
    a = _fp8_from_codes(a_km).T
    b = _fp8_from_codes(b_kn).T
    a_scale = torch.from_numpy(as_qm).T
    b_scale = torch.from_numpy(bs_qq).T
    c = torch.zeros((m, n), dtype=torch.bfloat16)
    return (a, b, a_scale, b_scale, c)


def generate_input_reference_style(m, n, k, seed):
    """Reference-style inputs: fp8(bf16(randn)) data and signed N(0,1) scales (can be tiny or negative)."""
    qn = (n + BLOCK - 1) // BLOCK
    qk = (k + BLOCK - 1) // BLOCK
    a = torch.from_numpy(cref.randn(seed, k * m, offset=0).reshape(k, m)).to(torch.bfloat16).to(FP8)
    b = torch.from_numpy(cref.randn(seed, k * n, offset=1 << 40).reshape(k, n)).to(torch.bfloat16).to(FP8)
    a_scale = torch.from_numpy(cref.randn(seed, qk * m, offset=2 << 40).reshape(qk, m))
    b_scale = torch.from_numpy(cref.randn(seed, qk * qn, offset=3 << 40).reshape(qk, qn))
    c = torch.zeros((m, n), dtype=torch.bfloat16)
    return (a.T, b.T, a_scale.T, b_scale.T, c)


def ref_kernel(data):
    """Dequantise-then-fp32-matmul. data = (a, b, a_scale, b_scale, c); writes and returns c."""
    a, b, a_scale, b_scale, c = data
    a = a.contiguous()
    a_scale = a_scale.contiguous()
    b_scale = b_scale.contiguous()
    m, k = a.shape
    n = b.shape[0]
    scale_n, scale_k = b_scale.shape
    a_sc = a_scale.unsqueeze(-1).repeat(1, 1, BLOCK).reshape(m, scale_k * BLOCK)[:, :k]
    a32 = a.to(torch.float32) * a_sc
    b_sc = (b_scale.view(-1, 1).repeat(1, BLOCK * BLOCK).view(scale_n, scale_k, BLOCK, BLOCK)
            .permute(0, 2, 1, 3).reshape(scale_n * BLOCK, scale_k * BLOCK))[:n, :k]
    b32 = b.to(torch.float32) * b_sc
    c[...] = (a32 @ b32.T).to(torch.bfloat16)
    return c


def verbose_allclose(received, expected, rtol=1e-5, atol=1e-8, max_print=5):
    """Returns a list of mismatch messages (empty when the tensors match)."""
    if received.shape != expected.shape:
        return ["SIZE MISMATCH"]
    r32, e32 = received.to(torch.float32), expected.to(torch.float32)
    diff = torch.abs(r32 - e32)
    tol = atol + rtol * torch.abs(e32)
    bad = (diff > tol) | (torch.isnan(r32) ^ torch.isnan(e32)) | \
          (torch.isposinf(r32) ^ torch.isposinf(e32)) | (torch.isneginf(r32) ^ torch.isneginf(e32))
    nbad = int(bad.sum())
    if nbad == 0:
        return []
    idx = torch.nonzero(bad)
    msgs = ["Number of mismatched elements: %d" % nbad]
    for i in idx[:max_print]:
        t = tuple(i.tolist())
        msgs.append("ERROR at %s: %r %r" % (t, float(r32[t]), float(e32[t])))
    return msgs


def check_implementation(data, output, rtol=2e-2, atol=1e-3):
    """Returns '' when output matches ref_kernel(data) under the reference's rule, else the reasons."""
    a, b, a_scale, b_scale, c = data
    expected = ref_kernel((a, b, a_scale, b_scale, torch.zeros_like(c)))
    reasons = verbose_allclose(output.cpu(), expected, rtol=rtol, atol=atol)
    return "mismatch found! custom implementation doesn't match reference: " + " ".join(reasons) if reasons else ""


def raw_layouts(data):
    """Numpy views of the underlying storage in the launcher's layouts:
    a [K][M] uint8, b [K][N] uint8, a_scale [QK][M] f32, b_scale [QK][QN] f32."""
    a, b, a_scale, b_scale, _ = data
    return (a.T.contiguous().view(torch.uint8).numpy(), b.T.contiguous().view(torch.uint8).numpy(),
            a_scale.T.contiguous().numpy(), b_scale.T.contiguous().numpy())
