"""ctypes binding of oracle/liboracle.so (the plain-C restatement).

Test infrastructure only; see fp8_blockscale_oracle.c for what each function restates.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force=False):
    """Compile liboracle.so with gcc (seconds)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, sz, i32, f32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_float
        L.rfo_e4m3fn_to_f32_array.argtypes = [vp, vp, sz]
        L.rfo_f32_to_e4m3fn_array.argtypes = [vp, vp, sz]
        L.rfo_f32_to_bf16_array.argtypes = [vp, vp, sz]
        L.rfo_f32_to_bf16_fast_array.argtypes = [vp, vp, sz]
        L.rfo_bf16_to_f32_array.argtypes = [vp, vp, sz]
        L.rfo_hash64.argtypes = [ctypes.c_uint64, ctypes.c_uint64]
        L.rfo_hash64.restype = ctypes.c_uint64
        L.rfo_randn.argtypes = [ctypes.c_uint64, ctypes.c_uint64, sz, vp]
        L.rfo_quantize_a.argtypes = [vp, i32, i32, vp, vp]
        L.rfo_quantize_b.argtypes = [vp, i32, i32, vp, vp]
        L.rfo_ref_gemm_f32.argtypes = [vp, vp, vp, vp, i32, i32, i32, vp, i32, vp, vp]
        L.rfo_ref_gemm_f64.argtypes = [vp, vp, vp, vp, i32, i32, i32, vp, i32, vp]
        L.rfo_ref_gemm_blockfold.argtypes = [vp, vp, vp, vp, i32, i32, i32, vp, i32, vp, vp]
        L.rfo_allclose.argtypes = [vp, vp, sz, f32, f32, ctypes.POINTER(f32), ctypes.POINTER(ctypes.c_long)]
        L.rfo_allclose.restype = ctypes.c_long
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


def e4m3fn_to_f32(codes):
    codes = _c(codes, np.uint8)
    out = np.empty(codes.shape, np.float32)
    lib().rfo_e4m3fn_to_f32_array(_p(codes), _p(out), codes.size)
    return out


def f32_to_e4m3fn(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint8)
    lib().rfo_f32_to_e4m3fn_array(_p(x), _p(out), x.size)
    return out


def f32_to_bf16(x, fast=False):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    (lib().rfo_f32_to_bf16_fast_array if fast else lib().rfo_f32_to_bf16_array)(_p(x), _p(out), x.size)
    return out


def bf16_to_f32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().rfo_bf16_to_f32_array(_p(h), _p(out), h.size)
    return out


def hash64(seed, i):
    return int(lib().rfo_hash64(seed, i))


def randn(seed, n, offset=0):
    out = np.empty(int(n), np.float32)
    lib().rfo_randn(seed, offset, out.size, _p(out))
    return out


def quantize_a(A32):
    """A32 [M][K] fp32 -> (a [K][M] uint8 e4m3fn codes, a_scale [QK][M] fp32)."""
    A32 = _c(A32, np.float32)
    M, K = A32.shape
    a = np.empty((K, M), np.uint8)
    s = np.empty((K // 128, M), np.float32)
    lib().rfo_quantize_a(_p(A32), M, K, _p(a), _p(s))
    return a, s


def quantize_b(B32):
    """B32 [N][K] fp32 -> (b [K][N] uint8 codes, b_scale [QK][QN] fp32)."""
    B32 = _c(B32, np.float32)
    N, K = B32.shape
    b = np.empty((K, N), np.uint8)
    s = np.empty((K // 128, (N + 127) // 128), np.float32)
    lib().rfo_quantize_b(_p(B32), N, K, _p(b), _p(s))
    return b, s


def _rows(rows, M):
    if rows is None:
        return None, M, None
    r = _c(rows, np.int32)
    return r, r.size, _p(r)


def _check(a, b, a_s, b_s):
    a = _c(a, np.uint8); b = _c(b, np.uint8); a_s = _c(a_s, np.float32); b_s = _c(b_s, np.float32)
    K, M = a.shape
    K2, N = b.shape
    assert K == K2 and K % 128 == 0
    assert a_s.shape == (K // 128, M), a_s.shape
    assert b_s.shape == (K // 128, (N + 127) // 128), b_s.shape
    return a, b, a_s, b_s, M, N, K


def ref_gemm_f32(a, b, a_s, b_s, rows=None):
    """Oracle: returns (fp32 [R][N], bf16 bits [R][N]) in the launcher's layouts (a [K][M], b [K][N])."""
    a, b, a_s, b_s, M, N, K = _check(a, b, a_s, b_s)
    r, nr, rp = _rows(rows, M)
    o32 = np.empty((nr, N), np.float32); o16 = np.empty((nr, N), np.uint16)
    lib().rfo_ref_gemm_f32(_p(a), _p(b), _p(a_s), _p(b_s), M, N, K, rp, nr, _p(o32), _p(o16))
    return o32, o16


def ref_gemm_f64(a, b, a_s, b_s, rows=None):
    a, b, a_s, b_s, M, N, K = _check(a, b, a_s, b_s)
    r, nr, rp = _rows(rows, M)
    o = np.empty((nr, N), np.float64)
    lib().rfo_ref_gemm_f64(_p(a), _p(b), _p(a_s), _p(b_s), M, N, K, rp, nr, _p(o))
    return o


def ref_gemm_blockfold(a, b, a_s, b_s, rows=None):
    a, b, a_s, b_s, M, N, K = _check(a, b, a_s, b_s)
    r, nr, rp = _rows(rows, M)
    o32 = np.empty((nr, N), np.float32); o16 = np.empty((nr, N), np.uint16)
    lib().rfo_ref_gemm_blockfold(_p(a), _p(b), _p(a_s), _p(b_s), M, N, K, rp, nr, _p(o32), _p(o16))
    return o32, o16


def allclose(got_bf16, exp_bf16, rtol=2e-2, atol=1e-3):
    """Reference checker rule on bf16 bit patterns. Returns (n_mismatch, max_abs_err, first_bad_index)."""
    g = _c(got_bf16, np.uint16); e = _c(exp_bf16, np.uint16)
    assert g.shape == e.shape
    mx = ctypes.c_float(0); fb = ctypes.c_long(-1)
    bad = lib().rfo_allclose(_p(g), _p(e), g.size, rtol, atol, ctypes.byref(mx), ctypes.byref(fb))
    return int(bad), float(mx.value), int(fb.value)
