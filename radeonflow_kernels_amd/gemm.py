"""Host-side mirror of the reference's Python operator boundary, over the C ABI of libgemm.so.

Mirrors the torch extension the reference generates (scripts/gen_submission.py:248-262,327-330):
  fp8_mm(a, b, a_scale, b_scale, c)   m=a.size(0), n=b.size(0), k=a.size(1); current stream; run(...)
  custom_kernel(data) -> c
Tensors carry the reference's strides: a [m,k] and b [n,k] are transposed views of [K][M] / [K][N]
fp8 storage, a_scale [m,k/128] and b_scale [ceil(n/128),k/128] are transposed views of [QK][M] /
[QK][QN] fp32 storage, c is contiguous bf16 [m,n]. PyTorch is used for device memory and streams only.
There is no CPU or PyTorch fallback: a missing library or a non-GPU tensor raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libgemm.so")
_lib = None

RF_OK = 0


class GemmConfig(ctypes.Structure):
    """rf_gemm_config of include/rf_gemm.h. stream_k is the schedule: 0 one workgroup per tile (and K split),
    1 stream-K, 2 persistent, 3 persistent with a last round of half tiles, 4 skinny K (K = 128 ... 512, variant 0)."""
    _fields_ = [("variant", ctypes.c_int), ("split_k", ctypes.c_int), ("group_m", ctypes.c_int),
                ("stream_k", ctypes.c_int)]

    def __repr__(self):
        return "GemmConfig(variant=%d, split_k=%d, group_m=%d, stream_k=%d)" % (self.variant, self.split_k,
                                                                                 self.group_m, self.stream_k)


class PerfMetricEntry(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 20), ("time", ctypes.c_float), ("gflops", ctypes.c_float)]


class PerfMetrics(ctypes.Structure):
    _fields_ = [("count", ctypes.c_int), ("entries", PerfMetricEntry * 20)]


EXPORTS = ("run", "rf_fp8_gemm", "rf_fp8_gemm_ex", "rf_gemm_select_config", "rf_gemm_num_variants",
           "rf_gemm_variant_info", "rf_gemm_variant_has_stream_k", "rf_gemm_variant_has_persistent", "rf_gemm_workspace_bytes", "rf_gemm_init", "rf_gemm_destroy",
           "rf_gemm_last_error", "rf_fp8_gemm_grouped", "rf_quantize_a_f32", "rf_quantize_a_bf16", "rf_quantize_b_f32", "rf_quantize_b_bf16",
           "rf_cast_f32_to_e4m3fn", "rf_gemm_load_plans", "rf_gemm_clear_plans", "rf_fp8_gemm_time", "rf_fp8_gemm_static",
           "rf_gemm_static_scratch_bytes", "rf_grouped_padded_offsets", "rf_quantize_a_grouped_f32",
           "rf_quantize_a_grouped_bf16", "rf_fp8_gemm_grouped_padded", "rf_gemm_plan_for", "rf_gemm_variant_k_groups",
           "rf_grouped_variant_for")


def lib():
    """Loads libgemm.so (built by radeonflow_kernels_amd.build). Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libgemm.so is missing at %s: build it with `python -m radeonflow_kernels_amd.build`"
                               % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        vp, i32 = ctypes.c_void_p, ctypes.c_int
        L.run.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, ctypes.POINTER(PerfMetrics), vp]
        L.run.restype = None
        L.rf_fp8_gemm.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, vp]
        L.rf_fp8_gemm.restype = i32
        L.rf_fp8_gemm_static.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, vp]
        L.rf_fp8_gemm_static.restype = i32
        L.rf_gemm_static_scratch_bytes.argtypes = []
        L.rf_gemm_static_scratch_bytes.restype = ctypes.c_size_t
        L.rf_fp8_gemm_ex.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, ctypes.POINTER(GemmConfig), vp]
        L.rf_fp8_gemm_ex.restype = i32
        L.rf_fp8_gemm_time.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, ctypes.POINTER(GemmConfig), i32, i32,
                                       ctypes.POINTER(ctypes.c_float), vp]
        L.rf_fp8_gemm_time.restype = i32
        L.rf_gemm_select_config.argtypes = [i32, i32, i32, ctypes.POINTER(GemmConfig)]
        L.rf_gemm_select_config.restype = i32
        L.rf_gemm_plan_for.argtypes = [i32, i32, i32, i32, ctypes.POINTER(GemmConfig)]
        L.rf_gemm_plan_for.restype = i32
        L.rf_gemm_load_plans.argtypes = [ctypes.c_char_p, ctypes.POINTER(i32)]
        L.rf_gemm_load_plans.restype = i32
        L.rf_gemm_clear_plans.restype = None
        L.rf_gemm_num_variants.restype = i32
        L.rf_gemm_variant_info.argtypes = [i32] + [ctypes.POINTER(i32)] * 5
        L.rf_gemm_variant_info.restype = i32
        L.rf_gemm_variant_has_stream_k.argtypes = [i32]
        L.rf_gemm_variant_has_stream_k.restype = i32
        L.rf_gemm_variant_k_groups.argtypes = [i32]
        L.rf_gemm_variant_k_groups.restype = i32
        L.rf_gemm_variant_has_persistent.argtypes = [i32]
        L.rf_gemm_variant_has_persistent.restype = i32
        L.rf_gemm_workspace_bytes.argtypes = [i32, i32, i32]
        L.rf_gemm_workspace_bytes.restype = ctypes.c_size_t
        L.rf_gemm_init.argtypes = [ctypes.c_size_t]
        L.rf_gemm_init.restype = i32
        L.rf_gemm_destroy.restype = None
        L.rf_gemm_last_error.restype = ctypes.c_char_p
        L.rf_fp8_gemm_grouped.argtypes = [ctypes.c_void_p] * 5 + [ctypes.POINTER(i32), i32, i32, i32, i32, ctypes.c_void_p]
        L.rf_fp8_gemm_grouped.restype = i32
        L.rf_fp8_gemm_grouped_padded.argtypes = [ctypes.c_void_p] * 5 + [ctypes.POINTER(i32), i32, i32, i32, i32, ctypes.c_void_p]
        L.rf_fp8_gemm_grouped_padded.restype = i32
        L.rf_grouped_padded_offsets.argtypes = [ctypes.POINTER(i32), i32, ctypes.POINTER(i32)]
        L.rf_grouped_padded_offsets.restype = i32
        L.rf_grouped_variant_for.argtypes = [ctypes.POINTER(i32), i32, i32, i32, i32, ctypes.POINTER(i32)]
        L.rf_grouped_variant_for.restype = i32
        for name in ("rf_quantize_a_grouped_f32", "rf_quantize_a_grouped_bf16"):
            f = getattr(L, name)
            f.argtypes = [ctypes.c_void_p, ctypes.POINTER(i32), i32, i32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
            f.restype = i32
        for name in ("rf_quantize_a_f32", "rf_quantize_a_bf16", "rf_quantize_b_f32", "rf_quantize_b_bf16"):
            f = getattr(L, name)
            f.argtypes = [ctypes.c_void_p, i32, i32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
            f.restype = i32
        L.rf_cast_f32_to_e4m3fn.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p]
        L.rf_cast_f32_to_e4m3fn.restype = i32
        _lib = L
    return _lib


def last_error():
    return lib().rf_gemm_last_error().decode()


def _check_layout(a, b, a_scale, b_scale, c):
    if not (a.is_cuda and b.is_cuda and a_scale.is_cuda and b_scale.is_cuda and c.is_cuda):
        raise ValueError("fp8_mm needs GPU tensors")
    m, k = a.shape
    n = b.shape[0]
    qk, qn = k // 128, (n + 127) // 128
    if a.element_size() != 1 or b.element_size() != 1:
        raise ValueError("a and b must be 1-byte fp8 (e4m3fn) tensors")
    if b.shape[1] != k or tuple(a_scale.shape) != (m, qk) or tuple(b_scale.shape) != (qn, qk) or tuple(c.shape) != (m, n):
        raise ValueError("inconsistent shapes")
    if a_scale.dtype != torch.float32 or b_scale.dtype != torch.float32 or c.dtype != torch.bfloat16:
        raise ValueError("scales must be fp32 and c bf16")
    # the launcher reads [K][M], [K][N], [QK][M], [QK][QN] storage: the tensors must be transposed views of that
    def colmajor(t):
        r, cdim = t.shape
        return (t.stride(0) == 1 or r == 1) and (t.stride(1) == r or cdim == 1)
    if not (colmajor(a) and colmajor(b) and colmajor(a_scale) and colmajor(b_scale) and c.is_contiguous()):
        raise ValueError("a, b, a_scale, b_scale must be column-major (transposed views), c row-major contiguous")
    return m, n, k


def fp8_mm(a, b, a_scale, b_scale, c, config=None):
    """c[m,n] = bf16(sum_kb a_scale*b_scale * (A_kb . B_kb^T)) on the current HIP stream; returns None."""
    m, n, k = _check_layout(a, b, a_scale, b_scale, c)
    stream = ctypes.c_void_p(torch.cuda.current_stream(a.device).cuda_stream)
    L = lib()
    cfg = ctypes.byref(config) if config is not None else None
    with torch.cuda.device(a.device):
        rc = L.rf_fp8_gemm_ex(a.data_ptr(), b.data_ptr(), a_scale.data_ptr(), b_scale.data_ptr(), c.data_ptr(),
                              m, n, k, cfg, stream)
    if rc != RF_OK:
        raise RuntimeError("rf_fp8_gemm failed (%d): %s" % (rc, last_error()))


def fp8_mm_static(a, b, a_scale, b_scale, c):
    """fp8_mm through rf_fp8_gemm_static: same result, no device memory is allocated or freed by the call (temporary
    data lives in a static 32 MiB device array; shapes that need more raise)."""
    m, n, k = _check_layout(a, b, a_scale, b_scale, c)
    stream = ctypes.c_void_p(torch.cuda.current_stream(a.device).cuda_stream)
    with torch.cuda.device(a.device):
        rc = lib().rf_fp8_gemm_static(a.data_ptr(), b.data_ptr(), a_scale.data_ptr(), b_scale.data_ptr(), c.data_ptr(),
                                      m, n, k, stream)
    if rc != RF_OK:
        raise RuntimeError("rf_fp8_gemm_static failed (%d): %s" % (rc, last_error()))


def fp8_mm_time(a, b, a_scale, b_scale, c, config=None, warmup=3, iters=20):
    """Average microseconds per launch of fp8_mm over `iters` back-to-back launches timed inside the library (no
    per-launch Python overhead, which exceeds the GPU time of small shapes)."""
    m, n, k = _check_layout(a, b, a_scale, b_scale, c)
    stream = ctypes.c_void_p(torch.cuda.current_stream(a.device).cuda_stream)
    us = ctypes.c_float(0.0)
    cfg = ctypes.byref(config) if config is not None else None
    with torch.cuda.device(a.device):
        rc = lib().rf_fp8_gemm_time(a.data_ptr(), b.data_ptr(), a_scale.data_ptr(), b_scale.data_ptr(), c.data_ptr(),
                                    m, n, k, cfg, warmup, iters, ctypes.byref(us), stream)
    if rc != RF_OK:
        raise RuntimeError("rf_fp8_gemm_time failed (%d): %s" % (rc, last_error()))
    return us.value


def fp8_mm_grouped(a, b, a_scale, b_scale, c, row_offsets, variant=-1):
    """Grouped GEMM: rows row_offsets[g]..row_offsets[g+1]-1 of a / a_scale / c belong to group g and are multiplied
    with b[g], b_scale[g].
      a [M_total, K] fp8 stride (1, M_total); a_scale [M_total, K/128] fp32 stride (1, M_total);
      b [G, N, K] fp8 stride (K*N, 1, N); b_scale [G, ceil(N/128), K/128] fp32 stride (QK*QN, 1, QN);
      c [M_total, N] bf16 contiguous; row_offsets: sequence of G+1 ints on the host."""
    m_total, k = a.shape
    groups, n, _ = b.shape
    qk, qn = k // 128, (n + 127) // 128
    ok = (a.dtype == torch.float8_e4m3fn and b.dtype == torch.float8_e4m3fn and c.dtype == torch.bfloat16
          and a_scale.dtype == torch.float32 and b_scale.dtype == torch.float32
          and tuple(b.shape) == (groups, n, k) and tuple(c.shape) == (m_total, n) and c.is_contiguous()
          and (m_total <= 1 or k == 1 or a.stride() == (1, m_total)) and tuple(a_scale.shape) == (m_total, qk)
          and (m_total <= 1 or qk == 1 or a_scale.stride() == (1, m_total))
          and (b.stride() == (k * n, 1, n) or (groups == 1 and b.stride()[1:] == (1, n))) and tuple(b_scale.shape) == (groups, qn, qk)
          and (b_scale.stride() == (qk * qn, 1, qn) or qn == 1 or qk == 1 or (groups == 1 and b_scale.stride()[1:] == (1, qn))) and len(row_offsets) == groups + 1)
    if not ok:
        raise ValueError("fp8_mm_grouped: operands do not have the documented dtypes / shapes / strides")
    offs = (ctypes.c_int32 * (groups + 1))(*[int(x) for x in row_offsets])
    stream = ctypes.c_void_p(torch.cuda.current_stream(a.device).cuda_stream)
    with torch.cuda.device(a.device):
        rc = lib().rf_fp8_gemm_grouped(a.data_ptr(), b.data_ptr(), a_scale.data_ptr(), b_scale.data_ptr(), c.data_ptr(),
                                       offs, groups, n, k, variant, stream)
    if rc != RF_OK:
        raise RuntimeError("rf_fp8_gemm_grouped failed (%d): %s" % (rc, last_error()))


def grouped_variant_for(row_offsets, n, k, num_cu=256):
    """The tile form fp8_mm_grouped takes with variant=-1 for groups of these sizes on a device with num_cu compute
    units (0..3: 256x256, 128x256, 128x128, 128x64 tiles; 4: 256-row tiles with a 128-row last tile; 5: the queue form).
    Host arithmetic only."""
    groups = len(row_offsets) - 1
    offs = (ctypes.c_int32 * (groups + 1))(*[int(x) for x in row_offsets])
    out = ctypes.c_int32(-1)
    rc = lib().rf_grouped_variant_for(offs, groups, n, k, num_cu, ctypes.byref(out))
    if rc != RF_OK:
        raise RuntimeError("rf_grouped_variant_for failed (%d): %s" % (rc, last_error()))
    return out.value


def grouped_padded_offsets(row_offsets):
    """Row offsets of the padded layout: every group starts at a multiple of 16 (list of len(row_offsets) ints)."""
    groups = len(row_offsets) - 1
    offs = (ctypes.c_int32 * (groups + 1))(*[int(x) for x in row_offsets])
    out = (ctypes.c_int32 * (groups + 1))()
    rc = lib().rf_grouped_padded_offsets(offs, groups, out)
    if rc != RF_OK:
        raise RuntimeError("rf_grouped_padded_offsets failed (%d): %s" % (rc, last_error()))
    return list(out)


def quantize_a_grouped(x, row_offsets):
    """Activations [M_total, K] (fp32 or bf16, contiguous, on the GPU) of groups that own rows row_offsets[g] ..
    row_offsets[g+1]-1 -> (a, a_scale) in the padded layout fp8_mm_grouped_padded takes: a [M_pad, K] stride (1, M_pad),
    a_scale [M_pad, K/128] stride (1, M_pad); padding rows hold zeros with scale 1."""
    if x.dim() != 2 or not x.is_contiguous() or x.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("source must be a contiguous 2-D fp32 or bf16 tensor [rows, K]")
    rows, k = x.shape
    if k < 128 or k % 128 or int(row_offsets[-1]) != rows:
        raise ValueError("K must be a positive multiple of 128 and row_offsets must end at the number of rows")
    groups = len(row_offsets) - 1
    m_pad = grouped_padded_offsets(row_offsets)[-1]
    a = torch.empty((k, m_pad), dtype=torch.float8_e4m3fn, device=x.device)
    a_scale = torch.empty((k // 128, m_pad), dtype=torch.float32, device=x.device)
    offs = (ctypes.c_int32 * (groups + 1))(*[int(v) for v in row_offsets])
    name = "rf_quantize_a_grouped_%s" % ("f32" if x.dtype == torch.float32 else "bf16")
    stream = ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
    with torch.cuda.device(x.device):
        rc = getattr(lib(), name)(x.data_ptr(), offs, groups, k, a.data_ptr(), a_scale.data_ptr(), stream)
    if rc != RF_OK:
        raise RuntimeError("%s failed (%d): %s" % (name, rc, last_error()))
    return a.T, a_scale.T


def fp8_mm_grouped_padded(a, b, a_scale, b_scale, c, row_offsets, variant=-1):
    """fp8_mm_grouped on activations already in the padded layout (quantize_a_grouped): a [M_pad, K] stride (1, M_pad),
    a_scale [M_pad, K/128] stride (1, M_pad); b, b_scale, c and row_offsets as for fp8_mm_grouped."""
    m_pad, k = a.shape
    groups, n, _ = b.shape
    qk, qn = k // 128, (n + 127) // 128
    m_total = int(row_offsets[-1])
    ok = (a.dtype == torch.float8_e4m3fn and b.dtype == torch.float8_e4m3fn and c.dtype == torch.bfloat16
          and a_scale.dtype == torch.float32 and b_scale.dtype == torch.float32 and len(row_offsets) == groups + 1
          and m_pad == grouped_padded_offsets(row_offsets)[-1] and a.stride() == (1, m_pad)
          and tuple(a_scale.shape) == (m_pad, qk) and (qk == 1 or a_scale.stride() == (1, m_pad))
          and tuple(b.shape) == (groups, n, k) and (b.stride() == (k * n, 1, n) or (groups == 1 and b.stride()[1:] == (1, n)))
          and tuple(b_scale.shape) == (groups, qn, qk) and (b_scale.stride() == (qk * qn, 1, qn) or qn == 1 or qk == 1 or (groups == 1 and b_scale.stride()[1:] == (1, qn)))
          and tuple(c.shape) == (m_total, n) and c.is_contiguous())
    if not ok:
        raise ValueError("fp8_mm_grouped_padded: operands do not have the documented dtypes / shapes / strides")
    offs = (ctypes.c_int32 * (groups + 1))(*[int(x) for x in row_offsets])
    stream = ctypes.c_void_p(torch.cuda.current_stream(a.device).cuda_stream)
    with torch.cuda.device(a.device):
        rc = lib().rf_fp8_gemm_grouped_padded(a.data_ptr(), b.data_ptr(), a_scale.data_ptr(), b_scale.data_ptr(),
                                              c.data_ptr(), offs, groups, n, k, variant, stream)
    if rc != RF_OK:
        raise RuntimeError("rf_fp8_gemm_grouped_padded failed (%d): %s" % (rc, last_error()))


def custom_kernel(data):
    """The contest entry point: data = (a, b, a_scale, b_scale, c); returns c."""
    a, b, a_scale, b_scale, c = data
    fp8_mm(a, b, a_scale, b_scale, c)
    return c


def run_with_metrics(a, b, a_scale, b_scale, c):
    """Calls the drop-in `run` entry with a PerfMetrics record; returns (time_ms, gflops) after a sync."""
    m, n, k = _check_layout(a, b, a_scale, b_scale, c)
    pm = PerfMetrics()
    stream = ctypes.c_void_p(torch.cuda.current_stream(a.device).cuda_stream)
    with torch.cuda.device(a.device):
        lib().run(a.data_ptr(), b.data_ptr(), a_scale.data_ptr(), b_scale.data_ptr(), c.data_ptr(), m, n, k,
                  ctypes.byref(pm), stream)
        torch.cuda.synchronize(a.device)
    return pm.entries[0].time, pm.entries[0].gflops, pm.count


def _quantize(x, per_row):
    if x.dim() != 2 or not x.is_contiguous() or x.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("source must be a contiguous 2-D fp32 or bf16 tensor [rows, K]")
    rows, k = x.shape
    if k < 128 or k % 128:
        raise ValueError("K must be a positive multiple of 128")
    q = torch.empty((k, rows), dtype=torch.float8_e4m3fn, device=x.device)
    nscale = rows if per_row else (rows + 127) // 128
    scales = torch.empty((k // 128, nscale), dtype=torch.float32, device=x.device)
    name = "rf_quantize_%s_%s" % ("a" if per_row else "b", "f32" if x.dtype == torch.float32 else "bf16")
    stream = ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
    with torch.cuda.device(x.device):
        rc = getattr(lib(), name)(x.data_ptr(), rows, k, q.data_ptr(), scales.data_ptr(), stream)
    if rc != RF_OK:
        raise RuntimeError("%s failed (%d): %s" % (name, rc, last_error()))
    return q.T, scales.T         # the transposed views fp8_mm takes: [rows, K] stride (1, rows), [rows or QN, K/128]


def cast_to_e4m3fn(x):
    """fp32 tensor (contiguous, on the GPU) -> torch.float8_e4m3fn tensor of the same shape, round to nearest even."""
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise ValueError("source must be a contiguous fp32 tensor")
    out = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
    stream = ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
    with torch.cuda.device(x.device):
        rc = lib().rf_cast_f32_to_e4m3fn(x.data_ptr(), x.numel(), out.data_ptr(), stream)
    if rc != RF_OK:
        raise RuntimeError("rf_cast_f32_to_e4m3fn failed (%d): %s" % (rc, last_error()))
    return out


def quantize_a(x):
    """Activations [M, K] (fp32 or bf16, on the GPU) -> (a, a_scale) as fp8_mm takes them: one scale per
    (row, 128-wide K block), scale = amax/448, value = e4m3fn_rne(x / scale)."""
    return _quantize(x, True)


def quantize_b(w):
    """Weights [N, K] -> (b, b_scale): one scale per 128x128 block."""
    return _quantize(w, False)


def select_config(m, n, k):
    cfg = GemmConfig()
    rc = lib().rf_gemm_select_config(m, n, k, ctypes.byref(cfg))
    if rc != RF_OK:
        raise RuntimeError("rf_gemm_select_config failed (%d): %s" % (rc, last_error()))
    return cfg


def plan_for(m, n, k, num_cu):
    """The plan for (m, n, k) on a device with num_cu compute units, worked out on the host alone (rf_gemm_plan_for)."""
    cfg = GemmConfig()
    rc = lib().rf_gemm_plan_for(m, n, k, num_cu, ctypes.byref(cfg))
    if rc != RF_OK:
        raise RuntimeError("rf_gemm_plan_for failed (%d): %s" % (rc, last_error()))
    return cfg


def load_plans(path):
    """Adds the measured plans of a file ("M N K variant split_k group_m stream_k" per line, as written by the tuner's
    --emit-file) in front of the built-in table; returns how many were added."""
    n = ctypes.c_int(0)
    rc = lib().rf_gemm_load_plans(os.fsencode(path), ctypes.byref(n))
    if rc != RF_OK:
        raise RuntimeError("rf_gemm_load_plans failed (%d): %s" % (rc, last_error()))
    return n.value


def clear_plans():
    lib().rf_gemm_clear_plans()


def plan_can_run(v, split, k):
    """Whether variant v (an entry of variants()) takes `split` K parts at this K under the tile schedule: a variant that
    splits K between wave groups of one workgroup takes split 1 only, and K/128 must be a multiple of its group count."""
    if split > k // 128:
        return False
    return v["k_groups"] == 1 or (split == 1 and (k // 128) % v["k_groups"] == 0)


def variants():
    L = lib()
    out = []
    for v in range(L.rf_gemm_num_variants()):
        vals = [ctypes.c_int() for _ in range(5)]
        L.rf_gemm_variant_info(v, *[ctypes.byref(x) for x in vals])
        out.append(dict(variant=v, block_m=vals[0].value, block_n=vals[1].value, waves_m=vals[2].value,
                        waves_n=vals[3].value, lds_bytes=vals[4].value,
                        stream_k=bool(L.rf_gemm_variant_has_stream_k(v)),
                        persistent=bool(L.rf_gemm_variant_has_persistent(v)),
                        k_groups=L.rf_gemm_variant_k_groups(v)))
    return out
