"""MI355X-native FP8 blockwise-scaled GEMM (libgemm.so + a thin host mirror of the reference's operator API)."""
from .gemm import (fp8_mm, fp8_mm_static, fp8_mm_time, fp8_mm_grouped, fp8_mm_grouped_padded, quantize_a_grouped, grouped_padded_offsets, grouped_variant_for, custom_kernel, select_config, variants, quantize_a, quantize_b, cast_to_e4m3fn, GemmConfig,  # noqa: F401
                   PerfMetrics, lib, load_plans, clear_plans, plan_for, plan_can_run)
