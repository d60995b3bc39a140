"""Writes the small committed fixtures (inputs in the launcher's layouts + the oracle's bf16 output).

Run from the repo root:  python tests/golden/make_golden.py
Fixtures: a [K][M] uint8 e4m3fn codes, b [K][N] uint8, a_scale [QK][M] f32, b_scale [QK][QN] f32,
c_bf16 [M][N] uint16 bit patterns from oracle.cref.ref_gemm_f32 (dequantise-then-fp32-matmul).
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from oracle import cref, ref_kernel as rk  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = [
    # name, generator, m, n, k, seed   (shapes from the reference's test list where small enough)
    ("blockquant_m64_n64_k128", rk.generate_input_blockquant, 64, 64, 128, 6635),
    ("refstyle_m64_n64_k128", rk.generate_input_reference_style, 64, 64, 128, 6635),
    ("blockquant_m96_n576_k256_raggedN", rk.generate_input_blockquant, 96, 576, 256, 542),
    ("refstyle_m48_n200_k384_odd", rk.generate_input_reference_style, 48, 200, 384, 99),
]

if __name__ == "__main__":
    for name, gen, m, n, k, seed in CASES:
        a, b, sa, sb = rk.raw_layouts(gen(m, n, k, seed))
        _, c16 = cref.ref_gemm_f32(a, b, sa, sb)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), a=a, b=b, a_scale=sa, b_scale=sb, c_bf16=c16)
        print(name, a.shape, b.shape, c16.shape)
