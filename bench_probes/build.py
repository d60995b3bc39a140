"""Builds bench_probes/mfma_ceiling: what the whole chip sustains on the GEMM's MFMA from registers alone, with and
without the folds and LDS reads of the GEMM's inner loop (bench.py --all reports it beside the GEMM).

Run:  python bench_probes/build.py
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def build_probe(verbose=False):
    from radeonflow_kernels_amd.build import HIPCC_FLAGS, _run, hipcc
    out = os.path.join(HERE, "mfma_ceiling")
    flags = [f for f in HIPCC_FLAGS if f != "-fPIC"]
    res = _run([hipcc()] + flags + ["-o", out, os.path.join(HERE, "mfma_ceiling.hip")])
    if verbose and res:
        print(res)
    return out


if __name__ == "__main__":
    print("built", build_probe(verbose=True))
