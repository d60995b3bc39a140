"""Builds tests/probes/mfma_precision (test infrastructure: the matrix unit's summation precision, one wave).

Run:  python tests/probes/build.py
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def build_probes(verbose=False):
    from radeonflow_kernels_amd.build import HIPCC_FLAGS, _run, hipcc
    out = os.path.join(HERE, "mfma_precision")
    flags = [f for f in HIPCC_FLAGS if f != "-fPIC"]
    res = _run([hipcc()] + flags + ["-o", out, os.path.join(HERE, "mfma_precision.hip")])
    if verbose and res:
        print(res)
    return out


if __name__ == "__main__":
    print("built", build_probes(verbose=True))
