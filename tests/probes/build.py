"""Builds the probes under tests/probes (test infrastructure): mfma_precision (the matrix unit's summation precision, one
wave) and lds_dma_order (completion order of LDS-DMA loads).

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
    flags = [f for f in HIPCC_FLAGS if f != "-fPIC"]
    outs = []
    for name in ("mfma_precision", "lds_dma_order"):
        out = os.path.join(HERE, name)
        res = _run([hipcc()] + flags + ["-o", out, os.path.join(HERE, name + ".hip")])
        if verbose and res:
            print(res)
        outs.append(out)
    return outs


if __name__ == "__main__":
    print("built", build_probes(verbose=True))
