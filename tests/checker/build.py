"""Builds tests/checker/gemm_checker: the native harness (test infrastructure; links the C oracle, dlopens libgemm.so).

Run:  python tests/checker/build.py        (after python -m radeonflow_kernels_amd.build)
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def build_checker(verbose=False):
    from radeonflow_kernels_amd.build import _run, hipcc
    src = os.path.join(HERE, "gemm_checker.cpp")
    oracle = os.path.join(ROOT, "oracle", "fp8_blockscale_oracle.c")
    out = os.path.join(HERE, "gemm_checker")
    obj = os.path.join(HERE, "oracle.o")
    _run(["gcc", "-O2", "-fopenmp", "-std=c11", "-ffp-contract=off", "-c", oracle, "-o", obj])
    rocm = os.path.dirname(os.path.dirname(os.path.realpath(hipcc())))
    # host-only program: plain g++ against the HIP runtime library
    cmd = ["g++", "-O2", "-std=c++17", "-fopenmp", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(rocm, "include"),
           "-o", out, src, obj, "-L" + os.path.join(rocm, "lib"), "-lamdhip64", "-ldl", "-lm",
           "-Wl,-rpath," + os.path.join(rocm, "lib"), "-Wl,-rpath,$ORIGIN/../../radeonflow_kernels_amd/lib"]
    res = _run(cmd)
    if verbose and res:
        print(res)
    return out


if __name__ == "__main__":
    print("built", build_checker(verbose=True))
