"""Builds libgemm.so (the HIP kernels + C ABI) for gfx950 with hipcc.

hipcc cross-compiles without a GPU. The library is written in-tree to radeonflow_kernels_amd/lib/.
Run:  python -m radeonflow_kernels_amd.build
"""
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libgemm.so")

# -packed-fp32-ops off: v_pk_{add,mul,fma}_f32 are kept out of the generated code on purpose.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "is not a recognized feature" not in l)
    if p.returncode != 0:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_lib(verbose=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [hipcc()] + HIPCC_FLAGS + ["-shared", "-o", LIB_PATH, os.path.join(CSRC, "gemm_launcher.hip")]
    out = _run(cmd)
    if verbose and out:
        print(out)
    return LIB_PATH


def build_checker(verbose=False):
    """tests/checker/gemm_checker: native harness (test infrastructure; links the C oracle, dlopens libgemm.so)."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "tests", "checker", "gemm_checker.cpp")
    oracle = os.path.join(root, "oracle", "fp8_blockscale_oracle.c")
    out = os.path.join(root, "tests", "checker", "gemm_checker")
    obj = os.path.join(root, "tests", "checker", "oracle.o")
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


def build_probe(verbose=False):
    """lib/mfma_ceiling: register-only MFMA throughput of the whole chip (bench.py --all reports it beside the GEMM)."""
    os.makedirs(LIB_DIR, exist_ok=True)
    out = os.path.join(LIB_DIR, "mfma_ceiling")
    res = _run([hipcc()] + HIPCC_FLAGS + ["-o", out, os.path.join(CSRC, "mfma_ceiling.hip")])
    if verbose and res:
        print(res)
    return out


def build_all(verbose=False):
    build_lib(verbose)
    build_probe(verbose)
    build_checker(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
    print("built", LIB_PATH)
