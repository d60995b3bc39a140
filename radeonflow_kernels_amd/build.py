"""Builds libgemm.so (the HIP kernels + C ABI) for gfx950 with hipcc.

hipcc cross-compiles without a GPU. The library is written in-tree to radeonflow_kernels_amd/lib/.
Run:  python -m radeonflow_kernels_amd.build
(The native test harness and the benchmark's probe have build scripts of their own: tests/checker/build.py,
bench_probes/build.py; __graft_entry__.build() runs all three.)
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


def build_all(verbose=False):
    build_lib(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
    print("built", LIB_PATH)
