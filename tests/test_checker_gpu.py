"""Runs the native harness (tests/checker/gemm_checker) on the GPU: the reference's `make test` path."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CHECKER = os.path.join(HERE, "checker", "gemm_checker")


@pytest.mark.gpu
def test_native_checker_single_run_mode_passes_all_cases():
    assert os.path.exists(CHECKER), "build it with python tests/checker/build.py"
    p = subprocess.run([CHECKER, "-b"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=900)
    print(p.stdout)
    assert p.returncode == 0, p.stdout
    assert "All 18 test cases passed" in p.stdout


@pytest.mark.gpu
def test_native_checker_prints_best_time_of_one_case():
    p = subprocess.run([CHECKER, "-c", "14", "-t", "0"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=300)
    assert p.returncode == 0, p.stdout
    assert 50.0 < float(p.stdout.strip().splitlines()[-1]) < 5000.0     # microseconds for 6144x4608x7168


def test_native_checker_usage_on_bad_flag():
    if not os.path.exists(CHECKER):
        pytest.skip("checker not built")
    p = subprocess.run([CHECKER, "-x"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert p.returncode != 0 and "Usage:" in p.stdout
