"""CPU oracle for the FP8 blockwise-scaled GEMM. Test infrastructure only.

Nothing under this package is imported by the shipped library. Only tests, the smoke
check and the benchmark's CPU-baseline leg use it, and only as the checker.
"""
