"""gfx950 plan sweep for the FP8 blockscale GEMM (replaces the reference's tuner/gemm_tuner.py + gemm_batch.py)."""
