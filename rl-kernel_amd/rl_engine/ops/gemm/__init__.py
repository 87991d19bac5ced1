"""Matrix multiplication operators of the deterministic dense path."""

from rl_engine.ops.gemm.det_gemm import DetGemmOp, deterministic_gemm

__all__ = ["DetGemmOp", "deterministic_gemm"]
