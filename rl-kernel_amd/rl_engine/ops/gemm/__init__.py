"""Matrix multiplication operators of the deterministic dense path."""

from rl_engine.ops.gemm import det_gemm as _det_gemm

DetGemmOp = _det_gemm.DetGemmOp
deterministic_gemm = _det_gemm.deterministic_gemm
__all__ = ["DetGemmOp", "deterministic_gemm"]
