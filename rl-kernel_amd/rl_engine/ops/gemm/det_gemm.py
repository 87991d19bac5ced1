"""Platform binding for the strict deterministic GEMM (gfx950 build: ROCm only).

Exports the same eight names as the reference module of this path
(rl_engine/ops/gemm/det_gemm.py:32-41).
"""

from rl_engine.backends.rocm.gemm.det_gemm import (
    DetGemmOp,
    det_gemm_backend,
    det_gemm_backend_id,
    det_gemm_fallback_reason,
    det_gemm_linear,
    det_gemm_linear_input_gradient,
    det_gemm_linear_weight_gradient,
    deterministic_gemm,
)

__all__ = [
    "DetGemmOp",
    "det_gemm_backend",
    "det_gemm_backend_id",
    "det_gemm_fallback_reason",
    "det_gemm_linear",
    "det_gemm_linear_input_gradient",
    "det_gemm_linear_weight_gradient",
    "deterministic_gemm",
]
