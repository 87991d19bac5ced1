"""The strict deterministic GEMM as the rest of the package imports it.

The reference binds this module to a platform backend at import time and exports eight names
(rl_engine/ops/gemm/det_gemm.py:32-41); this build has one backend, the gfx950 one, and takes
the same eight names from it.
"""

from rl_engine.backends.rocm.gemm import det_gemm as _gfx950

_EXPORTS = (
    "DetGemmOp", "deterministic_gemm",
    "det_gemm_linear", "det_gemm_linear_input_gradient", "det_gemm_linear_weight_gradient",
    "det_gemm_backend", "det_gemm_backend_id", "det_gemm_fallback_reason",
)  # fmt: skip
globals().update({name: getattr(_gfx950, name) for name in _EXPORTS})
__all__ = sorted(_EXPORTS)
