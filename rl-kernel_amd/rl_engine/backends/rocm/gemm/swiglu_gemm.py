"""Packed gate/up projection with the SwiGLU activation in the GEMM epilogue (gfx950).

Stands in for rl_engine/backends/rocm/gemm/swiglu_gemm.py:36-86 of the reference, whose
fused path serves decode-sized batches through split-K partials. Here one MFMA tile kernel
serves every batch above 128 rows (a workgroup owns the gate and the up projection of the
same 128 features, so the ``[M, 2 I]`` projection is never written), the streaming kernel
serves up to 16 rows the same way (eight gate and eight up rows per weight panel), and the
batches between run the GEMM for few tokens and the elementwise kernel. All three orders of
work give the same bits.
"""

from __future__ import annotations

import torch

from rl_engine import _C


def forward(a: torch.Tensor, weight: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """``swiglu(a @ weight[:I].T, a @ weight[I:].T)`` for packed gate/up rows ``[2 I, K]``."""
    if a.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("MFMA GEMM requires BF16 inputs")
    if a.dim() != 2 or weight.dim() != 2 or a.size(1) != weight.size(1):
        raise ValueError(f"MFMA GEMM expects [M,K] @ [K,N], got {tuple(a.shape)} and {tuple(weight.t().shape)}")
    if not (a.size(0) > 0 and weight.size(0) > 0 and weight.size(0) % 2 == 0):
        raise ValueError("fused SwiGLU requires a nonempty packed gate/up projection")
    return _C.det_gemm_swiglu(a, weight, out)


__all__ = ["forward"]
