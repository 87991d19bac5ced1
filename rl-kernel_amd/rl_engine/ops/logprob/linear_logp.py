"""Platform binding for the fused linear-LogP (gfx950 build: ROCm only)."""

from __future__ import annotations

from typing import Optional

import torch

from rl_engine.backends.rocm.logprob.linear_logp import (
    HipLinearLogpOp as LinearLogpOp,
    hip_deterministic_linear_logp as deterministic_linear_logp,
    linear_logp_contract_version,
)

_OP: LinearLogpOp | None = None


def linear_logp(
    hidden: torch.Tensor,
    lm_head_weight: torch.Tensor,
    target_ids: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Functional form of ``kernel_registry.get_op("linear_logp")(...)``."""
    global _OP
    if _OP is None:
        _OP = LinearLogpOp()
    return _OP(hidden, lm_head_weight, target_ids, bias)


__all__ = ["LinearLogpOp", "deterministic_linear_logp", "linear_logp", "linear_logp_contract_version"]
