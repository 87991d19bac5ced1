"""Selected-token log-probability operators (the reference leaves this package
as an empty extension point, rl_engine/ops/logprob/__init__.py)."""

from rl_engine.ops.logprob.linear_logp import (
    LinearLogpOp,
    deterministic_linear_logp,
    linear_logp,
    linear_logp_contract_version,
)

__all__ = ["LinearLogpOp", "deterministic_linear_logp", "linear_logp", "linear_logp_contract_version"]
