"""Selected-token log-probability operators (the reference leaves this package
as an empty extension point, rl_engine/ops/logprob/__init__.py)."""

from rl_engine.backends.rocm.logprob.vocab_parallel_logp import (
    RocmVocabParallelLogprobOp as VocabParallelLogprobOp,
    hip_deterministic_logp_from_logits as deterministic_logp_from_logits,
    merge_tile_partials,
)
from rl_engine.ops.logprob.linear_logp import (
    LinearLogpOp,
    deterministic_linear_logp,
    linear_logp,
    linear_logp_contract_version,
)

__all__ = [
    "LinearLogpOp",
    "VocabParallelLogprobOp",
    "deterministic_linear_logp",
    "deterministic_logp_from_logits",
    "linear_logp",
    "linear_logp_contract_version",
    "merge_tile_partials",
]
