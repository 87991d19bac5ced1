"""Loss epilogues of the deterministic dense path."""

from rl_engine.backends.rocm.loss.grpo import (
    GrpoLossOutput,
    compute_policy_ratio,
    compute_reference_kl,
    group_advantages,
    grpo_ratio_kl_loss,
)

__all__ = ["GrpoLossOutput", "compute_policy_ratio", "compute_reference_kl", "group_advantages", "grpo_ratio_kl_loss"]
