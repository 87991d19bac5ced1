"""GRPO ratio / k3-KL / clipped surrogate on per-token log-probs (gfx950).

Mirrors, on the GPU, the log-prob form of the reference loss:
``compute_policy_ratio`` / ``compute_reference_kl`` / ``masked_mean``
(rl_engine/reference/definitions.py:50-106) composed as in
tests/e2e/test_rl_kernel_loss_step.py:18-39 and NativeGRPOLossOp.apply
(rl_engine/reference/loss/grpo_loss.py:96-125). Forward only.
"""

from __future__ import annotations

from typing import NamedTuple, Optional

import torch

from rl_engine import _C


class GrpoLossOutput(NamedTuple):
    loss: torch.Tensor
    policy_loss: torch.Tensor
    kl: torch.Tensor
    ratio: torch.Tensor
    k3: torch.Tensor


def _as_2d(t: torch.Tensor) -> torch.Tensor:
    return t.reshape(1, -1) if t.dim() == 1 else t


def grpo_ratio_kl_loss(
    current_logps: torch.Tensor,
    old_logps: torch.Tensor,
    ref_logps: torch.Tensor,
    sample_advantages: torch.Tensor,
    completion_mask: Optional[torch.Tensor] = None,
    *,
    clip_eps: float = 0.2,
    beta: float = 0.0,
) -> GrpoLossOutput:
    """``(loss, policy_loss, kl, ratio, k3)`` from ``[rollouts, tokens]`` fp32 log-probs.

    ``sample_advantages`` holds one advantage per rollout and is broadcast over
    the rollout's tokens; masked tokens contribute zero and do not count.
    Defaults follow the reference (clip_eps 0.2, beta 0.0, grpo_loss.py:33-34).
    """
    if current_logps.dim() not in (1, 2):
        raise ValueError("log-probs must be [tokens] or [rollouts, tokens]")
    shape = current_logps.shape
    cur = _as_2d(current_logps.float())
    old = _as_2d(old_logps.float())
    ref = _as_2d(ref_logps.float())
    if old.shape != cur.shape or ref.shape != cur.shape:
        raise ValueError("current, old and reference log-probs must share one shape")
    adv = sample_advantages.float().reshape(-1)
    if adv.numel() != cur.size(0):
        raise ValueError(f"expected {cur.size(0)} per-rollout advantages, got {adv.numel()}")
    mask = None
    if completion_mask is not None:
        mask = _as_2d(completion_mask)
        if mask.shape != cur.shape:
            raise ValueError("completion_mask must match the log-prob shape")
    out3, ratio, k3 = _C.grpo_ratio_kl_loss(cur, old, ref, adv, mask, clip_eps, beta)
    return GrpoLossOutput(out3[0], out3[1], out3[2], ratio.reshape(shape), k3.reshape(shape))


def compute_policy_ratio(current_logps, old_logps, mask=None) -> torch.Tensor:
    """``exp(current - old)`` with masked entries set to zero."""
    zeros = torch.zeros(_as_2d(current_logps).size(0), dtype=torch.float32, device=current_logps.device)
    return grpo_ratio_kl_loss(current_logps, old_logps, current_logps, zeros, mask).ratio


def compute_reference_kl(current_logps, ref_logps, mask=None) -> torch.Tensor:
    """k3 estimator ``exp(d) - d - 1`` with ``d = ref - current``; masked entries zero."""
    zeros = torch.zeros(_as_2d(current_logps).size(0), dtype=torch.float32, device=current_logps.device)
    return grpo_ratio_kl_loss(current_logps, current_logps, ref_logps, zeros, mask).k3


__all__ = ["GrpoLossOutput", "compute_policy_ratio", "compute_reference_kl", "grpo_ratio_kl_loss"]
