"""GRPO ratio / k3-KL / clipped surrogate on per-token log-probs (gfx950).

Mirrors, on the GPU, the log-prob form of the reference loss:
``compute_policy_ratio`` / ``compute_reference_kl`` / ``masked_mean``
(rl_engine/reference/definitions.py:50-106) composed as in
tests/e2e/test_rl_kernel_loss_step.py:18-39 and NativeGRPOLossOp.apply
(rl_engine/reference/loss/grpo_loss.py:96-125). The three scalars are differentiable
with respect to the current log-probs, with the gradients torch's autograd gives the
reference's formula (``torch.minimum`` / ``torch.clamp`` conventions), so the loss
can sit on top of the differentiable fused linear-LogP in a training step.
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


def _bool_mask(mask: torch.Tensor, device: torch.device) -> torch.Tensor:
    """The mask as the reference reads it (``mask.bool()``, rl_engine/reference/definitions.py:50-70):
    any non-zero value, fractional or above 255 included, keeps the token, and keeps it with weight one."""
    return _as_2d(mask).to(device=device).bool()


class _GrpoLossAutograd(torch.autograd.Function):
    """Forward on the HIP kernel; backward elementwise on the saved per-token outputs.

    With ``r = exp(logp - old)``, ``d = ref - logp``, ``n = max(active, 1e-8)``:
    ``d policy_i / d logp_i = -A r_i`` where the unclipped branch is the minimum or ties it
    (inside the clip range, or outside it on the side the clip does not bind), else 0;
    ``d k3_i / d logp_i = 1 - exp(d_i)``; both times ``mask_i / n``.
    """

    @staticmethod
    def forward(ctx, cur, old, ref, adv, mask, clip_eps, beta):
        # `mask` is already the boolean mask (see _bool_mask): the kernel and the backward weigh with the same tensor
        out3, ratio, k3 = _C.grpo_ratio_kl_loss(cur, old, ref, adv, mask, clip_eps, beta)
        ctx.save_for_backward(cur, old, ref, adv, mask if mask is not None else torch.empty(0, device=cur.device))
        ctx.has_mask = mask is not None
        ctx.clip_eps, ctx.beta = float(clip_eps), float(beta)
        ctx.mark_non_differentiable(ratio, k3)
        return out3[0], out3[1], out3[2], ratio, k3

    @staticmethod
    def backward(ctx, g_loss, g_policy, g_kl, _g_ratio, _g_k3):
        cur, old, ref, adv, mask = ctx.saved_tensors
        keep = mask.to(torch.float32) if ctx.has_mask else torch.ones_like(cur)
        count = torch.clamp(keep.sum(), min=1e-8)
        a = adv.reshape(-1, 1)
        r = torch.exp(cur - old)
        lo, hi = 1.0 - ctx.clip_eps, 1.0 + ctx.clip_eps
        flows = ((r >= lo) & (r <= hi)) | ((r > hi) & (a < 0)) | ((r < lo) & (a > 0))
        d_policy = -(a * r) * flows.to(torch.float32)
        d_kl = 1.0 - torch.exp(ref - cur)
        zero = torch.zeros((), dtype=torch.float32, device=cur.device)
        g_loss = zero if g_loss is None else g_loss
        w_policy = g_loss + (zero if g_policy is None else g_policy)
        w_kl = ctx.beta * g_loss + (zero if g_kl is None else g_kl)
        grad = (w_policy * d_policy + w_kl * d_kl) * keep / count
        return grad, None, None, None, None, None, None


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
        mask = _bool_mask(completion_mask, cur.device)
        if mask.shape != cur.shape:
            raise ValueError("completion_mask must match the log-prob shape")
    if torch.is_grad_enabled() and cur.requires_grad:
        loss, policy, kl, ratio, k3 = _GrpoLossAutograd.apply(
            cur, old.detach(), ref.detach(), adv.detach(), mask, float(clip_eps), float(beta)
        )
        return GrpoLossOutput(loss, policy, kl, ratio.reshape(shape), k3.reshape(shape))
    out3, ratio, k3 = _C.grpo_ratio_kl_loss(cur, old, ref, adv, mask, clip_eps, beta)
    return GrpoLossOutput(out3[0], out3[1], out3[2], ratio.reshape(shape), k3.reshape(shape))


def group_advantages(
    rewards: torch.Tensor,
    *,
    samples_per_prompt: Optional[int] = None,
    group_boundaries=None,
    eps: float = 1e-6,
) -> torch.Tensor:
    """Per-sequence rewards normalised inside each generation group:
    ``(r - mean_g) / sqrt(max(E_g[r^2] - mean_g^2, eps^2))``, fp32, one value per sequence.

    Same arguments, checks and messages as ``NativeGRPOLossOp.group_advantages``
    (rl_engine/reference/loss/grpo_loss.py:53-84, 170-206). The group sums are plain
    reductions over each group's slice (no atomics), so the result is the same from run to run.
    """
    flat = rewards.reshape(-1).float()
    n = flat.numel()
    if (samples_per_prompt is not None) + (group_boundaries is not None) != 1:
        raise ValueError("Provide exactly one of samples_per_prompt or group_boundaries.")
    if samples_per_prompt is not None:
        if samples_per_prompt < 2:
            raise ValueError("samples_per_prompt must be at least 2 for group normalization.")
        if n % samples_per_prompt != 0:
            raise ValueError(f"num_sequences ({n}) must be divisible by samples_per_prompt ({samples_per_prompt}).")
        sizes = [int(samples_per_prompt)] * (n // int(samples_per_prompt))
    else:
        b = torch.as_tensor(group_boundaries, dtype=torch.long).cpu()
        if b.ndim != 1 or b.numel() < 2:
            raise ValueError("group_boundaries must be a 1D tensor of length num_groups + 1.")
        # Only the differences count, as in the reference (repeat_interleave over the sizes): group g is the
        # run of sizes[g] sequences after the groups before it, wherever the boundaries themselves start.
        sizes = [int(v) for v in (b[1:] - b[:-1]).tolist()]
        if sum(sizes) != n:
            raise ValueError(f"group sizes sum to {sum(sizes)} but there are {n} sequences.")
        if any(size < 1 for size in sizes):
            raise ValueError("each group must contain at least one sequence.")
    if n == 0:
        return flat.clone()

    def _normalise(g: torch.Tensor, size: int) -> torch.Tensor:  # g: [groups, size]
        mean = g.sum(dim=1, keepdim=True) / size
        var = (g * g).sum(dim=1, keepdim=True) / size - mean * mean
        return (g - mean) / var.clamp_min(eps**2).sqrt()

    if len(set(sizes)) == 1:
        return _normalise(flat.view(-1, sizes[0]), sizes[0]).reshape(-1)
    pieces, start = [], 0
    for size in sizes:
        pieces.append(_normalise(flat[start : start + size].view(1, size), size).reshape(-1))
        start += size
    return torch.cat(pieces)


def compute_policy_ratio(current_logps, old_logps, mask=None) -> torch.Tensor:
    """``exp(current - old)`` with masked entries set to zero."""
    zeros = torch.zeros(_as_2d(current_logps).size(0), dtype=torch.float32, device=current_logps.device)
    return grpo_ratio_kl_loss(current_logps, old_logps, current_logps, zeros, mask).ratio


def compute_reference_kl(current_logps, ref_logps, mask=None) -> torch.Tensor:
    """k3 estimator ``exp(d) - d - 1`` with ``d = ref - current``; masked entries zero."""
    zeros = torch.zeros(_as_2d(current_logps).size(0), dtype=torch.float32, device=current_logps.device)
    return grpo_ratio_kl_loss(current_logps, current_logps, ref_logps, zeros, mask).k3


__all__ = ["GrpoLossOutput", "compute_policy_ratio", "compute_reference_kl", "group_advantages", "grpo_ratio_kl_loss"]
