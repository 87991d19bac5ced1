"""Fused linear-LogP on gfx950: lm_head GEMM -> fixed-order LSE -> target gather.

The function and class below keep the call contracts of the reference's strict
entry points for this op:

* ``hip_deterministic_linear_logp`` has the signature, validation, return
  convention and error types of ``triton_deterministic_linear_logp``
  (rl_engine/backends/shared/triton/logprob/linear_logp.py:496-521, 631-700);
* ``HipLinearLogpOp`` has the ``__call__`` / ``apply`` signature the runtime
  registry expects of a ``linear_logp`` op
  (rl_engine/reference/logprob/linear_logp.py:731-773).

Unlike the reference's ROCm route (bf16 logits written to HBM, then a tile-stats
scan, rl_engine/integrations/common/linear_logp.py:1083-1102) the logits stay in
registers and the target logit is the fp32 accumulator value.
"""

from __future__ import annotations

from typing import Any, Optional

import torch

from rl_engine import _C, _lib


def linear_logp_contract_version() -> str:
    return _lib.load().rlk_linear_logp_contract_id().decode()


def _prepare(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    target_ids: torch.Tensor,
    temperature: Optional[torch.Tensor],
    validate: bool,
):
    if hidden.device.type != "cuda":
        raise RuntimeError(f"deterministic HIP linear_logp requires a GPU tensor, got device '{hidden.device}'.")
    if hidden.dim() < 1:
        raise ValueError("hidden must have at least one dimension")
    if weight.dim() != 2 or weight.size(-1) != hidden.size(-1):
        raise ValueError(f"hidden dim {hidden.size(-1)} must match lm_head_weight dim {weight.size(-1)}")
    if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("deterministic HIP linear_logp requires BF16 hidden and lm_head_weight")
    # the usual call hands over what the kernel takes; only other layouts pay for a reshape or a copy
    hidden_2d = hidden if hidden.dim() == 2 and hidden.is_contiguous() else hidden.reshape(-1, hidden.size(-1)).contiguous()
    weight_c = weight if weight.is_contiguous() else weight.contiguous()
    if target_ids.dim() == 1 and target_ids.dtype == torch.long and target_ids.device == hidden_2d.device and target_ids.is_contiguous():
        target_1d = target_ids
    else:
        target_1d = target_ids.reshape(-1).to(device=hidden_2d.device, dtype=torch.long).contiguous()
    if target_1d.numel() != hidden_2d.size(0):
        raise ValueError("target_ids must have one id per hidden row")
    temp_arg = None
    if temperature is not None:
        temp_arg = torch.as_tensor(temperature).to(device=hidden_2d.device, dtype=torch.float32).reshape(-1)
        if temp_arg.numel() == 1:
            temp_arg = temp_arg.expand(hidden_2d.size(0)).contiguous()
        else:
            temp_arg = temp_arg.contiguous()
        if temp_arg.numel() != hidden_2d.size(0) or (validate and bool((temp_arg <= 0).any().item())):
            raise ValueError("temperature must be positive and scalar or per-token")
    return hidden_2d, weight_c, target_1d, temp_arg


def _requires_grad(*tensors: Optional[torch.Tensor]) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


class _HipLinearLogpAutograd(torch.autograd.Function):
    """Differentiable ``(logp, lse)``: forward and backward both on the HIP library.

    Mirrors ``_DetTritonLinearLogpAutograd``
    (rl_engine/backends/shared/triton/logprob/linear_logp.py:573-628): the backward
    recomputes the logits from the saved ``lse`` and returns gradients in the dtypes
    of ``hidden``, ``lm_head_weight`` and ``bias``; the clamp ``logp = min(., 0)`` is
    not differentiated.
    """

    @staticmethod
    def forward(ctx, hidden_2d, weight, bias, target_1d, temp_arg, real_vocab, vocab_start, config):
        bias_c = bias.contiguous() if bias is not None else None
        logp, lse = _C.fused_linear_logp(
            hidden_2d, weight, target_1d, bias_c, temp_arg, False, real_vocab,
            vocab_start_index=vocab_start, config=config,
        )  # fmt: skip
        ctx.save_for_backward(
            hidden_2d,
            weight,
            bias_c if bias_c is not None else hidden_2d.new_empty(0),
            target_1d,
            lse,
            temp_arg if temp_arg is not None else hidden_2d.new_empty(0),
        )
        ctx.has_bias = bias is not None
        ctx.bias_dtype = bias.dtype if bias is not None else None
        ctx.real_vocab = real_vocab
        ctx.vocab_start = vocab_start
        ctx.config = config
        ctx.mark_non_differentiable(target_1d)
        return logp, lse

    @staticmethod
    def backward(ctx, grad_logp, grad_lse):
        if grad_logp is None and grad_lse is None:
            return (None,) * 8
        hidden_2d, weight, bias, target_1d, lse, temp = ctx.saved_tensors
        need_h, need_w, need_b = ctx.needs_input_grad[0], ctx.needs_input_grad[1], ctx.needs_input_grad[2]
        with torch.no_grad():
            grad_hidden, grad_weight, grad_bias = _C.fused_linear_logp_bwd(
                hidden_2d,
                weight,
                target_1d,
                lse,
                grad_logp,
                grad_lse,
                bias if ctx.has_bias else None,
                temp if temp.numel() else None,
                ctx.real_vocab,
                vocab_start_index=ctx.vocab_start,
                need_grad_hidden=need_h,
                need_grad_weight=need_w,
                need_grad_bias=bool(ctx.has_bias and need_b),
                config=ctx.config,
            )
        if grad_bias is not None:
            grad_bias = grad_bias.to(ctx.bias_dtype)
        return grad_hidden, grad_weight, grad_bias, None, None, None, None, None


def hip_deterministic_linear_logp(
    hidden: torch.Tensor,
    lm_head_weight: torch.Tensor,
    target_ids: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    *,
    temperature: Optional[torch.Tensor] = None,
    return_logits: bool = False,
    real_vocab_size: int = -1,
    vocab_start_index: int = 0,
    config: str | int = 0,
    validate: bool = False,
):
    """Strict entry: returns fp32 ``(logp, lse)`` (plus logits on request); differentiable
    with respect to ``hidden``, ``lm_head_weight`` and ``bias``.

    Two callers with byte-identical ``hidden`` rows, ``lm_head_weight``,
    ``target_ids`` and ``temperature`` receive bitwise-identical results for a
    row whatever batch it arrives in. ``real_vocab_size`` masks padded vocabulary
    lanes out of the LSE; ``-1`` disables masking.

    Values of ``target_ids`` and ``temperature``: the reference's strict entry reads them back from the device
    before it launches and raises ``ValueError`` for an id outside the real vocabulary or a temperature that is
    not positive (rl_engine/backends/shared/triton/logprob/linear_logp.py:516-517, 666-672). That read-back is a
    host synchronisation on every call, so here it is opt-in: ``validate=True`` does exactly that; by default
    nothing is read back (the call can be captured in a HIP graph) and the kernel marks such a row instead -
    ``logp`` is NaN for an id outside ``[vocab_start_index, vocab_start_index + real_vocab_size)``, ``logp`` and
    ``lse`` are NaN for a temperature that is not a positive number.
    """
    hidden_2d, weight, target_1d, temp_arg = _prepare(hidden, lm_head_weight, target_ids, temperature, bool(validate))
    lead_shape = hidden.shape[:-1]
    real_vocab = weight.size(0) if int(real_vocab_size) < 0 else int(real_vocab_size)
    if not 0 < real_vocab <= weight.size(0):
        raise ValueError(f"real_vocab_size must be in [1, {weight.size(0)}], got {real_vocab_size}")
    if validate and target_1d.numel():
        lo = int(vocab_start_index)
        bad = (target_1d < lo) | (target_1d >= lo + real_vocab)
        if bool(bad.any().item()):
            raise ValueError(
                f"target_ids must be in the real vocabulary [{lo}, {lo + real_vocab}), "
                f"got [{int(target_1d.min().item())}, {int(target_1d.max().item())}]"
            )
    if isinstance(config, str):
        config = _lib.LOGP_CONFIGS[config]
    if _requires_grad(hidden, lm_head_weight, bias):
        if return_logits:
            raise RuntimeError("return_logits=True is inference-only: call it under torch.no_grad()")
        logp, lse = _HipLinearLogpAutograd.apply(
            hidden_2d, weight, bias, target_1d, temp_arg, real_vocab, int(vocab_start_index), int(config)
        )
        return logp.reshape(lead_shape), lse.reshape(lead_shape)
    outputs = _C.fused_linear_logp(
        hidden_2d,
        weight,
        target_1d,
        bias.contiguous() if bias is not None else None,
        temp_arg,
        return_logits,
        real_vocab,
        vocab_start_index=int(vocab_start_index),
        config=int(config),
    )
    if hidden.dim() == 2:
        logp, lse = outputs[0], outputs[1]
    else:
        logp, lse = outputs[0].reshape(lead_shape), outputs[1].reshape(lead_shape)
    if return_logits:
        return logp, lse, outputs[2].reshape(*lead_shape, weight.size(0))
    return logp, lse


class HipLinearLogpOp:
    """``linear_logp`` operator object (registry shape) on the fused HIP kernel."""

    contract_version = property(lambda self: linear_logp_contract_version())

    def __init__(self) -> None:
        _lib.load()
        self.has_hardware_op = True

    def __call__(
        self,
        hidden: torch.Tensor,
        lm_head_weight: torch.Tensor,
        target_ids: torch.Tensor,
        bias: Optional[torch.Tensor] = None,
        *,
        tp_group: Any = None,
        vocab_start_index: int = 0,
        global_vocab_size: Optional[int] = None,
    ) -> torch.Tensor:
        return self.apply(
            hidden,
            lm_head_weight,
            target_ids,
            bias,
            tp_group=tp_group,
            vocab_start_index=vocab_start_index,
            global_vocab_size=global_vocab_size,
        )

    def apply(
        self,
        hidden: torch.Tensor,
        lm_head_weight: torch.Tensor,
        target_ids: torch.Tensor,
        bias: Optional[torch.Tensor] = None,
        *,
        tp_group: Any = None,
        vocab_start_index: int = 0,
        global_vocab_size: Optional[int] = None,
    ) -> torch.Tensor:
        """Selected-token log-prob ``z[t] - logsumexp(z)`` in float32, shape ``hidden.shape[:-1]``."""
        if hidden.shape[:-1] != target_ids.shape:
            raise ValueError(
                f"hidden leading shape {tuple(hidden.shape[:-1])} must match "
                f"target_ids shape {tuple(target_ids.shape)}"
            )
        if lm_head_weight.size(-1) != hidden.size(-1):
            raise ValueError(
                f"hidden dim {hidden.size(-1)} must match lm_head_weight dim {lm_head_weight.size(-1)}"
            )
        sharded = tp_group is not None and (
            int(vocab_start_index) != 0
            or (global_vocab_size is not None and int(global_vocab_size) != lm_head_weight.size(0))
        )
        if sharded:
            raise RuntimeError(
                "vocabulary-parallel linear_logp needs a collective; this build runs on one GPU "
                "with the full vocabulary"
            )
        logp, _ = hip_deterministic_linear_logp(hidden, lm_head_weight, target_ids, bias)
        return logp


LinearLogpOp = HipLinearLogpOp

__all__ = [
    "HipLinearLogpOp",
    "LinearLogpOp",
    "hip_deterministic_linear_logp",
    "linear_logp_contract_version",
]
