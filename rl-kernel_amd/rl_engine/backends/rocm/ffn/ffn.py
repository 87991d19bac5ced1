"""Bias-free gated FFN assembled from the deterministic gfx950 kernels.

The one-GPU share of rl_engine/backends/rocm/ffn/ffn.py of the reference: the packed
inference entry (:69-113, 303-330), the differentiable ``qwen3_ffn`` (:674-975, 976-1050)
and ``Qwen3FFNOp`` (:1073-1230). Tensor-, context- and sequence-parallel groups need
collectives, which this build does not have: a group with more than one rank is refused.

Forward:  gate_up = x @ W_gu^T -> SwiGLU -> @ W_down^T, every GEMM under the det_gemm
contract, so a token's output never depends on the batch it arrives in. Inference fuses the
activation into the gate/up GEMM; training keeps ``gate_up`` for the backward
(``swiglu_packed_backward``, two input-gradient and three weight-gradient GEMMs, the gate
and up input gradients added in bf16 as the reference does, ffn.py:960-975).
"""

from __future__ import annotations

from typing import Any

import torch
from torch import Tensor

from rl_engine import _C, _lib
from rl_engine._checks import enforce
from rl_engine.backends.rocm.gemm import swiglu_gemm
from rl_engine.backends.rocm.gemm.det_gemm import (
    det_gemm_linear,
    det_gemm_linear_input_gradient,
    det_gemm_linear_weight_gradient,
)

QWEN3_8B_HIDDEN_SIZE = 4096
QWEN3_8B_INTERMEDIATE_SIZE = 12288
BACKEND_ID = "rlkernel.ffn.qwen3.deterministic.hip_gfx950.v1"


def _single_rank(group: Any, name: str) -> None:
    if group is None:
        return
    dist = torch.distributed
    if dist.is_available() and dist.is_initialized() and dist.get_world_size(group=group) > 1:
        raise RuntimeError(f"{name}-parallel FFN needs a collective; this build runs on one GPU")


def _validate_ffn_inputs(rmsnorm_output, gate_weight, up_weight, down_weight, fused_gate_up_weight) -> None:
    """The checks, exception types and messages of the reference's _validate_ffn_inputs (ffn.py:585-640),
    written as one table per stage: argument types, ranks, shapes, then dtype and placement of every tensor."""
    named = [("rmsnorm_output", rmsnorm_output), ("gate_weight", gate_weight), ("up_weight", up_weight),
             ("down_weight", down_weight)]  # fmt: skip
    if fused_gate_up_weight is not None:
        named.append(("fused_gate_up_weight", fused_gate_up_weight))
    enforce((isinstance(t, Tensor), TypeError, f"{name} must be a torch.Tensor, got {type(t)!r}.") for name, t in named)
    enforce([
        (rmsnorm_output.dim() >= 1, ValueError, "rmsnorm_output must have at least one dimension."),
        (rmsnorm_output.numel() > 0, ValueError, "rmsnorm_output must contain at least one token."),
    ])  # fmt: skip
    enforce((t.dim() == 2, ValueError, f"{name} must be 2-D, got shape {tuple(t.shape)}.") for name, t in named[1:4])
    hidden, inter = rmsnorm_output.size(-1), gate_weight.size(0)
    wanted = {"gate_weight": (inter, hidden), "up_weight": (inter, hidden), "down_weight": (hidden, inter),
              "fused_gate_up_weight": (2 * inter, hidden)}  # fmt: skip
    enforce(
        (tuple(t.shape) == wanted[name], ValueError, f"{name} must have shape {wanted[name]}, got {tuple(t.shape)}.")
        for name, t in named[1:]
    )
    home = rmsnorm_output.device
    for name, t in named:
        enforce([
            (t.dtype == torch.bfloat16, TypeError, f"{name} must have dtype bfloat16, got {t.dtype}."),
            (t.is_cuda, RuntimeError, f"{name} must be on a CUDA/ROCm GPU device, got '{t.device}'."),
            (t.device == home, RuntimeError, f"all FFN inputs must be on {home}, got {name} on {t.device}."),
        ])  # fmt: skip


# ---------------------------------------------------------------------------
# Inference: packed weight, activation fused into the gate/up GEMM
# ---------------------------------------------------------------------------


def _packed_ffn(hidden_2d: Tensor, fused_gate_up_weight: Tensor, down_weight: Tensor, out: Tensor | None) -> Tensor:
    activated = swiglu_gemm.forward(hidden_2d, fused_gate_up_weight)
    return det_gemm_linear(activated, down_weight, out=out)


@torch.library.custom_op("rl_kernel::qwen3_ffn_packed_inference", mutates_args=())
def _qwen3_ffn_packed_inference(rmsnorm_output: Tensor, fused_gate_up_weight: Tensor, down_weight: Tensor) -> Tensor:
    """Graph-safe compute of the strict rollout FFN (no host sync; no workspace for M > 128 or M <= 16)."""
    shape = rmsnorm_output.shape
    hidden_2d = rmsnorm_output.reshape(-1, shape[-1]).contiguous()
    output = _packed_ffn(hidden_2d, fused_gate_up_weight, down_weight, None)
    return output.reshape(*shape[:-1], output.size(-1))


@_qwen3_ffn_packed_inference.register_fake
def _(rmsnorm_output, fused_gate_up_weight, down_weight):
    del fused_gate_up_weight
    return rmsnorm_output.new_empty((*rmsnorm_output.shape[:-1], down_weight.shape[0]))


@torch.library.custom_op("rl_kernel::qwen3_ffn_packed_inference_to_staging", mutates_args={"output"})
def _qwen3_ffn_packed_inference_to_staging(
    rmsnorm_output: Tensor, fused_gate_up_weight: Tensor, down_weight: Tensor, output: Tensor,
) -> None:
    """Same with the down projection written into a caller-owned staging buffer."""
    hidden_2d = rmsnorm_output.reshape(-1, rmsnorm_output.shape[-1]).contiguous()
    _packed_ffn(hidden_2d, fused_gate_up_weight, down_weight, output)


@_qwen3_ffn_packed_inference_to_staging.register_fake
def _(rmsnorm_output, fused_gate_up_weight, down_weight, output):
    return None


def qwen3_ffn_packed_inference(
    rmsnorm_output: Tensor, fused_gate_up_weight: Tensor, down_weight: Tensor, *, collective_handle: int = 0,
    tp_world_size: int = 1, collective: Any | None = None,
) -> Tensor:
    """Inference-only packed FFN entry (ffn.py:303-330 of the reference), one rank."""
    del collective_handle, collective
    if tp_world_size != 1:
        raise RuntimeError("packed rollout FFN with tensor parallelism needs a collective; this build runs on one GPU")
    operands = {"rmsnorm_output": rmsnorm_output, "fused_gate_up_weight": fused_gate_up_weight, "down_weight": down_weight}
    enforce(
        (t.dtype == torch.bfloat16, TypeError, f"{name} must have dtype bfloat16, got {t.dtype}.")
        for name, t in operands.items()
    )
    return torch.ops.rl_kernel.qwen3_ffn_packed_inference(rmsnorm_output, fused_gate_up_weight, down_weight)


# ---------------------------------------------------------------------------
# Training: differentiable FFN
# ---------------------------------------------------------------------------


class _DeterministicFFNFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rmsnorm_output, gate_weight, up_weight, down_weight, fused_gate_up_weight):
        shape = rmsnorm_output.shape
        x = rmsnorm_output.reshape(-1, shape[-1]).contiguous()
        packed = fused_gate_up_weight is not None
        if packed:
            gate_up = det_gemm_linear(x, fused_gate_up_weight)
            activated = _C.swiglu_packed_forward(gate_up)
            ctx.save_for_backward(x, gate_up, activated, gate_weight, up_weight, down_weight)
        else:
            gate = det_gemm_linear(x, gate_weight)
            up = det_gemm_linear(x, up_weight)
            activated = _C.swiglu_forward(gate, up)
            ctx.save_for_backward(x, gate, up, activated, gate_weight, up_weight, down_weight)
        output = det_gemm_linear(activated, down_weight)
        ctx.packed = packed
        ctx.input_shape = shape
        return output.reshape(*shape[:-1], output.size(-1))

    @staticmethod
    def backward(ctx, grad_output):
        if ctx.packed:
            x, gate_up, activated, gate_weight, up_weight, down_weight = ctx.saved_tensors
        else:
            x, gate, up, activated, gate_weight, up_weight, down_weight = ctx.saved_tensors
        grad_output = grad_output.reshape(-1, grad_output.size(-1)).to(torch.bfloat16).contiguous()
        grad_activated = det_gemm_linear_input_gradient(grad_output, down_weight)
        if ctx.packed:
            grad_gate, grad_up = _C.swiglu_packed_backward(grad_activated, gate_up)
        else:
            grad_gate, grad_up = _C.swiglu_backward(grad_activated, gate, up)
        need = ctx.needs_input_grad
        grad_down_weight = det_gemm_linear_weight_gradient(activated, grad_output) if need[3] else None
        grad_gate_weight = det_gemm_linear_weight_gradient(x, grad_gate) if need[1] else None
        grad_up_weight = det_gemm_linear_weight_gradient(x, grad_up) if need[2] else None
        grad_x = None
        if need[0]:
            grad_x = det_gemm_linear_input_gradient(grad_gate, gate_weight)
            grad_x.add_(det_gemm_linear_input_gradient(grad_up, up_weight))
            grad_x = grad_x.reshape(ctx.input_shape)
        return grad_x, grad_gate_weight, grad_up_weight, grad_down_weight, None


def qwen3_ffn(
    rmsnorm_output: Tensor, gate_weight: Tensor, up_weight: Tensor, down_weight: Tensor, *,
    fused_gate_up_weight: Tensor | None = None, tp_group: Any = None, cp_group: Any = None,
    sequence_parallel: bool = False, deterministic: bool | None = None, disable_split_k: bool | None = None,
) -> Tensor:
    """SiLU-gated FFN ``down(swiglu(gate(x), up(x)))`` with deterministic forward and backward.

    Signature of ``qwen3_ffn`` (ffn.py:976-1050 of the reference). ``fused_gate_up_weight``
    (``[2 I, H]`` = ``cat(gate_weight, up_weight)``) lets the forward run one GEMM while the
    gradients are still returned for the separate gate / up weights.
    """
    if not isinstance(sequence_parallel, bool):
        raise TypeError("sequence_parallel must be a bool.")
    for name, value in (("deterministic", deterministic), ("disable_split_k", disable_split_k)):
        if value is not None and not isinstance(value, bool):
            raise TypeError(f"{name} must be a bool or None.")
    if deterministic is False or (deterministic is None and disable_split_k is False):
        raise RuntimeError("this build has the deterministic FFN only (deterministic=False is not served)")
    if sequence_parallel:
        raise ValueError("sequence_parallel requires a tensor-parallel group.")
    _single_rank(tp_group, "tensor")
    _single_rank(cp_group, "context")
    _validate_ffn_inputs(rmsnorm_output, gate_weight, up_weight, down_weight, fused_gate_up_weight)
    _lib.load()
    return _DeterministicFFNFunction.apply(rmsnorm_output, gate_weight, up_weight, down_weight, fused_gate_up_weight)


class Qwen3FFNOp:
    """Operator object over :func:`qwen3_ffn` / :func:`qwen3_ffn_packed_inference`."""

    op_class = "ffn"
    is_batch_invariant = True
    backend_id = BACKEND_ID

    def __init__(self) -> None:
        _lib.load()

    def packed_inference(self, rmsnorm_output: Tensor, fused_gate_up_weight: Tensor, down_weight: Tensor, **kwargs):
        return qwen3_ffn_packed_inference(rmsnorm_output, fused_gate_up_weight, down_weight, **kwargs)

    def apply(self, rmsnorm_output, gate_weight, up_weight, down_weight, **kwargs) -> Tensor:
        return qwen3_ffn(rmsnorm_output, gate_weight, up_weight, down_weight, **kwargs)

    __call__ = apply


__all__ = ["BACKEND_ID", "Qwen3FFNOp", "qwen3_ffn", "qwen3_ffn_packed_inference"]
