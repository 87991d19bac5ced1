"""Selected-token log-probabilities from materialised logits on gfx950.

The one-GPU share of the reference's ROCm vocab-parallel logprob op
(rl_engine/backends/rocm/logprob/vocab_parallel_logp.py:308-477) and of
``LinearLogpWrapper.from_local_logits``
(rl_engine/integrations/common/linear_logp.py:750-815, 817-923): the sampler path
that reuses LM-head logits instead of running the GEMM again. Tile statistics,
the ascending tile merge and the target gather run in one pass over the logits;
a temperature scales them by its reciprocal in registers (the scaling of the fused
linear-LogP), so no fp32 copy of the logits is made.

The cross-rank exchange of the reference (an all-gather of per-tile partials) is
not part of this build: ``tp_group`` must describe a single rank.
"""

from __future__ import annotations

from typing import Any, Optional

import torch

from rl_engine import _C, _lib

BACKEND_ID = "rlkernel.vocab_parallel_logp.hip_gfx950.v1"
DEFAULT_NUM_VOCAB_TILES = 64  # rl_engine/reference/logprob/vocab_parallel_logp.py:52


def merge_tile_partials(m_all: torch.Tensor, s_all: torch.Tensor) -> torch.Tensor:
    """``lse`` from per-tile ``(max, sumexp)`` of shape ``[n, tiles]``.

    The formula of ``_merge_tile_partials``
    (rl_engine/reference/logprob/vocab_parallel_logp.py:355-363), kept for callers
    that hold tile statistics; :func:`hip_deterministic_logp_from_logits` merges on
    the GPU in ascending tile order instead.
    """
    big = m_all.max(dim=1).values
    finite = big > float("-inf")
    safe = torch.where(finite, big, torch.zeros_like(big))
    terms = s_all * (m_all - safe.unsqueeze(1)).exp()
    return big + terms.sum(dim=1).log()


def _temperature_rows(temperature, rows: int, device) -> Optional[torch.Tensor]:
    if temperature is None:
        return None
    if not isinstance(temperature, torch.Tensor):
        if float(temperature) == 1.0:
            return None
        temperature = torch.tensor(float(temperature))
    temp = temperature.to(device=device, dtype=torch.float32).reshape(-1)
    if temp.numel() == 1:
        temp = temp.expand(rows)
    if temp.numel() != rows or bool((temp <= 0).any().item()):
        raise ValueError("temperature must be positive and scalar or per-token")
    return temp.contiguous()


class _HipLogpFromLogits(torch.autograd.Function):
    """``(logp, lse)`` of materialised logits; the backward writes d(logits) in their dtype
    (_RocmVocabParallelLogprobFunction, vocab_parallel_logp.py:308-383 of the reference)."""

    @staticmethod
    def forward(ctx, logits, target_1d, temp, vocab_start, real_vocab, num_tiles):
        logp, lse = _C.hip_deterministic_logp_from_logits(
            logits, target_1d, vocab_start, real_vocab, num_tiles, temperature=temp
        )
        ctx.save_for_backward(logits, lse, target_1d, temp if temp is not None else logits.new_empty(0))
        ctx.vocab_start = vocab_start
        ctx.real_vocab = real_vocab
        ctx.set_materialize_grads(False)
        return logp, lse

    @staticmethod
    def backward(ctx, grad_logp, grad_lse):
        if not ctx.needs_input_grad[0] or (grad_logp is None and grad_lse is None):
            return None, None, None, None, None, None
        logits, lse, target_1d, temp = ctx.saved_tensors
        rows, local_vocab = logits.shape
        start = ctx.vocab_start
        if grad_logp is not None:
            coef_logp = grad_logp.reshape(-1).float().contiguous()
            owns = (target_1d >= start) & (target_1d < start + local_vocab)
            target_local = torch.where(owns, target_1d - start, torch.full_like(target_1d, -1)).contiguous()
        else:
            coef_logp = lse.new_zeros((rows,))
            target_local = torch.full((rows,), -1, dtype=torch.long, device=logits.device)
        has_lse_grad = grad_lse is not None
        coef_lse = grad_lse.reshape(-1).float().contiguous() if has_lse_grad else lse.new_zeros((rows,))
        grad = _C.hip_deterministic_logp_backward(
            logits, lse.contiguous(), coef_logp, coef_lse, target_local, start, ctx.real_vocab, has_lse_grad,
            temperature=temp if temp.numel() else None,
        )  # fmt: skip
        return grad, None, None, None, None, None


def hip_deterministic_logp_from_logits(
    local_logits: torch.Tensor,
    target_ids: torch.Tensor,
    *,
    vocab_start_index: int = 0,
    real_vocab_size: Optional[int] = None,
    temperature: float | torch.Tensor | None = None,
    num_vocab_tiles: int = DEFAULT_NUM_VOCAB_TILES,
    tp_group: Any = None,
):
    """fp32 ``(logp, lse)`` for ``local_logits [rows, V]`` (bf16 / fp16 / fp32) and global
    ``target_ids``; a row's result never depends on the rest of the batch.

    Validation follows ``LinearLogpWrapper.from_local_logits``
    (rl_engine/integrations/common/linear_logp.py:833-858).
    """
    if local_logits.ndim != 2 or local_logits.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise TypeError("strict reused LM-head logits must be 2-D bf16/fp16/fp32")
    if not local_logits.is_cuda:
        raise RuntimeError("strict reused LM-head logits require CUDA/ROCm")
    if target_ids.device != local_logits.device:
        raise ValueError("linear_logp target_ids must share the logits device")
    if tp_group is not None and torch.distributed.is_initialized() and torch.distributed.get_world_size(tp_group) > 1:
        raise RuntimeError("vocabulary-parallel logp needs a collective; this build runs on one GPU")
    rows, local_vocab = local_logits.shape
    real = local_vocab + int(vocab_start_index) if real_vocab_size is None else int(real_vocab_size)
    if not 0 < real <= int(vocab_start_index) + local_vocab:
        raise ValueError("real_vocab_size must be within the padded global vocabulary")
    if local_vocab % int(num_vocab_tiles) != 0:
        raise ValueError(f"local vocabulary {local_vocab} must be divisible by num_vocab_tiles={num_vocab_tiles}")
    target_1d = target_ids.reshape(-1).to(dtype=torch.long)
    if target_1d.numel() != rows:
        raise ValueError("target_ids must have one id per logits row")
    if rows and bool(((target_1d < 0) | (target_1d >= real)).any().item()):
        raise ValueError(f"target_ids must be in the real vocabulary [0, {real})")
    temp = _temperature_rows(temperature, rows, local_logits.device)
    logp, lse = _HipLogpFromLogits.apply(
        local_logits, target_1d, temp, int(vocab_start_index), real, int(num_vocab_tiles)
    )
    return logp.reshape(target_ids.shape), lse.reshape(target_ids.shape)


class RocmVocabParallelLogprobOp:
    """Operator object over :func:`hip_deterministic_logp_from_logits` (one rank)."""

    op_class = "logprob"
    is_batch_invariant = True
    backend_id = BACKEND_ID

    def __init__(self) -> None:
        _lib.load()

    def apply(
        self,
        local_logits: torch.Tensor,
        target_ids: torch.Tensor,
        *,
        vocab_start_index: int = 0,
        real_vocab_size: Optional[int] = None,
        temperature: float | torch.Tensor | None = None,
        tp_group: Any = None,
        num_vocab_tiles: int = DEFAULT_NUM_VOCAB_TILES,
    ) -> tuple[torch.Tensor, torch.Tensor]:
        return hip_deterministic_logp_from_logits(
            local_logits,
            target_ids,
            vocab_start_index=vocab_start_index,
            real_vocab_size=real_vocab_size,
            temperature=temperature,
            num_vocab_tiles=num_vocab_tiles,
            tp_group=tp_group,
        )

    __call__ = apply


__all__ = [
    "BACKEND_ID",
    "DEFAULT_NUM_VOCAB_TILES",
    "RocmVocabParallelLogprobOp",
    "hip_deterministic_logp_from_logits",
    "merge_tile_partials",
]
