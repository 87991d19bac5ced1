"""Argument checking for the host-side facades, written as tables.

A facade states what it requires as rows ``(holds, exception type, message)`` and hands them to
:func:`enforce`, which raises for the first row that does not hold. The exception types and the
message texts are part of the interface the facades keep (callers and tests match on them); the
tables keep them in one place per entry point instead of a chain of ``if`` statements.

``holds`` and ``message`` may be zero-argument callables, evaluated only when the row is reached:
use that for a condition that is only meaningful once the rows before it have passed (a size that
needs a 2-D tensor, a device comparison that needs a tensor at all).
"""

from __future__ import annotations

from collections.abc import Callable, Iterable
from typing import Union

import torch

Lazy = Union[bool, Callable[[], bool]]
Text = Union[str, Callable[[], str]]
Rule = tuple[Lazy, type, Text]


def enforce(rules: Iterable[Rule]) -> None:
    """Raise ``exception(message)`` of the first rule whose condition does not hold."""
    for holds, exception, message in rules:
        if callable(holds):
            holds = holds()
        if not holds:
            raise exception(message() if callable(message) else message)


def assert_async_or_raise(condition: torch.Tensor, exception: type, message: str, host_message: str | None = None) -> None:
    """A value check on a 0-d boolean tensor: a device-side assertion for a GPU tensor (the call never
    waits for the host, so it can sit inside a captured graph), an ordinary exception for a CPU one."""
    if condition.is_cuda:
        torch._assert_async(condition, message)
    elif not bool(condition):
        raise exception(host_message or message)


def output_buffer_rules(out: torch.Tensor, shape: tuple[int, int], device: torch.device, what: str) -> list[Rule]:
    """Rules for a caller-owned bf16 ``[M, N]`` output with contiguous rows (``what`` prefixes the messages)."""
    return [
        (tuple(out.shape) == tuple(shape), ValueError, f"{what} output must have shape {tuple(shape)}, got {tuple(out.shape)}"),
        (out.dtype == torch.bfloat16, TypeError, f"{what} output must be BF16, got {out.dtype}"),
        (out.device == device, RuntimeError, f"{what} output must live on the input device"),
        (lambda: out.stride(1) == 1, ValueError, f"{what} output rows must be contiguous"),
        (not out.requires_grad, ValueError, f"{what} output buffer must not require gradients"),
    ]
