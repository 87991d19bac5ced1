"""Strict deterministic GEMM facade for ROCm, gfx950 build.

Public names, argument meaning and error behaviour follow the reference facade
(rl_engine/backends/rocm/gemm/det_gemm.py:32-105, 178-197, 411-465, 491-593) and its MFMA
host layer (rl_engine/backends/rocm/gemm/mfma_gemm.py:277-458). Two contracts, both HIP
kernels of librlk_gfx950.so, selected by ``RL_KERNEL_DET_GEMM_BACKEND`` as in the
reference; neither ever falls back.

``hip_mfma`` (default; the reference's ``triton_mfma`` role): bf16 operands, one fp32
accumulator per output element updated by ascending 32-wide MFMA steps over the whole K
range, one rounding to bf16. A row's result does not depend on how many other rows share
the call.

``hip_tree`` (the reference's ``triton_tree`` role): fp32 scalar-FMA leaves of at most 32 K
values rounded to bf16, combined by the bf16 midpoint tree over K. Batch invariant as well,
and invariant to the tensor-parallel degree of a K-sharded layer; about 20 times slower.
"""

from __future__ import annotations

import os
from collections.abc import Callable, Iterable
from threading import Lock

import torch

from rl_engine import _C, _lib

_BACKEND_ENV = "RL_KERNEL_DET_GEMM_BACKEND"
_AUTO_BACKEND = "auto"
_HIP_BACKEND = "hip_mfma"
_TREE_BACKEND = "hip_tree"
# Names the reference accepts (rl_engine/backends/rocm/gemm/det_gemm.py:33-48) select the
# contract that plays the same role here; "auto" is the MFMA contract on gfx950.
_BACKEND_ALIASES = {
    "rocm": _TREE_BACKEND,
    "triton": _TREE_BACKEND,
    "tree": _TREE_BACKEND,
    "triton_tree": _TREE_BACKEND,
    "mfma": _HIP_BACKEND,
    "triton_mfma": _HIP_BACKEND,
}
_ROUTE_REPORTED = False
_ROUTE_REPORT_LOCK = Lock()
_WEIGHT_TRANSPOSE_CACHE: dict[tuple[int, str, tuple[int, ...], torch.dtype], tuple[int | None, torch.Tensor]] = {}
_WEIGHT_TRANSPOSE_CACHE_LIMIT = 256


def _resolve_backend_request(value: str) -> str:
    value = value.strip().lower()
    value = _BACKEND_ALIASES.get(value, value)
    if value not in {_AUTO_BACKEND, _HIP_BACKEND, _TREE_BACKEND}:
        raise RuntimeError(
            f"{_BACKEND_ENV} must be '{_AUTO_BACKEND}', '{_TREE_BACKEND}' or '{_HIP_BACKEND}' "
            f"on the gfx950 build, got {value!r}"
        )
    return value


def _requested_backend() -> str:
    return _resolve_backend_request(os.getenv(_BACKEND_ENV, _AUTO_BACKEND))


_REQUESTED_BACKEND = _requested_backend()


def det_gemm_backend() -> str:
    """Name of the strict GEMM implementation in use."""
    return _TREE_BACKEND if _REQUESTED_BACKEND == _TREE_BACKEND else _HIP_BACKEND


def _use_tree() -> bool:
    return det_gemm_backend() == _TREE_BACKEND


def det_gemm_fallback_reason() -> str | None:
    return None


def det_gemm_backend_id() -> str:
    """Arithmetic-contract id reported in provenance records."""
    lib = _lib.load()
    return (lib.rlk_det_gemm_tree_contract_id() if _use_tree() else lib.rlk_contract_id()).decode()


def _report_strict_route_once() -> None:
    global _ROUTE_REPORTED
    if os.getenv("RL_KERNEL_ROUTE_REPORT", "").strip().lower() not in {"1", "true", "yes", "on"}:
        return
    with _ROUTE_REPORT_LOCK:
        if _ROUTE_REPORTED:
            return
        _ROUTE_REPORTED = True
    print(
        f"[RL-Kernel][route] mode={os.getenv('RL_KERNEL_MODE', 'strict')} module=gemm "
        f"requested={_REQUESTED_BACKEND} actual={det_gemm_backend_id()} fallback=false",
        flush=True,
    )


# ---------------------------------------------------------------------------
# Core strided GEMM with the reference's validation
# ---------------------------------------------------------------------------


def _validate_operands(a: torch.Tensor, b: torch.Tensor) -> None:
    if a.dim() != 2 or b.dim() != 2:
        raise ValueError("MFMA GEMM expects two 2-D tensors")
    if a.size(1) != b.size(0):
        raise ValueError(f"MFMA GEMM K mismatch: {a.size(1)} and {b.size(0)}")
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise TypeError("MFMA GEMM requires BF16 inputs")
    if not a.is_cuda or not b.is_cuda or a.device != b.device:
        raise RuntimeError("MFMA GEMM inputs must share one ROCm device")
    for name, tensor in (("a", a), ("b", b)):
        if min(tensor.stride()) < 0:
            raise ValueError(f"MFMA GEMM operand {name} must not use negative strides")
        if tensor.stride(0) != 1 and tensor.stride(1) != 1 and tensor.numel() > 1:
            raise ValueError(f"MFMA GEMM operand {name} needs one unit-stride dimension")


def mfma_gemm(
    a: torch.Tensor,
    b: torch.Tensor,
    *,
    out: torch.Tensor | None = None,
    config: str | int | None = None,
) -> torch.Tensor:
    """``a[M,K] @ b[K,N]`` in bf16 under the pinned MFMA contract.

    Both operands may be strided views (``weight.t()`` of a native ``[N,K]``
    weight is the fast layout). ``out`` may be a caller-owned bf16 ``[M,N]``
    buffer with contiguous rows, for instance a narrowed staging view.
    ``config`` names a tile configuration; it never changes a result bit.
    """
    _validate_operands(a, b)
    m_size, k_size = a.shape
    n_size = b.size(1)
    if out is None:
        out = torch.empty((m_size, n_size), dtype=torch.bfloat16, device=a.device)
    else:
        if tuple(out.shape) != (m_size, n_size):
            raise ValueError(f"MFMA GEMM output must have shape {(m_size, n_size)}, got {tuple(out.shape)}")
        if out.dtype != torch.bfloat16:
            raise TypeError(f"MFMA GEMM output must be BF16, got {out.dtype}")
        if out.device != a.device:
            raise RuntimeError("MFMA GEMM output must live on the input device")
        if out.stride(1) != 1:
            raise ValueError("MFMA GEMM output rows must be contiguous")
        if out.requires_grad:
            raise ValueError("MFMA GEMM output buffer must not require gradients")
    if m_size == 0 or n_size == 0:
        return out
    if isinstance(config, str):
        config = _lib.GEMM_CONFIGS[config]
    _C.gemm_strided(a, b, out, config=int(config or 0))
    return out


def tree_gemm(a: torch.Tensor, b: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """``a[M,K] @ b[K,N]`` in bf16 under the k-tree contract (any strided views).

    Equals the specification the reference's tests evaluate
    (tests/ops/gemm/test_det_gemm.py:156-168) bit for bit; a contiguous half of K is
    exactly one child of the root, so K-sharded partial results combined by bf16
    adds in a balanced rank tree reproduce the unsharded result.
    """
    _validate_operands(a, b)
    m_size, n_size = a.size(0), b.size(1)
    if out is None:
        out = torch.empty((m_size, n_size), dtype=torch.bfloat16, device=a.device)
    else:
        if tuple(out.shape) != (m_size, n_size):
            raise ValueError(f"MFMA GEMM output must have shape {(m_size, n_size)}, got {tuple(out.shape)}")
        if out.dtype != torch.bfloat16:
            raise TypeError(f"MFMA GEMM output must be BF16, got {out.dtype}")
        if out.device != a.device:
            raise RuntimeError("MFMA GEMM output must live on the input device")
        if out.stride(1) != 1:
            raise ValueError("MFMA GEMM output rows must be contiguous")
        if out.requires_grad:
            raise ValueError("MFMA GEMM output buffer must not require gradients")
    if m_size == 0 or n_size == 0:
        return out
    return _C.gemm_tree_strided(a, b, out)


def _strict_gemm(a: torch.Tensor, b: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """``a @ b`` under the contract selected at import."""
    if _use_tree():
        return tree_gemm(a, b, out=out)
    return mfma_gemm(a, b, out=out)


def _reduction_major(tensor: torch.Tensor) -> torch.Tensor:
    """``tensor.t()`` for a GEMM that reduces over ``tensor``'s rows: the plain view when
    the library's K-major loader can take it, else a value-preserving copy."""
    return _C._reduction_major(tensor)


def mfma_linear(a: torch.Tensor, weight: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """``a @ weight.T`` for a native ``[N,K]`` weight, no transpose copy."""
    return _strict_gemm(a, weight.t(), out=out)


def mfma_linear_input_gradient(grad_output: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``dX = dY @ W`` with ``W`` in native ``[N,K]`` layout."""
    if _use_tree():
        return tree_gemm(grad_output, weight)
    # The reduction runs over N, the slow axis of W: a K-major operand of the kernel.
    return mfma_gemm(grad_output, _reduction_major(weight).t())


def mfma_linear_weight_gradient(a: torch.Tensor, grad_output: torch.Tensor) -> torch.Tensor:
    """``dW = dY.T @ X`` returned in native ``[N,K]`` layout."""
    if _use_tree():
        return tree_gemm(grad_output.t(), a)
    return mfma_gemm(_reduction_major(grad_output), _reduction_major(a).t())


# ---------------------------------------------------------------------------
# Weight-transpose cache (inference only)
# ---------------------------------------------------------------------------


def _tensor_version(tensor: torch.Tensor) -> int | None:
    try:
        return int(tensor._version)
    except RuntimeError:  # inference tensors carry no version counter
        return None


def _cache_key(weight: torch.Tensor):
    return (weight.data_ptr(), str(weight.device), tuple(weight.shape), weight.dtype)


@torch.inference_mode()
def refresh_cached_weight_transposes(weights: Iterable[object]) -> int:
    """Re-copy cached ``[K,N]`` transposes after an in-place weight update.

    Same role as the reference function of this name
    (rl_engine/backends/rocm/gemm/det_gemm.py:143-159): the buffers keep their
    addresses so HIP graphs captured against them stay valid.
    """
    refreshed = 0
    for weight in weights:
        if not isinstance(weight, torch.Tensor) or weight.ndim != 2:
            continue
        cached = _WEIGHT_TRANSPOSE_CACHE.get(_cache_key(weight))
        if cached is None:
            continue
        cached[1].copy_(weight.t())
        _WEIGHT_TRANSPOSE_CACHE[_cache_key(weight)] = (_tensor_version(weight), cached[1])
        refreshed += 1
    return refreshed


def prepare_det_gemm_linear_weight(weight: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """Materialise a stable contiguous ``[K,N]`` inference weight from ``[N,K]``.

    Checks and error types follow the reference
    (rl_engine/backends/rocm/gemm/det_gemm.py:345-408). The caller owns freshness.
    """
    if weight.dim() != 2:
        raise ValueError("prepared deterministic linear weights must be 2-D")
    if weight.dtype != torch.bfloat16:
        raise TypeError("prepared deterministic linear weights must be BF16")
    if not weight.is_cuda:
        raise RuntimeError("prepared deterministic linear weights must be on ROCm")
    if not weight.is_contiguous():
        raise ValueError("source deterministic linear weights must be contiguous")
    expected_shape = (weight.size(1), weight.size(0))
    if out is None:
        with torch.inference_mode(False), torch.no_grad():
            out = torch.empty(expected_shape, dtype=weight.dtype, device=weight.device)
    else:
        if tuple(out.shape) != expected_shape:
            raise ValueError(
                f"prepared deterministic linear weight must have shape {expected_shape}, got {tuple(out.shape)}"
            )
        if out.dtype != weight.dtype:
            raise TypeError("prepared deterministic linear weight dtype must match its source")
        if out.device != weight.device:
            raise RuntimeError("prepared deterministic linear weight device must match its source")
        if not out.is_contiguous():
            raise ValueError("prepared deterministic linear weight must be contiguous")
        if out.requires_grad:
            raise ValueError("prepared deterministic linear weight must not require gradients")
        if torch._C._overlaps(out, weight):
            raise ValueError("prepared deterministic linear weight must not alias its source")
    with torch.no_grad():
        out.copy_(weight.t())
        cached = _WEIGHT_TRANSPOSE_CACHE.get(_cache_key(weight))
        if cached is not None:
            if cached[1] is not out:
                cached[1].copy_(weight.t())
            _WEIGHT_TRANSPOSE_CACHE[_cache_key(weight)] = (_tensor_version(weight), cached[1])
    return out


# ---------------------------------------------------------------------------
# Linear entry points
# ---------------------------------------------------------------------------


def det_gemm_linear(
    a: torch.Tensor,
    weight: torch.Tensor,
    *,
    native_op: Callable[[torch.Tensor, torch.Tensor], torch.Tensor] | None = None,
    out: torch.Tensor | None = None,
    inference_schedule: bool = False,
) -> torch.Tensor:
    """Apply a native ``[N,K]`` weight: ``a @ weight.T``."""
    del native_op, inference_schedule
    return mfma_linear(a, weight, out=out)


def det_gemm_linear_prepared(a: torch.Tensor, weight_t: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """Apply a lifecycle-managed contiguous ``[K,N]`` inference weight."""
    if torch.is_grad_enabled() and (a.requires_grad or weight_t.requires_grad):
        raise RuntimeError("prepared deterministic linear GEMM is inference-only")
    if not weight_t.is_contiguous():
        raise ValueError("prepared deterministic linear weight must be contiguous")
    if out is not None and (torch._C._overlaps(out, a) or torch._C._overlaps(out, weight_t)):
        raise ValueError("prepared deterministic linear output must not alias its inputs")
    return _strict_gemm(a, weight_t, out=out)


def det_gemm_linear_input_gradient(
    grad_output: torch.Tensor,
    weight: torch.Tensor,
    *,
    native_op: Callable[[torch.Tensor, torch.Tensor], torch.Tensor] | None = None,
) -> torch.Tensor:
    """``dX = dY @ weight``."""
    del native_op
    return mfma_linear_input_gradient(grad_output, weight)


def det_gemm_linear_weight_gradient(
    a: torch.Tensor,
    grad_output: torch.Tensor,
    *,
    native_op: Callable[[torch.Tensor, torch.Tensor], torch.Tensor] | None = None,
) -> torch.Tensor:
    """``dWeight = dY.T @ X`` in native ``[N,K]`` layout."""
    del native_op
    return mfma_linear_weight_gradient(a, grad_output)


@torch.library.custom_op("rl_kernel::rocm_det_gemm_linear_inference", mutates_args=())
def _det_gemm_linear_inference(a: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    return det_gemm_linear(a, weight, inference_schedule=True)


@_det_gemm_linear_inference.register_fake
def _det_gemm_linear_inference_fake(a: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    return a.new_empty((a.shape[0], weight.shape[0]))


@torch.library.custom_op("rl_kernel::rocm_det_gemm_linear_inference_out", mutates_args={"out"})
def _det_gemm_linear_inference_out(a: torch.Tensor, weight: torch.Tensor, out: torch.Tensor) -> None:
    det_gemm_linear(a, weight, out=out, inference_schedule=True)


@_det_gemm_linear_inference_out.register_fake
def _det_gemm_linear_inference_out_fake(a: torch.Tensor, weight: torch.Tensor, out: torch.Tensor) -> None:
    del a, weight, out


def _as_bf16_grad(grad_out: torch.Tensor) -> torch.Tensor:
    if grad_out.dtype != torch.bfloat16:
        grad_out = grad_out.to(torch.bfloat16)
    if grad_out.stride(1) != 1 and grad_out.stride(0) != 1:
        grad_out = grad_out.contiguous()
    return grad_out


class MfmaLinearFn(torch.autograd.Function):
    """``a @ weight.T`` with deterministic dgrad / wgrad."""

    @staticmethod
    def forward(ctx, a: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
        ctx.save_for_backward(a, weight)
        return mfma_linear(a, weight)

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        a, weight = ctx.saved_tensors
        grad_out = _as_bf16_grad(grad_out)
        da = mfma_linear_input_gradient(grad_out, weight) if ctx.needs_input_grad[0] else None
        dw = mfma_linear_weight_gradient(a, grad_out) if ctx.needs_input_grad[1] else None
        return da, dw


class MfmaGemmFn(torch.autograd.Function):
    """``a @ b`` with deterministic gradients for both operands."""

    @staticmethod
    def forward(ctx, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        ctx.save_for_backward(a, b)
        return _strict_gemm(a, b)

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        a, b = ctx.saved_tensors
        grad_out = _as_bf16_grad(grad_out)
        if _use_tree():
            da = tree_gemm(grad_out, b.t()) if ctx.needs_input_grad[0] else None
            db = tree_gemm(a.t(), grad_out) if ctx.needs_input_grad[1] else None
            return da, db
        da = mfma_gemm(grad_out, b.t()) if ctx.needs_input_grad[0] else None
        db = mfma_gemm(_reduction_major(a), _reduction_major(grad_out).t()) if ctx.needs_input_grad[1] else None
        return da, db


class RocmDetGemmOp:
    """Batch-invariant deterministic GEMM backed by the gfx950 HIP kernel."""

    def __init__(self):
        _lib.load()
        self.op = self
        self.has_hardware_op = True
        _report_strict_route_once()

    def __call__(self, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        assert a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16, "BF16 only"
        assert a.is_cuda and b.is_cuda, "Inputs must be on ROCm device"
        return deterministic_gemm(a, b)

    def linear(self, a: torch.Tensor, weight: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
        """Apply a native ``[N,K]`` linear weight."""
        assert a.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16, "BF16 only"
        assert a.is_cuda and weight.is_cuda, "Inputs must be on ROCm device"
        a = a.contiguous()
        weight = weight.contiguous()
        if out is not None:
            if torch.is_grad_enabled() and (a.requires_grad or weight.requires_grad):
                raise RuntimeError("direct-output deterministic GEMM is inference-only")
            _det_gemm_linear_inference_out(a, weight, out)
            return out
        if not torch.is_grad_enabled() or not (a.requires_grad or weight.requires_grad):
            return _det_gemm_linear_inference(a, weight)
        return MfmaLinearFn.apply(a, weight)

    def linear_prepared(self, a: torch.Tensor, weight_t: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
        """Apply a post-load prepared ``[K,N]`` weight."""
        assert a.dtype == torch.bfloat16 and weight_t.dtype == torch.bfloat16, "BF16 only"
        assert a.is_cuda and weight_t.is_cuda, "Inputs must be on ROCm device"
        return det_gemm_linear_prepared(a.contiguous(), weight_t, out=out)

    def forward_fp32(self, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        """The fp32 accumulator of ``a @ b`` stored without the bf16 rounding."""
        assert a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16, "BF16 only"
        assert a.is_cuda and b.is_cuda, "Inputs must be on ROCm device"
        return _C.det_gemm_fwd_out_fp32(a, b)

    def forward_accum_fp32(self, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
            raise TypeError("FP32-accumulation GEMM requires BF16 inputs on the gfx950 build")
        assert a.is_cuda and b.is_cuda, "Inputs must be on ROCm device"
        return _C.det_gemm_fwd_out_fp32(a, b).to(a.dtype)

    def parameter_vjp_contributions_fp32(self, *, a, b, grad_output):
        del b
        rows_a = a.float()
        rows_g = grad_output.float()
        return {"b": rows_a[:, :, None] * rows_g[:, None, :]}


DetGemmOp = RocmDetGemmOp


def deterministic_gemm(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Functional strict GEMM entry for ``[M,K] @ [K,N]``."""
    if torch.is_grad_enabled() and (a.requires_grad or b.requires_grad):
        return MfmaGemmFn.apply(a, b)
    return _strict_gemm(a, b)


__all__ = [
    "DetGemmOp",
    "RocmDetGemmOp",
    "MfmaGemmFn",
    "MfmaLinearFn",
    "det_gemm_backend",
    "det_gemm_backend_id",
    "tree_gemm",
    "det_gemm_fallback_reason",
    "det_gemm_linear",
    "det_gemm_linear_prepared",
    "det_gemm_linear_input_gradient",
    "det_gemm_linear_weight_gradient",
    "deterministic_gemm",
    "mfma_gemm",
    "mfma_linear",
    "prepare_det_gemm_linear_weight",
    "refresh_cached_weight_transposes",
]
