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
import weakref
from collections.abc import Callable, Iterable
from threading import Lock

import torch

from rl_engine import _C, _lib
from rl_engine._checks import enforce, output_buffer_rules

_HIP_BACKEND = "hip_mfma"
_TREE_BACKEND = "hip_tree"
# RL_KERNEL_DET_GEMM_BACKEND: every value the reference accepts (rl_engine/backends/rocm/gemm/det_gemm.py:33-48)
# selects the contract that plays the same role here; "auto" is the MFMA contract on gfx950.
_CONTRACT_OF_REQUEST = {
    "auto": _HIP_BACKEND, _HIP_BACKEND: _HIP_BACKEND, "mfma": _HIP_BACKEND, "triton_mfma": _HIP_BACKEND,
    _TREE_BACKEND: _TREE_BACKEND, "tree": _TREE_BACKEND, "triton_tree": _TREE_BACKEND, "triton": _TREE_BACKEND,
    "rocm": _TREE_BACKEND,
}  # fmt: skip
# Prepared [K,N] copies by source weight: what refresh_cached_weight_transposes re-copies. The kernels read
# the native [N,K] layout directly, so no transpose is ever made behind the caller's back; the only
# transposed buffers alive are the ones prepare_det_gemm_linear_weight handed out. A source is identified by
# its storage object (plus offset, shape, strides and dtype inside it), not by its address: an entry dies with
# the storage, so a later tensor that the allocator places at the same address is a different source. Buffers
# are held weakly as well: one the caller dropped is forgotten.
_PREPARED_TRANSPOSES: dict[tuple, tuple[weakref.ReferenceType, list[weakref.ReferenceType]]] = {}
_PREPARED_LOCK = Lock()


def _resolve_backend_request(value: str) -> str:
    """The request as written (normalised), refused when it names no contract of this build."""
    key = value.strip().lower()
    if key not in _CONTRACT_OF_REQUEST:
        raise RuntimeError(
            f"RL_KERNEL_DET_GEMM_BACKEND must be 'auto', '{_TREE_BACKEND}' or '{_HIP_BACKEND}' "
            f"on the gfx950 build, got {key!r}"
        )
    return "auto" if key == "auto" else _CONTRACT_OF_REQUEST[key]


def _requested_backend() -> str:
    return _resolve_backend_request(os.getenv("RL_KERNEL_DET_GEMM_BACKEND", "auto"))


_REQUESTED_BACKEND = _requested_backend()  # read once, at import, as in the reference


def det_gemm_backend() -> str:
    """Name of the strict GEMM implementation in use."""
    return _CONTRACT_OF_REQUEST[_REQUESTED_BACKEND]


def _use_tree() -> bool:
    return det_gemm_backend() == _TREE_BACKEND


def det_gemm_fallback_reason() -> str | None:
    return None


def det_gemm_backend_id() -> str:
    """Arithmetic-contract id reported in provenance records."""
    lib = _lib.load()
    return (lib.rlk_det_gemm_tree_contract_id() if _use_tree() else lib.rlk_contract_id()).decode()


_route_line_pending = [True]  # one route line per process (RL_KERNEL_ROUTE_REPORT), whoever constructs first


def _report_strict_route_once() -> None:
    if os.getenv("RL_KERNEL_ROUTE_REPORT", "").strip().lower() not in {"1", "true", "yes", "on"}:
        return
    with _PREPARED_LOCK:
        first, _route_line_pending[0] = _route_line_pending[0], False
    if first:
        mode = os.getenv("RL_KERNEL_MODE", "strict")
        print(f"[RL-Kernel][route] mode={mode} module=gemm requested={_REQUESTED_BACKEND} "
              f"actual={det_gemm_backend_id()} fallback=false", flush=True)  # fmt: skip


# ---------------------------------------------------------------------------
# Core strided GEMM with the reference's validation
# ---------------------------------------------------------------------------


def _operand_rules(a: torch.Tensor, b: torch.Tensor) -> list:
    def strides_ok(t: torch.Tensor):
        return lambda: min(t.stride()) >= 0

    def one_unit_stride(t: torch.Tensor):
        return lambda: t.numel() <= 1 or 1 in t.stride()

    return [
        (a.dim() == 2 and b.dim() == 2, ValueError, "MFMA GEMM expects two 2-D tensors"),
        (lambda: a.size(1) == b.size(0), ValueError, lambda: f"MFMA GEMM K mismatch: {a.size(1)} and {b.size(0)}"),
        (a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16, TypeError, "MFMA GEMM requires BF16 inputs"),
        (a.is_cuda and b.is_cuda and a.device == b.device, RuntimeError, "MFMA GEMM inputs must share one ROCm device"),
        (strides_ok(a), ValueError, "MFMA GEMM operand a must not use negative strides"),
        (one_unit_stride(a), ValueError, "MFMA GEMM operand a needs one unit-stride dimension"),
        (strides_ok(b), ValueError, "MFMA GEMM operand b must not use negative strides"),
        (one_unit_stride(b), ValueError, "MFMA GEMM operand b needs one unit-stride dimension"),
    ]


def _validate_operands(a: torch.Tensor, b: torch.Tensor) -> None:
    enforce(_operand_rules(a, b))


def _checked_output(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor | None) -> torch.Tensor:
    """Operand checks of both contracts, then the caller's output buffer (checked) or a fresh one."""
    enforce(_operand_rules(a, b))
    shape = (a.size(0), b.size(1))
    if out is None:
        return torch.empty(shape, dtype=torch.bfloat16, device=a.device)
    enforce(output_buffer_rules(out, shape, a.device, "MFMA GEMM"))
    return out


def mfma_gemm(
    a: torch.Tensor, b: torch.Tensor, *, out: torch.Tensor | None = None, config: str | int | None = None,
) -> torch.Tensor:
    """``a[M,K] @ b[K,N]`` in bf16 under the pinned MFMA contract.

    Both operands may be strided views (``weight.t()`` of a native ``[N,K]``
    weight is the fast layout). ``out`` may be a caller-owned bf16 ``[M,N]``
    buffer with contiguous rows, for instance a narrowed staging view.
    ``config`` names a tile configuration; it never changes a result bit.
    """
    out = _checked_output(a, b, out)
    if out.numel() == 0:
        return out
    code = _lib.GEMM_CONFIGS[config] if isinstance(config, str) else int(config or 0)
    _C.gemm_strided(a, b, out, config=code)
    return out


def tree_gemm(a: torch.Tensor, b: torch.Tensor, *, out: torch.Tensor | None = None, leaf_space: bool = False) -> torch.Tensor:
    """``a[M,K] @ b[K,N]`` in bf16 under the k-tree contract (any strided views).

    Equals the specification the reference's tests evaluate
    (tests/ops/gemm/test_det_gemm.py:156-168) bit for bit; a contiguous half of K is
    exactly one child of the root, so K-sharded partial results combined by bf16
    adds in a balanced rank tree reproduce the unsharded result.

    ``leaf_space=True`` splits the tree over the fixed 32-wide K tiles instead of over elements, the shape of
    the reference's ``DetGemmTreeReferenceOp`` (rl_engine/reference/gemm/det_gemm.py:29-60): the same result
    when K / 32 is a power of two, another tree (and contract id, ``tree_leaf_space_contract_id()``) otherwise.
    """
    out = _checked_output(a, b, out)
    if out.numel() == 0:
        return out
    return _C.gemm_tree_strided(a, b, out, _lib.TREE_LEAF_SPACE if leaf_space else 0)


def tree_leaf_space_contract_id() -> str:
    return _lib.load().rlk_det_gemm_tree_leaf_space_contract_id().decode()


def _strict_gemm(a: torch.Tensor, b: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """``a @ b`` under the contract selected at import."""
    if _use_tree():
        return tree_gemm(a, b, out=out)
    return mfma_gemm(a, b, out=out)


def _fp32_gemm(a: torch.Tensor, b: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """``a @ b`` accumulated in fp32 and never rounded below it (one rounding to ``out_dtype`` when that is
    bf16), in the arithmetic family of the selected backend.

    MFMA backend, bf16 operands: the fp32 accumulator of the MFMA chain. k-tree backend, or any fp32 operand:
    one fp32 fused multiply-add per k, k ascending, from +0 (the chain a k-tree leaf is made of, here over the
    whole of K) - the arithmetic of the reference's native round-once twin (csrc/musa/det_gemm.mu:25-48).
    Neither ever runs in place of the other; ``det_gemm_fp32_backend_id`` names the one in use.
    """
    if not _use_tree() and a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16:
        return _C.det_gemm_fwd_out_fp32(a, b) if out_dtype == torch.float32 else _C.det_gemm_fwd(a, b)
    return _C.det_gemm_seq(a, b, out_dtype)


def det_gemm_fp32_backend_id(a_dtype: torch.dtype = torch.bfloat16, b_dtype: torch.dtype = torch.bfloat16) -> str:
    """Contract id of ``DetGemmOp.forward_fp32`` / ``forward_accum_fp32`` for these operand dtypes."""
    lib = _lib.load()
    if not _use_tree() and a_dtype == torch.bfloat16 and b_dtype == torch.bfloat16:
        return lib.rlk_contract_id().decode()
    return lib.rlk_det_gemm_seq_contract_id().decode()


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
# Prepared (transposed) inference weights and their refresh
# ---------------------------------------------------------------------------


def _source_key(weight: torch.Tensor):
    storage = weight.untyped_storage()
    return storage, (storage._cdata, weight.storage_offset(), tuple(weight.shape), tuple(weight.stride()), weight.dtype)


def _forget_source(key) -> None:
    with _PREPARED_LOCK:
        _PREPARED_TRANSPOSES.pop(key, None)


def _live_prepared(weight: torch.Tensor) -> list[torch.Tensor]:
    """Prepared copies of ``weight`` that are still alive (dead entries are dropped on the way)."""
    storage, key = _source_key(weight)
    with _PREPARED_LOCK:
        entry = _PREPARED_TRANSPOSES.get(key)
        if entry is None or entry[0]() is not storage:
            return []
        alive = [(ref, ref()) for ref in entry[1]]
        kept = [ref for ref, buf in alive if buf is not None]
        if kept:
            _PREPARED_TRANSPOSES[key] = (entry[0], kept)
        else:
            _PREPARED_TRANSPOSES.pop(key, None)
    return [buf for _, buf in alive if buf is not None]


def _remember_prepared(weight: torch.Tensor, prepared: torch.Tensor) -> None:
    storage, key = _source_key(weight)
    with _PREPARED_LOCK:
        entry = _PREPARED_TRANSPOSES.get(key)
        if entry is None or entry[0]() is not storage:
            # the entry goes when the source's storage is freed (the callback runs outside this lock's holder:
            # a storage dies when its last tensor does, never inside these functions, which hold `weight`)
            entry = (weakref.ref(storage, lambda _ref, key=key: _forget_source(key)), [])
        refs = [ref for ref in entry[1] if ref() is not None]
        if not any(ref() is prepared for ref in refs):
            refs.append(weakref.ref(prepared))
        _PREPARED_TRANSPOSES[key] = (entry[0], refs)


@torch.inference_mode()
def refresh_cached_weight_transposes(weights: Iterable[object]) -> int:
    """Re-copy, in place, every live prepared ``[K,N]`` buffer of the given ``[N,K]`` weights after an
    in-place weight update; returns how many weights had one.

    Same role as the reference function of this name
    (rl_engine/backends/rocm/gemm/det_gemm.py:143-159): the buffers keep their addresses, so HIP
    graphs captured against them stay valid. Weights that were never prepared are skipped; the
    native-layout paths read the weight itself and have nothing to refresh.
    """
    refreshed = 0
    for weight in weights:
        if not isinstance(weight, torch.Tensor) or weight.ndim != 2:
            continue
        buffers = _live_prepared(weight)
        for buf in buffers:
            buf.copy_(weight.t())
        refreshed += 1 if buffers else 0
    return refreshed


def prepare_det_gemm_linear_weight(weight: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """Materialise a stable contiguous ``[K,N]`` inference weight from ``[N,K]``.

    Checks and error types follow the reference
    (rl_engine/backends/rocm/gemm/det_gemm.py:345-408). The caller owns freshness: call this again
    with ``out=`` or :func:`refresh_cached_weight_transposes` after the source changes.
    """
    what = "prepared deterministic linear weight"
    enforce([
        (weight.dim() == 2, ValueError, f"{what}s must be 2-D"),
        (weight.dtype == torch.bfloat16, TypeError, f"{what}s must be BF16"),
        (weight.is_cuda, RuntimeError, f"{what}s must be on ROCm"),
        (weight.is_contiguous(), ValueError, "source deterministic linear weights must be contiguous"),
    ])  # fmt: skip
    transposed_shape = tuple(reversed(weight.shape))
    if out is not None:
        enforce([
            (tuple(out.shape) == transposed_shape, ValueError, f"{what} must have shape {transposed_shape}, got {tuple(out.shape)}"),
            (out.dtype == weight.dtype, TypeError, f"{what} dtype must match its source"),
            (out.device == weight.device, RuntimeError, f"{what} device must match its source"),
            (out.is_contiguous(), ValueError, f"{what} must be contiguous"),
            (not out.requires_grad, ValueError, f"{what} must not require gradients"),
            (lambda: not torch._C._overlaps(out, weight), ValueError, f"{what} must not alias its source"),
        ])  # fmt: skip
    else:
        # Post-load hooks run under inference mode; an ordinary tensor can be refreshed in place later.
        with torch.inference_mode(False), torch.no_grad():
            out = torch.empty(transposed_shape, dtype=weight.dtype, device=weight.device)
    with torch.no_grad():
        # Only `out` is written, as in the reference: an earlier prepared copy of the same source keeps its bits
        # (it may be a deliberate snapshot) until refresh_cached_weight_transposes, or another call with it as
        # `out`, re-copies it.
        out.copy_(weight.t())
    _remember_prepared(weight, out)
    return out


# ---------------------------------------------------------------------------
# Linear entry points
# ---------------------------------------------------------------------------


def det_gemm_linear(
    a: torch.Tensor, weight: torch.Tensor, *, native_op: Callable[[torch.Tensor, torch.Tensor],
    torch.Tensor] | None = None, out: torch.Tensor | None = None, inference_schedule: bool = False,
) -> torch.Tensor:
    """Apply a native ``[N,K]`` weight: ``a @ weight.T``."""
    del native_op, inference_schedule
    # the everyday call (fresh output, MFMA contract, plain row-major operands) skips the rule tables and the
    # transposed view: same library call, same result, about half the host time per call
    if out is None and _CONTRACT_OF_REQUEST[_REQUESTED_BACKEND] == _HIP_BACKEND:
        result = _C.linear_plain(a, weight)
        if result is not None:
            return result
    return mfma_linear(a, weight, out=out)


def det_gemm_linear_prepared(a: torch.Tensor, weight_t: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """Apply a lifecycle-managed contiguous ``[K,N]`` inference weight."""
    tracked = torch.is_grad_enabled() and (a.requires_grad or weight_t.requires_grad)
    enforce([
        (not tracked, RuntimeError, "prepared deterministic linear GEMM is inference-only"),
        (weight_t.is_contiguous(), ValueError, "prepared deterministic linear weight must be contiguous"),
        (lambda: out is None or not (torch._C._overlaps(out, a) or torch._C._overlaps(out, weight_t)),
         ValueError, "prepared deterministic linear output must not alias its inputs"),
    ])  # fmt: skip
    return _strict_gemm(a, weight_t, out=out)


def det_gemm_linear_input_gradient(
    grad_output: torch.Tensor, weight: torch.Tensor, *, native_op: Callable[[torch.Tensor, torch.Tensor],
    torch.Tensor] | None = None,
) -> torch.Tensor:
    """``dX = dY @ weight``."""
    del native_op
    return mfma_linear_input_gradient(grad_output, weight)


def det_gemm_linear_weight_gradient(
    a: torch.Tensor, grad_output: torch.Tensor, *, native_op: Callable[[torch.Tensor, torch.Tensor],
    torch.Tensor] | None = None,
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


def _assert_bf16_on_gpu(*tensors: torch.Tensor) -> None:
    # AssertionError with the reference's two messages (backends/rocm/gemm/det_gemm.py:505-506)
    assert all(t.dtype == torch.bfloat16 for t in tensors), "BF16 only"
    assert all(t.is_cuda for t in tensors), "Inputs must be on ROCm device"


class RocmDetGemmOp:
    """Batch-invariant deterministic GEMM backed by the gfx950 HIP kernel."""

    def __init__(self):
        _lib.load()
        self.op = self
        self.has_hardware_op = True
        _report_strict_route_once()

    def __call__(self, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        _assert_bf16_on_gpu(a, b)
        return deterministic_gemm(a, b)

    def linear(self, a: torch.Tensor, weight: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
        """Apply a native ``[N,K]`` linear weight."""
        _assert_bf16_on_gpu(a, weight)
        a, weight = a.contiguous(), weight.contiguous()
        differentiable = torch.is_grad_enabled() and (a.requires_grad or weight.requires_grad)
        if out is None:
            # one opaque custom op for inference (Dynamo / graph capture), autograd otherwise
            return MfmaLinearFn.apply(a, weight) if differentiable else _det_gemm_linear_inference(a, weight)
        if differentiable:
            raise RuntimeError("direct-output deterministic GEMM is inference-only")
        _det_gemm_linear_inference_out(a, weight, out)
        return out

    def linear_prepared(self, a: torch.Tensor, weight_t: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
        """Apply a post-load prepared ``[K,N]`` weight."""
        _assert_bf16_on_gpu(a, weight_t)
        return det_gemm_linear_prepared(a.contiguous(), weight_t, out=out)

    def forward_fp32(self, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        """``a @ b`` as fp32, never rounded to bf16: the fp32 chain of the selected backend's kernel family
        (the MFMA accumulator, or the sequential fp32 fused-multiply-add chain when the k-tree is selected)."""
        _assert_bf16_on_gpu(a, b)
        return _fp32_gemm(a, b)

    def forward_accum_fp32(self, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        """fp32 accumulation, result in the dtype of ``a``; bf16 or fp32 operands, as in the reference
        (backends/rocm/gemm/det_gemm.py:548-555). An fp32 operand always takes the sequential fp32 chain."""
        allowed = (torch.bfloat16, torch.float32)
        if a.dtype not in allowed or b.dtype not in allowed:
            raise TypeError("FP32-accumulation GEMM requires BF16 or FP32 inputs")
        assert a.is_cuda and b.is_cuda, "Inputs must be on ROCm device"
        return _fp32_gemm(a, b, a.dtype)

    def parameter_vjp_contributions_fp32(self, *, a, b, grad_output):
        """Per-row outer products ``a_i (x) g_i`` in fp32: the summands of the weight gradient."""
        del b
        return {"b": torch.einsum("mk,mn->mkn", a.float(), grad_output.float())}


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
    "det_gemm_fp32_backend_id",
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
