"""Tensor-level native entry points, named as the reference's ``rl_engine._C``.

The reference module is a pybind extension (csrc/bindings/ops.cpp:504-761,
stub rl_engine/_C.pyi). This one has the same function names, argument order,
return shapes and error strings for the deterministic dense path, and forwards
to the C ABI of librlk_gfx950.so with raw device pointers; PyTorch only supplies
device memory and the current stream.
"""

from __future__ import annotations

from typing import List, Optional

import torch

from rl_engine import _lib

_BF16 = torch.bfloat16


def _stream_handle(device: torch.device) -> int:
    """The raw handle of ``device``'s current stream (what ``torch.cuda.current_stream(device).cuda_stream`` holds,
    without building the stream object: this runs on every call)."""
    return torch._C._cuda_getCurrentRawStream(device.index)


class _NoSwitch:
    """A context manager that does nothing: the device is already current."""

    __slots__ = ()

    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on(device: torch.device):
    """``torch.cuda.device(device)`` for the launch, or nothing at all when that device is current already (the
    usual case; entering and leaving the guard costs several microseconds per call)."""
    if device.index == torch._C._cuda_getDevice():
        return _NO_SWITCH
    return torch.cuda.device(device)


def _check_in(t: torch.Tensor, name: str) -> None:
    # Same wording as check_in, csrc/cuda/gemm/det_gemm_kernel.cu:437-440.
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be CUDA")
    if t.dtype != _BF16:
        raise RuntimeError(f"{name} must be bf16")


def _raw_gemm(
    a: torch.Tensor,
    a_row_stride: int,
    a_k_stride: int,
    b: torch.Tensor,
    b_k_stride: int,
    b_n_stride: int,
    out: torch.Tensor,
    m: int,
    n: int,
    k: int,
    config: int = 0,
) -> None:
    """One call of rlk_det_gemm_bf16 on the current stream of ``a``'s device."""
    lib = _lib.load()
    with _on(a.device):
        status = lib.rlk_det_gemm_bf16(
            a.data_ptr(),
            a_row_stride,
            a_k_stride,
            b.data_ptr(),
            b_k_stride,
            b_n_stride,
            out.data_ptr(),
            out.stride(0) if out.dim() == 2 else n,
            m,
            n,
            k,
            1 if out.dtype == torch.float32 else 0,
            config,
            _stream_handle(a.device),
        )
    _lib.check(status, "rlk_det_gemm_bf16 failed")


def gemm_strided(
    a: torch.Tensor,
    b: torch.Tensor,
    out: torch.Tensor,
    *,
    config: int = 0,
) -> torch.Tensor:
    """``out[M,N] = a[M,K] @ b[K,N]`` for arbitrary non-negative strides."""
    m, k = a.shape
    n = b.shape[1]
    if m == 0 or n == 0:
        return out
    _raw_gemm(a, a.stride(0), a.stride(1), b, b.stride(0), b.stride(1), out, m, n, k, config)
    return out


_gemm_entry = None  # rlk_det_gemm_bf16, looked up once


def linear_plain(a: torch.Tensor, weight: torch.Tensor) -> Optional[torch.Tensor]:
    """``a[M,K] @ weight[N,K].T`` into a fresh bf16 ``[M,N]`` for the everyday operands - two non-empty 2-D bf16
    tensors on one GPU with matching K and contiguous rows - or ``None`` for anything else (including everything
    that has to raise: the long way words the errors). The same call of rlk_det_gemm_bf16 that
    :func:`gemm_strided` makes for ``(a, weight.t())``, without the rule tables and the transposed view."""
    global _gemm_entry
    sa, sw = a.stride(), weight.stride()
    if len(sa) != 2 or len(sw) != 2 or sa[1] != 1 or sw[1] != 1 or sa[0] < 0 or sw[0] < 0:
        return None
    if a.dtype is not _BF16 or weight.dtype is not _BF16:
        return None
    device = a.device
    if device.type != "cuda" or weight.device != device:
        return None
    m, k = a.shape
    n, kw = weight.shape
    if k != kw or m == 0 or n == 0 or k == 0:
        return None
    if _gemm_entry is None:
        _gemm_entry = _lib.load().rlk_det_gemm_bf16
    out = torch.empty((m, n), dtype=_BF16, device=device)
    with _on(device):
        status = _gemm_entry(
            a.data_ptr(), sa[0], 1, weight.data_ptr(), 1, sw[0], out.data_ptr(), n, m, n, k, 0, 0,
            torch._C._cuda_getCurrentRawStream(device.index),
        )  # fmt: skip
    if status:
        _lib.check(status, "rlk_det_gemm_bf16 failed")
    return out


def gemm_tree_strided(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor, config: int = 0) -> torch.Tensor:
    """``out[M,N] = a[M,K] @ b[K,N]`` under the k-tree contract, arbitrary non-negative strides.

    ``config`` (``rlk_tree_config``; the same bits whichever runs): 0 picks the kernel, 1 forces the
    vector-ALU tiled kernel, 2 the fp32 matrix-pipe tiled kernel, 3 / 4 the node-per-wave kernels for up
    to 16 rows / any row count (``ValueError`` when the operands are not eligible)."""
    m, k = a.shape
    n = b.shape[1]
    if m == 0 or n == 0:
        return out
    lib = _lib.load()
    with _on(a.device):
        status = lib.rlk_det_gemm_tree_bf16_config(
            a.data_ptr(),
            a.stride(0),
            a.stride(1),
            b.data_ptr(),
            b.stride(0),
            b.stride(1),
            out.data_ptr(),
            out.stride(0),
            m,
            n,
            k,
            int(config),
            _stream_handle(a.device),
        )
    _lib.check(status, "rlk_det_gemm_tree_bf16 failed")
    return out


def det_gemm_sm90_compiled() -> bool:
    """Always False here (csrc/cuda/gemm/det_gemm_kernel.cu:511-517): no SM90 code exists."""
    return False


def det_gemm_fwd(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """``a[M,K] @ b[K,N] -> [M,N]`` bf16 (det_gemm_kernel.cu:519-525)."""
    _check_in(a, "A")
    _check_in(b, "B")
    if a.dim() != 2 or b.dim() != 2:
        raise RuntimeError("det_gemm_fwd: expect 2D [M,K]@[K,N]")
    if b.size(0) != a.size(1):
        raise RuntimeError("det_gemm_fwd: K mismatch")
    out = torch.empty((a.size(0), b.size(1)), dtype=_BF16, device=a.device)
    return gemm_strided(a, b, out)


def det_gemm_fwd_rhs_transposed(a: torch.Tensor, bt: torch.Tensor) -> torch.Tensor:
    """``a[M,K] @ bt[N,K].T -> [M,N]`` (det_gemm_kernel.cu:527-534)."""
    _check_in(a, "A")
    _check_in(bt, "Bt")
    if a.dim() != 2 or bt.dim() != 2:
        raise RuntimeError("det_gemm_fwd_rhs_transposed: expect A[M,K] and Bt[N,K]")
    if bt.size(1) != a.size(1):
        raise RuntimeError("det_gemm_fwd_rhs_transposed: K mismatch")
    out = torch.empty((a.size(0), bt.size(0)), dtype=_BF16, device=a.device)
    return gemm_strided(a, bt.t(), out)


def det_gemm_fwd_out_fp32(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """``a[M,K] @ b[K,N]`` with the fp32 accumulator stored unrounded.

    Serves DetGemmOp.forward_fp32 (rl_engine/backends/rocm/gemm/det_gemm.py:545-548).
    """
    _check_in(a, "A")
    _check_in(b, "B")
    if a.dim() != 2 or b.dim() != 2:
        raise RuntimeError("det_gemm_fwd_out_fp32: expect 2D [M,K]@[K,N]")
    if b.size(0) != a.size(1):
        raise RuntimeError("det_gemm_fwd_out_fp32: K mismatch")
    out = torch.empty((a.size(0), b.size(1)), dtype=torch.float32, device=a.device)
    return gemm_strided(a, b, out)


_SEQ_DTYPES = {torch.bfloat16: _lib.DTYPE_BF16, torch.float32: _lib.DTYPE_FP32}


def det_gemm_seq(a: torch.Tensor, b: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """``a[M,K] @ b[K,N]`` with one fp32 fused multiply-add per k, k ascending, nothing rounded below fp32;
    bf16 or fp32 operands (any strides), fp32 result or one rounding to bf16 (rlk_det_gemm_seq)."""
    for name, t in (("A", a), ("B", b)):
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be CUDA")
        if t.dtype not in _SEQ_DTYPES:
            raise RuntimeError(f"{name} must be bf16 or fp32")
    if a.dim() != 2 or b.dim() != 2:
        raise RuntimeError("det_gemm_fwd_fp32: expect 2D [M,K]@[K,N]")
    if b.size(0) != a.size(1):
        raise RuntimeError("det_gemm_fwd_fp32: K mismatch")
    if out_dtype not in _SEQ_DTYPES:
        raise RuntimeError("det_gemm_fwd_fp32: output must be bf16 or fp32")
    m, k = a.shape
    n = b.size(1)
    out = torch.empty((m, n), dtype=out_dtype, device=a.device)
    if m == 0 or n == 0:
        return out
    with _on(a.device):
        status = _lib.load().rlk_det_gemm_seq(
            a.data_ptr(), _SEQ_DTYPES[a.dtype], a.stride(0), a.stride(1), b.data_ptr(), _SEQ_DTYPES[b.dtype],
            b.stride(0), b.stride(1), out.data_ptr(), _SEQ_DTYPES[out_dtype], n, m, n, k, _stream_handle(a.device),
        )  # fmt: skip
    _lib.check(status, "rlk_det_gemm_seq failed")
    return out


def det_gemm_fwd_fp32(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """fp32 ``a @ b`` from bf16 or fp32 operands, sequential fp32 chain (rl_engine/_C.pyi:244;
    csrc/musa/det_gemm.mu:25-48)."""
    return det_gemm_seq(a, b, torch.float32)


def det_gemm_accum_fwd_fp32(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """The same chain, result rounded once to the dtype of ``a`` (rl_engine/_C.pyi:245-248)."""
    return det_gemm_seq(a, b, a.dtype if a.dtype in _SEQ_DTYPES else torch.float32)


# the name the facade uses for the fp32-result path
det_gemm_seq_fp32 = det_gemm_fwd_fp32


def _reduction_major(t: torch.Tensor) -> torch.Tensor:
    """``t.t()`` ready for a GEMM whose reduction runs over ``t``'s rows.

    A row-major ``t[M, C]`` with ``C % 8 == 0`` and 16-byte aligned rows is passed as the
    plain view ``t.t()``: the library reads such a K-major operand through transposing LDS
    loads, whole 64-row tiles directly and the rest of an ``M`` that 64 does not divide
    through registers. Anything else gets a value-preserving copy with the
    reduction axis contiguous.
    """
    tt = t.t()
    if tt.stride(1) == 1:
        return tt
    if (
        t.stride(1) == 1
        and t.size(1) % 8 == 0
        and t.size(0) >= 1
        and t.stride(0) % 8 == 0
        and t.data_ptr() % 16 == 0
    ):
        return tt
    return tt.contiguous()


def det_gemm_da(dc: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """``dA[M,K] = dC[M,N] @ B[K,N].T`` (det_gemm_kernel.cu:545-554)."""
    _check_in(dc, "dC")
    _check_in(b, "B")
    if dc.dim() != 2 or b.dim() != 2:
        raise RuntimeError("det_gemm_da: expect dC[M,N] and B[K,N]")
    if b.size(1) != dc.size(1):
        raise RuntimeError("det_gemm_da: N mismatch")
    out = torch.empty((dc.size(0), b.size(0)), dtype=_BF16, device=dc.device)
    return gemm_strided(dc, b.t(), out)


def det_gemm_db(a: torch.Tensor, dc: torch.Tensor) -> torch.Tensor:
    """``dB[K,N] = A[M,K].T @ dC[M,N]`` (det_gemm_kernel.cu:556-565)."""
    _check_in(a, "A")
    _check_in(dc, "dC")
    if a.dim() != 2 or dc.dim() != 2:
        raise RuntimeError("det_gemm_db: expect A[M,K] and dC[M,N]")
    if dc.size(0) != a.size(0):
        raise RuntimeError("det_gemm_db: M mismatch")
    # Reduction runs over tokens: make that axis contiguous in both operands so
    # the vector loader applies (the copies change no value).
    at = _reduction_major(a)  # [K, M]
    dct = _reduction_major(dc)  # [N, M]
    out = torch.empty((a.size(1), dc.size(1)), dtype=_BF16, device=a.device)
    return gemm_strided(at, dct.t(), out)


def det_gemm_db_transposed(a: torch.Tensor, dc: torch.Tensor) -> torch.Tensor:
    """``dW[N,K] = dC[M,N].T @ A[M,K]``, contiguous (det_gemm_kernel.cu:567-602)."""
    _check_in(a, "A")
    _check_in(dc, "dC")
    if a.dim() != 2 or dc.dim() != 2:
        raise RuntimeError("det_gemm_db_transposed: expect A[M,K] and dC[M,N]")
    if dc.size(0) != a.size(0):
        raise RuntimeError("det_gemm_db_transposed: M mismatch")
    at = _reduction_major(a)  # [K, M]
    dct = _reduction_major(dc)  # [N, M]
    out = torch.empty((dc.size(1), a.size(1)), dtype=_BF16, device=a.device)
    return gemm_strided(dct, at.t(), out)


def det_gemm_pick_config(m: int, n: int, k: int) -> int:
    return int(_lib.load().rlk_det_gemm_pick_config(int(m), int(n), int(k)))


def linear_logp_split_count(vocab: int) -> int:
    return int(_lib.load().rlk_linear_logp_split_count(int(vocab)))


def _linear_logp_forward(
    who: str,
    entry: str,
    hidden: torch.Tensor,
    weight: torch.Tensor,
    target: torch.Tensor,
    bias: Optional[torch.Tensor],
    temperature: Optional[torch.Tensor],
    real_vocab_size: int,
    vocab_start_index: int,
    config: int,
    want_logits: bool = False,
):
    """Checks shared by the fused linear-LogP entries, then one call of ``entry`` in the C ABI.

    Returns ``(first, lse, logits)``; ``first`` is logp or the target logit, whichever ``entry``
    writes; ``logits`` is the fp32 ``[N, V]`` tensor the same pass stored when ``want_logits``, else None."""
    if not hidden.is_cuda or not weight.is_cuda or not target.is_cuda:
        raise RuntimeError(f"{who}: hidden, weight and target must be CUDA tensors")
    if hidden.dtype != _BF16 or weight.dtype != _BF16:
        raise RuntimeError(f"{who}: hidden and weight must be bf16")
    if hidden.dim() != 2 or weight.dim() != 2:
        raise RuntimeError(f"{who}: expect hidden [N,D] and weight [V,D]")
    if not hidden.is_contiguous() or not weight.is_contiguous():
        raise RuntimeError(f"{who}: hidden and weight must be contiguous")
    n, d = hidden.shape
    v = weight.size(0)
    if weight.size(1) != d:
        raise RuntimeError(f"{who}: hidden dim must match weight dim")
    if target.numel() != n:
        raise RuntimeError(f"{who}: target must have one id per row")
    real_vocab = v if int(real_vocab_size) < 0 else int(real_vocab_size)
    if not 0 < real_vocab <= v:
        raise RuntimeError(f"{who}: real_vocab_size must be in [1, {v}]")
    target_i64 = target.reshape(-1).to(torch.int64).contiguous()
    bias_f32 = None
    if bias is not None:
        if bias.numel() != v:
            raise RuntimeError(f"{who}: bias must have V elements")
        bias_f32 = bias.to(device=hidden.device, dtype=torch.float32).contiguous()
    temp_f32 = None
    if temperature is not None:
        if temperature.dtype != torch.float32 or temperature.numel() != n:
            raise RuntimeError(f"{who}: temperature must be fp32 with one value per row")
        temp_f32 = temperature.to(hidden.device).contiguous()

    lib = _lib.load()
    first = torch.empty((n,), dtype=torch.float32, device=hidden.device)
    lse = torch.empty((n,), dtype=torch.float32, device=hidden.device)
    logits = torch.empty((n, v), dtype=torch.float32, device=hidden.device) if want_logits else None
    ws_bytes = int(lib.rlk_linear_logp_workspace_bytes(n, v))
    workspace = torch.empty((max(ws_bytes, 4) // 4,), dtype=torch.float32, device=hidden.device)
    if n > 0:
        head = (
            hidden.data_ptr(), hidden.stride(0), weight.data_ptr(), weight.stride(0), target_i64.data_ptr(),
            bias_f32.data_ptr() if bias_f32 is not None else None,
            temp_f32.data_ptr() if temp_f32 is not None else None,
            first.data_ptr(), lse.data_ptr(),
        )  # fmt: skip
        tail = (workspace.data_ptr(), ws_bytes, n, d, v, int(vocab_start_index), real_vocab, config, _stream_handle(hidden.device))
        with _on(hidden.device):
            if want_logits:  # the logits come out of the same pass: entry + "_logits"
                entry = entry + "_logits"
                status = getattr(lib, entry)(*head, logits.data_ptr(), logits.stride(0), *tail)
            else:
                status = getattr(lib, entry)(*head, *tail)
        _lib.check(status, f"{entry} failed")
    return first, lse, logits


def fused_linear_logp(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    target: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    temperature: Optional[torch.Tensor] = None,
    return_logits: bool = False,
    real_vocab_size: int = -1,
    *,
    vocab_start_index: int = 0,
    config: int = 0,
) -> List[torch.Tensor]:
    """Fused lm_head GEMM + fixed-order log-sum-exp + target gather -> ``[logp, lse]``.

    Same arguments, checks and return convention as ``_C.fused_linear_logp_sm90``
    (csrc/bindings/ops.cpp:514-520; csrc/cuda/logprob/fused_linear_logp_sm90.cu:2040-2176).
    ``return_logits=True`` appends the unscaled fp32 logits ``[N, V]`` (bias applied, padded
    lanes -inf), stored by the same kernel pass from the accumulators the reduction sees
    (rlk_linear_logp_fwd_logits; no second GEMM); it does not change logp / lse.
    """
    logp, lse, logits = _linear_logp_forward(
        "fused_linear_logp", "rlk_linear_logp_fwd", hidden, weight, target, bias, temperature,
        real_vocab_size, vocab_start_index, config, want_logits=bool(return_logits),
    )  # fmt: skip
    return [logp, lse, logits] if return_logits else [logp, lse]


# The name the reference's CUDA build binds the same function under (csrc/bindings/ops.cpp:514).
fused_linear_logp_sm90 = fused_linear_logp


def fused_linear_logp_sm90_global_target(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    target: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    vocab_start_index: int = 0,
    temperature: Optional[torch.Tensor] = None,
    real_vocab_size: int = -1,
    *,
    config: int = 0,
) -> List[torch.Tensor]:
    """One vocabulary shard's ``[target_logit, lse]`` for targets given in global ids.

    ``weight`` holds lm_head rows ``[vocab_start_index, vocab_start_index + V)``.
    ``target_logit`` is the scaled, unclamped logit of a target this shard owns and 0
    otherwise; ``lse`` covers the shard's real columns. The caller merges both across
    shards (_merge_tp_local_logp, rl_engine/backends/cuda/logprob/linear_logp.py:711-740).
    Argument order and return convention of ``_C.fused_linear_logp_sm90_global_target``
    (csrc/bindings/ops.cpp:522-526; csrc/cuda/logprob/fused_linear_logp_sm90.cu:2169-2176).
    """
    target_logit, lse, _ = _linear_logp_forward(
        "fused_linear_logp_sm90_global_target", "rlk_linear_logp_fwd_shard", hidden, weight, target, bias,
        temperature, real_vocab_size, vocab_start_index, config,
    )  # fmt: skip
    return [target_logit, lse]


def fused_linear_logp_bwd(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    target: torch.Tensor,
    lse: torch.Tensor,
    grad_logp: Optional[torch.Tensor],
    grad_lse: Optional[torch.Tensor],
    bias: Optional[torch.Tensor] = None,
    temperature: Optional[torch.Tensor] = None,
    real_vocab_size: int = -1,
    *,
    vocab_start_index: int = 0,
    need_grad_hidden: bool = True,
    need_grad_weight: bool = True,
    need_grad_bias: bool = False,
    config: int = 0,
) -> List[Optional[torch.Tensor]]:
    """Backward of :func:`fused_linear_logp` -> ``[grad_hidden, grad_weight, grad_bias]``.

    ``lse`` is the forward's result; ``grad_logp`` / ``grad_lse`` are fp32 ``[N]`` or
    ``None``. ``grad_hidden`` / ``grad_weight`` are bf16, ``grad_bias`` fp32; an entry
    that was not asked for is ``None``. Stands in for
    ``_DetTritonLinearLogpAutograd.backward``
    (rl_engine/backends/shared/triton/logprob/linear_logp.py:600-628) and
    ``chunked_linear_logp_backward`` (rl_engine/reference/logprob/linear_logp.py:642-715).
    """
    if not hidden.is_cuda or not weight.is_cuda or not target.is_cuda or not lse.is_cuda:
        raise RuntimeError("fused_linear_logp_bwd: hidden, weight, target and lse must be CUDA tensors")
    if hidden.dtype != _BF16 or weight.dtype != _BF16:
        raise RuntimeError("fused_linear_logp_bwd: hidden and weight must be bf16")
    if hidden.dim() != 2 or weight.dim() != 2:
        raise RuntimeError("fused_linear_logp_bwd: expect hidden [N,D] and weight [V,D]")
    if not hidden.is_contiguous() or not weight.is_contiguous():
        raise RuntimeError("fused_linear_logp_bwd: hidden and weight must be contiguous")
    n, d = hidden.shape
    v = weight.size(0)
    if weight.size(1) != d:
        raise RuntimeError("fused_linear_logp_bwd: hidden dim must match weight dim")
    if target.numel() != n or lse.numel() != n:
        raise RuntimeError("fused_linear_logp_bwd: target and lse must have one value per row")
    real_vocab = v if int(real_vocab_size) < 0 else int(real_vocab_size)
    if not 0 < real_vocab <= v:
        raise RuntimeError(f"fused_linear_logp_bwd: real_vocab_size must be in [1, {v}]")

    def _per_row(t: Optional[torch.Tensor], name: str) -> Optional[torch.Tensor]:
        if t is None:
            return None
        if t.numel() != n:
            raise RuntimeError(f"fused_linear_logp_bwd: {name} must have one value per row")
        return t.reshape(-1).to(device=hidden.device, dtype=torch.float32).contiguous()

    target_i64 = target.reshape(-1).to(torch.int64).contiguous()
    lse_f32 = _per_row(lse, "lse")
    g_logp = _per_row(grad_logp, "grad_logp")
    g_lse = _per_row(grad_lse, "grad_lse")
    temp_f32 = _per_row(temperature, "temperature")
    bias_f32 = None
    if bias is not None:
        if bias.numel() != v:
            raise RuntimeError("fused_linear_logp_bwd: bias must have V elements")
        bias_f32 = bias.to(device=hidden.device, dtype=torch.float32).contiguous()

    lib = _lib.load()
    grad_hidden = torch.empty((n, d), dtype=_BF16, device=hidden.device) if need_grad_hidden else None
    grad_weight = torch.empty((v, d), dtype=_BF16, device=hidden.device) if need_grad_weight else None
    grad_bias = torch.empty((v,), dtype=torch.float32, device=hidden.device) if need_grad_bias else None
    ws_bytes = int(lib.rlk_linear_logp_bwd_workspace_bytes(n, v, 1 if need_grad_bias else 0))
    # torch's allocator hands out 512-byte aligned blocks, which covers the 256 the library asks for
    workspace = torch.empty((max(ws_bytes, 256),), dtype=torch.uint8, device=hidden.device)

    def _ptr(t: Optional[torch.Tensor]):
        return t.data_ptr() if t is not None else None

    if n == 0:  # no tokens: the token-summed gradients are zero
        if grad_weight is not None:
            grad_weight.zero_()
        if grad_bias is not None:
            grad_bias.zero_()
        return [grad_hidden, grad_weight, grad_bias]
    with _on(hidden.device):
        status = lib.rlk_linear_logp_bwd(
            hidden.data_ptr(),
            hidden.stride(0),
            weight.data_ptr(),
            weight.stride(0),
            target_i64.data_ptr(),
            _ptr(bias_f32),
            _ptr(temp_f32),
            lse_f32.data_ptr(),
            _ptr(g_logp),
            _ptr(g_lse),
            _ptr(grad_hidden),
            d,
            _ptr(grad_weight),
            d,
            _ptr(grad_bias),
            workspace.data_ptr(),
            ws_bytes,
            n,
            d,
            v,
            int(vocab_start_index),
            real_vocab,
            int(config),
            _stream_handle(hidden.device),
        )
    _lib.check(status, "rlk_linear_logp_bwd failed")
    return [grad_hidden, grad_weight, grad_bias]


def fused_linear_logp_sm90_backward(
    grad_logp: torch.Tensor,
    hidden: torch.Tensor,
    weight: torch.Tensor,
    target: torch.Tensor,
    lse: torch.Tensor,
    bias: Optional[torch.Tensor],
    vocab_start_index: int,
    compute_grad_hidden: bool,
    compute_grad_weight: bool,
    compute_grad_bias: bool,
    use_global_lse: bool,
) -> List[torch.Tensor]:
    """:func:`fused_linear_logp_bwd` under the reference's CUDA name and argument order
    (csrc/bindings/ops.cpp:33-43, 527-528): ``[grad_hidden, grad_weight, grad_bias]`` with an
    empty fp32 tensor in place of a gradient that was not asked for
    (csrc/cuda/logprob/fused_linear_logp_sm90.cu:2185-2215, 2307).

    ``target`` is in global ids and ``lse`` is the value to differentiate against: the
    shard-merged one when ``use_global_lse``, else this weight's own. The reference
    recomputes the latter from its backward logits; here the forward's ``lse`` is already
    the value of the same MFMA chain, so it is used as given in both cases.
    """
    del use_global_lse
    if grad_logp.numel() != hidden.size(0):
        raise RuntimeError("fused_linear_logp_sm90_backward: grad_logp must have one value per token")
    grads = fused_linear_logp_bwd(
        hidden, weight, target, lse, grad_logp.reshape(-1), None, bias,
        vocab_start_index=int(vocab_start_index), need_grad_hidden=bool(compute_grad_hidden),
        need_grad_weight=bool(compute_grad_weight), need_grad_bias=bool(compute_grad_bias),
    )  # fmt: skip
    empty = torch.empty((0,), dtype=torch.float32, device=hidden.device)
    return [empty if g is None else g for g in grads]


def _logits_dtype_code(logits: torch.Tensor) -> int:
    if not logits.is_cuda:
        raise RuntimeError("logits must be a ROCm tensor")
    if logits.dim() != 2:
        raise RuntimeError("logits must be 2D [tokens, local_vocab]")
    codes = {torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_FP16, torch.float32: _lib.DTYPE_FP32}
    if logits.dtype not in codes:
        raise RuntimeError("logits must be float16, bfloat16, or float32")
    return codes[logits.dtype]


def _row_contiguous(logits: torch.Tensor) -> torch.Tensor:
    return logits if logits.stride(1) == 1 and logits.stride(0) >= logits.size(1) else logits.contiguous()


def hip_deterministic_logp_tile_stats(
    logits: torch.Tensor,
    vocab_start: int,
    real_vocab: int,
    num_tiles: int,
    *,
    temperature: Optional[torch.Tensor] = None,
) -> List[torch.Tensor]:
    """``[tile_max, tile_sum]``, each fp32 ``[rows, num_tiles]``, of materialised logits.

    Same signature, checks and messages as ``_C.hip_deterministic_logp_tile_stats``
    (csrc/bindings/ops.cpp:122-126; csrc/rocm/logprob/hip_deterministic_logp_kernel.hip:550-588).
    ``temperature`` (fp32, one value per row) scales the logits by its reciprocal in registers.
    """
    code = _logits_dtype_code(logits)
    if not (int(vocab_start) >= 0 and int(real_vocab) > 0 and int(num_tiles) > 0):
        raise RuntimeError("invalid vocabulary metadata")
    rows, local_vocab = logits.shape
    if not (local_vocab > 0 and local_vocab % int(num_tiles) == 0):
        raise RuntimeError("local_vocab must be divisible by num_tiles")
    if int(num_tiles) > 65535:
        raise RuntimeError("num_tiles must fit the launch grid")
    src = _row_contiguous(logits)
    tile_max = torch.empty((rows, int(num_tiles)), dtype=torch.float32, device=logits.device)
    tile_sum = torch.empty((rows, int(num_tiles)), dtype=torch.float32, device=logits.device)
    if rows == 0:
        return [tile_max, tile_sum]
    temp = None
    if temperature is not None:
        if temperature.numel() != rows:
            raise RuntimeError("temperature must have one value per row")
        temp = temperature.reshape(-1).to(device=logits.device, dtype=torch.float32).contiguous()
    with _on(logits.device):
        status = _lib.load().rlk_logits_tile_stats(
            src.data_ptr(), code, src.stride(0), temp.data_ptr() if temp is not None else None, rows, local_vocab,
            int(vocab_start), int(real_vocab), int(num_tiles), tile_max.data_ptr(), tile_sum.data_ptr(),
            _stream_handle(logits.device),
        )  # fmt: skip
    _lib.check(status, "rlk_logits_tile_stats failed")
    return [tile_max, tile_sum]


def hip_deterministic_logp_from_logits(
    logits: torch.Tensor,
    target: torch.Tensor,
    vocab_start: int,
    real_vocab: int,
    num_tiles: int,
    *,
    temperature: Optional[torch.Tensor] = None,
) -> List[torch.Tensor]:
    """``[logp, lse]`` (fp32 ``[rows]``) from materialised logits: tile statistics, ascending
    tile merge and target gather in one pass over the logits. ``target`` holds global ids."""
    code = _logits_dtype_code(logits)
    if not (int(vocab_start) >= 0 and int(real_vocab) > 0 and int(num_tiles) > 0):
        raise RuntimeError("invalid vocabulary metadata")
    rows, local_vocab = logits.shape
    if not (local_vocab > 0 and local_vocab % int(num_tiles) == 0):
        raise RuntimeError("local_vocab must be divisible by num_tiles")
    if target.numel() != rows:
        raise RuntimeError("target must have one id per row")
    src = _row_contiguous(logits)
    logp = torch.empty((rows,), dtype=torch.float32, device=logits.device)
    lse = torch.empty((rows,), dtype=torch.float32, device=logits.device)
    if rows == 0:
        return [logp, lse]
    target_i64 = target.reshape(-1).to(device=logits.device, dtype=torch.int64).contiguous()
    temp = None
    if temperature is not None:
        if temperature.numel() != rows:
            raise RuntimeError("temperature must have one value per row")
        temp = temperature.reshape(-1).to(device=logits.device, dtype=torch.float32).contiguous()
    lib = _lib.load()
    ws_bytes = int(lib.rlk_logp_from_logits_workspace_bytes(rows, int(num_tiles)))
    workspace = torch.empty((ws_bytes // 4,), dtype=torch.float32, device=logits.device)
    with _on(logits.device):
        status = lib.rlk_logp_from_logits(
            src.data_ptr(), code, src.stride(0), target_i64.data_ptr(), temp.data_ptr() if temp is not None else None,
            rows, local_vocab, int(vocab_start), int(real_vocab), int(num_tiles), logp.data_ptr(), lse.data_ptr(),
            workspace.data_ptr(), ws_bytes, _stream_handle(logits.device),
        )  # fmt: skip
    _lib.check(status, "rlk_logp_from_logits failed")
    return [logp, lse]


def hip_deterministic_logp_backward(
    logits: torch.Tensor,
    lse: torch.Tensor,
    coef_logp: torch.Tensor,
    coef_lse: torch.Tensor,
    target_local: torch.Tensor,
    vocab_start: int,
    real_vocab: int,
    has_lse_grad: bool,
    *,
    temperature: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``grad = coef_logp * (onehot - p) + coef_lse * p`` in the dtype of ``logits``.

    Same signature, checks and messages as ``_C.hip_deterministic_logp_backward``
    (csrc/bindings/ops.cpp:127-135; hip_deterministic_logp_kernel.hip:590-640).
    """
    code = _logits_dtype_code(logits)
    if not (int(vocab_start) >= 0 and int(real_vocab) > 0):
        raise RuntimeError("invalid vocabulary metadata")
    src = _row_contiguous(logits)
    rows, local_vocab = src.shape

    def _check_row_vector(t: torch.Tensor, dtype: torch.dtype, name: str) -> None:
        if not t.is_cuda or t.device != src.device:
            raise RuntimeError(f"{name} must live on the logits device")
        if t.dtype != dtype:
            raise RuntimeError(f"{name} has the wrong dtype")
        if t.dim() != 1 or t.size(0) != rows:
            raise RuntimeError(f"{name} must have one entry per token")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")

    _check_row_vector(lse, torch.float32, "lse")
    _check_row_vector(coef_logp, torch.float32, "coef_logp")
    _check_row_vector(coef_lse, torch.float32, "coef_lse")
    _check_row_vector(target_local, torch.int64, "target_local")
    grad = torch.empty((rows, local_vocab), dtype=src.dtype, device=src.device)
    if rows == 0 or local_vocab == 0:
        return grad
    temp = None
    if temperature is not None:
        if temperature.numel() != rows:
            raise RuntimeError("temperature must have one value per row")
        temp = temperature.reshape(-1).to(device=src.device, dtype=torch.float32).contiguous()
    with _on(src.device):
        status = _lib.load().rlk_logits_logp_backward(
            src.data_ptr(), code, src.stride(0), lse.data_ptr(), coef_logp.data_ptr(),
            coef_lse.data_ptr() if has_lse_grad else None, target_local.data_ptr(),
            temp.data_ptr() if temp is not None else None, grad.data_ptr(), grad.stride(0), rows, local_vocab,
            int(vocab_start), int(real_vocab), _stream_handle(src.device),
        )  # fmt: skip
    _lib.check(status, "rlk_logits_logp_backward failed")
    return grad


def _check_act(t: torch.Tensor, name: str) -> None:
    """Checks of check_cuda_contig (csrc/cuda/activation/activation.cu:145-156)."""
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if t.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise RuntimeError(f"{name} must be fp16, bf16, or fp32, got {t.dtype}")


def _act_dtype_code(t: torch.Tensor) -> int:
    return {torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_FP16, torch.float32: _lib.DTYPE_FP32}[t.dtype]


def _same_act_dtype(first: torch.Tensor, first_name: str, other: torch.Tensor, other_name: str) -> None:
    if other.dtype != first.dtype:
        raise RuntimeError(f"{other_name} and {first_name} must share dtype")


def _rows_cols(t: torch.Tensor) -> tuple:
    cols = t.size(-1) if t.dim() else 1
    return (t.numel() // cols if cols else 0), cols


def swiglu_forward(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``silu(gate) * up`` elementwise (csrc/bindings/ops.cpp:400-402; activation.cu:211-240)."""
    _check_act(gate, "gate")
    _check_act(up, "up")
    if gate.device != up.device:
        raise RuntimeError(f"gate and up must be on the same CUDA device, got {gate.device} and {up.device}")
    if gate.shape != up.shape:
        raise RuntimeError("gate and up must share shape")
    _same_act_dtype(gate, "gate", up, "up")
    y = torch.empty_like(gate)
    rows, cols = _rows_cols(gate)
    if gate.numel():
        with _on(gate.device):
            status = _lib.load().rlk_swiglu_fwd(
                gate.data_ptr(), cols, up.data_ptr(), cols, y.data_ptr(), cols, rows, cols,
                _act_dtype_code(gate), _stream_handle(gate.device),
            )  # fmt: skip
        _lib.check(status, "rlk_swiglu_fwd failed")
    return y


def swiglu_backward(dy: torch.Tensor, gate: torch.Tensor, up: torch.Tensor) -> List[torch.Tensor]:
    """``[d_gate, d_up]`` of :func:`swiglu_forward` (ops.cpp:404-409; activation.cu:242-284)."""
    _check_act(dy, "dy")
    _check_act(gate, "gate")
    _check_act(up, "up")
    if gate.shape != up.shape:
        raise RuntimeError("gate and up must share shape")
    if dy.shape != gate.shape:
        raise RuntimeError("dy and gate must share shape")
    _same_act_dtype(gate, "gate", dy, "dy")
    _same_act_dtype(gate, "gate", up, "up")
    d_gate, d_up = torch.empty_like(gate), torch.empty_like(up)
    rows, cols = _rows_cols(gate)
    if gate.numel():
        with _on(gate.device):
            status = _lib.load().rlk_swiglu_bwd(
                dy.data_ptr(), cols, gate.data_ptr(), cols, up.data_ptr(), cols, d_gate.data_ptr(), cols,
                d_up.data_ptr(), cols, rows, cols, _act_dtype_code(gate), _stream_handle(gate.device),
            )  # fmt: skip
        _lib.check(status, "rlk_swiglu_bwd failed")
    return [d_gate, d_up]


def swiglu_packed_forward(gate_up: torch.Tensor) -> torch.Tensor:
    """SwiGLU of a packed ``[rows, 2 * intermediate]`` projection -> ``[rows, intermediate]``
    (ops.cpp:411-413; activation.cu:286-320)."""
    _check_act(gate_up, "gate_up")
    if gate_up.dim() != 2:
        raise RuntimeError("gate_up must be [rows, 2 * intermediate]")
    if gate_up.size(1) % 2:
        raise RuntimeError("gate_up width must be even")
    rows, width = gate_up.size(0), gate_up.size(1) // 2
    y = torch.empty((rows, width), dtype=gate_up.dtype, device=gate_up.device)
    if y.numel():
        base = gate_up.data_ptr()
        with _on(gate_up.device):
            status = _lib.load().rlk_swiglu_fwd(
                base, 2 * width, base + gate_up.element_size() * width, 2 * width, y.data_ptr(), width, rows, width,
                _act_dtype_code(gate_up), _stream_handle(gate_up.device),
            )  # fmt: skip
        _lib.check(status, "rlk_swiglu_fwd failed")
    return y


def swiglu_packed_backward(dy: torch.Tensor, gate_up: torch.Tensor) -> List[torch.Tensor]:
    """``[d_gate, d_up]`` (each ``[rows, intermediate]``) of :func:`swiglu_packed_forward`
    (ops.cpp:415-419; activation.cu:322-370)."""
    _check_act(dy, "dy")
    _check_act(gate_up, "gate_up")
    if gate_up.dim() != 2 or dy.dim() != 2:
        raise RuntimeError("gate_up must be [rows, 2 * intermediate]")
    if gate_up.size(1) % 2:
        raise RuntimeError("gate_up width must be even")
    rows, width = gate_up.size(0), gate_up.size(1) // 2
    if tuple(dy.shape) != (rows, width):
        raise RuntimeError("dy must be [rows, intermediate]")
    _same_act_dtype(gate_up, "gate_up", dy, "dy")
    d_gate = torch.empty((rows, width), dtype=gate_up.dtype, device=gate_up.device)
    d_up = torch.empty_like(d_gate)
    if d_gate.numel():
        base = gate_up.data_ptr()
        with _on(gate_up.device):
            status = _lib.load().rlk_swiglu_bwd(
                dy.data_ptr(), width, base, 2 * width, base + gate_up.element_size() * width, 2 * width,
                d_gate.data_ptr(), width, d_up.data_ptr(), width, rows, width, _act_dtype_code(gate_up),
                _stream_handle(gate_up.device),
            )  # fmt: skip
        _lib.check(status, "rlk_swiglu_bwd failed")
    return [d_gate, d_up]


def det_gemm_swiglu(a: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``swiglu(a @ weight[:I].T, a @ weight[I:].T)`` for a packed ``[2 I, K]`` gate/up weight.

    Equals ``swiglu_packed_forward(det_gemm_fwd_rhs_transposed(a, weight))`` bit for bit; with
    contiguous operands, ``K % 64 == 0`` and more than 16 rows the ``[M, 2 I]`` projection is
    never written (rl_engine/backends/rocm/gemm/swiglu_gemm.py:36-86).
    """
    _check_in(a, "A")
    _check_in(weight, "weight")
    if a.dim() != 2 or weight.dim() != 2:
        raise RuntimeError("det_gemm_swiglu: expect a[M,K] and weight[2I,K]")
    if weight.size(1) != a.size(1):
        raise RuntimeError("det_gemm_swiglu: K mismatch")
    if weight.size(0) % 2:
        raise RuntimeError("det_gemm_swiglu: packed gate/up weight needs an even number of rows")
    a_c = a if a.stride(1) == 1 else a.contiguous()
    w_c = weight if weight.stride(1) == 1 else weight.contiguous()
    m, k = a_c.shape
    inter = w_c.size(0) // 2
    if out is None:
        out = torch.empty((m, inter), dtype=_BF16, device=a.device)
    elif tuple(out.shape) != (m, inter) or out.dtype != _BF16 or out.stride(1) != 1:
        raise RuntimeError(f"det_gemm_swiglu: out must be a row-contiguous bf16 [{m}, {inter}] tensor")
    if m == 0 or inter == 0:
        return out
    lib = _lib.load()
    ws_bytes = int(lib.rlk_det_gemm_swiglu_workspace_bytes(a_c.data_ptr(), a_c.stride(0), w_c.data_ptr(), w_c.stride(0), m, inter, k))
    workspace = torch.empty((ws_bytes // 2,), dtype=_BF16, device=a.device) if ws_bytes else None
    with _on(a.device):
        status = lib.rlk_det_gemm_swiglu_bf16(
            a_c.data_ptr(), a_c.stride(0), w_c.data_ptr(), w_c.stride(0), out.data_ptr(), out.stride(0),
            workspace.data_ptr() if workspace is not None else None, ws_bytes, m, inter, k, _stream_handle(a.device),
        )  # fmt: skip
    _lib.check(status, "rlk_det_gemm_swiglu_bf16 failed")
    return out


def grpo_ratio_kl_loss(
    logp: torch.Tensor,
    old_logp: torch.Tensor,
    ref_logp: torch.Tensor,
    advantages: torch.Tensor,
    mask: Optional[torch.Tensor],
    clip_eps: float,
    beta: float,
) -> List[torch.Tensor]:
    """GRPO epilogue on log-probs -> ``[loss3, ratio, k3]`` (loss3 = loss, policy, kl).

    ``logp`` / ``old_logp`` / ``ref_logp`` are fp32 ``[rollouts, tokens]``,
    ``advantages`` fp32 ``[rollouts]``, ``mask`` bool/uint8 ``[rollouts, tokens]`` or None.
    """
    for name, t in (("logp", logp), ("old_logp", old_logp), ("ref_logp", ref_logp), ("advantages", advantages)):
        if not t.is_cuda:
            raise RuntimeError(f"grpo_ratio_kl_loss: {name} must be a CUDA tensor")
        if t.dtype != torch.float32:
            raise RuntimeError(f"grpo_ratio_kl_loss: {name} must be fp32")
    if logp.dim() != 2 or old_logp.shape != logp.shape or ref_logp.shape != logp.shape:
        raise RuntimeError("grpo_ratio_kl_loss: logp, old_logp, ref_logp must share one [rollouts, tokens] shape")
    rollouts, tokens = logp.shape
    if advantages.numel() != rollouts:
        raise RuntimeError("grpo_ratio_kl_loss: one advantage per rollout expected")
    logp_c, old_c, ref_c = logp.contiguous(), old_logp.contiguous(), ref_logp.contiguous()
    adv_c = advantages.reshape(-1).contiguous()
    mask_u8 = None
    if mask is not None:
        if tuple(mask.shape) != (rollouts, tokens):
            raise RuntimeError("grpo_ratio_kl_loss: mask shape must match logp")
        # any non-zero mask value keeps the token (mask.bool(), rl_engine/reference/definitions.py:50-70)
        mask_u8 = mask.to(device=logp.device).bool().to(torch.uint8).contiguous()
    lib = _lib.load()
    ratio = torch.empty_like(logp_c)
    k3 = torch.empty_like(logp_c)
    out3 = torch.empty((3,), dtype=torch.float32, device=logp.device)
    ws_bytes = int(lib.rlk_grpo_workspace_bytes(rollouts))
    workspace = torch.empty((max(ws_bytes, 4) // 4,), dtype=torch.float32, device=logp.device)
    with _on(logp.device):
        status = lib.rlk_grpo_ratio_kl_loss(
            logp_c.data_ptr(),
            old_c.data_ptr(),
            ref_c.data_ptr(),
            adv_c.data_ptr(),
            mask_u8.data_ptr() if mask_u8 is not None else None,
            rollouts,
            tokens,
            float(clip_eps),
            float(beta),
            ratio.data_ptr(),
            k3.data_ptr(),
            out3.data_ptr(),
            workspace.data_ptr(),
            ws_bytes,
            _stream_handle(logp.device),
        )
    _lib.check(status, "rlk_grpo_ratio_kl_loss failed")
    return [out3, ratio, k3]
