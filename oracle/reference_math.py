"""CPU oracle for the deterministic dense path -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module. The product (``librlk_gfx950.so`` and the
``rl_engine`` package) never does, and fails loudly instead of falling back.

It restates, with numpy on the host, the arithmetic of the reference
(ryankert01/RL-Kernel) for three things:

* the round-once bf16 GEMM (``det_gemm``),
* the linear-LogP (lm_head GEMM -> log-sum-exp over the vocabulary -> target gather),
* the GRPO ratio / k3-KL / clipped-surrogate epilogue,

each function citing the reference file:line it follows. bf16 tensors travel as
numpy ``uint16`` bit patterns so that rounding is explicit.

Pinning (which check fixes which function; see tests/test_oracle.py):

* ``f32_to_bf16`` / ``bf16_to_f32``: known bit patterns, round-to-nearest-even ties.
* ``det_gemm_ref`` / C ``oracle_gemm_seq_f32``: K=1 exact products, one-hot rows,
  power-of-two integer sums, the fp64 brute force, and the reference's own
  equality demand at [4,16]x[9,16] (tests/test_musa_det_gemm.py:133-140).
* ``k_tree_gemm``: K <= 32 reduces to ``det_gemm`` of one leaf; element- and
  leaf-space trees agree when K/32 is a power of two and differ at K=12288 by the
  leaf widths the reference states (tests/ops/gemm/test_det_gemm.py:282-283).
* ``linear_logp_chunked`` / ``linear_logp_dense``: uniform logits (logp = -log V),
  probabilities summing to one, the fp64 brute force, agreement between the
  chunked and the dense form, chunk-size independence.
* ``linear_logp_dlogits`` / ``linear_logp_backward``: central finite differences of
  ``linear_logp_f64`` in hidden, weight and bias; rows of d(logits) summing to
  ``grad_lse / temperature``; zero hidden gradient when every weight row is the same.
* ``logits_tile_stats`` / ``merge_tile_partials`` / ``logp_from_logits`` /
  ``logits_logp_backward``: scipy's logsumexp on the real columns, tile-count
  independence of the merged lse, the all-padding tile identity, central finite
  differences of logsumexp and the gathered logit.
* ``swiglu`` / ``swiglu_backward`` / ``swiglu_packed`` / ``gated_ffn``: silu(0) = 0,
  silu(x) -> x and -> 0 in the tails, linearity in ``up``, central finite differences of
  the fp64 formula, and ``gated_ffn`` against an fp64 evaluation.
* ``grpo_ratio_kl_loss`` / ``group_advantages`` / ``masked_mean``: the reference's
  hand examples (tests/reference/test_reference_ops.py:77-98,
  tests/ops/loss/test_grpo_loss.py:112-119) and closed forms (old == logp gives
  ratio 1, ref == logp gives k3 0, clip saturation).

* ``det_gemm_ref_torch`` / ``native_gemm_torch`` / ``linear_logp_chunked_torch`` (the torch forms the CPU baseline
  times): against the numpy forms on seeded inputs (tests/test_oracle.py).

One function is "parity unpinned" against the reference: ``det_gemm_seq_f32`` with general fp32 operands
(``oracle_gemm_seq_fma_f32in``). Its step is one fused multiply-add; the sources it follows
(csrc/musa/det_gemm.mu:43-44, ``_det_gemm_fp32_kernel``) leave fusion to their compilers and the reference holds
no fixture with fp32 operands. The function itself is pinned (exact small-integer products, an order-sensitive
case, a case where fused and unfused steps differ); with bf16-valued operands products are exact and the
question does not arise. Every other function here is pinned against the reference as listed above.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from pathlib import Path

import numpy as np

ORACLE_DIR = Path(__file__).resolve().parent
_C_SOURCE = ORACLE_DIR / "rlk_oracle.c"
_C_LIB = ORACLE_DIR / "librlk_oracle.so"

# ---------------------------------------------------------------------------
# bf16 <-> fp32
# ---------------------------------------------------------------------------


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns, round to nearest even, NaN -> quiet NaN.

    The rounding torch applies in ``.to(torch.bfloat16)``, which is the single
    rounding of the round-once contract (rl_engine/reference/embedding/matmul.py:22-28).
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    out = np.where(nan, (u >> 16) | 0x0040, rounded)
    return out.astype(np.uint16)


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << 16).view(np.float32)


def randn_bf16(rng: np.random.Generator, shape, scale: float = 1.0) -> np.ndarray:
    """Seeded N(0, scale^2) values generated in fp32 and rounded to bf16 bits."""
    return f32_to_bf16(rng.standard_normal(shape, dtype=np.float32) * np.float32(scale))


# ---------------------------------------------------------------------------
# C restatement (sequential fp32 / fp64 / k-tree GEMMs)
# ---------------------------------------------------------------------------


def build_c_oracle(force: bool = False) -> Path:
    """Compile rlk_oracle.c with gcc into librlk_oracle.so next to it."""
    if force or not _C_LIB.exists() or _C_LIB.stat().st_mtime < _C_SOURCE.stat().st_mtime:
        cmd = [
            os.environ.get("CC", "gcc"),
            "-O2",
            "-fPIC",
            "-shared",
            "-ffp-contract=off",
            "-o",
            str(_C_LIB),
            str(_C_SOURCE),
            "-lm",
        ]
        subprocess.run(cmd, check=True)
    return _C_LIB


_clib = None


def _c():
    global _clib
    if _clib is None:
        if not _C_LIB.exists():
            build_c_oracle()
        lib = ctypes.CDLL(str(_C_LIB))
        u16p = ctypes.POINTER(ctypes.c_uint16)
        lib.oracle_gemm_seq_f32.argtypes = [u16p, u16p, u16p, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        lib.oracle_gemm_seq_f32.restype = None
        lib.oracle_gemm_f64.argtypes = [
            u16p,
            u16p,
            ctypes.POINTER(ctypes.c_double),
            ctypes.c_int,
            ctypes.c_int,
            ctypes.c_int,
        ]
        lib.oracle_gemm_f64.restype = None
        lib.oracle_gemm_ktree.argtypes = [u16p, u16p, u16p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        lib.oracle_gemm_ktree.restype = None
        _clib = lib
    return _clib


def _u16(a: np.ndarray):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16))


def _prep(a_bits: np.ndarray, bt_bits: np.ndarray):
    a = np.ascontiguousarray(a_bits, dtype=np.uint16)
    bt = np.ascontiguousarray(bt_bits, dtype=np.uint16)
    if a.ndim != 2 or bt.ndim != 2 or a.shape[1] != bt.shape[1]:
        raise ValueError(f"expected A[M,K] and Bt[N,K], got {a.shape} and {bt.shape}")
    return a, bt


def det_gemm_seq(a_bits: np.ndarray, bt_bits: np.ndarray) -> np.ndarray:
    """Round-once GEMM, strictly sequential fp32 sum (csrc/musa/det_gemm.mu:25-48)."""
    a, bt = _prep(a_bits, bt_bits)
    out = np.empty((a.shape[0], bt.shape[0]), dtype=np.uint16)
    _c().oracle_gemm_seq_f32(_u16(a), _u16(bt), _u16(out), a.shape[0], bt.shape[0], a.shape[1])
    return out


def det_gemm_seq_f32(a: np.ndarray, bt: np.ndarray) -> np.ndarray:
    """fp32 ``a[M,K] @ bt[N,K].T`` by one fused multiply-add per k, k ascending from +0, unrounded fp32 result
    (the float instantiation of csrc/musa/det_gemm.mu:25-48; the role of _det_gemm_fp32_kernel,
    rl_engine/backends/shared/triton/gemm/det_gemm.py:680-749). Operands are float32 arrays (widen bf16
    bit patterns with bf16_to_f32 first)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    bt = np.ascontiguousarray(bt, dtype=np.float32)
    assert a.ndim == 2 and bt.ndim == 2 and a.shape[1] == bt.shape[1]
    out = np.empty((a.shape[0], bt.shape[0]), dtype=np.float32)
    f32p = ctypes.POINTER(ctypes.c_float)
    lib = _c()
    lib.oracle_gemm_seq_fma_f32in.argtypes = [f32p, f32p, f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int]
    lib.oracle_gemm_seq_fma_f32in.restype = None
    lib.oracle_gemm_seq_fma_f32in(a.ctypes.data_as(f32p), bt.ctypes.data_as(f32p), out.ctypes.data_as(f32p), a.shape[0], bt.shape[0], a.shape[1])
    return out


def det_gemm_f64(a_bits: np.ndarray, bt_bits: np.ndarray) -> np.ndarray:
    """The exact products accumulated in fp64, unrounded (brute-force anchor)."""
    a, bt = _prep(a_bits, bt_bits)
    out = np.empty((a.shape[0], bt.shape[0]), dtype=np.float64)
    _c().oracle_gemm_f64(
        _u16(a), _u16(bt), out.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), a.shape[0], bt.shape[0], a.shape[1]
    )
    return out


def k_tree_gemm(a_bits: np.ndarray, bt_bits: np.ndarray, *, leaf_space: bool = False) -> np.ndarray:
    """Legacy k-tree contract: 32-wide fp32 leaves rounded to bf16, bf16 midpoint tree.

    Element-space split: tests/ops/gemm/test_det_gemm.py:156-168,
    csrc/cuda/gemm/det_gemm_kernel.cu:74-85. Leaf-space split:
    rl_engine/reference/gemm/det_gemm.py:29-60.
    """
    a, bt = _prep(a_bits, bt_bits)
    out = np.empty((a.shape[0], bt.shape[0]), dtype=np.uint16)
    _c().oracle_gemm_ktree(_u16(a), _u16(bt), _u16(out), a.shape[0], bt.shape[0], a.shape[1], int(leaf_space))
    return out


# ---------------------------------------------------------------------------
# det_gemm
# ---------------------------------------------------------------------------


def det_gemm_ref_f32(a_bits: np.ndarray, bt_bits: np.ndarray) -> np.ndarray:
    """``a.float() @ b.float()`` before the rounding: fp32 [M,N].

    NativeMatmulOp.forward_fp32, rl_engine/reference/embedding/matmul.py:22-28.
    The fp32 summation order inside the BLAS is implementation defined; the
    round-once family only fixes that there is one rounding at the end.
    """
    a, bt = _prep(a_bits, bt_bits)
    return bf16_to_f32(a) @ bf16_to_f32(bt).T


def det_gemm_ref(a_bits: np.ndarray, bt_bits: np.ndarray) -> np.ndarray:
    """``(a.float() @ b.float()).to(bf16)`` as bf16 bits.

    The round-once GEMM of the reference: NativeMatmulOp
    (rl_engine/reference/embedding/matmul.py:10-28), NativeGemmOp on upcast inputs
    (rl_engine/reference/gemm/det_gemm.py:15-23) and the MFMA contract
    (rl_engine/backends/rocm/gemm/mfma_gemm.py:5-13). ``bt_bits`` is the right-hand
    side stored [N,K] (the native linear weight), i.e. the result is a @ bt.T.
    """
    return f32_to_bf16(det_gemm_ref_f32(a_bits, bt_bits))


def bf16_ulp_distance(x_bits: np.ndarray, y_bits: np.ndarray) -> np.ndarray:
    """Distance in bf16 units in the last place between two bit-pattern arrays."""

    def ordered(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)

    return np.abs(ordered(np.asarray(x_bits)) - ordered(np.asarray(y_bits)))


# ---------------------------------------------------------------------------
# The same two paths written with torch on the CPU, the way the reference itself writes them. They exist for
# the CPU baseline (timed on the host cores next to the GPU) and are pinned against the numpy forms above.
# ---------------------------------------------------------------------------


def cpu_model_string() -> str:
    """The host CPU's model name (first ``model name`` line of /proc/cpuinfo), or ``"unknown"``."""
    try:
        for line in Path("/proc/cpuinfo").read_text().splitlines():
            if line.lower().startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def det_gemm_ref_torch(a, bt):
    """``(a.float() @ b.float()).to(torch.bfloat16)`` on CPU bf16 tensors ``a[M,K]``, ``bt[N,K]`` (the native linear
    weight, b = bt.t()): NativeMatmulOp, rl_engine/reference/embedding/matmul.py:22-28."""
    import torch

    return (a.float() @ bt.float().t()).to(torch.bfloat16)


def native_gemm_torch(a, bt):
    """``torch.matmul(a, b)`` on the bf16 tensors themselves: NativeGemmOp, rl_engine/reference/gemm/det_gemm.py:15-23.
    Its summation order (and whether partial sums are rounded to bf16) is the CPU BLAS's own."""
    import torch

    return torch.matmul(a, bt.t())


def linear_logp_chunked_torch(h, w, target, *, chunk_elems: int = 1 << 24):
    """_chunked_local_linear_logp_stats (rl_engine/reference/logprob/linear_logp.py:259-308) in torch on CPU tensors:
    the recurrence of ``linear_logp_chunked`` above, operands upcast to fp32 (:31-36). Returns ``(logp, lse)``."""
    import torch

    h32, n, v = h.float(), h.shape[0], w.shape[0]
    target = target.long().reshape(-1)
    local_max = torch.full((n,), float("-inf"))
    local_sum = torch.zeros((n,))
    target_logit = torch.zeros((n,))
    rows = torch.arange(n)
    chunk = max(1, min(v, chunk_elems // max(n, 1)))
    for v0 in range(0, v, chunk):
        v1 = min(v0 + chunk, v)
        logits = h32 @ w[v0:v1].float().t()
        new_max = torch.maximum(local_max, logits.max(dim=-1).values)
        local_sum = local_sum * torch.exp(local_max - new_max) + torch.exp(logits - new_max[:, None]).sum(dim=-1)
        local_max = new_max
        owns = (target >= v0) & (target < v1)
        safe = (target - v0).clamp(0, v1 - v0 - 1)
        target_logit = torch.where(owns, logits[rows, safe], target_logit)
    lse = local_max + torch.log(local_sum)
    return target_logit - lse, lse


# ---------------------------------------------------------------------------
# linear-LogP
# ---------------------------------------------------------------------------

BWD_CHUNK_ELEMS = 1 << 24  # rl_engine/reference/logprob/linear_logp.py:16


def linear_logp_chunked(
    h_bits: np.ndarray,
    w_bits: np.ndarray,
    target: np.ndarray,
    bias: np.ndarray | None = None,
    *,
    vocab_start_index: int = 0,
    chunk_elems: int = BWD_CHUNK_ELEMS,
):
    """Chunked online log-sum-exp in ascending vocabulary order.

    Restates _chunked_local_linear_logp_stats
    (rl_engine/reference/logprob/linear_logp.py:259-308): vocabulary chunk of
    ``max(1, min(V, chunk_elems // N))`` weight rows (:281); per chunk fp32 logits
    from the fp32-upcast operands (:31-36, :279); ``tile_max``,
    ``new_max = max(m, tile_max)``,
    ``s = s * exp(m - new_max) + sum(exp(z - new_max))`` (:292-297); the target
    logit is captured by the owning chunk (:299-304). The caller forms
    ``lse = max + log(sum)`` and ``logp = target_logit - lse`` (:561-562).

    Returns ``(logp, lse, local_max, local_sum, target_logit)`` as fp32 arrays.
    """
    h = bf16_to_f32(np.ascontiguousarray(h_bits, dtype=np.uint16))
    w = bf16_to_f32(np.ascontiguousarray(w_bits, dtype=np.uint16))
    target = np.asarray(target, dtype=np.int64).reshape(-1)
    n, v = h.shape[0], w.shape[0]
    if target.shape[0] != n:
        raise ValueError("target must have one id per hidden row")
    local_max = np.full((n,), -np.inf, dtype=np.float32)
    local_sum = np.zeros((n,), dtype=np.float32)
    target_logit = np.zeros((n,), dtype=np.float32)
    rows = np.arange(n)
    chunk = max(1, min(v, chunk_elems // max(n, 1)))
    for v0 in range(0, v, chunk):
        v1 = min(v0 + chunk, v)
        logits = h @ w[v0:v1].T
        if bias is not None:
            logits = logits + np.asarray(bias, dtype=np.float32)[v0:v1]
        logits = logits.astype(np.float32, copy=False)
        tile_max = logits.max(axis=-1)
        new_max = np.maximum(local_max, tile_max)
        with np.errstate(invalid="ignore"):
            scale = np.exp(local_max - new_max)
        local_sum = (local_sum * scale + np.exp(logits - new_max[:, None]).sum(axis=-1, dtype=np.float32)).astype(
            np.float32
        )
        local_max = new_max
        g0 = vocab_start_index + v0
        g1 = vocab_start_index + v1
        owns = (target >= g0) & (target < g1)
        safe = np.clip(target - g0, 0, max(v1 - v0 - 1, 0))
        target_logit = np.where(owns, logits[rows, safe], target_logit).astype(np.float32)
    lse = (local_max + np.log(local_sum)).astype(np.float32)
    logp = (target_logit - lse).astype(np.float32)
    return logp, lse, local_max, local_sum, target_logit


def linear_logp_dense(
    h_bits: np.ndarray,
    w_bits: np.ndarray,
    target: np.ndarray,
    bias: np.ndarray | None = None,
    *,
    temperature: np.ndarray | float | None = None,
    real_vocab_size: int = -1,
):
    """``log_softmax(F.linear(h, W, b).float())[target]`` on fp32-upcast inputs.

    NativeLinearLogpOp.apply, rl_engine/reference/logprob/linear_logp.py:790-796,
    called the way the reference's tests call it (``.float()`` inputs,
    tests/ops/logprob/test_linear_logp.py:615,715). ``temperature`` and
    ``real_vocab_size`` follow the strict contract: padded lanes are -inf and the
    logits are multiplied by ``1 / temperature`` in fp32
    (rl_engine/backends/shared/triton/logprob/linear_logp.py:251-275, 351-367).
    Returns ``(logp, lse)`` fp32.
    """
    h = bf16_to_f32(np.ascontiguousarray(h_bits, dtype=np.uint16))
    w = bf16_to_f32(np.ascontiguousarray(w_bits, dtype=np.uint16))
    target = np.asarray(target, dtype=np.int64).reshape(-1)
    logits = (h @ w.T).astype(np.float32)
    if bias is not None:
        logits = logits + np.asarray(bias, dtype=np.float32)
    if real_vocab_size is not None and real_vocab_size >= 0:
        logits[:, real_vocab_size:] = -np.inf
    if temperature is not None:
        inv_t = (np.float32(1.0) / np.broadcast_to(np.asarray(temperature, dtype=np.float32), (h.shape[0],))).astype(
            np.float32
        )
        logits = logits * inv_t[:, None]
    m = logits.max(axis=-1)
    lse = (m + np.log(np.exp(logits - m[:, None]).sum(axis=-1, dtype=np.float32))).astype(np.float32)
    zt = logits[np.arange(h.shape[0]), target]
    return (zt - lse).astype(np.float32), lse


def linear_logp_f64(h_bits, w_bits, target, bias=None, *, temperature=None, real_vocab_size=-1):
    """fp64 brute force of the same quantity (anchor, not a reference restatement)."""
    h = bf16_to_f32(np.ascontiguousarray(h_bits, dtype=np.uint16)).astype(np.float64)
    w = bf16_to_f32(np.ascontiguousarray(w_bits, dtype=np.uint16)).astype(np.float64)
    target = np.asarray(target, dtype=np.int64).reshape(-1)
    logits = h @ w.T
    if bias is not None:
        logits = logits + np.asarray(bias, dtype=np.float32).astype(np.float64)
    if real_vocab_size is not None and real_vocab_size >= 0:
        logits[:, real_vocab_size:] = -np.inf
    if temperature is not None:
        inv_t = np.float32(1.0) / np.broadcast_to(np.asarray(temperature, dtype=np.float32), (h.shape[0],))
        logits = logits * inv_t.astype(np.float64)[:, None]
    m = logits.max(axis=-1)
    lse = m + np.log(np.exp(logits - m[:, None]).sum(axis=-1))
    zt = logits[np.arange(h.shape[0]), target]
    return zt - lse, lse


def linear_logp_dlogits(
    h_bits,
    w_bits,
    target,
    lse,
    grad_logp=None,
    grad_lse=None,
    bias=None,
    *,
    temperature=None,
    real_vocab_size=-1,
    dtype=np.float32,
):
    """d(logits) of the strict linear-LogP, recomputed from a saved ``lse``.

    Restates _det_reference_dlogits
    (rl_engine/backends/shared/triton/logprob/linear_logp.py:522-570): logits from the
    fp32-upcast operands, divided by the temperature, padded lanes -inf;
    ``probs = exp(logits - lse)``; ``dlogits = probs * (grad_lse - grad_logp)``, plus
    ``grad_logp`` at the target column, divided by the temperature once more.
    ``dtype`` float64 turns the same formula into the exact anchor.
    """
    h = bf16_to_f32(np.ascontiguousarray(h_bits, dtype=np.uint16)).astype(dtype)
    w = bf16_to_f32(np.ascontiguousarray(w_bits, dtype=np.uint16)).astype(dtype)
    target = np.asarray(target, dtype=np.int64).reshape(-1)
    n = h.shape[0]
    logits = h @ w.T
    if bias is not None:
        logits = logits + np.asarray(bias, dtype=np.float32).astype(dtype)
    temp = None
    if temperature is not None:
        temp = np.broadcast_to(np.asarray(temperature, dtype=np.float32), (n,)).astype(dtype)
        logits = logits / temp[:, None]
    if real_vocab_size is not None and 0 <= real_vocab_size < logits.shape[1]:
        logits[:, real_vocab_size:] = -np.inf
    probs = np.exp(logits - np.asarray(lse, dtype=dtype).reshape(-1, 1))
    g_logp = np.zeros((n,), dtype=dtype) if grad_logp is None else np.asarray(grad_logp, dtype=np.float32).astype(dtype)
    g_lse = np.zeros((n,), dtype=dtype) if grad_lse is None else np.asarray(grad_lse, dtype=np.float32).astype(dtype)
    dlogits = probs * (g_lse - g_logp)[:, None]
    dlogits[np.arange(n), target] += g_logp
    if temp is not None:
        dlogits = dlogits / temp[:, None]
    return dlogits.astype(dtype)


def linear_logp_backward(
    h_bits,
    w_bits,
    target,
    lse,
    grad_logp=None,
    grad_lse=None,
    bias=None,
    *,
    temperature=None,
    real_vocab_size=-1,
    round_dlogits_to_bf16: bool = True,
):
    """``(grad_hidden, grad_weight, grad_bias, dlogits)`` of the strict linear-LogP.

    ``grad_hidden = dlogits @ W``, ``grad_weight = dlogits.T @ H``,
    ``grad_bias = dlogits.sum(0)``
    (_DetTritonLinearLogpAutograd.backward,
    rl_engine/backends/shared/triton/logprob/linear_logp.py:600-628). With
    ``round_dlogits_to_bf16`` the d(logits) are rounded to the weight dtype before the
    two products, which is the bf16 branch of chunked_linear_logp_backward
    (rl_engine/reference/logprob/linear_logp.py:698-703; its bias gradient sums the
    unrounded values, :704-705). Products accumulate in fp64 here, so what is left to
    the implementation under test is its summation order and the final rounding.
    Gradients are returned as float64 arrays, dlogits as float32.
    """
    dz = linear_logp_dlogits(
        h_bits, w_bits, target, lse, grad_logp, grad_lse, bias, temperature=temperature, real_vocab_size=real_vocab_size
    )
    h = bf16_to_f32(np.ascontiguousarray(h_bits, dtype=np.uint16)).astype(np.float64)
    w = bf16_to_f32(np.ascontiguousarray(w_bits, dtype=np.uint16)).astype(np.float64)
    used = bf16_to_f32(f32_to_bf16(dz)) if round_dlogits_to_bf16 else dz
    used = used.astype(np.float64)
    grad_hidden = used @ w
    grad_weight = used.T @ h
    grad_bias = dz.astype(np.float64).sum(axis=0)
    return grad_hidden, grad_weight, grad_bias, dz


# ---------------------------------------------------------------------------
# log-probabilities from materialised logits (the stage that reuses LM-head logits)
# ---------------------------------------------------------------------------


def logits_tile_stats(logits, vocab_start: int, real_vocab: int, num_tiles: int, *, temperature=None):
    """Per-row, per-tile ``(max, sum of exp(z - max))`` over the real-vocabulary part of a tile.

    Restates hip_tile_stats_kernel
    (csrc/rocm/logprob/hip_deterministic_logp_kernel.hip:389-467): tile ``t`` covers
    columns ``[t * V / tiles, (t + 1) * V / tiles)`` cut at ``real_vocab - vocab_start``;
    an all-padding tile reports ``(-inf, 0)``. ``logits`` is a float array (already
    upcast); ``temperature`` divides it first, as the wrapper does
    (rl_engine/integrations/common/linear_logp.py:777-785). fp32 throughout.
    """
    z = np.asarray(logits, dtype=np.float32)
    rows, v = z.shape
    if v % num_tiles:
        raise ValueError("local_vocab must be divisible by num_tiles")
    if temperature is not None:
        z = (z / np.broadcast_to(np.asarray(temperature, dtype=np.float32), (rows,))[:, None]).astype(np.float32)
    tile = v // num_tiles
    real_cols = max(int(real_vocab) - int(vocab_start), 0)
    tile_max = np.full((rows, num_tiles), -np.inf, dtype=np.float32)
    tile_sum = np.zeros((rows, num_tiles), dtype=np.float32)
    for t in range(num_tiles):
        lo, hi = t * tile, min((t + 1) * tile, real_cols)
        if hi <= lo:
            continue
        part = z[:, lo:hi]
        m = part.max(axis=1)
        tile_max[:, t] = m
        with np.errstate(invalid="ignore"):
            s = np.exp(part - m[:, None]).sum(axis=1, dtype=np.float32)
        tile_sum[:, t] = np.where(np.isfinite(m), s, 0.0)
    return tile_max, tile_sum


def merge_tile_partials(m_all, s_all):
    """``lse = M + log(sum_t s_t * exp(m_t - M))`` with ``M = max_t m_t``.

    _merge_tile_partials, rl_engine/reference/logprob/vocab_parallel_logp.py:355-363.
    """
    m_all = np.asarray(m_all, dtype=np.float32)
    s_all = np.asarray(s_all, dtype=np.float32)
    big = m_all.max(axis=1)
    safe = np.where(big > -np.inf, big, 0.0).astype(np.float32)
    with np.errstate(divide="ignore"):
        terms = s_all * np.exp(m_all - safe[:, None])
        return (big + np.log(terms.sum(axis=1, dtype=np.float32))).astype(np.float32)


def logp_from_logits(logits, target, vocab_start: int, real_vocab: int, num_tiles: int, *, temperature=None):
    """``(logp, lse)`` of materialised logits: tile statistics, merge, target gather
    (_RocmVocabParallelLogprobFunction.forward,
    rl_engine/backends/rocm/logprob/vocab_parallel_logp.py:311-352, single rank)."""
    z = np.asarray(logits, dtype=np.float32)
    rows = z.shape[0]
    m_all, s_all = logits_tile_stats(z, vocab_start, real_vocab, num_tiles, temperature=temperature)
    lse = merge_tile_partials(m_all, s_all)
    local = np.asarray(target, dtype=np.int64).reshape(-1) - int(vocab_start)
    zt = z[np.arange(rows), np.clip(local, 0, z.shape[1] - 1)]
    if temperature is not None:
        zt = (zt / np.broadcast_to(np.asarray(temperature, dtype=np.float32), (rows,))).astype(np.float32)
    owned = (local >= 0) & (local < min(z.shape[1], max(int(real_vocab) - int(vocab_start), 0)))
    zt = np.where(owned, zt, np.float32(0.0)).astype(np.float32)
    return (zt - lse).astype(np.float32), lse


def logits_logp_backward(
    logits, lse, coef_logp, coef_lse, target_local, vocab_start: int, real_vocab: int, *, temperature=None,
    dtype=np.float32,
):  # fmt: skip
    """``grad = coef_logp * (onehot - p) + coef_lse * p`` with ``p = exp(z - lse)`` on finite
    rows, 0 on padded columns (hip_backward_kernel,
    csrc/rocm/logprob/hip_deterministic_logp_kernel.hip:472-540). With a temperature the
    logits are divided by it first and the gradient once more (chain rule)."""
    z = np.asarray(logits, dtype=dtype)
    rows, v = z.shape
    temp = None
    if temperature is not None:
        temp = np.broadcast_to(np.asarray(temperature, dtype=np.float32), (rows,)).astype(dtype)
        z = z / temp[:, None]
    lse = np.asarray(lse, dtype=dtype).reshape(-1)
    finite = np.isfinite(lse)
    with np.errstate(over="ignore", invalid="ignore"):
        p = np.where(finite[:, None], np.exp(z - np.where(finite, lse, 0.0)[:, None]), 0.0)
    g_logp = np.asarray(coef_logp, dtype=dtype).reshape(-1)
    g_lse = np.zeros((rows,), dtype=dtype) if coef_lse is None else np.asarray(coef_lse, dtype=dtype).reshape(-1)
    onehot = np.zeros((rows, v), dtype=dtype)
    hit = np.asarray(target_local, dtype=np.int64).reshape(-1)
    ok = hit >= 0
    onehot[np.arange(rows)[ok], hit[ok]] = 1.0
    grad = g_logp[:, None] * (onehot - p) + g_lse[:, None] * p
    real_end = min(v, max(int(real_vocab) - int(vocab_start), 0))
    grad[:, real_end:] = 0.0
    if temp is not None:
        grad = grad / temp[:, None]
    return grad.astype(dtype)


# ---------------------------------------------------------------------------
# SwiGLU and the gated FFN
# ---------------------------------------------------------------------------


def _sigmoid_f32(x: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        return (np.float32(1.0) / (np.float32(1.0) + np.exp(-x, dtype=np.float32))).astype(np.float32)


def swiglu(gate_bits, up_bits) -> np.ndarray:
    """``silu(gate) * up`` with fp32 math on the bf16 inputs, rounded once to bf16.

    swiglu_forward_kernel / silu_f32, csrc/cuda/activation/activation.cu:20-24, 62-75:
    ``s = 1 / (1 + expf(-g))``, ``y = (g * s) * u``.
    """
    g = bf16_to_f32(np.ascontiguousarray(gate_bits, dtype=np.uint16))
    u = bf16_to_f32(np.ascontiguousarray(up_bits, dtype=np.uint16))
    return f32_to_bf16(((g * _sigmoid_f32(g)).astype(np.float32) * u).astype(np.float32))


def swiglu_backward(dy_bits, gate_bits, up_bits):
    """``(d_gate, d_up)`` as bf16 bits: ``d_up = dy * silu(g)``,
    ``d_gate = dy * u * s * (1 + g * (1 - s))`` (activation.cu:26-31, 77-95)."""
    dy = bf16_to_f32(np.ascontiguousarray(dy_bits, dtype=np.uint16))
    g = bf16_to_f32(np.ascontiguousarray(gate_bits, dtype=np.uint16))
    u = bf16_to_f32(np.ascontiguousarray(up_bits, dtype=np.uint16))
    s = _sigmoid_f32(g)
    d_up = (dy * (g * s)).astype(np.float32)
    d_gate = ((dy * u) * (s * (np.float32(1.0) + g * (np.float32(1.0) - s)))).astype(np.float32)
    return f32_to_bf16(d_gate), f32_to_bf16(d_up)


def swiglu_values(gate, up, dy=None):
    """The same formulas on fp32 arrays, unrounded fp32 results: ``y`` or, with ``dy``,
    ``(d_gate, d_up)``. What the fp16 / fp32 instantiations of the reference kernels
    compute before their cast to the element type (activation.cu:62-95)."""
    g = np.asarray(gate, dtype=np.float32)
    u = np.asarray(up, dtype=np.float32)
    s = _sigmoid_f32(g)
    if dy is None:
        return ((g * s).astype(np.float32) * u).astype(np.float32)
    d = np.asarray(dy, dtype=np.float32)
    d_up = (d * (g * s)).astype(np.float32)
    d_gate = ((d * u) * (s * (np.float32(1.0) + g * (np.float32(1.0) - s)))).astype(np.float32)
    return d_gate, d_up


def swiglu_packed(gate_up_bits) -> np.ndarray:
    """SwiGLU of a packed ``[rows, 2 I]`` projection: columns ``[0, I)`` gate, ``[I, 2 I)`` up
    (swiglu_packed_forward_kernel, activation.cu:97-112)."""
    gu = np.ascontiguousarray(gate_up_bits, dtype=np.uint16)
    width = gu.shape[1] // 2
    return swiglu(gu[:, :width], gu[:, width:])


def gated_ffn(x_bits, gate_up_weight_bits, down_weight_bits) -> np.ndarray:
    """``down(swiglu(x @ W_gu^T))`` with every projection rounded once to bf16
    (_packed_gate_up_inference + det_gemm_linear, rl_engine/backends/rocm/ffn/ffn.py:69-104)."""
    gate_up = det_gemm_ref(x_bits, gate_up_weight_bits)
    return det_gemm_ref(swiglu_packed(gate_up), down_weight_bits)


# ---------------------------------------------------------------------------
# GRPO epilogue
# ---------------------------------------------------------------------------


def compute_policy_ratio(current, old, mask=None):
    """``exp(current - old)`` with masked entries zeroed (rl_engine/reference/definitions.py:82-93)."""
    ratio = np.exp(np.asarray(current, np.float32) - np.asarray(old, np.float32)).astype(np.float32)
    if mask is not None:
        ratio = np.where(np.asarray(mask).astype(bool), ratio, np.float32(0.0))
    return ratio


def compute_reference_kl(current, ref, mask=None):
    """k3 estimator ``exp(d) - d - 1`` with ``d = ref - current`` (definitions.py:96-106)."""
    diff = (np.asarray(ref, np.float32) - np.asarray(current, np.float32)).astype(np.float32)
    kl = (np.exp(diff) - diff - np.float32(1.0)).astype(np.float32)
    if mask is not None:
        kl = np.where(np.asarray(mask).astype(bool), kl, np.float32(0.0))
    return kl


def masked_mean(values, mask=None, eps: float = 1e-8):
    """Masked mean with the denominator clamped at ``eps`` (definitions.py:50-79)."""
    values = np.asarray(values, np.float32)
    if mask is None:
        count = np.float32(values.size)
        total = values.sum(dtype=np.float32)
    else:
        m = np.asarray(mask).astype(bool)
        count = np.float32(m.sum())
        total = np.where(m, values, np.float32(0.0)).sum(dtype=np.float32)
    return np.float32(total / max(count, np.float32(eps)))


def grpo_ratio_kl_loss(logp, old_logp, ref_logp, advantages, mask=None, *, clip_eps=0.2, beta=0.0):
    """Clipped surrogate on per-token log-probs.

    ``logp``/``old_logp``/``ref_logp`` are ``[rollouts, tokens]``, ``advantages``
    is ``[rollouts]``. Follows NativeGRPOLossOp.apply
    (rl_engine/reference/loss/grpo_loss.py:96-125): per-sequence advantages
    broadcast over tokens with masked tokens zeroed, ``-min(ratio * A,
    clamp(ratio, 1 - eps, 1 + eps) * A)``, masked means (:162-168), and
    ``loss = policy_loss + beta * kl``; composed on log-probs exactly as
    tests/e2e/test_rl_kernel_loss_step.py:18-39 does.
    Returns ``(loss, policy_loss, kl, ratio, k3)``.
    """
    logp = np.asarray(logp, np.float32)
    if mask is None:
        mask = np.ones(logp.shape, dtype=bool)
    mask = np.asarray(mask).astype(bool)
    ratio = compute_policy_ratio(logp, old_logp, mask)
    k3 = compute_reference_kl(logp, ref_logp, mask)
    adv = np.broadcast_to(np.asarray(advantages, np.float32).reshape(-1, 1), logp.shape)
    adv = np.where(mask, adv, np.float32(0.0)).astype(np.float32)
    unclipped = ratio * adv
    clipped = np.clip(ratio, np.float32(1.0 - clip_eps), np.float32(1.0 + clip_eps)) * adv
    terms = -np.minimum(unclipped, clipped)
    policy_loss = masked_mean(terms, mask)
    kl = masked_mean(k3, mask)
    loss = np.float32(policy_loss + np.float32(beta) * kl)
    return loss, policy_loss, kl, ratio, k3


def group_advantages(rewards, *, samples_per_prompt=None, group_boundaries=None, eps: float = 1e-6):
    """Per-group reward normalisation with the population variance.

    NativeGRPOLossOp.group_advantages, rl_engine/reference/loss/grpo_loss.py:53-84:
    ``(r - mean_g) / sqrt(max(E[r^2] - mean_g^2, eps^2))``.
    """
    r = np.asarray(rewards, np.float32).reshape(-1)
    if (samples_per_prompt is None) == (group_boundaries is None):
        raise ValueError("give exactly one of samples_per_prompt / group_boundaries")
    if samples_per_prompt is not None:
        bounds = list(range(0, r.size + 1, int(samples_per_prompt)))
    else:
        # only the differences count (repeat_interleave over the sizes, grpo_loss.py:189-206)
        raw = [int(b) for b in group_boundaries]
        bounds = [b - raw[0] for b in raw]
    out = np.empty_like(r)
    for lo, hi in zip(bounds[:-1], bounds[1:]):
        g = r[lo:hi]
        count = np.float32(hi - lo)
        mean = g.sum(dtype=np.float32) / count
        var = (g * g).sum(dtype=np.float32) / count - mean * mean
        std = np.sqrt(max(var, np.float32(eps) ** 2))
        out[lo:hi] = (g - mean) / std
    return out
