"""ctypes binding of librlk_gfx950.so (the C ABI declared in include/rlk.h).

The library is looked up next to the package (built in-tree by
``rl-kernel_amd/build.py``). Nothing here computes: a missing library is an
error, never a reason to fall back to another implementation.
"""

from __future__ import annotations

import ctypes
import os
from pathlib import Path

_PKG_ROOT = Path(__file__).resolve().parent.parent
LIB_NAME = "librlk_gfx950.so"

# rlk_status
RLK_OK = 0
RLK_ERR_INVALID_ARGUMENT = -1
RLK_ERR_DEVICE = -2
RLK_ERR_UNSUPPORTED = -3

# rlk_gemm_config
GEMM_CONFIGS = {
    "auto": 0,
    "256x256": 1,
    "256x128": 2,
    "128x128": 3,
    "128x64": 4,
    "64x64": 5,
    "64x16": 6,
    "16x16": 7,
    "stream16_deep": 8,
    "stream16": 9,
    "256x64": 10,
    "64x64_deep": 11,
    "128x64_deep": 12,
    "128x128_deep": 13,
    "stream64": 14,
    "256x256_solo": 15,
    "192x256": 16,
    "shortk": 17,
    "192x128": 18,
}
# OR-ed into a GEMM or LogP configuration: register-staged main loop (bit-neutral).
FORCE_STAGED = 0x100
TREE_LEAF_SPACE = 0x100  # RLK_TREE_CFG_LEAF_SPACE: OR-ed into rlk_tree_config 0 (auto) or 2 (matrix pipe)
NOALLOC_SCRATCH_BYTES = 32 << 20  # RLK_NOALLOC_SCRATCH_BYTES
# rlk_dtype (element types of materialised logits)
DTYPE_BF16, DTYPE_FP16, DTYPE_FP32 = 0, 1, 2
# rlk_logp_config
LOGP_CONFIGS = {"auto": 0, "256": 1, "128": 2, "64": 3, "16": 4, "64_streams": 5, "128_streams": 6, "256_streams": 7}

EXPORTED_SYMBOLS = (
    "rlk_contract_id",
    "rlk_version",
    "rlk_last_error",
    "rlk_det_gemm_bf16",
    "rlk_det_gemm_pick_config",
    "rlk_det_gemm_tree_bf16",
    "rlk_det_gemm_tree_bf16_config",
    "rlk_det_gemm_tree_contract_id",
    "rlk_det_gemm_tree_leaf_space_contract_id",
    "rlk_det_gemm_seq",
    "rlk_det_gemm_seq_contract_id",
    "rlk_linear_logp_contract_id",
    "rlk_linear_logp_split_count",
    "rlk_linear_logp_workspace_bytes",
    "rlk_linear_logp_fwd",
    "rlk_linear_logp_fwd_logits",
    "rlk_linear_logp_fwd_shard",
    "rlk_linear_logp_fwd_noalloc",
    "rlk_linear_logp_bwd_workspace_bytes",
    "rlk_linear_logp_bwd",
    "rlk_logits_tile_stats",
    "rlk_logits_logp_contract_id",
    "rlk_logp_from_logits_workspace_bytes",
    "rlk_logp_from_logits",
    "rlk_logits_logp_backward",
    "rlk_swiglu_fwd",
    "rlk_swiglu_bwd",
    "rlk_det_gemm_swiglu_workspace_bytes",
    "rlk_det_gemm_swiglu_bf16",
    "rlk_grpo_workspace_bytes",
    "rlk_grpo_ratio_kl_loss",
)


class RlkLibraryMissing(RuntimeError):
    """librlk_gfx950.so has not been built."""


def library_path() -> Path:
    override = os.environ.get("RLK_LIBRARY")
    return Path(override) if override else _PKG_ROOT / LIB_NAME


_lib = None


def load() -> ctypes.CDLL:
    """Load the library once and declare every prototype."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not path.exists():
        raise RlkLibraryMissing(
            f"{path} not found: build it with `python rl-kernel_amd/build.py` "
            "(hipcc --offload-arch=gfx950). There is no fallback implementation."
        )
    lib = ctypes.CDLL(str(path))
    c = ctypes
    vp, i64, i32, sz, f32 = c.c_void_p, c.c_int64, c.c_int, c.c_size_t, c.c_float

    lib.rlk_contract_id.restype = c.c_char_p
    lib.rlk_contract_id.argtypes = []
    lib.rlk_version.restype = c.c_char_p
    lib.rlk_version.argtypes = []
    lib.rlk_last_error.restype = c.c_char_p
    lib.rlk_last_error.argtypes = []

    lib.rlk_det_gemm_bf16.restype = i32
    lib.rlk_det_gemm_bf16.argtypes = [vp, i64, i64, vp, i64, i64, vp, i64, i32, i32, i32, i32, i32, vp]
    lib.rlk_det_gemm_tree_bf16.restype = i32
    lib.rlk_det_gemm_tree_bf16.argtypes = [vp, i64, i64, vp, i64, i64, vp, i64, i32, i32, i32, vp]
    lib.rlk_det_gemm_tree_bf16_config.restype = i32
    lib.rlk_det_gemm_tree_bf16_config.argtypes = [vp, i64, i64, vp, i64, i64, vp, i64, i32, i32, i32, i32, vp]
    lib.rlk_det_gemm_tree_contract_id.restype = c.c_char_p
    lib.rlk_det_gemm_tree_contract_id.argtypes = []
    lib.rlk_det_gemm_tree_leaf_space_contract_id.restype = c.c_char_p
    lib.rlk_det_gemm_tree_leaf_space_contract_id.argtypes = []
    lib.rlk_det_gemm_seq.restype = i32
    lib.rlk_det_gemm_seq.argtypes = [vp, i32, i64, i64, vp, i32, i64, i64, vp, i32, i64, i32, i32, i32, vp]
    lib.rlk_det_gemm_seq_contract_id.restype = c.c_char_p
    lib.rlk_det_gemm_seq_contract_id.argtypes = []
    lib.rlk_det_gemm_pick_config.restype = i32
    lib.rlk_det_gemm_pick_config.argtypes = [i32, i32, i32]

    lib.rlk_linear_logp_contract_id.restype = c.c_char_p
    lib.rlk_linear_logp_contract_id.argtypes = []
    lib.rlk_linear_logp_split_count.restype = i32
    lib.rlk_linear_logp_split_count.argtypes = [i32]
    lib.rlk_linear_logp_workspace_bytes.restype = sz
    lib.rlk_linear_logp_workspace_bytes.argtypes = [i32, i32]
    lib.rlk_linear_logp_fwd.restype = i32
    lib.rlk_linear_logp_fwd.argtypes = [vp, i64, vp, i64, vp, vp, vp, vp, vp, vp, sz, i32, i32, i32, i64, i32, i32, vp]
    lib.rlk_linear_logp_fwd_shard.restype = i32
    lib.rlk_linear_logp_fwd_shard.argtypes = lib.rlk_linear_logp_fwd.argtypes
    lib.rlk_linear_logp_fwd_logits.restype = i32
    lib.rlk_linear_logp_fwd_logits.argtypes = [
        vp, i64, vp, i64, vp, vp, vp, vp, vp, vp, i64, vp, sz, i32, i32, i32, i64, i32, i32, vp,
    ]  # fmt: skip
    lib.rlk_linear_logp_fwd_noalloc.restype = i32
    lib.rlk_linear_logp_fwd_noalloc.argtypes = [vp, i64, vp, i64, vp, vp, vp, vp, vp, i32, i32, i32, i64, i32, i32, vp]

    lib.rlk_linear_logp_bwd_workspace_bytes.restype = sz
    lib.rlk_linear_logp_bwd_workspace_bytes.argtypes = [i32, i32, i32]
    lib.rlk_linear_logp_bwd.restype = i32
    lib.rlk_linear_logp_bwd.argtypes = [
        vp, i64, vp, i64, vp, vp, vp, vp, vp, vp, vp, i64, vp, i64, vp, vp, sz, i32, i32, i32, i64, i32, i32, vp,
    ]  # fmt: skip

    lib.rlk_logits_tile_stats.restype = i32
    lib.rlk_logits_tile_stats.argtypes = [vp, i32, i64, vp, i32, i64, i64, i64, i32, vp, vp, vp]
    lib.rlk_logits_logp_contract_id.restype = c.c_char_p
    lib.rlk_logits_logp_contract_id.argtypes = []
    lib.rlk_logp_from_logits_workspace_bytes.restype = sz
    lib.rlk_logp_from_logits_workspace_bytes.argtypes = [i32, i32]
    lib.rlk_logp_from_logits.restype = i32
    lib.rlk_logp_from_logits.argtypes = [vp, i32, i64, vp, vp, i32, i64, i64, i64, i32, vp, vp, vp, sz, vp]
    lib.rlk_logits_logp_backward.restype = i32
    lib.rlk_logits_logp_backward.argtypes = [vp, i32, i64, vp, vp, vp, vp, vp, vp, i64, i32, i64, i64, i64, vp]

    lib.rlk_swiglu_fwd.restype = i32
    lib.rlk_swiglu_fwd.argtypes = [vp, i64, vp, i64, vp, i64, i32, i32, i32, vp]
    lib.rlk_swiglu_bwd.restype = i32
    lib.rlk_swiglu_bwd.argtypes = [vp, i64, vp, i64, vp, i64, vp, i64, vp, i64, i32, i32, i32, vp]
    lib.rlk_det_gemm_swiglu_workspace_bytes.restype = sz
    lib.rlk_det_gemm_swiglu_workspace_bytes.argtypes = [vp, i64, vp, i64, i32, i32, i32]
    lib.rlk_det_gemm_swiglu_bf16.restype = i32
    lib.rlk_det_gemm_swiglu_bf16.argtypes = [vp, i64, vp, i64, vp, i64, vp, sz, i32, i32, i32, vp]

    lib.rlk_grpo_workspace_bytes.restype = sz
    lib.rlk_grpo_workspace_bytes.argtypes = [i32]
    lib.rlk_grpo_ratio_kl_loss.restype = i32
    lib.rlk_grpo_ratio_kl_loss.argtypes = [vp, vp, vp, vp, vp, i32, i32, f32, f32, vp, vp, vp, vp, sz, vp]
    _lib = lib
    return lib


def last_error() -> str:
    return load().rlk_last_error().decode("utf-8", "replace")


def check(status: int, what: str) -> None:
    """Turn a non-zero rlk_status into the exception the reference raises there."""
    if status == RLK_OK:
        return
    message = last_error() or what
    if status == RLK_ERR_INVALID_ARGUMENT:
        raise ValueError(message)
    raise RuntimeError(message)
