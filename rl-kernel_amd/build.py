"""Build librlk_gfx950.so (the C-ABI HIP library) in-tree with hipcc.

Usage: python rl-kernel_amd/build.py            (or __graft_entry__.build())
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "librlk_gfx950.so"
SOURCES = ["det_gemm.hip", "det_gemm_stream.hip", "det_gemm_tree.hip", "linear_logp.hip",
    "linear_logp_bwd.hip", "logits_logp.hip", "swiglu.hip", "grpo.hip", "rlk_api.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # Floating-point contraction off: every fused multiply-add in the kernels is
    # written explicitly, so the same expression rounds the same way in every
    # template instantiation.
    "-ffp-contract=off",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; set HIPCC or install ROCm")


def build(verbose: bool = True) -> Path:
    """Compile every HIP source for gfx950 into one shared library."""
    cmd = [find_hipcc(), *HIPCC_FLAGS, "-o", str(LIB_PATH), *[str(CSRC / s) for s in SOURCES]]
    if verbose:
        print("[rlk build]", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(
        line for line in proc.stdout.splitlines() if "packed-fp32-ops" not in line and line.strip()
    )
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{out}")
    if verbose and out:
        print(out, flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
