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
OBJ_DIR = PKG_DIR / "build"  # object files (git-ignored)
SOURCES = ["det_gemm.hip", "det_gemm_stream.hip", "det_gemm_shortk.hip", "det_gemm_tree.hip", "det_gemm_seq.hip", "linear_logp.hip",
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


def _run(cmd: list[str]) -> str:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(line for line in proc.stdout.splitlines() if "packed-fp32-ops" not in line and line.strip())
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    return out


def build(verbose: bool = True, only: list[str] | None = None) -> Path:
    """Compile every HIP source for gfx950 (one hipcc per source, side by side) and link them into
    one shared library. `only` names the sources to recompile; the objects of the others are reused
    when they exist and are newer than every header under csrc/ and include/ (a developer's
    shortcut, the default recompiles everything)."""
    from concurrent.futures import ThreadPoolExecutor

    hipcc = find_hipcc()
    OBJ_DIR.mkdir(exist_ok=True)
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    headers = [*CSRC.glob("*.h"), *(PKG_DIR.parent / "include").glob("*.h")]
    newest_header = max((h.stat().st_mtime for h in headers), default=0.0)
    jobs = []
    for src in SOURCES:
        obj = OBJ_DIR / (src + ".o")
        fresh = obj.exists() and obj.stat().st_mtime > max(newest_header, (CSRC / src).stat().st_mtime)
        if only is not None and src not in only and fresh:
            continue
        jobs.append([hipcc, *compile_flags, "-c", "-o", str(obj), str(CSRC / src)])
    if verbose:
        for cmd in jobs:
            print("[rlk build]", " ".join(cmd), flush=True)
    workers = max(1, min(len(jobs), int(os.environ.get("MAX_JOBS", "0")) or os.cpu_count() or 1))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        outs = list(pool.map(_run, jobs))
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH),
            *[str(OBJ_DIR / (s + ".o")) for s in SOURCES]]
    if verbose:
        print("[rlk build]", " ".join(link), flush=True)
    outs.append(_run(link))
    if verbose:
        for out in outs:
            if out:
                print(out, flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build(only=sys.argv[1:] or None)
    sys.exit(0)
