"""MI355X (gfx950) implementation of RL-Kernel's batch-invariant dense path.

Keeps the reference's import paths for that path only:
``rl_engine.ops.gemm.det_gemm``, ``rl_engine.backends.rocm.gemm.det_gemm`` and
``rl_engine._C`` (reference rl_engine/ops/gemm/det_gemm.py:9-41,
rl_engine/backends/rocm/gemm/det_gemm.py:577-593, rl_engine/_C.pyi), plus the
fused linear-LogP and GRPO entry points under ``rl_engine.ops.logprob`` /
``rl_engine.ops.loss``. All compute runs in librlk_gfx950.so (hand-written HIP);
there is no CPU or PyTorch fallback.
"""

__version__ = "0.1.0"
