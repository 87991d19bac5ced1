"""Gated FFN operators (gfx950 build: ROCm only)."""

from rl_engine.backends.rocm.ffn.ffn import BACKEND_ID, Qwen3FFNOp, qwen3_ffn, qwen3_ffn_packed_inference

__all__ = ["BACKEND_ID", "Qwen3FFNOp", "qwen3_ffn", "qwen3_ffn_packed_inference"]
