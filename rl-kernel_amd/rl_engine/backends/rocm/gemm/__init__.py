"""Deterministic GEMM for ROCm gfx950 (hand-written HIP behind a C ABI)."""
