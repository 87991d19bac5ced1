"""GRPO loss epilogue for ROCm gfx950."""
