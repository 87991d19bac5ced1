"""Fused linear-LogP for ROCm gfx950."""
