"""Seeded random sweep over shapes, strides, offsets and every forced configuration, on a real MI355X.

A configuration is a work split, never a different result: every GEMM configuration
must give the bits of the one-wave tile kernel with the element-wise loader, every
linear-LogP configuration the bits of the 16-token one, and the values must stay
within the tolerances of this path (LogP 1e-3 nats against fp64). Shapes are drawn
from continuous ranges so that edges no hand-written case lists come up."""

from __future__ import annotations

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _bits(x):
    return x.contiguous().view(torch.int32 if x.dtype == torch.float32 else torch.int16)


def _same(x, y):
    return torch.equal(_bits(x), _bits(y))


class _Draw:
    def __init__(self, seed):
        self.rng = np.random.default_rng(seed)
        self.gen = torch.Generator(device=DEV).manual_seed(seed)

    def bf16(self, *shape, scale=1.0):
        return (torch.randn(*shape, device=DEV, generator=self.gen) * scale).to(torch.bfloat16)

    def dim(self, big=False):
        r = self.rng.random()
        if r < 0.25:
            return int(self.rng.integers(1, 20))
        if r < 0.6:
            return int(self.rng.integers(1, 300))
        if r < 0.9 or not big:
            return int(self.rng.integers(1, 700))
        return int(self.rng.integers(700, 20000))

    def depth(self):
        r = self.rng.random()
        if r < 0.3:
            return int(self.rng.integers(1, 300))
        if r < 0.7:
            return 64 * int(self.rng.integers(1, 40))
        if r < 0.85:
            return 8 * int(self.rng.integers(1, 300))
        return 256 * int(self.rng.integers(1, 12))

    def view(self, rows, k, layout, scale):
        """0 contiguous, 1 other axis contiguous, 2 odd offset + padded rows, 3 aligned offset + padded rows."""
        if layout == 0:
            return self.bf16(rows, k, scale=scale)
        if layout == 1:
            return self.bf16(k, rows, scale=scale).t()
        if layout == 2:
            off, pad = int(self.rng.integers(0, 9)), int(self.rng.integers(0, 40))
            return self.bf16(rows + 1, k + pad + off, scale=scale)[1:, off : off + k]
        off, pad = 8 * int(self.rng.integers(0, 3)), 8 * int(self.rng.integers(0, 5))
        return self.bf16(rows, k + pad + off, scale=scale)[:, off : off + k]


def test_gemm_configurations_strides_and_output_pitch():
    from rl_engine import _C, _lib

    d = _Draw(9100)
    reference = _lib.GEMM_CONFIGS["16x16"] | _lib.FORCE_STAGED
    for case in range(160):
        m, n, k = d.dim(), d.dim(big=True), d.depth()
        if m * n > 4e6:
            n = max(1, int(4e6 // m))
        la, lb = int(d.rng.integers(0, 4)), int(d.rng.integers(0, 4))
        a, w = d.view(m, k, la, 1.0), d.view(n, k, lb, 0.05)
        dtype = torch.float32 if d.rng.random() < 0.25 else torch.bfloat16
        pitch_pad = int(d.rng.choice([0, 0, 8, 3]))
        want = torch.empty(m, n, device=DEV, dtype=dtype)
        _C.gemm_strided(a, w.t(), want, config=reference)
        for name, code in _lib.GEMM_CONFIGS.items():
            for staged in (0, _lib.FORCE_STAGED):
                if staged and d.rng.random() < 0.7:
                    continue
                buf = torch.full((m, n + pitch_pad), 7.0, device=DEV, dtype=dtype)
                got = buf[:, :n]
                _C.gemm_strided(a, w.t(), got, config=code | staged)
                where = (case, m, n, k, la, lb, str(dtype), name, staged, pitch_pad)
                assert _same(got, want), where
                assert pitch_pad == 0 or bool((buf[:, n:] == 7.0).all()), where  # nothing written past a row


def test_linear_logp_configurations_and_values():
    from rl_engine import _C, _lib

    d = _Draw(9200)
    for case in range(120):
        t = d.dim() if d.rng.random() < 0.8 else int(d.rng.integers(1, 1300))
        v, hidden = int(d.rng.integers(1, 6000)), 32 * int(d.rng.integers(1, 20))
        h, w = d.bf16(t, hidden), d.bf16(v, hidden, scale=0.1)
        real = v if d.rng.random() < 0.5 else int(d.rng.integers(1, v + 1))
        start = 0 if d.rng.random() < 0.6 else int(d.rng.integers(0, 100000))
        tgt = torch.randint(max(start - 3, 0), start + real + 3, (t,), device=DEV, generator=d.gen)
        bias = torch.randn(v, device=DEV, generator=d.gen) if d.rng.random() < 0.4 else None
        temp = (torch.rand(t, device=DEV, generator=d.gen) + 0.5) if d.rng.random() < 0.4 else None
        where = (case, t, v, hidden, real, start, bias is not None, temp is not None)
        base = None
        for name, code in _lib.LOGP_CONFIGS.items():
            logp, lse = _C.fused_linear_logp(h, w, tgt, bias, temp, False, real, vocab_start_index=start, config=code)
            if base is None:
                base = (logp, lse)
            assert _same(logp, base[0]) and _same(lse, base[1]), where + (name,)
        z = h.double() @ w[:real].double().t()
        if bias is not None:
            z = z + bias[:real].double()
        if temp is not None:
            z = z / temp.double()[:, None]
        lse64 = torch.logsumexp(z, dim=-1)
        assert (base[1].double() - lse64).abs().max().item() <= 1e-3, where
        local = tgt - start
        owned = (local >= 0) & (local < real)
        zt = z.gather(1, local.clamp(0, real - 1)[:, None])[:, 0]
        assert ((base[0].double() - (zt - lse64)).abs() * owned).max().item() <= 1e-3, where


def test_gated_projection_and_k_tree_rows():
    from rl_engine import _C, _lib

    d = _Draw(9300)
    reference = _lib.GEMM_CONFIGS["16x16"] | _lib.FORCE_STAGED
    for case in range(120):
        m, inter, k = d.dim(), int(d.rng.integers(1, 500)), d.depth()
        a, w = d.bf16(m, k), d.bf16(2 * inter, k, scale=0.1)
        proj = torch.empty(m, 2 * inter, device=DEV, dtype=torch.bfloat16)
        _C.gemm_strided(a, w.t(), proj, config=reference)
        assert _same(_C.det_gemm_swiglu(a, w), _C.swiglu_packed_forward(proj)), (case, m, inter, k)
        tree = torch.empty(m, inter, device=DEV, dtype=torch.bfloat16)
        _C.gemm_tree_strided(a, w[:inter].t(), tree)
        row = int(d.rng.integers(0, m))
        alone = torch.empty(1, inter, device=DEV, dtype=torch.bfloat16)
        _C.gemm_tree_strided(a[row : row + 1], w[:inter].t(), alone)
        assert _same(tree[row : row + 1], alone), (case, m, inter, k, row)
