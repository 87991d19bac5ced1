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
        # a target outside the real vocabulary is marked with NaN; every other row carries its log-prob
        assert torch.equal(torch.isnan(base[0]), ~owned), where
        if bool(owned.any()):
            assert (base[0].double() - (zt - lse64)).abs()[owned].max().item() <= 1e-3, where


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


def test_k_tree_leaf_loops_over_layouts_and_depths(oracle):
    # The matrix-pipe leaf loop (16-byte chunks where the layout allows, elements elsewhere) against
    # the vector-ALU one over contiguous, transposed, offset and padded operands; small cases also
    # bit for bit against the CPU oracle.
    from rl_engine import _C

    d = _Draw(9350)
    for case in range(90):
        m, n, k = d.dim(), d.dim(), d.depth()
        if case % 9 == 0:
            k = int(d.rng.integers(1, 9)) * 4096 + (0 if case % 2 else 8 * int(d.rng.integers(0, 5)))
            m, n = min(m, 200), min(n, 200)
        a = d.view(m, k, int(d.rng.integers(0, 4)), 1.0)
        w = d.view(n, k, int(d.rng.integers(0, 4)), 0.1)
        outs = []
        for config in (1, 2, 0):
            out = torch.full((m, n + 3), 7.0, device=DEV, dtype=torch.bfloat16)[:, :n]
            outs.append(_C.gemm_tree_strided(a, w.t(), out, config))
            assert bool((out.as_strided((m, 3), (n + 3, 1), n) == 7.0).all()), (case, "wrote past N")
        assert _same(outs[0], outs[1]) and _same(outs[0], outs[2]), (case, m, n, k, a.stride(), w.stride())
        if m * n * k <= 4_000_000:
            want = oracle.k_tree_gemm(
                a.contiguous().view(torch.int16).cpu().numpy().view(np.uint16),
                w.contiguous().view(torch.int16).cpu().numpy().view(np.uint16),
            )
            got = outs[1].contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
            assert np.array_equal(got, want), (case, m, n, k)


def test_linear_logp_backward_configurations_rows_and_values():
    from rl_engine import _C, _lib

    d = _Draw(9400)
    for case in range(80):
        t = int(d.rng.integers(1, 400)) if d.rng.random() < 0.85 else int(d.rng.integers(400, 1400))
        v, hidden = int(d.rng.integers(1, 5000)), 32 * int(d.rng.integers(1, 16))
        h, w = d.bf16(t, hidden), d.bf16(v, hidden, scale=0.1)
        real = v if d.rng.random() < 0.5 else int(d.rng.integers(1, v + 1))
        start = 0 if d.rng.random() < 0.6 else int(d.rng.integers(0, 100000))
        tgt = torch.randint(max(start - 3, 0), start + real + 3, (t,), device=DEV, generator=d.gen)
        bias = torch.randn(v, device=DEV, generator=d.gen) if d.rng.random() < 0.4 else None
        temp = (torch.rand(t, device=DEV, generator=d.gen) + 0.5) if d.rng.random() < 0.4 else None
        g_logp = torch.randn(t, device=DEV, generator=d.gen) if d.rng.random() < 0.8 else None
        g_lse = torch.randn(t, device=DEV, generator=d.gen) if (d.rng.random() < 0.4 or g_logp is None) else None
        where = (case, t, v, hidden, real, start, bias is not None, temp is not None, g_logp is None, g_lse is None)
        _, lse = _C.fused_linear_logp(h, w, tgt, bias, temp, False, real, vocab_start_index=start)
        base = None
        for name, code in _lib.LOGP_CONFIGS.items():
            for staged in (0, _lib.FORCE_STAGED):
                if staged and d.rng.random() < 0.6:
                    continue
                out = _C.fused_linear_logp_bwd(
                    h, w, tgt, lse, g_logp, g_lse, bias, temp, real, vocab_start_index=start,
                    need_grad_bias=bias is not None, config=code | staged,
                )  # fmt: skip
                if base is None:
                    base = out
                for got, want in zip(out, base):
                    assert (got is None) == (want is None), where + (name, staged)
                    assert got is None or _same(got, want), where + (name, staged)
        row = int(d.rng.integers(0, t))
        cut = slice(row, row + 1)
        alone = _C.fused_linear_logp_bwd(
            h[cut].contiguous(), w, tgt[cut].contiguous(), lse[cut].contiguous(),
            None if g_logp is None else g_logp[cut].contiguous(), None if g_lse is None else g_lse[cut].contiguous(),
            bias, None if temp is None else temp[cut].contiguous(), real, vocab_start_index=start, need_grad_weight=False,
        )  # fmt: skip
        assert _same(alone[0], base[0][cut]), where + (row,)
        # values: fp64 gradients of the bf16-rounded d(logits)
        z = h.double() @ w.double().t()
        if bias is not None:
            z = z + bias.double()
        z[:, real:] = float("-inf")
        if temp is not None:
            z = z / temp.double()[:, None]
        p = torch.exp(z - lse.double()[:, None])
        gl = torch.zeros(t, device=DEV, dtype=torch.float64) if g_logp is None else g_logp.double()
        gs = torch.zeros(t, device=DEV, dtype=torch.float64) if g_lse is None else g_lse.double()
        dz = p * (gs - gl)[:, None]
        local = tgt - start
        owned = (local >= 0) & (local < real)
        dz[torch.arange(t, device=DEV)[owned], local[owned]] += gl[owned]
        if temp is not None:
            dz = dz / temp.double()[:, None]
        dz = dz.to(torch.bfloat16).double()
        for got, ref in ((base[0], dz @ w.double()), (base[1], dz.t() @ h.double())):
            scale = max(ref.abs().max().item(), 1e-6)
            assert (got.double() - ref).abs().max().item() <= 2.0**-6 * scale, where


def test_logits_side_kernels_dtypes_pitches_and_rows():
    from rl_engine import _C

    d = _Draw(9500)
    for case in range(150):
        rows, tiles = int(d.rng.integers(1, 300)), int(d.rng.choice([1, 2, 8, 64]))
        v = tiles * int(d.rng.integers(1, 120))
        dtype = [torch.bfloat16, torch.float16, torch.float32][int(d.rng.integers(0, 3))]
        pad = int(d.rng.choice([0, 0, 8, 5]))
        logits = (torch.randn(rows, v + pad, device=DEV, generator=d.gen) * 3).to(dtype)[:, :v]
        real = int(d.rng.integers(1, v + 1)) if d.rng.random() < 0.5 else v
        start = 0 if d.rng.random() < 0.6 else int(d.rng.integers(0, 100000))
        tgt = torch.randint(start, start + real, (rows,), device=DEV, generator=d.gen)
        temp = (torch.rand(rows, device=DEV, generator=d.gen) + 0.5) if d.rng.random() < 0.4 else None
        where = (case, rows, v, tiles, real, start, str(dtype), pad, temp is not None)
        logp, lse = _C.hip_deterministic_logp_from_logits(logits, tgt, start, start + real, tiles, temperature=temp)
        z = logits.double()[:, :real]
        if temp is not None:
            z = z / temp.double()[:, None]
        lse64 = torch.logsumexp(z, -1)
        zt = z.gather(1, (tgt - start)[:, None])[:, 0]
        tol = 1e-3 if dtype == torch.float32 else 2e-3
        assert (lse.double() - lse64).abs().max().item() <= tol, where
        assert (logp.double() - (zt - lse64)).abs().max().item() <= tol, where
        row = int(d.rng.integers(0, rows))
        cut = slice(row, row + 1)
        lp1, lse1 = _C.hip_deterministic_logp_from_logits(
            logits[cut], tgt[cut].contiguous(), start, start + real, tiles,
            temperature=None if temp is None else temp[cut].contiguous(),
        )  # fmt: skip
        assert _same(lp1, logp[cut]) and _same(lse1, lse[cut]), where + (row,)
        c_logp = torch.randn(rows, device=DEV, generator=d.gen)
        c_lse = torch.randn(rows, device=DEV, generator=d.gen)
        with_lse = bool(d.rng.random() < 0.5)
        grad = _C.hip_deterministic_logp_backward(
            logits, lse, c_logp, c_lse, (tgt - start).contiguous(), start, start + real, with_lse, temperature=temp
        )
        p = torch.exp(z - lse.double()[:, None])
        ref = torch.zeros(rows, v, device=DEV, dtype=torch.float64)
        ref[:, :real] = p * ((c_lse.double() if with_lse else 0.0) - c_logp.double())[:, None]
        ref[torch.arange(rows, device=DEV), tgt - start] += c_logp.double()
        if temp is not None:
            ref = ref / temp.double()[:, None]
        eps = {torch.bfloat16: 2.0**-7, torch.float16: 2.0**-9, torch.float32: 1e-4}[dtype]
        scale = max(ref.abs().max().item(), c_logp.abs().max().item(), c_lse.abs().max().item())
        assert (grad.double() - ref).abs().max().item() <= eps * scale + 1e-6, where
