"""Log-probabilities from materialised logits on a real MI355X, through the C ABI.

Tolerance: tile maxima are exact; tile sums, lse and logp within 1e-5 relative /
2e-5 nats of the CPU oracle (fp32 arithmetic on both sides, different summation
orders); the gradient within one rounding of the logits dtype. Determinism and
batch invariance are bit-exact."""

from __future__ import annotations

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"


@pytest.fixture(scope="module")
def native():
    from rl_engine import _C

    return _C


@pytest.fixture(scope="module")
def logp_mod():
    from rl_engine.ops import logprob

    return logprob


def _logits(rows, v, seed, dtype, scale=4.0):
    gen = torch.Generator().manual_seed(seed)
    return (torch.randn(rows, v, generator=gen) * scale).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(37, 4096, 64, 4096), (5, 2374 * 4, 4, 9000), (64, 1000, 8, 700), (3, 151936, 64, 151000)])
def test_tile_stats_match_the_oracle(native, oracle, dtype, shape):
    rows, v, tiles, real = shape
    z = _logits(rows, v, 7000 + rows, dtype)
    tile_max, tile_sum = native.hip_deterministic_logp_tile_stats(z.to(DEV), 0, real, tiles)
    assert tile_max.shape == (rows, tiles) and tile_max.dtype == torch.float32
    ref_max, ref_sum = oracle.logits_tile_stats(z.float().numpy(), 0, real, tiles)
    assert np.array_equal(tile_max.cpu().numpy(), ref_max)
    assert np.allclose(tile_sum.cpu().numpy(), ref_sum, rtol=1e-5, atol=0)
    # a shard that starts beyond the real vocabulary is all padding
    pad_max, pad_sum = native.hip_deterministic_logp_tile_stats(z.to(DEV), real, real, tiles)
    assert bool(torch.isneginf(pad_max).all()) and not bool(pad_sum.any())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_logp_from_logits_parity_invariance_and_temperature(native, logp_mod, oracle, dtype):
    rows, v, real, start = 200, 2374 * 32, 75000, 0
    z = _logits(rows, v, 7100, dtype)
    gen = torch.Generator().manual_seed(7101)
    target = torch.randint(0, real, (rows,), generator=gen)
    temp = torch.rand(rows, generator=gen) * 1.5 + 0.5
    zd, td, tempd = z.to(DEV), target.to(DEV), temp.to(DEV)
    for tiles in (1, 8, 64):
        logp, lse = logp_mod.deterministic_logp_from_logits(zd, td, real_vocab_size=real, temperature=tempd, num_vocab_tiles=tiles)
        ref_logp, ref_lse = oracle.logp_from_logits(z.float().numpy(), target.numpy(), start, real, tiles, temperature=temp.numpy())
        assert np.abs(lse.cpu().numpy() - ref_lse).max() < 2e-5
        assert np.abs(logp.cpu().numpy() - ref_logp).max() < 2e-5
        # the GPU merge agrees with the reference's torch merge of the GPU tile statistics
        m, s = native.hip_deterministic_logp_tile_stats(zd, start, real, tiles, temperature=tempd)
        assert torch.allclose(logp_mod.merge_tile_partials(m, s), lse, atol=1e-5, rtol=0)
        # run to run and row by row: same bits
        again = logp_mod.deterministic_logp_from_logits(zd, td, real_vocab_size=real, temperature=tempd, num_vocab_tiles=tiles)
        assert torch.equal(again[0].view(torch.int32), logp.view(torch.int32))
        for r in (0, 37, rows - 1):
            one = logp_mod.deterministic_logp_from_logits(
                zd[r : r + 1], td[r : r + 1], real_vocab_size=real, temperature=tempd[r : r + 1], num_vocab_tiles=tiles
            )
            assert torch.equal(one[0].view(torch.int32), logp[r : r + 1].view(torch.int32)), (tiles, r)
            assert torch.equal(one[1].view(torch.int32), lse[r : r + 1].view(torch.int32)), (tiles, r)
    # a row-strided view (the narrowed staging buffer of a padded vocabulary) and an unaligned base
    wide = torch.zeros((rows, v + 24), dtype=dtype, device=DEV)
    wide[:, 8 : 8 + v] = zd
    base = logp_mod.deterministic_logp_from_logits(zd, td, real_vocab_size=real, num_vocab_tiles=64)
    view = logp_mod.deterministic_logp_from_logits(wide[:, 8 : 8 + v], td, real_vocab_size=real, num_vocab_tiles=64)
    shifted = logp_mod.deterministic_logp_from_logits(wide[:, 9 : 9 + v].copy_(zd), td, real_vocab_size=real, num_vocab_tiles=64)
    for other in (view, shifted):
        assert torch.equal(other[0].view(torch.int32), base[0].view(torch.int32))
        assert torch.equal(other[1].view(torch.int32), base[1].view(torch.int32))
    # temperature 1.0 as a python float is the untempered path
    plain = logp_mod.deterministic_logp_from_logits(zd, td, real_vocab_size=real, temperature=1.0, num_vocab_tiles=64)
    assert torch.equal(plain[0].view(torch.int32), base[0].view(torch.int32))


def test_from_logits_agrees_with_the_fused_linear_logp(native, logp_mod):
    import inputs

    h, w, target = inputs.logp_inputs(96, vocab=4096, hidden=256, seed=7200, rms_norm=False)
    w = (w.float() * 2.5).to(torch.bfloat16)
    hd, wd, td = h.to(DEV), w.to(DEV), target.to(DEV)
    fused_logp, fused_lse, logits = logp_mod.deterministic_linear_logp(hd, wd, td, return_logits=True)
    logp, lse = logp_mod.deterministic_logp_from_logits(logits, td, num_vocab_tiles=64)
    assert torch.allclose(logp, fused_logp, atol=2e-5, rtol=0) and torch.allclose(lse, fused_lse, atol=2e-5, rtol=0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_backward_matches_the_oracle_and_autograd_wiring(native, logp_mod, oracle, dtype):
    rows, v, real = 48, 2048, 2000
    z = _logits(rows, v, 7300, dtype)
    gen = torch.Generator().manual_seed(7301)
    target = torch.randint(0, real, (rows,), generator=gen)
    temp = torch.rand(rows, generator=gen) * 1.5 + 0.5
    g_logp = torch.randn(rows, generator=gen)
    g_lse = torch.randn(rows, generator=gen) * 0.5
    zd = z.to(DEV).requires_grad_(True)
    logp, lse = logp_mod.deterministic_logp_from_logits(zd, target.to(DEV), real_vocab_size=real, temperature=temp.to(DEV))
    ((logp * g_logp.to(DEV)).sum() + (lse * g_lse.to(DEV)).sum()).backward()
    assert zd.grad.dtype == dtype and zd.grad.shape == z.shape
    ref = oracle.logits_logp_backward(
        z.float().numpy(), lse.detach().cpu().numpy(), g_logp.numpy(), g_lse.numpy(), target.numpy(), 0, real,
        temperature=temp.numpy(), dtype=np.float64,
    )  # fmt: skip
    got = zd.grad.double().cpu().numpy()
    ulp = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11, torch.float32: 2.0**-23}[dtype]
    assert np.all(np.abs(got - ref) <= ulp * np.abs(ref) + 1e-5 * np.abs(ref) + 1e-7)
    assert not bool(zd.grad[:, real:].any())
    # logp only: target_local = -1 rows (a target owned elsewhere) get -coef * p everywhere
    lse_d = lse.detach().contiguous()
    none = torch.full((rows,), -1, dtype=torch.long, device=DEV)
    zero = torch.zeros(rows, device=DEV)
    grad = native.hip_deterministic_logp_backward(zd.detach(), lse_d, g_logp.to(DEV), zero, none, 0, real, False)
    assert bool((grad.float() * g_logp.to(DEV)[:, None] <= 0).all())


def test_argument_errors(native, logp_mod):
    z = torch.zeros((4, 64), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="divisible by num_tiles"):
        native.hip_deterministic_logp_tile_stats(z, 0, 64, 7)
    with pytest.raises(RuntimeError, match="invalid vocabulary metadata"):
        native.hip_deterministic_logp_tile_stats(z, -1, 64, 8)
    with pytest.raises(RuntimeError, match="float16, bfloat16, or float32"):
        native.hip_deterministic_logp_tile_stats(z.to(torch.float64), 0, 64, 8)
    with pytest.raises(RuntimeError, match="2D"):
        native.hip_deterministic_logp_tile_stats(z[0], 0, 64, 8)
    with pytest.raises(TypeError, match="2-D bf16/fp16/fp32"):
        logp_mod.deterministic_logp_from_logits(z.double(), torch.zeros(4, dtype=torch.long, device=DEV))
    with pytest.raises(ValueError, match="real vocabulary"):
        logp_mod.deterministic_logp_from_logits(z, torch.full((4,), 64, device=DEV))
    with pytest.raises(RuntimeError, match="coef_logp has the wrong dtype"):
        native.hip_deterministic_logp_backward(
            z, torch.zeros(4, device=DEV), torch.zeros(4, device=DEV, dtype=torch.float64), torch.zeros(4, device=DEV),
            torch.zeros(4, dtype=torch.long, device=DEV), 0, 64, False,
        )  # fmt: skip
    empty = native.hip_deterministic_logp_tile_stats(z[:0], 0, 64, 8)
    assert tuple(empty[0].shape) == (0, 8)


def test_full_size_rows_are_batch_invariant_and_normalised(native, logp_mod):
    """bf16 logits [8192, 151936] (2.5 GB): a row's (logp, lse) has the same bits alone, in a cut and
    in another packing; exp(logp) over every target id of a row sums to one."""
    rows, v = 8192, 151936
    gen = torch.Generator(device=DEV).manual_seed(7400)
    z = torch.empty((rows, v), dtype=torch.bfloat16, device=DEV)
    for r0 in range(0, rows, 1024):
        z[r0 : r0 + 1024] = (torch.randn((1024, v), generator=gen, device=DEV) * 3).to(torch.bfloat16)
    target = torch.randint(0, v, (rows,), generator=gen, device=DEV)
    logp, lse = logp_mod.deterministic_logp_from_logits(z, target)
    assert bool(torch.isfinite(logp).all()) and bool((logp <= 1e-6).all())
    for lo, hi in ((0, 1), (4095, 4102), (8191, 8192)):
        part = logp_mod.deterministic_logp_from_logits(z[lo:hi], target[lo:hi])
        assert torch.equal(part[0].view(torch.int32), logp[lo:hi].view(torch.int32))
        assert torch.equal(part[1].view(torch.int32), lse[lo:hi].view(torch.int32))
    perm = torch.randperm(rows, generator=torch.Generator().manual_seed(7401))[:512].to(DEV)
    packed = logp_mod.deterministic_logp_from_logits(z[perm], target[perm])
    assert torch.equal(packed[0].view(torch.int32), logp[perm].view(torch.int32))
    total = (z[77].float() - lse[77]).double().exp().sum()
    assert abs(float(total) - 1.0) < 1e-4
