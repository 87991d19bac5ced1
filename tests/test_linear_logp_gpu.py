"""Fused linear-LogP and the GRPO epilogue on a real MI355X, through the C ABI.

Tolerance for this path: |logp - oracle| <= 1e-3 nats (the reference's own bar
against the fp32-upcast native op is 2e-2, tests/ops/logprob/test_linear_logp.py:617);
determinism and batch invariance are bit-exact."""

from __future__ import annotations

from pathlib import Path

import numpy as np
import pytest
import torch

import inputs

pytestmark = pytest.mark.gpu

DEV = "cuda"
TOL_NATS = 1e-3
GOLDEN = Path(__file__).parent / "golden"


@pytest.fixture(scope="module")
def logp_mod():
    from rl_engine.ops import logprob

    return logprob


@pytest.fixture(scope="module")
def loss_mod():
    from rl_engine.ops import loss

    return loss


def _same_bits(x: torch.Tensor, y: torch.Tensor) -> bool:
    return torch.equal(x.contiguous().view(torch.int32), y.contiguous().view(torch.int32))


def test_golden_small_case(logp_mod):
    d = np.load(GOLDEN / "small_linear_logp.npz")
    h = inputs.from_bits(d["hidden_bits"], DEV)
    w = inputs.from_bits(d["weight_bits"], DEV)
    t = torch.from_numpy(d["target"]).to(DEV)
    logp, lse = logp_mod.deterministic_linear_logp(h, w, t)
    assert logp.dtype == torch.float32 and logp.shape == (48,)
    assert np.abs(logp.cpu().numpy() - d["logp"]).max() < 1e-4
    assert np.abs(lse.cpu().numpy() - d["lse"]).max() < 1e-4
    logp2, lse2 = logp_mod.deterministic_linear_logp(
        h,
        w,
        t % 1900,
        torch.from_numpy(d["bias"]).to(DEV),
        temperature=torch.from_numpy(d["temperature"]).to(DEV),
        real_vocab_size=1900,
    )
    assert np.abs(logp2.cpu().numpy() - d["logp_bias_temp_pad"]).max() < 1e-4
    assert np.abs(lse2.cpu().numpy() - d["lse_bias_temp_pad"]).max() < 1e-4
    assert bool((logp2 <= 0).all())


@pytest.mark.parametrize("shape", [(40, 3000, 264), (300, 2500, 128), (5, 1024, 64), (130, 5000, 512), (96, 4099, 320), (700, 9000, 256)])
def test_parity_with_oracle_and_config_neutrality(logp_mod, oracle, shape):
    from rl_engine import _lib

    t, v, d = shape
    h, w, target = inputs.logp_inputs(t, vocab=v, hidden=d, seed=4200 + t, rms_norm=False)
    w = (w.float() * 2.5).to(torch.bfloat16)  # sigma 0.05: a wider logit spread than N(0, 0.02)
    ref_logp, ref_lse = oracle.linear_logp_chunked(inputs.bits(h), inputs.bits(w), target.numpy(), chunk_elems=t * 700)[:2]
    dense_logp = oracle.linear_logp_dense(inputs.bits(h), inputs.bits(w), target.numpy())[0]
    h_d, w_d, t_d = h.to(DEV), w.to(DEV), target.to(DEV)
    base = None
    for name in ("256", "128", "64", "16", "64_streams", "128_streams", "256_streams", "auto"):
        logp, lse = logp_mod.deterministic_linear_logp(h_d, w_d, t_d, config=name)
        assert np.abs(logp.cpu().numpy() - ref_logp).max() <= TOL_NATS
        assert np.abs(lse.cpu().numpy() - ref_lse).max() <= TOL_NATS
        assert np.abs(logp.cpu().numpy() - dense_logp).max() <= TOL_NATS
        if base is None:
            base = (logp, lse)
        assert _same_bits(logp, base[0]) and _same_bits(lse, base[1]), name
        if name != "auto":
            staged = logp_mod.deterministic_linear_logp(h_d, w_d, t_d, config=_lib.LOGP_CONFIGS[name] | _lib.FORCE_STAGED)
            assert _same_bits(staged[0], base[0]) and _same_bits(staged[1], base[1]), f"{name} staged"
    assert np.abs(base[0].cpu().numpy() - ref_logp).max() < 5e-5  # what the kernel actually achieves


def test_row_alone_equals_row_in_batch_with_bias_temperature_padding(logp_mod):
    # The strict-contract invariance check: row 37 alone vs inside N=96, int32 views,
    # with bias + temperature + padded vocabulary (tests/ops/logprob/test_linear_logp.py:1428-1463).
    n, d, v, real = 96, 256, 3072, 3000
    h, w, target = inputs.logp_inputs(n, vocab=v, hidden=d, seed=4300, rms_norm=False)
    target = target % real
    g = torch.Generator().manual_seed(4301)
    bias = (torch.randn(v, generator=g) * 0.3).to(DEV)
    temp = (0.5 + torch.rand(n, generator=g)).to(DEV)
    h_d, w_d, t_d = h.to(DEV), w.to(DEV), target.to(DEV)
    logp, lse = logp_mod.deterministic_linear_logp(h_d, w_d, t_d, bias, temperature=temp, real_vocab_size=real)
    for row in (0, 37, 95):
        one_lp, one_lse = logp_mod.deterministic_linear_logp(
            h_d[row : row + 1], w_d, t_d[row : row + 1], bias, temperature=temp[row : row + 1], real_vocab_size=real
        )
        assert _same_bits(one_lp, logp[row : row + 1]) and _same_bits(one_lse, lse[row : row + 1]), row
    # return_logits must not change logp / lse bits and exposes unscaled, bias-applied, padded logits
    lp2, lse2, logits = logp_mod.deterministic_linear_logp(
        h_d, w_d, t_d, bias, temperature=temp, real_vocab_size=real, return_logits=True
    )
    assert _same_bits(lp2, logp) and _same_bits(lse2, lse)
    assert logits.shape == (n, v) and bool(torch.isinf(logits[:, real:]).all()) and bool((logp <= 0).all())
    probs = torch.softmax(logits.double() * (1.0 / temp.double())[:, None], dim=-1)
    picked = probs[torch.arange(n, device=DEV), t_d].log()
    assert float((picked - logp.double()).abs().max()) < 1e-4


@pytest.mark.parametrize("shape", [(40, 3000, 256, 2990), (1100, 2500, 128, 2500), (300, 4099, 320, 4000), (1, 1024, 64, 1024), (2050, 1030, 64, 1001)])
def test_logits_come_out_of_the_same_pass_bit_for_bit(logp_mod, shape):
    """return_logits: the fp32 logits are the accumulators the reduction sees (bias added, padded lanes -inf,
    no temperature), stored by the fused kernel itself: equal to the fp32-output GEMM plus bias bit for bit,
    for the stream-group grid (up to 1024 tokens) and the split grid, aligned and unaligned vocabulary sizes,
    every configuration; logp and lse keep their bits."""
    from rl_engine import _C, _lib

    n, v, d, real = shape
    h, w, target = inputs.logp_inputs(n, vocab=v, hidden=d, seed=4900 + n, rms_norm=False)
    target = target % real
    g = torch.Generator().manual_seed(4901 + n)
    bias = (torch.randn(v, generator=g) * 0.3).to(DEV)
    temp = (0.5 + torch.rand(n, generator=g)).to(DEV)
    h_d, w_d, t_d = h.to(DEV), w.to(DEV), target.to(DEV)
    plain = _C.det_gemm_fwd_out_fp32(h_d, w_d.t())
    for extra, want in (({}, plain), ({"bias": bias, "temperature": temp, "real_vocab_size": real}, plain + bias)):
        want = want.clone()
        if extra:
            want[:, real:] = float("-inf")
        base = logp_mod.deterministic_linear_logp(h_d, w_d, t_d, **extra)
        for name in ("auto", "256", "128", "64", "16", "64_streams", "256_streams"):
            lp, lse, logits = logp_mod.deterministic_linear_logp(h_d, w_d, t_d, return_logits=True, config=name, **extra)
            assert logits.dtype == torch.float32 and logits.shape == (n, v)
            assert _same_bits(logits, want), (name, sorted(extra))
            assert _same_bits(lp, base[0]) and _same_bits(lse, base[1]), (name, sorted(extra))
        staged = _lib.LOGP_CONFIGS["64"] | _lib.FORCE_STAGED
        assert _same_bits(logp_mod.deterministic_linear_logp(h_d, w_d, t_d, return_logits=True, config=staged, **extra)[2], want)


@pytest.mark.parametrize(
    "shape",
    [(1, 5000, 256, 4900), (17, 3072, 128, 3000), (64, 9001, 320, 9001), (33, 1024, 64, 1000), (130, 4608, 128, 4500), (700, 2300, 192, 2290)],
)
def test_stream_group_split_keeps_the_bits(logp_mod, oracle, shape):
    # For few token tiles the vocabulary splits are cut into four stream groups, one workgroup each:
    # a different work split, the same contract. Bias, temperature and padded vocabulary included.
    n, v, d, real = shape
    h, w, target = inputs.logp_inputs(n, vocab=v, hidden=d, seed=4350 + n, rms_norm=False)
    target = target % real
    target[0] = real - 1
    g = torch.Generator().manual_seed(4351 + n)
    bias = torch.randn(v, generator=g) * 0.3
    temp = 0.5 + torch.rand(n, generator=g)
    ref_logp, ref_lse = oracle.linear_logp_dense(
        inputs.bits(h), inputs.bits(w), target.numpy(), bias.numpy(), temperature=temp.numpy(), real_vocab_size=real
    )
    h_d, w_d, t_d, b_d, tmp_d = h.to(DEV), w.to(DEV), target.to(DEV), bias.to(DEV), temp.to(DEV)
    for extra in ({}, {"bias": b_d, "temperature": tmp_d, "real_vocab_size": real}):
        base = logp_mod.deterministic_linear_logp(h_d, w_d, t_d, config="256", **extra)
        for name in ("64_streams", "128_streams", "256_streams", "auto"):
            got = logp_mod.deterministic_linear_logp(h_d, w_d, t_d, config=name, **extra)
            assert _same_bits(got[0], base[0]) and _same_bits(got[1], base[1]), (name, sorted(extra))
    assert np.abs(got[0].cpu().numpy() - ref_logp).max() <= TOL_NATS
    assert np.abs(got[1].cpu().numpy() - ref_lse).max() <= TOL_NATS


def test_seeded_random_shapes_match_the_smallest_tile_with_the_staged_loop(logp_mod):
    """Whatever grid and tile the picker chooses for a token count, hidden size and vocabulary, with or
    without bias, temperature and padding, logp and lse have the bits of the 16-token tile kernel."""
    from rl_engine import _lib

    rng = np.random.default_rng(4700)
    reference_config = _lib.LOGP_CONFIGS["16"] | _lib.FORCE_STAGED
    for case in range(40):
        n = int(rng.choice([1, 5, 16, 33, 64, 65, 128, 129, 300, 700, 1025, 1300]))
        v = int(rng.choice([40, 256, 1000, 1024, 2500, 4099, 6000]))
        d = int(rng.choice([8, 64, 72, 128, 320, 512]))
        h, w, target = inputs.logp_inputs(n, vocab=v, hidden=d, seed=4701 + case, rms_norm=False)
        real = v if case % 3 else max(1, v - int(rng.integers(1, 30)))
        target = target % real
        extra = {}
        if case % 2:
            g = torch.Generator().manual_seed(4800 + case)
            extra = {"bias": (torch.randn(v, generator=g) * 0.2).to(DEV), "temperature": (0.5 + torch.rand(n, generator=g)).to(DEV)}
        if real != v:
            extra["real_vocab_size"] = real
        h_d, w_d, t_d = h.to(DEV), w.to(DEV), target.to(DEV)
        want = logp_mod.deterministic_linear_logp(h_d, w_d, t_d, config=reference_config, **extra)
        got = logp_mod.deterministic_linear_logp(h_d, w_d, t_d, **extra)
        assert _same_bits(got[0], want[0]) and _same_bits(got[1], want[1]), (case, n, v, d, sorted(extra))


def test_layout_packing_invariance(logp_mod):
    # Rows permuted across [2,3] / [3,2] / [1,6] layouts give the same per-row bits
    # (tests/ops/logprob/test_linear_logp.py:339-367).
    h, w, target = inputs.logp_inputs(6, vocab=2048, hidden=128, seed=4400, rms_norm=False)
    h_d, w_d, t_d = h.to(DEV), w.to(DEV), target.to(DEV)
    flat, _ = logp_mod.deterministic_linear_logp(h_d, w_d, t_d)
    for lead in ((2, 3), (3, 2), (1, 6)):
        out, lse = logp_mod.deterministic_linear_logp(h_d.view(*lead, 128), w_d, t_d.view(*lead))
        assert out.shape == lead and lse.shape == lead and _same_bits(out.reshape(-1), flat)
    perm = torch.tensor([4, 0, 5, 2, 1, 3], device=DEV)
    out, _ = logp_mod.deterministic_linear_logp(h_d[perm], w_d, t_d[perm])
    assert _same_bits(out, flat[perm])
    op = logp_mod.LinearLogpOp()
    assert _same_bits(op(h_d.view(2, 3, 128), w_d, t_d.view(2, 3)).reshape(-1), flat)
    assert _same_bits(logp_mod.linear_logp(h_d, w_d, t_d), flat)


def test_uniform_logits_and_target_checks(logp_mod):
    v, d = 5000, 64
    h = torch.zeros((4, d), dtype=torch.bfloat16, device=DEV)
    w = inputs.randn_bf16(4500, v, d).to(DEV)
    t = torch.tensor([0, 1, 4999, 2500], device=DEV)
    logp, lse = logp_mod.deterministic_linear_logp(h, w, t)
    assert torch.allclose(logp, torch.full_like(logp, -float(np.log(v))), atol=1e-5)
    assert torch.allclose(lse, torch.full_like(lse, float(np.log(v))), atol=1e-5)
    # values are checked on the host (a read-back, as the reference's strict entry does) only on request ...
    bad_t = torch.tensor([0, 1, 5000, 2], device=DEV)
    bad_temp = torch.tensor([1.0, 0.0, 1.0, -2.0])
    with pytest.raises(ValueError, match="real vocabulary"):
        logp_mod.deterministic_linear_logp(h, w, bad_t, validate=True)
    with pytest.raises(ValueError, match="temperature"):
        logp_mod.deterministic_linear_logp(h, w, t, temperature=bad_temp, validate=True)
    # ... by default the kernel marks the offending rows, and only those, with NaN
    marked, lse_marked = logp_mod.deterministic_linear_logp(h, w, bad_t)
    assert bool(torch.isnan(marked[2])) and _same_bits(marked[[0, 1]], logp[[0, 1]]) and _same_bits(lse_marked, lse)
    marked, _ = logp_mod.deterministic_linear_logp(h, w, torch.tensor([-1, 1, 4990, 2], device=DEV), real_vocab_size=4990)
    assert torch.isnan(marked).tolist() == [True, False, True, False]
    marked, lse_marked = logp_mod.deterministic_linear_logp(h, w, t, temperature=bad_temp)
    assert torch.isnan(marked).tolist() == [False, True, False, True] and torch.isnan(lse_marked).tolist() == [False, True, False, True]
    assert _same_bits(marked[[0, 2]], logp[[0, 2]])
    with pytest.raises(ValueError, match="real_vocab_size"):
        logp_mod.deterministic_linear_logp(h, w, t, real_vocab_size=v + 1)
    with pytest.raises(ValueError, match="one id per hidden row"):
        logp_mod.deterministic_linear_logp(h, w, t[:3])
    hg = h.clone().requires_grad_(True)
    with pytest.raises(RuntimeError, match="inference-only"):
        logp_mod.deterministic_linear_logp(hg, w, t, return_logits=True)


def test_vocab_start_index_offsets_targets(logp_mod):
    h, w, target = inputs.logp_inputs(9, vocab=1500, hidden=64, seed=4600, rms_norm=False)
    h_d, w_d, t_d = h.to(DEV), w.to(DEV), target.to(DEV)
    base, _ = logp_mod.deterministic_linear_logp(h_d, w_d, t_d)
    shifted, _ = logp_mod.deterministic_linear_logp(h_d, w_d, t_d + 7000, vocab_start_index=7000)
    assert _same_bits(base, shifted)


@pytest.mark.parametrize("tokens", [5, 300, 1500])
def test_shard_entry_returns_the_terms_a_vocabulary_split_merges(tokens):
    """``fused_linear_logp_sm90_global_target`` against the whole-vocabulary entry and the dense
    formula: one shard reproduces logp bit for bit; three uneven shards (the last one padded,
    with bias and per-token temperature) merge to the whole vocabulary's logp within 1e-3 nats,
    and each target logit is owned by exactly one shard."""
    from rl_engine import _C

    vocab, hidden = 5000, 192
    h, w, target = inputs.logp_inputs(tokens, vocab=vocab, hidden=hidden, seed=4700 + tokens, rms_norm=False)
    g = torch.Generator().manual_seed(4701)
    bias = torch.randn((vocab,), generator=g) * 0.5
    temp = torch.rand((tokens,), generator=g) + 0.5
    h_d, w_d, t_d, b_d, temp_d = (x.to(DEV) for x in (h, w, target, bias, temp))

    logp, lse = _C.fused_linear_logp_sm90(h_d, w_d, t_d, b_d, temp_d)
    zt, lse1 = _C.fused_linear_logp_sm90_global_target(h_d, w_d, t_d, b_d, 0, temp_d)
    assert _same_bits(lse, lse1)
    assert _same_bits(logp, torch.clamp(zt - lse1, max=0.0))
    dense = (h.double() @ w.double().t() + bias.double()) / temp.double()[:, None]
    want_zt = dense.gather(1, target[:, None])[:, 0]
    assert (zt.cpu().double() - want_zt).abs().max().item() <= 2e-3 * max(1.0, want_zt.abs().max().item())

    bounds = [0, 1111, 3200, vocab]
    zts, lses = [], []
    for lo, hi in zip(bounds[:-1], bounds[1:]):
        rows = w_d[lo:hi]
        shard_bias = b_d[lo:hi]
        real = hi - lo
        if hi == vocab:  # the last shard carries 40 rows of padding that must not count
            rows = torch.cat([rows, torch.full((40, hidden), 3.0, dtype=torch.bfloat16, device=DEV)])
            shard_bias = torch.cat([shard_bias, torch.full((40,), 9.0, device=DEV)])
        a, b = _C.fused_linear_logp_sm90_global_target(h_d, rows.contiguous(), t_d, shard_bias, lo, temp_d, real)
        zts.append(a)
        lses.append(b)
        owned = (target >= lo) & (target < hi)
        assert torch.equal(a.cpu() != 0, owned & (want_zt != 0).cpu())
    owners = torch.stack([z != 0 for z in zts]).sum(0)
    assert int(owners.max()) <= 1
    merged = torch.stack(zts).double().sum(0) - torch.logsumexp(torch.stack(lses).double(), dim=0)
    want = torch.log_softmax(dense, dim=-1).gather(1, target[:, None])[:, 0]
    assert (merged.cpu() - want).abs().max().item() <= TOL_NATS
    assert (logp.cpu().double() - want).abs().max().item() <= TOL_NATS


def test_backward_under_the_reference_name_and_argument_order():
    from rl_engine import _C

    h, w, target = inputs.logp_inputs(70, vocab=1300, hidden=128, seed=4800, rms_norm=False)
    h_d, w_d, t_d = h.to(DEV), w.to(DEV), target.to(DEV)
    grad = torch.randn((70,), generator=torch.Generator().manual_seed(4801)).to(DEV)
    _, lse = _C.fused_linear_logp_sm90(h_d, w_d, t_d)
    gh, gw, gb = _C.fused_linear_logp_sm90_backward(grad, h_d, w_d, t_d, lse, None, 0, True, True, False, False)
    ours = _C.fused_linear_logp_bwd(h_d, w_d, t_d, lse, grad, None)
    assert torch.equal(gh, ours[0]) and torch.equal(gw, ours[1])
    assert gb.numel() == 0 and gb.dtype == torch.float32
    only_w = _C.fused_linear_logp_sm90_backward(grad, h_d, w_d, t_d, lse, None, 0, False, True, False, False)
    assert only_w[0].numel() == 0 and torch.equal(only_w[1], gw)
    # a shard's backward takes global ids and the shard's first row
    lo = 400
    half = _C.fused_linear_logp_sm90_backward(grad, h_d, w_d[lo:].contiguous(), t_d, lse, None, lo, False, True, False, True)
    zf = h.double() @ w.double().t()
    dz = -torch.exp(zf - lse.cpu().double()[:, None]) * grad.cpu().double()[:, None]
    dz[torch.arange(70), target] += grad.cpu().double()
    ref = dz[:, lo:].to(torch.bfloat16).double().t() @ h.double()
    assert (half[1].cpu().double() - ref).abs().max().item() <= 2.0**-7 * ref.abs().max().item()


# ---------------------------------------------------------------------------
# Config 4 at full size: T=8192, V=151936, D=4096
# ---------------------------------------------------------------------------


@pytest.fixture(scope="module")
def config4():
    h, w, target = inputs.logp_inputs(8192)
    return {"h": h, "w": w, "t": target, "h_d": h.to(DEV), "w_d": w.to(DEV), "t_d": target.to(DEV)}


def test_config4_full_size(logp_mod, oracle, config4):
    c = config4
    logp, lse = logp_mod.deterministic_linear_logp(c["h_d"], c["w_d"], c["t_d"])
    assert logp.shape == (8192,) and bool(torch.isfinite(logp).all()) and bool((logp <= 0).all())
    # bit-exact run to run
    logp_b, lse_b = logp_mod.deterministic_linear_logp(c["h_d"], c["w_d"], c["t_d"])
    assert _same_bits(logp, logp_b) and _same_bits(lse, lse_b)
    # bit-exact per row: M=1, M=7 and a ragged cut against the M=8192 batch
    for lo, hi in ((0, 1), (0, 7), (4095, 4096), (8191, 8192), (5000, 5130)):
        part, part_lse = logp_mod.deterministic_linear_logp(c["h_d"][lo:hi], c["w_d"], c["t_d"][lo:hi])
        assert _same_bits(part, logp[lo:hi]) and _same_bits(part_lse, lse[lo:hi]), (lo, hi)
    # a different packing of the same rows
    perm = torch.randperm(8192, generator=torch.Generator().manual_seed(4002)).to(DEV)
    packed, _ = logp_mod.deterministic_linear_logp(c["h_d"][perm], c["w_d"], c["t_d"][perm])
    assert _same_bits(packed, logp[perm])
    # parity with the oracle's chunked online LSE on a random 256-row sample
    # plus the rows on both sides of every token-tile seam and the last rows
    sample = torch.randperm(8192, generator=torch.Generator().manual_seed(4003))[:256]
    edges = torch.tensor([0, 15, 16, 63, 64, 127, 128, 255, 256, 257, 511, 512, 4095, 4096, 7935, 7936, 8190, 8191])
    sample = torch.unique(torch.cat([sample, edges]))
    ref_logp, ref_lse = oracle.linear_logp_chunked(
        inputs.bits(c["h"][sample]), inputs.bits(c["w"]), c["t"][sample].numpy(), chunk_elems=256 * 2048
    )[:2]
    err = np.abs(logp.cpu().numpy()[sample.numpy()] - ref_logp).max()
    err_lse = np.abs(lse.cpu().numpy()[sample.numpy()] - ref_lse).max()
    assert err <= TOL_NATS and err_lse <= TOL_NATS, (err, err_lse)
    assert err < 1e-4, err


def test_config4_probabilities_of_all_columns_sum_to_one(logp_mod, config4):
    # size-independent property: for one row, exp(logp) summed over every target id is 1
    c = config4
    v = c["w"].size(0)
    ids = torch.arange(v, device=DEV)
    row = c["h_d"][123:124].expand(4096, -1).contiguous()
    total = 0.0
    lse0 = None
    for v0 in range(0, v, 4096):
        chunk = ids[v0 : v0 + 4096]
        lp, lse = logp_mod.deterministic_linear_logp(row[: chunk.numel()], c["w_d"], chunk)
        total += float(lp.double().exp().sum())
        lse0 = lse[0] if lse0 is None else lse0
        assert bool((lse == lse0).all())  # the same row gives the same lse in every slot
    assert abs(total - 1.0) < 1e-4


# ---------------------------------------------------------------------------
# GRPO epilogue and config 5
# ---------------------------------------------------------------------------


def test_grpo_golden_small_case(loss_mod):
    d = np.load(GOLDEN / "small_grpo.npz")
    out = loss_mod.grpo_ratio_kl_loss(
        torch.from_numpy(d["logp"]).to(DEV),
        torch.from_numpy(d["old"]).to(DEV),
        torch.from_numpy(d["ref"]).to(DEV),
        torch.from_numpy(d["adv"]).to(DEV),
        torch.from_numpy(d["mask"]).to(DEV),
        clip_eps=0.2,
        beta=0.01,
    )
    got3 = torch.stack([out.loss, out.policy_loss, out.kl]).cpu().numpy()
    assert np.allclose(got3, d["loss3"], rtol=2e-5, atol=1e-7)
    assert np.allclose(out.ratio.cpu().numpy(), d["ratio"], rtol=2e-6, atol=0)
    assert np.allclose(out.k3.cpu().numpy(), d["k3"], rtol=0, atol=3e-7)
    again = loss_mod.grpo_ratio_kl_loss(
        torch.from_numpy(d["logp"]).to(DEV),
        torch.from_numpy(d["old"]).to(DEV),
        torch.from_numpy(d["ref"]).to(DEV),
        torch.from_numpy(d["adv"]).to(DEV),
        torch.from_numpy(d["mask"]).to(DEV),
        clip_eps=0.2,
        beta=0.01,
    )
    assert _same_bits(again.loss.reshape(1), out.loss.reshape(1)) and _same_bits(again.ratio, out.ratio)


def test_grpo_closed_forms(loss_mod):
    g = torch.Generator().manual_seed(5200)
    logp = (-torch.randn((7, 130), generator=g).abs()).to(DEV)
    adv = torch.randn(7, generator=g).to(DEV)
    same = loss_mod.grpo_ratio_kl_loss(logp, logp, logp, adv, beta=0.5)
    assert bool((same.ratio == 1.0).all()) and bool((same.k3 == 0.0).all()) and float(same.kl) == 0.0
    assert float(same.policy_loss) == pytest.approx(-float(adv.mean()), rel=1e-5)
    hi = loss_mod.grpo_ratio_kl_loss(logp, logp - 1.0, logp, torch.full((7,), 2.0, device=DEV), clip_eps=0.2)
    assert float(hi.policy_loss) == pytest.approx(-2.4, rel=1e-6)
    lo = loss_mod.grpo_ratio_kl_loss(logp, logp - 1.0, logp, torch.full((7,), -2.0, device=DEV), clip_eps=0.2)
    assert float(lo.policy_loss) == pytest.approx(2.0 * float(np.e), rel=1e-6)
    mask = torch.zeros((7, 130), dtype=torch.bool, device=DEV)
    none = loss_mod.grpo_ratio_kl_loss(logp, logp - 1.0, logp + 0.3, adv, mask, beta=0.1)
    assert float(none.loss) == 0.0 and bool((none.ratio == 0).all()) and bool((none.k3 == 0).all())
    quarter = loss_mod.compute_policy_ratio(logp, logp - 0.25)
    assert torch.allclose(quarter, torch.full_like(quarter, float(np.exp(0.25))), rtol=1e-6)
    assert bool((loss_mod.compute_reference_kl(logp, logp + 0.01) >= 0).all())


def _reference_rl_loss(logp, old, ref, adv, mask, eps, beta):
    """The reference's minimal RL loss in torch (tests/e2e/test_rl_kernel_loss_step.py:18-39 on
    rl_engine/reference/definitions.py:50-106): differentiable through torch's own autograd."""
    keep = mask.to(logp.dtype)
    ratio = torch.exp(logp - old) * keep
    a = adv.reshape(-1, 1).to(logp.dtype)
    policy = -torch.minimum(ratio * a, torch.clamp(ratio, 1.0 - eps, 1.0 + eps) * a)
    d = (ref - logp) * keep
    kl = (torch.exp(d) - d - 1.0) * keep
    count = torch.clamp(keep.sum(), min=1e-8)
    policy_loss, kl_mean = (policy * keep).sum() / count, kl.sum() / count
    return policy_loss + beta * kl_mean, policy_loss, kl_mean


def test_grpo_loss_gradients_match_torch_autograd(loss_mod):
    g = torch.Generator().manual_seed(5300)
    rollouts, tokens = 9, 70
    base = -torch.randn((rollouts, tokens), generator=g).abs()
    old = (base + 0.3 * torch.randn((rollouts, tokens), generator=g)).to(DEV)  # ratios on both sides of the clip range
    ref = (base + 0.2 * torch.randn((rollouts, tokens), generator=g)).to(DEV)
    adv = torch.randn(rollouts, generator=g).to(DEV)
    adv[3] = 0.0
    mask = (torch.rand((rollouts, tokens), generator=g) < 0.75).to(DEV)
    for which, beta in ((0, 0.01), (0, 0.0), (1, 0.3), (2, 0.3)):
        cur = base.to(DEV).clone().requires_grad_(True)
        out = loss_mod.grpo_ratio_kl_loss(cur, old, ref, adv, mask, clip_eps=0.2, beta=beta)
        assert out.loss.requires_grad and not out.ratio.requires_grad
        (out.loss, out.policy_loss, out.kl)[which].backward()
        cur64 = base.to(DEV).double().requires_grad_(True)
        want = _reference_rl_loss(cur64, old.double(), ref.double(), adv.double(), mask, 0.2, beta)
        want[which].backward()
        assert float(out.loss.detach()) == pytest.approx(float(want[0].detach()), rel=1e-5, abs=1e-7)
        assert (cur.grad.double() - cur64.grad).abs().max().item() <= 1e-6 * max(1.0, cur64.grad.abs().max().item())
        assert bool((cur.grad[~mask] == 0).all())
    # the forward values under autograd are the inference values, bit for bit
    cur = base.to(DEV).clone().requires_grad_(True)
    a = loss_mod.grpo_ratio_kl_loss(cur, old, ref, adv, mask, beta=0.01)
    b = loss_mod.grpo_ratio_kl_loss(cur.detach(), old, ref, adv, mask, beta=0.01)
    assert _same_bits(a.loss.detach().reshape(1), b.loss.reshape(1)) and _same_bits(a.k3, b.k3)


def test_grpo_mask_is_read_as_a_boolean_in_forward_and_backward(loss_mod):
    """A mask with values other than 0 / 1 (2, 0.5, 256) keeps those tokens with weight one, forward and
    backward alike: the reference reads every mask through ``mask.bool()`` (reference/definitions.py:50-70)."""
    g = torch.Generator().manual_seed(5310)
    rollouts, tokens = 5, 40
    base = -torch.randn((rollouts, tokens), generator=g).abs()
    old = (base + 0.2 * torch.randn((rollouts, tokens), generator=g)).to(DEV)
    ref = (base + 0.2 * torch.randn((rollouts, tokens), generator=g)).to(DEV)
    adv = torch.randn(rollouts, generator=g).to(DEV)
    keep = (torch.rand((rollouts, tokens), generator=g) < 0.7).to(DEV)
    values = torch.tensor([2.0, 0.5, 256.0, 1.0], device=DEV)
    odd = keep.float() * values[torch.arange(rollouts * tokens, device=DEV).view(rollouts, tokens) % 4]
    assert bool(((odd != 0) == keep).all())
    results = []
    for mask in (keep, odd, odd.to(torch.int32)):
        cur = base.to(DEV).clone().requires_grad_(True)
        out = loss_mod.grpo_ratio_kl_loss(cur, old, ref, adv, mask, beta=0.05)
        out.loss.backward()
        results.append((out.loss.detach().reshape(1), out.ratio, out.k3, cur.grad))
    # int32 truncates 0.5 to 0 before the library sees it, exactly as `.to(int32).bool()` does in the reference
    as_int = odd.to(torch.int32).bool()
    for got, want in zip(results[1], results[0]):
        assert _same_bits(got, want)
    cur = base.to(DEV).clone().requires_grad_(True)
    out = loss_mod.grpo_ratio_kl_loss(cur, old, ref, adv, as_int, beta=0.05)
    out.loss.backward()
    for got, want in zip(results[2], (out.loss.detach().reshape(1), out.ratio, out.k3, cur.grad)):
        assert _same_bits(got, want)


def test_rl_loss_step_end_to_end(logp_mod, loss_mod):
    """hidden, lm_head -> fused linear-LogP -> GRPO loss -> backward: the training step of
    tests/e2e/test_rl_kernel_loss_step.py on this path, against fp64 autograd of the same formula."""
    rollouts, tokens, hidden, vocab = 8, 40, 128, 3000
    g = torch.Generator().manual_seed(5400)
    h0 = inputs.randn_bf16(5401, rollouts * tokens, hidden).to(DEV)
    w0 = inputs.randn_bf16(5402, vocab, hidden, 0.1).to(DEV)
    target = torch.randint(0, vocab, (rollouts, tokens), generator=g).to(DEV)
    mask = (torch.rand((rollouts, tokens), generator=g) < 0.75).to(DEV)
    adv = torch.randn(rollouts, generator=g).to(DEV)
    with torch.no_grad():
        logp0, _ = logp_mod.deterministic_linear_logp(h0, w0, target.reshape(-1))
    old = logp0.view(rollouts, tokens) + 0.15 * torch.randn((rollouts, tokens), generator=g).to(DEV)
    ref = logp0.view(rollouts, tokens) + 0.15 * torch.randn((rollouts, tokens), generator=g).to(DEV)

    h = h0.clone().requires_grad_(True)
    w = w0.clone().requires_grad_(True)
    logp, _ = logp_mod.deterministic_linear_logp(h.view(rollouts, tokens, hidden), w, target)
    out = loss_mod.grpo_ratio_kl_loss(logp, old, ref, adv, mask, clip_eps=0.2, beta=0.01)
    out.loss.backward()
    assert torch.isfinite(out.loss) and h.grad.dtype == torch.bfloat16 and w.grad.shape == w.shape
    assert bool((out.ratio[~mask] == 0).all()) and bool((out.k3[~mask] == 0).all())

    h64 = h0.double().requires_grad_(True)
    w64 = w0.double().requires_grad_(True)
    logp64 = torch.log_softmax(h64 @ w64.t(), dim=-1).gather(1, target.reshape(-1, 1)).view(rollouts, tokens)
    want = _reference_rl_loss(logp64, old.double(), ref.double(), adv.double(), mask, 0.2, 0.01)
    want[0].backward()
    assert float(out.loss.detach()) == pytest.approx(float(want[0].detach()), rel=1e-4, abs=1e-6)
    for got, exact in ((h.grad, h64.grad), (w.grad, w64.grad)):
        scale = exact.abs().max().item()
        assert (got.double() - exact).abs().max().item() <= 2.0**-6 * scale  # d(logits) and the gradients are bf16
    masked_rows = (~mask).reshape(-1)
    assert bool((h.grad[masked_rows] == 0).all())  # masked tokens do not reach the hidden states

    # masked positions do not affect the loss, whatever they hold (reference test, :94-131)
    wild_old, wild_ref = old.clone(), ref.clone()
    wild_old[~mask], wild_ref[~mask] = -1000.0, 500.0
    again = loss_mod.grpo_ratio_kl_loss(logp.detach(), wild_old, wild_ref, adv, mask, clip_eps=0.2, beta=0.01)
    assert _same_bits(again.loss.reshape(1), out.loss.detach().reshape(1))


def test_config5_rollout_scale(logp_mod, loss_mod, oracle, config4):
    """64 rollouts x 1024 tokens through linear-LogP then the GRPO epilogue."""
    rollouts, per = 64, 1024
    tokens = rollouts * per
    h = inputs.hidden_states(tokens, seed=5001, rms_norm=False)
    gt = torch.Generator().manual_seed(5003)
    target = torch.randint(0, inputs.QWEN3_VOCAB, (tokens,), generator=gt)
    w, w_d = config4["w"], config4["w_d"]
    h_d, t_d = h.to(DEV), target.to(DEV)
    logp, lse = logp_mod.deterministic_linear_logp(h_d, w_d, t_d)
    assert logp.shape == (tokens,) and bool(torch.isfinite(logp).all()) and bool((logp <= 0).all())
    # per-rollout recomputation is bit-identical to the packed 65536-token call
    for r in (0, 31, 63):
        part, _ = logp_mod.deterministic_linear_logp(h_d[r * per : (r + 1) * per], w_d, t_d[r * per : (r + 1) * per])
        assert _same_bits(part, logp[r * per : (r + 1) * per]), r
    sample = torch.randperm(tokens, generator=torch.Generator().manual_seed(5004))[:128].sort().values
    ref_logp = oracle.linear_logp_chunked(inputs.bits(h[sample]), inputs.bits(w), target[sample].numpy(), chunk_elems=128 * 2048)[0]
    assert np.abs(logp.cpu().numpy()[sample.numpy()] - ref_logp).max() <= TOL_NATS

    old, ref, adv = inputs.grpo_side_inputs(logp, rollouts)
    lp2d = logp.view(rollouts, per)
    for beta in (0.0, 0.01):
        out = loss_mod.grpo_ratio_kl_loss(lp2d, old.view(rollouts, per).to(DEV), ref.view(rollouts, per).to(DEV), adv.to(DEV), clip_eps=0.2, beta=beta)
        e_loss, e_policy, e_kl, e_ratio, e_k3 = oracle.grpo_ratio_kl_loss(
            lp2d.cpu().numpy(), old.view(rollouts, per).numpy(), ref.view(rollouts, per).numpy(), adv.numpy(), clip_eps=0.2, beta=beta
        )
        assert np.allclose(out.ratio.cpu().numpy(), e_ratio, rtol=2e-6)
        assert np.allclose(out.k3.cpu().numpy(), e_k3, atol=3e-7)
        assert float(out.policy_loss) == pytest.approx(float(e_policy), rel=1e-4, abs=1e-6)
        assert float(out.kl) == pytest.approx(float(e_kl), rel=1e-4)
        assert float(out.loss) == pytest.approx(float(e_loss), rel=1e-4, abs=1e-6)
        rerun = loss_mod.grpo_ratio_kl_loss(lp2d, old.view(rollouts, per).to(DEV), ref.view(rollouts, per).to(DEV), adv.to(DEV), clip_eps=0.2, beta=beta)
        assert _same_bits(rerun.loss.reshape(1), out.loss.reshape(1))


# ---------------------------------------------------------------------------
# Engine-facing wrapper
# ---------------------------------------------------------------------------


def test_linear_logp_wrapper_entries(logp_mod):
    from rl_engine.integrations.common.linear_logp import LinearLogpWrapper

    h, w, target = inputs.logp_inputs(48, vocab=4096, hidden=256, seed=4600, rms_norm=False)
    hd, wd, td = h.to(DEV), w.to(DEV), target.to(DEV) % 4000
    wrapper = LinearLogpWrapper()
    temp = torch.rand(48, generator=torch.Generator().manual_seed(4601)).to(DEV) + 0.5
    out = wrapper(hd, wd, td, real_vocab_size=4000, temperature=temp, target="rollout")
    want, lse = logp_mod.deterministic_linear_logp(hd, wd, td, temperature=temp, real_vocab_size=4000)
    assert out.dtype == torch.float32 and _same_bits(out, want)
    prov = wrapper.provenance
    assert prov["deterministic_linear_logp"] is True and prov["real_vocab_size"] == 4000 and prov["target"] == "rollout"
    assert prov["logits_materialized"] is False and prov["hidden_shape"] == [48, 256]
    assert _same_bits(wrapper(hd, wd, td, real_vocab_size=4000, temperature=1.0), logp_mod.deterministic_linear_logp(hd, wd, td, real_vocab_size=4000)[0])
    # reused logits: same numbers as the from-logits operator, lse on request
    _, _, logits = logp_mod.deterministic_linear_logp(hd, wd, td, return_logits=True)
    got, got_lse = wrapper.from_local_logits(
        logits, td, tp_group=None, vocab_start_index=0, global_vocab_size=4096, real_vocab_size=4000, return_lse=True
    )
    ref = logp_mod.deterministic_logp_from_logits(logits, td, real_vocab_size=4000)
    assert _same_bits(got, ref[0]) and _same_bits(got_lse, ref[1])
    assert wrapper.provenance["lm_head_result_reused"] is True
    # training: gradients flow through the wrapper
    hg = hd.clone().requires_grad_(True)
    wrapper(hg, wd, td).sum().backward()
    assert hg.grad is not None and hg.grad.dtype == torch.bfloat16
    # contract errors keep the reference's wording
    with pytest.raises(ValueError, match="complete local vocab at offset zero"):
        wrapper(hd, wd, td, vocab_start_index=8)
    with pytest.raises(ValueError, match="real_vocab_size must be in"):
        wrapper(hd, wd, td, real_vocab_size=5000)
    with pytest.raises(TypeError, match="bfloat16 hidden and LM-head"):
        wrapper(hd.float(), wd, td)
    with pytest.raises(ValueError, match="equal rank-ordered TP shards"):
        wrapper.from_local_logits(logits, td, tp_group=None, vocab_start_index=0, global_vocab_size=8192, real_vocab_size=4000)


def test_linear_logp_wrapper_is_graph_capturable():
    """No host synchronisation on the call path: value checks are device-side assertions."""
    from rl_engine.integrations.common.linear_logp import LinearLogpWrapper

    h, w, target = inputs.logp_inputs(16, vocab=2048, hidden=128, seed=4700, rms_norm=False)
    hd, wd, td = h.to(DEV), w.to(DEV), target.to(DEV)
    wrapper = LinearLogpWrapper()
    with torch.no_grad():
        eager = wrapper(hd, wd, td, temperature=0.7).clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            wrapper(hd, wd, td, temperature=0.7)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = wrapper(hd, wd, td, temperature=0.7)
        for _ in range(3):
            captured.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert _same_bits(captured, eager)
