"""Backward of the fused linear-LogP on a real MI355X, through the C ABI.

Parity bar: grad_hidden / grad_weight are bf16 results of a bf16 GEMM over d(logits)
that were themselves rounded to bf16 once, so against the exact (fp64) gradient of the
oracle every element must lie within
    half a bf16 ulp of itself  +  (2^-8 + K 2^-24 + 2e-5) * sum_k |dz_k| |operand_k|
(the second term: dz rounding, fp32 accumulation over K terms, fp32 exp / lse).
grad_bias is fp32 and sums the unrounded fp32 dz (as the reference does): within
(2e-5 + T 2^-24) * sum_t |dz|, i.e. fp32 exp / lse and fp32 accumulation only.
Determinism, batch invariance of grad_hidden rows and configuration neutrality are
bit-exact."""

from __future__ import annotations

import numpy as np
import pytest
import torch

import inputs

pytestmark = pytest.mark.gpu

DEV = "cuda"


@pytest.fixture(scope="module")
def logp_mod():
    from rl_engine.ops import logprob

    return logprob


@pytest.fixture(scope="module")
def native():
    from rl_engine import _C

    return _C


def _bits16(x: torch.Tensor) -> torch.Tensor:
    return x.contiguous().view(torch.int16)


def _case(t, v, d, seed, *, bias=False, temperature=False, real=None):
    h, w, target = inputs.logp_inputs(t, vocab=v, hidden=d, seed=seed, rms_norm=False)
    w = (w.float() * 2.5).to(torch.bfloat16)
    gen = torch.Generator().manual_seed(seed + 1)
    real = v if real is None else real
    target = target % real
    out = {
        "h": h,
        "w": w,
        "target": target,
        "g_logp": torch.randn(t, generator=gen),
        "g_lse": torch.randn(t, generator=gen) * 0.5,
        "bias": torch.randn(v, generator=gen) * 0.3 if bias else None,
        "temp": torch.rand(t, generator=gen) * 1.5 + 0.5 if temperature else None,
        "real": real,
    }
    return out


def _gpu_backward(native, c, *, config=0, need_bias=None, g_lse=True):
    dev = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    logp, lse = native.fused_linear_logp(dev["h"], dev["w"], dev["target"], dev["bias"], dev["temp"], False, c["real"])
    need_bias = (c["bias"] is not None) if need_bias is None else need_bias
    grads = native.fused_linear_logp_bwd(
        dev["h"], dev["w"], dev["target"], lse, dev["g_logp"], dev["g_lse"] if g_lse else None, dev["bias"], dev["temp"],
        c["real"], need_grad_bias=need_bias, config=config,
    )  # fmt: skip
    return lse, grads


def _assert_grad_parity(oracle, c, lse, grads, *, g_lse=True):
    gh, gw, gb = grads
    hb, wb = inputs.bits(c["h"]), inputs.bits(c["w"])
    args = dict(
        grad_logp=c["g_logp"].numpy(),
        grad_lse=c["g_lse"].numpy() if g_lse else None,
        bias=None if c["bias"] is None else c["bias"].numpy(),
        temperature=None if c["temp"] is None else c["temp"].numpy(),
        real_vocab_size=c["real"],
    )
    lse64 = lse.double().cpu().numpy()
    dz = oracle.linear_logp_dlogits(hb, wb, c["target"].numpy(), lse64, dtype=np.float64, **args)
    hf = oracle.bf16_to_f32(hb).astype(np.float64)
    wf = oracle.bf16_to_f32(wb).astype(np.float64)
    t, v = dz.shape
    slack = 2.0**-8 + 2e-5

    def check(got_bits, exact, abs_sum, k, tag):
        got = oracle.bf16_to_f32(got_bits).astype(np.float64)
        bound = 2.0**-8 * np.abs(got) + (slack + k * 2.0**-24) * abs_sum + 1e-30
        worst = float((np.abs(got - exact) / bound).max())
        assert worst <= 1.0, f"{tag}: error is {worst:.3f}x the rounding + accumulation bound"

    check(inputs.bits(gh), dz @ wf, np.abs(dz) @ np.abs(wf), v, "grad_hidden")
    check(inputs.bits(gw), dz.T @ hf, np.abs(dz).T @ np.abs(hf), t, "grad_weight")
    if gb is not None:
        exact = dz.sum(axis=0)
        bound = (2e-5 + t * 2.0**-24) * np.abs(dz).sum(axis=0) + 1e-30  # no bf16 rounding of dz in this sum
        worst = float((np.abs(gb.double().cpu().numpy() - exact) / bound).max())
        assert worst <= 1.0, f"grad_bias: error is {worst:.3f}x the bound"
    # the reference's own bf16-dz formulation as a second, looser witness (its ws1 bf16 tolerance)
    ref = oracle.linear_logp_backward(hb, wb, c["target"].numpy(), lse64, **args)
    assert np.allclose(gh.double().cpu().numpy(), ref[0], atol=5e-2, rtol=2e-2)
    assert np.allclose(gw.double().cpu().numpy(), ref[1], atol=5e-2, rtol=2e-2)


@pytest.mark.parametrize(
    "shape,opts",
    [
        ((64, 1024, 128), {}),
        ((192, 2048, 256), dict(bias=True, temperature=True, real=1900)),
        ((40, 3000, 264), dict(bias=True)),  # D % 64 != 0 and V % 64 != 0: staged / element loaders
        ((130, 5000, 512), dict(temperature=True)),  # T % 64 != 0: weight gradient on the element loader
        ((256, 4096, 320), dict(bias=True, temperature=True, real=4000)),
        # from 512 tokens on (T % 8 == 0) the weight gradient reads the hidden states from a transposed copy
        # that is staged in the grad_hidden buffer: T % 64 != 0 with D % 64 != 0, and whole tiles
        ((520, 2048, 264), dict(bias=True)),
        ((1024, 3000, 256), dict(bias=True, temperature=True, real=2900)),
    ],
)
def test_backward_parity_with_oracle(native, oracle, shape, opts):
    t, v, d = shape
    c = _case(t, v, d, 5100 + t, **opts)
    lse, grads = _gpu_backward(native, c)
    assert grads[0].dtype == torch.bfloat16 and tuple(grads[0].shape) == (t, d)
    assert grads[1].dtype == torch.bfloat16 and tuple(grads[1].shape) == (v, d)
    _assert_grad_parity(oracle, c, lse, grads)
    if c["real"] < v:  # padded vocabulary rows get exactly zero
        assert not bool(grads[1][c["real"] :].any())
        assert not bool(grads[2][c["real"] :].any())


def test_backward_is_bitwise_deterministic_and_config_neutral(native):
    from rl_engine import _lib

    # the second case is large enough for the transposed-hidden form of the weight gradient, which the
    # register-staged configurations do not take
    for shape in ((320, 3072, 256), (576, 2048, 328)):
        c = _case(*shape, 5200, bias=True, temperature=True, real=shape[1] - 72)
        _, base = _gpu_backward(native, c)
        for _ in range(3):
            _, again = _gpu_backward(native, c)
            for x, y in zip(base, again):
                assert torch.equal(x.view(torch.uint8), y.view(torch.uint8))
        for name, value in _lib.LOGP_CONFIGS.items():
            for flag in (0, _lib.FORCE_STAGED):
                _, other = _gpu_backward(native, c, config=value | flag)
                for x, y in zip(base, other):
                    assert torch.equal(x.view(torch.uint8), y.view(torch.uint8)), (shape, name, flag)


@pytest.mark.parametrize("tokens", (1040, 2100))
def test_bias_gradient_is_config_neutral_above_1024_tokens(native, tokens):
    # above 1024 tokens the bias partial rows are per 64-token tile, and a forced 16-token tile is remapped to 64:
    # grad_bias (and the other two gradients) must keep the bits of the automatic choice under every configuration
    from rl_engine import _lib

    c = _case(tokens, 1536, 128, 5250 + tokens, bias=True, temperature=True, real=1500)
    _, base = _gpu_backward(native, c)
    for name, value in _lib.LOGP_CONFIGS.items():
        for flag in (0, _lib.FORCE_STAGED):
            _, other = _gpu_backward(native, c, config=value | flag)
            for x, y in zip(base, other):
                assert torch.equal(x.view(torch.uint8), y.view(torch.uint8)), (tokens, name, flag)
    assert not bool(base[2][1500:].any()) and bool(torch.isfinite(base[2]).all())


def test_grad_hidden_rows_are_batch_invariant(native):
    c = _case(384, 4096, 256, 5300, temperature=True)
    _, (gh_full, _, _) = _gpu_backward(native, c)
    for start, rows in ((0, 1), (37, 1), (100, 17), (128, 256), (383, 1)):
        part = {k: (v[start : start + rows] if isinstance(v, torch.Tensor) and k in ("h", "target", "g_logp", "g_lse", "temp") else v) for k, v in c.items()}
        _, (gh, _, _) = _gpu_backward(native, part)
        assert torch.equal(_bits16(gh), _bits16(gh_full[start : start + rows])), (start, rows)


def test_closed_forms_on_the_gpu(native):
    # grad_lse only: d(logits) = softmax * g / T, so grad_bias sums to sum_t g_t / T_t
    c = _case(128, 2048, 128, 5400, bias=True, temperature=True)
    dev = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    _, lse = native.fused_linear_logp(dev["h"], dev["w"], dev["target"], dev["bias"], dev["temp"], False, c["real"])
    _, _, gb = native.fused_linear_logp_bwd(
        dev["h"], dev["w"], dev["target"], lse, None, dev["g_lse"], dev["bias"], dev["temp"], c["real"], need_grad_bias=True
    )
    expect = float((c["g_lse"].double() / c["temp"].double()).sum())
    assert abs(float(gb.double().sum()) - expect) < 2e-2 * float((c["g_lse"].abs().double() / c["temp"].double()).sum())
    # zero upstream gradients give exactly zero everywhere
    zero = torch.zeros(128, device=DEV)
    gh, gw, gb = native.fused_linear_logp_bwd(
        dev["h"], dev["w"], dev["target"], lse, zero, zero, dev["bias"], dev["temp"], c["real"], need_grad_bias=True
    )
    assert not bool(gh.any()) and not bool(gw.any()) and not bool(gb.any())
    # identical weight rows: logp = -log V for any hidden, so grad_hidden of logp is ~0
    same = dev["w"][:1].expand(2048, -1).contiguous()
    _, lse_same = native.fused_linear_logp(dev["h"], same, dev["target"])
    gh, _, _ = native.fused_linear_logp_bwd(dev["h"], same, dev["target"], lse_same, dev["g_logp"], None)
    scale = float(dev["g_logp"].abs().max() * same.float().abs().max())
    assert float(gh.float().abs().max()) <= 2.0**-7 * scale


def test_autograd_entry_matches_the_native_backward(logp_mod, native):
    c = _case(96, 2048, 128, 5500, bias=True, temperature=True, real=2000)
    dev = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    h = dev["h"].clone().requires_grad_(True)
    w = dev["w"].clone().requires_grad_(True)
    b = dev["bias"].clone().requires_grad_(True)
    logp, lse = logp_mod.deterministic_linear_logp(
        h.view(8, 12, 128), w, dev["target"].view(8, 12), b, temperature=dev["temp"], real_vocab_size=2000
    )
    assert logp.shape == (8, 12) and logp.requires_grad and lse.requires_grad
    loss = (logp * dev["g_logp"].view(8, 12)).sum() + (lse * dev["g_lse"].view(8, 12)).sum()
    loss.backward()
    assert h.grad.dtype == torch.bfloat16 and h.grad.shape == h.shape
    assert w.grad.dtype == torch.bfloat16 and b.grad.dtype == b.dtype
    _, (gh, gw, gb) = _gpu_backward(native, c)
    assert torch.equal(_bits16(h.grad), _bits16(gh))
    assert torch.equal(_bits16(w.grad), _bits16(gw))
    assert torch.equal(b.grad, gb)
    # forward values under autograd are the inference values, bit for bit
    with torch.no_grad():
        logp2, lse2 = logp_mod.deterministic_linear_logp(
            dev["h"], dev["w"], dev["target"], dev["bias"], temperature=dev["temp"], real_vocab_size=2000
        )
    assert torch.equal(logp.detach().reshape(-1).view(torch.int32), logp2.view(torch.int32))
    # only hidden needs a gradient: the weight-sized outputs are skipped
    h2 = dev["h"].clone().requires_grad_(True)
    out, _ = logp_mod.deterministic_linear_logp(h2, dev["w"], dev["target"])
    out.sum().backward()
    assert h2.grad is not None and dev["w"].grad is None


def test_backward_argument_errors(native):
    c = _case(16, 256, 64, 5600)
    dev = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    _, lse = native.fused_linear_logp(dev["h"], dev["w"], dev["target"])
    with pytest.raises(RuntimeError, match="must be bf16"):
        native.fused_linear_logp_bwd(dev["h"].float(), dev["w"], dev["target"], lse, dev["g_logp"], None)
    with pytest.raises(RuntimeError, match="one value per row"):
        native.fused_linear_logp_bwd(dev["h"], dev["w"], dev["target"], lse[:3], dev["g_logp"], None)
    with pytest.raises(RuntimeError, match="real_vocab_size"):
        native.fused_linear_logp_bwd(dev["h"], dev["w"], dev["target"], lse, dev["g_logp"], None, None, None, 9999)
    # empty batch: token-summed gradients are zero, grad_hidden is empty
    empty = native.fused_linear_logp_bwd(
        dev["h"][:0], dev["w"], dev["target"][:0], lse[:0], dev["g_logp"][:0], None, need_grad_bias=False
    )
    assert tuple(empty[0].shape) == (0, 64) and not bool(empty[1].any())


# ---------------------------------------------------------------------------
# Full size (T = 8192, V = 151936, D = 4096): size-independent properties and sampled parity
# ---------------------------------------------------------------------------


def test_full_size_backward_properties_and_sampled_parity(native, oracle):
    h, w, target = inputs.logp_inputs(8192)
    t, v, d = 8192, w.size(0), w.size(1)
    gen = torch.Generator().manual_seed(5701)
    g_logp = torch.randn(t, generator=gen)
    g_lse = torch.randn(t, generator=gen) * 0.25
    bias = torch.randn(v, generator=gen) * 0.1
    hd, wd, td, bd = h.to(DEV), w.to(DEV), target.to(DEV), bias.to(DEV)
    _, lse = native.fused_linear_logp(hd, wd, td, bd)
    gh, gw, gb = native.fused_linear_logp_bwd(hd, wd, td, lse, g_logp.to(DEV), g_lse.to(DEV), bd, need_grad_bias=True)
    assert tuple(gh.shape) == (t, d) and tuple(gw.shape) == (v, d) and tuple(gb.shape) == (v,)
    assert bool(torch.isfinite(gh.float()).all()) and bool(torch.isfinite(gw.float()).all())
    # run to run: every output bit
    gh2, gw2, gb2 = native.fused_linear_logp_bwd(hd, wd, td, lse, g_logp.to(DEV), g_lse.to(DEV), bd, need_grad_bias=True)
    assert torch.equal(_bits16(gh), _bits16(gh2)) and torch.equal(_bits16(gw), _bits16(gw2)) and torch.equal(gb, gb2)
    # rows of grad_hidden are bit-identical at M = 1, M = 7, a ragged cut and another packing
    for lo, hi in ((0, 1), (0, 7), (8191, 8192), (5000, 5130)):
        part, _, _ = native.fused_linear_logp_bwd(
            hd[lo:hi], wd, td[lo:hi], lse[lo:hi], g_logp[lo:hi].to(DEV), g_lse[lo:hi].to(DEV), bd, need_grad_weight=False
        )
        assert torch.equal(_bits16(part), _bits16(gh[lo:hi])), (lo, hi)
    perm = torch.randperm(t, generator=torch.Generator().manual_seed(5702)).to(DEV)
    packed, _, _ = native.fused_linear_logp_bwd(
        hd[perm], wd, td[perm], lse[perm], g_logp.to(DEV)[perm], g_lse.to(DEV)[perm], bd, need_grad_weight=False
    )
    assert torch.equal(_bits16(packed), _bits16(gh[perm]))
    # probabilities sum to one: the bias gradient summed over the vocabulary is sum_t g_lse[t]
    expect = float(g_lse.double().sum())
    scale = float(g_logp.abs().double().sum() * 2 + g_lse.abs().double().sum())
    assert abs(float(gb.double().sum()) - expect) <= 2.0**-8 * scale
    # sampled parity: four token rows of grad_hidden and six vocabulary rows of grad_weight
    lse64 = lse.double().cpu().numpy()
    hb, wb = inputs.bits(h), inputs.bits(w)
    rows = np.array([0, 1777, 4096, 8191])
    dz = oracle.linear_logp_dlogits(
        hb[rows], wb, target.numpy()[rows], lse64[rows], g_logp.numpy()[rows], g_lse.numpy()[rows], bias.numpy(),
        dtype=np.float64,
    )  # fmt: skip
    wf = oracle.bf16_to_f32(wb).astype(np.float64)
    want = dz @ wf
    bound = 2.0**-8 * np.abs(want) + (2.0**-8 + v * 2.0**-24 + 2e-5) * (np.abs(dz) @ np.abs(wf)) + 1e-30
    got = gh[torch.from_numpy(rows).to(DEV)].double().cpu().numpy()
    assert float((np.abs(got - want) / bound).max()) <= 1.0
    cols = np.array([0, 1, 70000, 151935] + [int(target[5]), int(target[4096])])
    hf = oracle.bf16_to_f32(hb).astype(np.float64)
    z = hf @ wf[cols].T + bias.numpy().astype(np.float64)[cols]  # [T, 6] logits of the sampled columns
    p = np.exp(z - lse64[:, None])
    dz_cols = p * (g_lse.numpy().astype(np.float64) - g_logp.numpy().astype(np.float64))[:, None]
    for j, col in enumerate(cols):
        hit = target.numpy() == col
        dz_cols[hit, j] += g_logp.numpy().astype(np.float64)[hit]
    want_w = dz_cols.T @ hf
    bound_w = 2.0**-8 * np.abs(want_w) + (2.0**-8 + t * 2.0**-24 + 2e-5) * (np.abs(dz_cols).T @ np.abs(hf)) + 1e-30
    got_w = gw[torch.from_numpy(cols).to(DEV)].double().cpu().numpy()
    assert float((np.abs(got_w - want_w) / bound_w).max()) <= 1.0
    want_b = dz_cols.sum(axis=0)
    got_b = gb[torch.from_numpy(cols).to(DEV)].double().cpu().numpy()
    assert np.all(np.abs(got_b - want_b) <= (2.0**-8 + t * 2.0**-24 + 2e-5) * np.abs(dz_cols).sum(axis=0) + 1e-30)
