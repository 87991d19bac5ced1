"""The committed fixtures against the oracle and the input generators (no GPU)."""

from __future__ import annotations

from pathlib import Path

import numpy as np

import inputs

GOLDEN = Path(__file__).parent / "golden"


def test_config1_fixture_matches_generators_and_oracle(oracle):
    data = np.load(GOLDEN / "config1_det_gemm.npz")
    a, b = inputs.config1()
    a_bits, bt_bits = inputs.bits(a), inputs.bits(b.t().contiguous())
    assert int(a_bits.astype(np.uint64).sum()) == int(data["a_checksum"])
    assert int(inputs.bits(b).astype(np.uint64).sum()) == int(data["b_checksum"])
    assert data["expected_bits"].shape == (128, 1024)
    # the sequential restatement and the fixture (BLAS order) are the same GEMM to rounding
    seq = oracle.det_gemm_seq(a_bits[:32], bt_bits)
    ulp = oracle.bf16_ulp_distance(seq, data["expected_bits"][:32])
    assert (ulp <= 1).mean() > 0.999 and ulp.max() <= int(data["max_ulp_allowed"])
    # and both sit within the accumulation bound of the exact value
    exact = oracle.det_gemm_f64(a_bits[:8], bt_bits)
    got = oracle.bf16_to_f32(data["expected_bits"][:8]).astype(np.float64)
    abs_sum = np.abs(oracle.bf16_to_f32(a_bits[:8])).astype(np.float64) @ np.abs(oracle.bf16_to_f32(bt_bits)).astype(np.float64).T
    assert np.all(np.abs(got - exact) <= 2.0**-8 * np.abs(got) + 1024 * 2.0**-24 * abs_sum)


def test_small_logp_fixture_matches_oracle(oracle):
    d = np.load(GOLDEN / "small_linear_logp.npz")
    logp, lse = oracle.linear_logp_chunked(d["hidden_bits"], d["weight_bits"], d["target"])[:2]
    assert np.allclose(logp, d["logp"], atol=2e-6, rtol=0) and np.allclose(lse, d["lse"], atol=2e-6, rtol=0)
    exact = oracle.linear_logp_f64(d["hidden_bits"], d["weight_bits"], d["target"])[0]
    assert np.abs(d["logp"] - exact).max() < 1e-5
    exact2 = oracle.linear_logp_f64(
        d["hidden_bits"], d["weight_bits"], d["target"] % 1900, d["bias"], temperature=d["temperature"], real_vocab_size=1900
    )[0]
    assert np.abs(d["logp_bias_temp_pad"] - exact2).max() < 1e-5


def test_small_grpo_fixture_matches_oracle(oracle):
    d = np.load(GOLDEN / "small_grpo.npz")
    loss, policy, kl, ratio, k3 = oracle.grpo_ratio_kl_loss(d["logp"], d["old"], d["ref"], d["adv"], d["mask"], clip_eps=0.2, beta=0.01)
    assert np.allclose([loss, policy, kl], d["loss3"], rtol=1e-6)
    assert np.array_equal(ratio, d["ratio"]) and np.array_equal(k3, d["k3"])
