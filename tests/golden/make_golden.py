"""Writes the fixtures under tests/golden/ from the CPU oracle.

The reference ships no stored vectors for this path (its tests/data/ holds only a
.gitkeep), so these are oracle outputs on seeded inputs: they freeze the oracle
and the input generators, and give the GPU tests a fixed target.

Run from the repository root:  python tests/golden/make_golden.py
"""

from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

import inputs  # noqa: E402
from oracle import reference_math as oracle  # noqa: E402


def config1():
    a, b = inputs.config1()
    a_bits, bt_bits = inputs.bits(a), inputs.bits(b.t().contiguous())
    expected = oracle.det_gemm_ref(a_bits, bt_bits)
    seq = oracle.det_gemm_seq(a_bits, bt_bits)
    # two legitimate fp32 summation orders differ by at most this many bf16 ulps here
    max_ulp = int(oracle.bf16_ulp_distance(expected, seq).max())
    np.savez_compressed(
        HERE / "config1_det_gemm.npz",
        expected_bits=expected,
        a_checksum=np.uint64(inputs.bits(a).astype(np.uint64).sum()),
        b_checksum=np.uint64(inputs.bits(b).astype(np.uint64).sum()),
        max_ulp_allowed=np.int64(max(2 * max_ulp, 4)),
    )


def small_logp():
    h, w, target = inputs.logp_inputs(48, vocab=2000, hidden=128, seed=4101)
    rng = np.random.default_rng(4102)
    bias = (rng.standard_normal(2000) * 0.2).astype(np.float32)
    temp = (0.5 + rng.random(48)).astype(np.float32)
    hb, wb = inputs.bits(h), inputs.bits(w)
    logp, lse = oracle.linear_logp_chunked(hb, wb, target.numpy())[:2]
    logp_bt, lse_bt = oracle.linear_logp_dense(hb, wb, target.numpy() % 1900, bias, temperature=temp, real_vocab_size=1900)
    np.savez_compressed(
        HERE / "small_linear_logp.npz",
        hidden_bits=hb,
        weight_bits=wb,
        target=target.numpy(),
        bias=bias,
        temperature=temp,
        logp=logp,
        lse=lse,
        logp_bias_temp_pad=logp_bt,
        lse_bias_temp_pad=lse_bt,
    )


def small_grpo():
    rng = np.random.default_rng(5101)
    rollouts, tokens = 6, 300
    logp = -np.abs(rng.standard_normal((rollouts, tokens))).astype(np.float32) * 2
    old = (logp + 0.05 * rng.standard_normal(logp.shape)).astype(np.float32)
    ref = (logp + 0.05 * rng.standard_normal(logp.shape)).astype(np.float32)
    adv = rng.standard_normal(rollouts).astype(np.float32)
    mask = rng.random(logp.shape) < 0.75
    loss, policy, kl, ratio, k3 = oracle.grpo_ratio_kl_loss(logp, old, ref, adv, mask, clip_eps=0.2, beta=0.01)
    np.savez_compressed(
        HERE / "small_grpo.npz",
        logp=logp,
        old=old,
        ref=ref,
        adv=adv,
        mask=mask,
        loss3=np.array([loss, policy, kl], np.float32),
        ratio=ratio,
        k3=k3,
    )


if __name__ == "__main__":
    config1()
    small_logp()
    small_grpo()
    for p in sorted(HERE.glob("*.npz")):
        print(p.name, p.stat().st_size, "bytes")
