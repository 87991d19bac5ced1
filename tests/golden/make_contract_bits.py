"""Writes tests/golden/contract_bits.json: SHA-256 of the raw output bytes of the GPU kernels
on the stored fixture inputs, one entry per arithmetic contract id.

The contracts promise bit-identical results for a given id across builds of the library; this
file freezes the bits the first shipped build produced, so a change of arithmetic that forgets
to bump the id fails tests/test_contract_bits_gpu.py. Needs an MI355X:

    python tests/golden/make_contract_bits.py [output.json]
"""

from __future__ import annotations

import hashlib
import json
import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
sys.path.insert(0, str(ROOT / "rl-kernel_amd"))
sys.path.insert(0, str(ROOT / "tests"))

import inputs  # noqa: E402


def _sha(t: torch.Tensor) -> str:
    raw = t.detach().contiguous().cpu()
    raw = raw.view(torch.int16) if raw.dtype == torch.bfloat16 else raw
    return hashlib.sha256(raw.numpy().tobytes()).hexdigest()


def contract_bits() -> dict:
    from rl_engine import _lib
    from rl_engine.backends.rocm.gemm import det_gemm as gemm
    from rl_engine.ops.logprob import deterministic_linear_logp

    dev = "cuda"
    lib = _lib.load()
    a, b = inputs.config1()  # seeded; config1_det_gemm.npz holds the checksums of these operands
    a, b = a.to(dev), b.to(dev)
    out = {}
    out[lib.rlk_contract_id().decode()] = {"config1_det_gemm": _sha(gemm.mfma_gemm(a, b))}
    out[lib.rlk_det_gemm_tree_contract_id().decode()] = {"config1_det_gemm": _sha(gemm.tree_gemm(a, b))}
    d = np.load(HERE / "small_linear_logp.npz")
    h = inputs.from_bits(d["hidden_bits"], dev)
    w = inputs.from_bits(d["weight_bits"], dev)
    t = torch.from_numpy(d["target"]).to(dev)
    logp, lse = deterministic_linear_logp(h, w, t)
    logp2, lse2 = deterministic_linear_logp(
        h, w, t % 1900, torch.from_numpy(d["bias"]).to(dev), temperature=torch.from_numpy(d["temperature"]).to(dev), real_vocab_size=1900
    )
    out[lib.rlk_linear_logp_contract_id().decode()] = {
        "small_linear_logp.logp": _sha(logp),
        "small_linear_logp.lse": _sha(lse),
        "small_linear_logp.logp_bias_temp_pad": _sha(logp2),
        "small_linear_logp.lse_bias_temp_pad": _sha(lse2),
    }
    # gradients of the fused linear-LogP (same contract id: the backward is part of it)
    from rl_engine import _C

    g = torch.linspace(-1.0, 1.0, h.size(0), device=dev)
    grad_h, grad_w, _ = _C.fused_linear_logp_bwd(h, w, t, lse, g, None)
    out[lib.rlk_linear_logp_contract_id().decode()]["small_linear_logp.grad_hidden"] = _sha(grad_h)
    out[lib.rlk_linear_logp_contract_id().decode()]["small_linear_logp.grad_weight"] = _sha(grad_w)
    # bias gradient (fp32 sums of the unrounded d(logits) in the fixed token tree) on the padded case
    bias = torch.from_numpy(d["bias"]).to(dev)
    temp = torch.from_numpy(d["temperature"]).to(dev)
    _, _, grad_b = _C.fused_linear_logp_bwd(h, w, t % 1900, lse2, g, None, bias, temp, 1900, need_grad_bias=True)
    out[lib.rlk_linear_logp_contract_id().decode()]["small_linear_logp.grad_bias_bias_temp_pad"] = _sha(grad_b)
    # log-probabilities from materialised logits (the fp32 logits of the same case, and their bf16 rounding)
    logits = _C.det_gemm_fwd_out_fp32(h, w.t())
    vocab = logits.size(1)
    tiles = next(n for n in (64, 16, 8, 1) if vocab % n == 0)
    entries = {}
    for name, z in (("fp32", logits), ("bf16", logits.to(torch.bfloat16))):
        lp, ls = _C.hip_deterministic_logp_from_logits(z, t, 0, vocab, tiles)
        tmax, tsum = _C.hip_deterministic_logp_tile_stats(z, 0, vocab - 37, tiles, temperature=temp)
        entries[f"small_linear_logp.from_{name}_logits.logp"] = _sha(lp)
        entries[f"small_linear_logp.from_{name}_logits.lse"] = _sha(ls)
        entries[f"small_linear_logp.from_{name}_logits.tile_max_temp_pad"] = _sha(tmax)
        entries[f"small_linear_logp.from_{name}_logits.tile_sum_temp_pad"] = _sha(tsum)
    out[lib.rlk_logits_logp_contract_id().decode()] = entries
    # the sequential fp32 chain (fully specified: the CPU suite checks the stored hash against the oracle)
    out[lib.rlk_det_gemm_seq_contract_id().decode()] = {"config1_det_gemm_fp32": _sha(_C.det_gemm_fwd_fp32(a, b))}
    # gated FFN on the same hidden states: packed gate/up projection + SwiGLU, then down
    from rl_engine.ops.ffn import qwen3_ffn_packed_inference

    w_gu = inputs.randn_bf16(9901, 2 * 192, h.size(1), 0.1).to(dev)
    w_d = inputs.randn_bf16(9902, h.size(1), 192, 0.1).to(dev)
    out[lib.rlk_contract_id().decode()]["small_gated_ffn"] = _sha(qwen3_ffn_packed_inference(h, w_gu, w_d))
    big = inputs.randn_bf16(9903, 200, h.size(1)).to(dev)  # above 128 tokens: the fused projection kernel
    out[lib.rlk_contract_id().decode()]["gated_ffn_200_tokens"] = _sha(qwen3_ffn_packed_inference(big, w_gu, w_d))
    return out


if __name__ == "__main__":
    target = Path(sys.argv[1]) if len(sys.argv) > 1 else HERE / "contract_bits.json"
    target.write_text(json.dumps(contract_bits(), indent=2, sort_keys=True) + "\n")
    print(target.read_text())
