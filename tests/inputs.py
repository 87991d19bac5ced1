"""Seeded synthetic inputs for the five benchmark configurations.

Values are drawn in fp32 from a host ``torch.Generator`` and rounded to bf16,
the pattern the reference's tests use (tests/ops/logprob/test_linear_logp.py:1419-1425).
Rows of a smaller token count are prefixes of the largest tensor of the same
seed, so a row can be compared across batch sizes.
"""

from __future__ import annotations

import numpy as np
import torch

QWEN3_HIDDEN = 4096
QWEN3_INTER = 12288
QWEN3_VOCAB = 151936
QWEN3_QKV_OUT = 6144  # 32 q heads + 8 kv heads (k and v), head_dim 128


def randn_bf16(seed: int, rows: int, cols: int, scale: float = 1.0) -> torch.Tensor:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    x = torch.randn((rows, cols), generator=g, dtype=torch.float32)
    if scale != 1.0:
        x = x * scale
    return x.to(torch.bfloat16)


def bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor (any device) -> numpy uint16 bit patterns on the host."""
    return t.detach().cpu().contiguous().view(torch.uint16).numpy().copy()


def from_bits(b: np.ndarray, device="cpu") -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(b, dtype=np.uint16)).view(torch.bfloat16).to(device)


def config1():
    """A [128,1024] ~N(0,1), B [1024,1024] ~N(0,0.02) (B returned as [K,N])."""
    a = randn_bf16(1001, 128, 1024)
    b = randn_bf16(1002, 1024, 1024, 0.02)
    return a, b


def ffn_weights(seed: int = 2000):
    """Qwen3-8B FFN weights in native [out,in] layout: gate_up [24576,4096], down [4096,12288]."""
    w_gu = randn_bf16(seed + 1, 2 * QWEN3_INTER, QWEN3_HIDDEN, 0.02)
    w_d = randn_bf16(seed + 2, QWEN3_HIDDEN, QWEN3_INTER, 0.02)
    return w_gu, w_d


def ffn_activations(tokens: int, seed: int = 2000):
    x = randn_bf16(seed + 3, tokens, QWEN3_HIDDEN)
    h = randn_bf16(seed + 4, tokens, QWEN3_INTER)
    return x, h


def ragged_lengths(total: int, lo: int = 64, hi: int = 2048, seed: int = 3001) -> list[int]:
    """Sequence lengths ~U[lo,hi] drawn until they sum to ``total`` (last one clipped)."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    out, acc = [], 0
    while acc < total:
        n = int(torch.randint(lo, hi + 1, (1,), generator=g).item())
        n = min(n, total - acc)
        out.append(n)
        acc += n
    return out


def packing_order(n_seqs: int, seed: int) -> list[int]:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return torch.randperm(n_seqs, generator=g).tolist()


def pack_rows(lengths: list[int], order: list[int]) -> torch.Tensor:
    """Row index map of a packing: position p of the packed batch holds canonical token map[p]."""
    starts = np.concatenate([[0], np.cumsum(lengths)[:-1]])
    parts = [torch.arange(int(starts[s]), int(starts[s]) + lengths[s]) for s in order]
    return torch.cat(parts)


def hidden_states(tokens: int, hidden: int = QWEN3_HIDDEN, seed: int = 4001, rms_norm: bool = True) -> torch.Tensor:
    """hidden [T,D] ~N(0,1), optionally RMS-normalised in fp32, rounded to bf16."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    h = torch.randn((tokens, hidden), generator=g, dtype=torch.float32)
    if rms_norm:
        h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + 1e-6)
    return h.to(torch.bfloat16)


def logp_inputs(tokens: int, vocab: int = QWEN3_VOCAB, hidden: int = QWEN3_HIDDEN, seed: int = 4001, rms_norm: bool = True):
    """hidden [T,D] (optionally RMS-normalised in fp32), lm_head W [V,D] ~N(0,0.02), targets ~U[0,V)."""
    h = hidden_states(tokens, hidden, seed, rms_norm)
    gw = torch.Generator(device="cpu")
    gw.manual_seed(seed + 1)
    w = torch.empty((vocab, hidden), dtype=torch.bfloat16)
    step = 8192
    for v0 in range(0, vocab, step):
        v1 = min(v0 + step, vocab)
        w[v0:v1] = (torch.randn((v1 - v0, hidden), generator=gw, dtype=torch.float32) * 0.02).to(torch.bfloat16)
    gt = torch.Generator(device="cpu")
    gt.manual_seed(seed + 2)
    target = torch.randint(0, vocab, (tokens,), generator=gt, dtype=torch.int64)
    return h, w, target


def grpo_side_inputs(logp: torch.Tensor, rollouts: int, seed: int = 5001):
    """old/ref log-probs = logp + N(0,0.05) and per-rollout advantages ~N(0,1)."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    lp = logp.detach().float().cpu()
    old = lp + 0.05 * torch.randn(lp.shape, generator=g)
    ref = lp + 0.05 * torch.randn(lp.shape, generator=g)
    adv = torch.randn((rollouts,), generator=g)
    return old, ref, adv
