"""Both ends of the size range, through the C ABI, on a real MI355X: buffers of more than
2**31 elements, and empty inputs.

The reference sizes its rollout case at 65536 tokens x 151936 vocabulary columns
(9.96e9 logits); every kernel that walks a [rows, columns] buffer must index it
in 64 bits. Each case here makes one buffer cross 2**31 elements and compares
its last rows (the ones a 32-bit offset would misplace) and its first rows with
the same rows computed alone: bit equality, the batch-invariance contract."""

from __future__ import annotations

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"
TAIL = 96  # rows compared at either end
VOCAB = 151936


def _randn(shape, seed, scale=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(torch.bfloat16).to(DEV)


def _same_bits(x: torch.Tensor, y: torch.Tensor) -> bool:
    if x.dtype == torch.float32:
        return torch.equal(x.contiguous().view(torch.int32), y.contiguous().view(torch.int32))
    return torch.equal(x.contiguous().view(torch.int16), y.contiguous().view(torch.int16))


@pytest.fixture(autouse=True)
def _release_memory():
    yield
    torch.cuda.empty_cache()


@pytest.fixture(scope="module")
def C():
    from rl_engine import _C

    return _C


def _ends(m):
    return (slice(0, TAIL), slice(m - TAIL, m))


def test_det_gemm_output_over_2g_elements(C):
    m, n, k = 40000, 60000, 64
    assert m * n > 2**31
    a, w = _randn((m, k), 11), _randn((n, k), 12, 0.05)
    out = C.det_gemm_fwd_rhs_transposed(a, w)
    for rows in _ends(m):
        assert _same_bits(out[rows], C.det_gemm_fwd_rhs_transposed(a[rows].contiguous(), w))
    # one closed form at the very last element: 64 exact products, fp32 sum, one rounding
    ref = (a[-1].float().double() * w[-1].float().double()).sum()
    assert abs(out[-1, -1].float().item() - ref.item()) <= 2.0**-7 * max(abs(ref.item()), 0.05)


def test_det_gemm_fp32_output_over_2g_elements(C):
    m, n, k = 36000, 60000, 64
    assert m * n > 2**31
    a, w = _randn((m, k), 13), _randn((n, k), 14, 0.05)
    out = C.det_gemm_fwd_out_fp32(a, w.t())
    assert out.dtype == torch.float32
    for rows in _ends(m):
        assert _same_bits(out[rows], C.det_gemm_fwd_out_fp32(a[rows].contiguous(), w.t()))


def test_det_gemm_tree_output_over_2g_elements(C):
    m, n, k = 40000, 60000, 64
    a, w = _randn((m, k), 15), _randn((n, k), 16, 0.05)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    C.gemm_tree_strided(a, w.t(), out)
    for rows in _ends(m):
        alone = torch.empty((TAIL, n), dtype=torch.bfloat16, device=DEV)
        C.gemm_tree_strided(a[rows], w.t(), alone)
        assert _same_bits(out[rows], alone)


def test_gated_projection_output_over_2g_elements(C):
    m, inter, k = 40000, 60000, 64
    a, w = _randn((m, k), 17), _randn((2 * inter, k), 18, 0.3)
    out = C.det_gemm_swiglu(a, w)
    for rows in _ends(m):
        # 96 rows alone take the projection + elementwise route: same bits by contract
        assert _same_bits(out[rows], C.det_gemm_swiglu(a[rows].contiguous(), w))


def test_swiglu_elementwise_over_2g_elements(C):
    rows_n, cols = 36000, 60000
    g = torch.Generator(device=DEV).manual_seed(19)
    gate_up = torch.randn((rows_n, 2 * cols), generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    y = C.swiglu_packed_forward(gate_up)
    dy = torch.randn((rows_n, cols), generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    dg, du = C.swiglu_packed_backward(dy, gate_up)
    for rows in _ends(rows_n):
        part = gate_up[rows].contiguous()
        assert _same_bits(y[rows], C.swiglu_packed_forward(part))
        dg1, du1 = C.swiglu_packed_backward(dy[rows].contiguous(), part)
        assert _same_bits(dg[rows], dg1) and _same_bits(du[rows], du1)


def test_linear_logp_and_logits_over_2g_elements(C):
    t, d = 16384, 128
    assert t * VOCAB > 2**31
    h, w = _randn((t, d), 21), _randn((VOCAB, d), 22, 0.2)
    g = torch.Generator(device="cpu").manual_seed(23)
    tgt = torch.randint(0, VOCAB, (t,), generator=g).to(DEV)
    logp, lse, logits = C.fused_linear_logp(h, w, tgt, return_logits=True)
    assert logits.shape == (t, VOCAB) and logits.dtype == torch.float32
    for rows in _ends(t):
        lp1, lse1, lg1 = C.fused_linear_logp(h[rows].contiguous(), w, tgt[rows].contiguous(), return_logits=True)
        assert _same_bits(logp[rows], lp1) and _same_bits(lse[rows], lse1) and _same_bits(logits[rows], lg1)
    # the last rows against the dense formula on the logits the library returned
    dense = torch.log_softmax(logits[-TAIL:].double(), dim=-1).gather(1, tgt[-TAIL:, None])[:, 0]
    assert (logp[-TAIL:].double() - dense).abs().max().item() <= 1e-3

    # the same buffer through the logits-side kernels (tile statistics + gather, then backward)
    lp2, lse2 = C.hip_deterministic_logp_from_logits(logits, tgt, 0, VOCAB, 64)
    for rows in _ends(t):
        a1, b1 = C.hip_deterministic_logp_from_logits(logits[rows].contiguous(), tgt[rows].contiguous(), 0, VOCAB, 64)
        assert _same_bits(lp2[rows], a1) and _same_bits(lse2[rows], b1)
    assert (lp2[-TAIL:].double() - dense).abs().max().item() <= 1e-3


def test_linear_logp_backward_over_2g_elements(C):
    t, d = 16384, 128
    h, w = _randn((t, d), 31), _randn((VOCAB, d), 32, 0.2)
    g = torch.Generator(device="cpu").manual_seed(33)
    tgt = torch.randint(0, VOCAB, (t,), generator=g).to(DEV)
    grad = torch.randn((t,), generator=g).to(DEV)
    _, lse = C.fused_linear_logp(h, w, tgt)
    gh, gw = C.fused_linear_logp_bwd(h, w, tgt, lse, grad, None)[:2]
    assert gh.shape == (t, d) and gw.shape == (VOCAB, d)
    for rows in _ends(t):
        gh1 = C.fused_linear_logp_bwd(
            h[rows].contiguous(), w, tgt[rows].contiguous(), lse[rows].contiguous(), grad[rows].contiguous(), None,
            need_grad_weight=False,
        )[0]  # fmt: skip
        assert _same_bits(gh[rows], gh1)
    # grad_weight rows at both ends of the vocabulary against fp64 on the bf16-rounded d(logits)
    for cols in (slice(0, 32), slice(VOCAB - 32, VOCAB)):
        z = h.double() @ w[cols].double().t()
        dz = -torch.exp(z - lse.double()[:, None]) * grad.double()[:, None]
        ids = torch.arange(cols.start, cols.stop, device=DEV)
        dz = dz + (tgt[:, None] == ids[None, :]).double() * grad.double()[:, None]
        ref = dz.to(torch.bfloat16).double().t() @ h.double()
        scale = ref.abs().max().item()
        assert (gw[cols].double() - ref).abs().max().item() <= 2.0**-7 * scale


def test_empty_inputs_through_every_entry(C):
    """The other end of the size range: zero rows (and zero columns where the shape allows it)
    return empty tensors of the right shape and dtype without a launch."""
    from rl_engine.ops import logprob, loss

    w = _randn((64, 128), 41, 0.1)
    none = torch.empty((0, 128), dtype=torch.bfloat16, device=DEV)
    no_ids = torch.empty((0,), dtype=torch.int64, device=DEV)
    assert C.det_gemm_fwd_rhs_transposed(none, w).shape == (0, 64)
    assert C.det_gemm_fwd_out_fp32(none, w.t()).dtype == torch.float32
    tree = torch.empty((0, 64), dtype=torch.bfloat16, device=DEV)
    assert C.gemm_tree_strided(none, w.t(), tree).shape == (0, 64)
    logp, lse = C.fused_linear_logp(none, w, no_ids)
    assert logp.shape == (0,) and lse.shape == (0,) and logp.dtype == torch.float32
    logp, lse = logprob.deterministic_linear_logp(none.view(0, 3, 128), w, no_ids.view(0, 3))
    assert logp.shape == (0, 3)
    assert C.det_gemm_swiglu(none, w).shape == (0, 32)
    assert C.swiglu_packed_forward(torch.empty((0, 64), dtype=torch.bfloat16, device=DEV)).shape == (0, 32)
    logits = torch.empty((0, 64), dtype=torch.bfloat16, device=DEV)
    a, b = C.hip_deterministic_logp_from_logits(logits, no_ids, 0, 64, 8)
    assert a.shape == (0,) and b.shape == (0,)
    stats = C.hip_deterministic_logp_tile_stats(logits, 0, 64, 8)
    assert stats[0].shape == (0, 8)
    out = loss.grpo_ratio_kl_loss(torch.empty((0, 5), device=DEV), torch.empty((0, 5), device=DEV),
                                  torch.empty((0, 5), device=DEV), torch.empty((0,), device=DEV))
    assert float(out.loss) == 0.0 and out.ratio.shape == (0, 5)
