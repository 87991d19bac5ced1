"""SwiGLU, the fused gate/up projection and the gated FFN on a real MI355X, through the C ABI.

Tolerance: the elementwise kernels are within 1 bf16 ulp of the CPU oracle (their only
difference is the last bit of the fp32 exponential); the fused GEMM + SwiGLU kernel equals
the GEMM followed by the elementwise kernel bit for bit; rows are bit-invariant across
batches; the FFN is held to the bf16 rounding bound of its three projections."""

from __future__ import annotations

import numpy as np
import pytest
import torch

import inputs

pytestmark = pytest.mark.gpu

DEV = "cuda"


@pytest.fixture(scope="module")
def native():
    from rl_engine import _C

    return _C


@pytest.fixture(scope="module")
def ffn_mod():
    from rl_engine.ops import ffn

    return ffn


def _same_bits(x, y):
    return torch.equal(x.contiguous().view(torch.int16), y.contiguous().view(torch.int16))


@pytest.mark.parametrize("shape", [(64, 256), (37, 1000), (5, 7), (1, 12288), (300, 24)])
def test_elementwise_forward_and_backward_match_the_oracle(native, oracle, shape):
    rows, cols = shape
    gate = inputs.randn_bf16(8100, rows, cols, 2.0)
    up = inputs.randn_bf16(8101, rows, cols)
    dy = inputs.randn_bf16(8102, rows, cols)
    y = native.swiglu_forward(gate.to(DEV), up.to(DEV))
    ref = oracle.swiglu(inputs.bits(gate), inputs.bits(up))
    assert oracle.bf16_ulp_distance(inputs.bits(y), ref).max() <= 1
    d_gate, d_up = native.swiglu_backward(dy.to(DEV), gate.to(DEV), up.to(DEV))
    ref_g, ref_u = oracle.swiglu_backward(inputs.bits(dy), inputs.bits(gate), inputs.bits(up))
    assert oracle.bf16_ulp_distance(inputs.bits(d_gate), ref_g).max() <= 1
    assert oracle.bf16_ulp_distance(inputs.bits(d_up), ref_u).max() <= 1
    # packed layout: same bits as the separate form; unaligned widths take the element path
    packed = torch.cat([gate, up], dim=1).to(DEV)
    assert _same_bits(native.swiglu_packed_forward(packed), y)
    pg, pu = native.swiglu_packed_backward(dy.to(DEV), packed)
    assert _same_bits(pg, d_gate) and _same_bits(pu, d_up)
    # a row alone equals the row in the batch
    assert _same_bits(native.swiglu_forward(gate[-1:].to(DEV), up[-1:].to(DEV)), y[-1:])


def test_elementwise_special_values(native):
    gate = torch.tensor([[0.0, -0.0, 50.0, -50.0, float("inf"), float("-inf"), float("nan"), 1.0]], dtype=torch.bfloat16, device=DEV)
    up = torch.tensor([[3.0, 3.0, 2.0, 2.0, 1.0, 1.0, 1.0, float("nan")]], dtype=torch.bfloat16, device=DEV)
    y = native.swiglu_forward(gate, up).float().cpu()[0]
    assert y[0] == 0 and y[1] == 0 and y[2] == 100.0 and abs(float(y[3])) < 1e-18
    assert y[4] == float("inf") and torch.isnan(y[5]) and torch.isnan(y[6]) and torch.isnan(y[7])


@pytest.mark.parametrize(
    "shape",
    [(300, 256, 256), (1024, 1000, 128), (17, 128, 64), (64, 136, 4096), (513, 3000, 512), (4096, 1536, 1024), (16, 512, 256), (1, 256, 4096), (40, 256, 72), (129, 4096, 128), (128, 4096, 128), (200, 136, 64),
     # up to 16 rows with K >= 1024: the streaming kernel with the gated panel (edges: I % 8, one feature)
     (16, 12288, 4096), (5, 13, 1024), (9, 100, 2048), (16, 1, 1088), (2, 8, 12288)],
)
def test_fused_projection_equals_gemm_then_activation(native, shape):
    m, inter, k = shape
    x = inputs.randn_bf16(8200, m, k).to(DEV)
    w = inputs.randn_bf16(8201, 2 * inter, k, 0.05).to(DEV)
    expected = native.swiglu_packed_forward(native.det_gemm_fwd_rhs_transposed(x, w))
    for _ in range(3):
        assert _same_bits(native.det_gemm_swiglu(x, w), expected)
    out = torch.full((m, inter + 8), 7.0, dtype=torch.bfloat16, device=DEV)
    native.det_gemm_swiglu(x, w, out[:, :inter])
    assert _same_bits(out[:, :inter], expected) and bool((out[:, inter:] == 7.0).all())
    # rows do not depend on the batch they are in
    for start, rows in ((0, 1), (m // 2, min(20, m - m // 2)), (m - 1, 1)):
        part = native.det_gemm_swiglu(x[start : start + rows], w)
        assert _same_bits(part, expected[start : start + rows]), (start, rows)


def test_packed_inference_ffn(native, ffn_mod, oracle):
    t, h, inter = 96, 256, 384
    x = inputs.randn_bf16(8300, t, h)
    w_gu = inputs.randn_bf16(8301, 2 * inter, h, 0.1)
    w_d = inputs.randn_bf16(8302, h, inter, 0.1)
    xd, gud, dd = x.to(DEV), w_gu.to(DEV), w_d.to(DEV)
    out = ffn_mod.qwen3_ffn_packed_inference(xd.view(8, 12, h), gud, dd)
    assert out.shape == (8, 12, h) and out.dtype == torch.bfloat16
    manual = native.det_gemm_fwd_rhs_transposed(native.swiglu_packed_forward(native.det_gemm_fwd_rhs_transposed(xd, gud)), dd)
    assert _same_bits(out.reshape(t, h), manual)
    # parity with the oracle's FFN: one bf16 ulp of the activation moves the output by at most
    # 2^-7 * sum |act| |w|; the rest is the output's own rounding
    ref = oracle.bf16_to_f32(oracle.gated_ffn(inputs.bits(x), inputs.bits(w_gu), inputs.bits(w_d))).astype(np.float64)
    got = out.reshape(t, h).double().cpu().numpy()
    act = oracle.bf16_to_f32(oracle.swiglu_packed(oracle.det_gemm_ref(inputs.bits(x), inputs.bits(w_gu)))).astype(np.float64)
    scale = np.abs(act) @ np.abs(oracle.bf16_to_f32(inputs.bits(w_d)).astype(np.float64)).T
    assert np.all(np.abs(got - ref) <= 2.0**-7 * np.abs(ref) + 2.0**-7 * scale + 1e-30)
    # batch invariance through the whole FFN, decode-sized batches included (other kernels)
    for rows in (1, 7, 16, 17, 64):
        part = ffn_mod.qwen3_ffn_packed_inference(xd[:rows], gud, dd)
        assert _same_bits(part, out.reshape(t, h)[:rows]), rows
    # the staging form writes into a caller-owned buffer
    staging = torch.zeros((t, h), dtype=torch.bfloat16, device=DEV)
    torch.ops.rl_kernel.qwen3_ffn_packed_inference_to_staging(xd, gud, dd, staging)
    assert _same_bits(staging, manual)


def test_training_ffn_forward_and_backward(native, ffn_mod):
    t, h, inter = 128, 128, 192
    x = inputs.randn_bf16(8400, t, h).to(DEV)
    wg = inputs.randn_bf16(8401, inter, h, 0.1).to(DEV)
    wu = inputs.randn_bf16(8402, inter, h, 0.1).to(DEV)
    wd = inputs.randn_bf16(8403, h, inter, 0.1).to(DEV)
    packed = torch.cat([wg, wu], dim=0).contiguous()
    params = [p.clone().requires_grad_(True) for p in (x, wg, wu, wd)]
    out = ffn_mod.qwen3_ffn(*params, fused_gate_up_weight=packed)
    assert _same_bits(out.detach(), ffn_mod.qwen3_ffn_packed_inference(x, packed, wd))
    dy = inputs.randn_bf16(8404, t, h).to(DEV)
    out.backward(dy)
    # separate gate / up weights: same forward and backward bits as the packed form
    params2 = [p.clone().requires_grad_(True) for p in (x, wg, wu, wd)]
    out2 = ffn_mod.qwen3_ffn(*params2)
    assert _same_bits(out2.detach(), out.detach())
    out2.backward(dy)
    for a, b in zip(params, params2):
        assert a.grad is not None and a.grad.dtype == torch.bfloat16 and _same_bits(a.grad, b.grad)
    # fp32 autograd of the same formula: gradients agree to bf16 accuracy
    ref = [p.detach().float().requires_grad_(True) for p in (x, wg, wu, wd)]
    g = ref[0] @ ref[1].t()
    u = ref[0] @ ref[2].t()
    ((torch.nn.functional.silu(g) * u) @ ref[3].t()).backward(dy.float())
    for got, want, name in zip(params, ref, ("x", "gate", "up", "down")):
        err = (got.grad.float() - want.grad).abs().max().item()
        assert err <= 3e-2 * want.grad.abs().max().item() + 1e-3, (name, err)
    # run to run
    params3 = [p.clone().requires_grad_(True) for p in (x, wg, wu, wd)]
    ffn_mod.qwen3_ffn(*params3, fused_gate_up_weight=packed).backward(dy)
    for a, b in zip(params, params3):
        assert _same_bits(a.grad, b.grad)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(64, 256), (37, 1000), (5, 7), (3, 4, 24)])
def test_swiglu_fp16_and_fp32_tensors(native, oracle, dtype, shape):
    """The reference's activation kernels dispatch on the element type (activation.cu:240-284): same
    fp32 arithmetic, one rounding to the element type. fp32: within 4 fp32 ulp-scale of the oracle
    (hardware exp and reciprocal); fp16: the oracle's value within half an fp16 ulp plus that."""
    g = torch.Generator().manual_seed(8600 + len(shape))
    gate = (torch.randn(shape, generator=g) * 2.0).to(dtype)
    up = torch.randn(shape, generator=g).to(dtype)
    dy = torch.randn(shape, generator=g).to(dtype)
    y = native.swiglu_forward(gate.to(DEV), up.to(DEV))
    d_gate, d_up = native.swiglu_backward(dy.to(DEV), gate.to(DEV), up.to(DEV))
    assert y.dtype == dtype and y.shape == gate.shape and d_gate.dtype == dtype and d_up.shape == up.shape
    want_y = oracle.swiglu_values(gate.float().numpy(), up.float().numpy())
    want_g, want_u = oracle.swiglu_values(gate.float().numpy(), up.float().numpy(), dy.float().numpy())
    eps = 2.0**-11 if dtype == torch.float16 else 0.0
    floor = 2.0**-25 if dtype == torch.float16 else 0.0  # half an fp16 subnormal step
    gf, uf, df = (np.abs(t.double().numpy()) for t in (gate, up, dy))
    # the sigmoid is good to about 2 fp32 ulp; silu'(g) = s (1 + g (1 - s)) can cancel, so its error is
    # absolute in (1 + |g|), not relative to the result
    scales = (gf * uf, df * uf * (1.0 + gf), df * gf)
    for got, want, scale in zip((y, d_gate, d_up), (want_y, want_g, want_u), scales):
        err = np.abs(got.double().cpu().numpy() - want.astype(np.float64))
        assert np.all(err <= eps * np.abs(want) + 2.0**-21 * scale + floor + 1e-30)
    if len(shape) == 2:
        packed = torch.cat([gate, up], dim=1).contiguous().to(DEV)
        assert torch.equal(native.swiglu_packed_forward(packed), y)
        pg, pu = native.swiglu_packed_backward(dy.to(DEV), packed)
        assert torch.equal(pg, d_gate) and torch.equal(pu, d_up)
    with pytest.raises(RuntimeError, match="must share dtype"):
        native.swiglu_forward(gate.to(DEV), up.to(DEV).to(torch.bfloat16))


def test_argument_errors(native, ffn_mod):
    x = torch.zeros((4, 64), dtype=torch.bfloat16, device=DEV)
    w = torch.zeros((32, 64), dtype=torch.bfloat16, device=DEV)
    wd = torch.zeros((64, 32), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="gate and up must share shape"):
        native.swiglu_forward(x, x[:, :32].contiguous())
    with pytest.raises(RuntimeError, match="width must be even"):
        native.swiglu_packed_forward(torch.zeros((4, 7), dtype=torch.bfloat16, device=DEV))
    with pytest.raises(RuntimeError, match="must be contiguous"):
        native.swiglu_forward(x[:, ::2], x[:, ::2])
    with pytest.raises(RuntimeError, match="K mismatch"):
        native.det_gemm_swiglu(x, torch.zeros((32, 48), dtype=torch.bfloat16, device=DEV))
    with pytest.raises(ValueError, match="gate_weight must have shape"):
        ffn_mod.qwen3_ffn(x, w[:, :32].contiguous(), w, wd)
    with pytest.raises(TypeError, match="dtype bfloat16"):
        ffn_mod.qwen3_ffn(x.float(), w, w, wd)
    with pytest.raises(ValueError, match="at least one token"):
        ffn_mod.qwen3_ffn(x[:0], w, w, wd)
    with pytest.raises(RuntimeError, match="deterministic FFN only"):
        ffn_mod.qwen3_ffn(x, w, w, wd, deterministic=False)


@pytest.mark.parametrize("rows", [8, 64, 300])
def test_ffn_and_logp_stages_replay_bit_identically_in_a_hip_graph(native, ffn_mod, rows):
    """The rollout path is captured once and replayed against capture-time addresses: the FFN
    (fused gate/up + SwiGLU, then down into a staging buffer), the LogP-from-logits stage and the
    fused linear-LogP must give the eager bits on every replay (eager work and synchronisations
    in between)."""
    # (the `_C` layer: the Python entry points above it validate targets on the host, which a
    # capture does not allow; the reference's wrapper has a `targets_validated` switch for this)
    h, inter, vocab = 256, 384, 2048
    x = inputs.randn_bf16(8500, rows, h).to(DEV)
    w_gu = inputs.randn_bf16(8501, 2 * inter, h, 0.1).to(DEV)
    w_d = inputs.randn_bf16(8502, h, inter, 0.1).to(DEV)
    w_lm = inputs.randn_bf16(8503, vocab, h, 0.1).to(DEV)
    target = torch.randint(0, vocab, (rows,), generator=torch.Generator().manual_seed(8504)).to(DEV)
    staging = torch.zeros((rows, h), dtype=torch.bfloat16, device=DEV)

    def step():
        torch.ops.rl_kernel.qwen3_ffn_packed_inference_to_staging(x, w_gu, w_d, staging)
        logp, lse, logits = native.fused_linear_logp(staging, w_lm, target, None, None, True)
        logp2, _ = native.hip_deterministic_logp_from_logits(logits, target, 0, vocab, 64)
        return logp, lse, logp2

    with torch.no_grad():
        eager = [t.clone() for t in step()]
        eager_staging = staging.clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()  # warm-up outside capture
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = step()
        for _ in range(3):
            staging.zero_()
            for t in captured:
                t.zero_()
            native.swiglu_forward(x, x)  # unrelated eager work between replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert _same_bits(staging, eager_staging)
            for got, want in zip(captured, eager):
                assert torch.equal(got.view(torch.int32), want.view(torch.int32))
