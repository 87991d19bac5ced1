"""det_gemm on a real MI355X: parity with the CPU oracle, bit-exact batch
invariance, layout / configuration neutrality and the reference's error
behaviour. Every call goes through the C ABI of librlk_gfx950.so."""

from __future__ import annotations

import numpy as np
import pytest
import torch

import inputs

pytestmark = pytest.mark.gpu

DEV = "cuda"


@pytest.fixture(scope="module")
def gemm():
    from rl_engine.backends.rocm.gemm import det_gemm

    return det_gemm


@pytest.fixture(scope="module")
def native():
    from rl_engine import _C

    return _C


def _same_bits(x: torch.Tensor, y: torch.Tensor) -> bool:
    return torch.equal(x.contiguous().view(torch.int16), y.contiguous().view(torch.int16))


def _assert_parity(oracle, got: torch.Tensor, a: torch.Tensor, w_nk: torch.Tensor, tag: str):
    """got[M,N] (bf16, GPU) against the round-once oracle of a @ w_nk.T.

    Tolerance (the bar for this path: bf16 output within 1 ulp-scale relative
    error of the CPU reference): the bf16 value must lie within half a bf16 ulp
    plus the fp32 summation bound K * 2^-24 * sum|a_k b_k| of the exact sum, and
    within 1 bf16 ulp of the oracle's bits wherever the result is not dominated
    by cancellation.
    """
    a_bits, w_bits, got_bits = inputs.bits(a), inputs.bits(w_nk), inputs.bits(got)
    k = a_bits.shape[1]
    af = oracle.bf16_to_f32(a_bits).astype(np.float64)
    wf = oracle.bf16_to_f32(w_bits).astype(np.float64)
    exact = af @ wf.T
    abs_sum = np.abs(af) @ np.abs(wf).T
    gotf = oracle.bf16_to_f32(got_bits).astype(np.float64)
    bound = 2.0**-8 * np.abs(gotf) + k * 2.0**-24 * abs_sum + 1e-30
    worst = float((np.abs(gotf - exact) / bound).max())
    assert worst <= 1.0, f"{tag}: |got - exact| exceeds rounding + accumulation bound ({worst:.3f}x)"
    ref_bits = oracle.det_gemm_ref(a_bits, w_bits)
    ulp = oracle.bf16_ulp_distance(got_bits, ref_bits)
    clean = np.abs(exact) > 2.0**-6 * abs_sum  # not a near-total cancellation
    assert ulp[clean].max(initial=0) <= 1, f"{tag}: more than 1 bf16 ulp from the oracle"
    assert (ulp > 1).mean() < 1e-3, f"{tag}: too many elements beyond 1 ulp"


# ---------------------------------------------------------------------------
# Config 1: [128,1024] x [1024,1024]
# ---------------------------------------------------------------------------


def test_config1_parity_and_batch_invariance(gemm, oracle):
    a, b = inputs.config1()
    a_d, b_d = a.to(DEV), b.to(DEV)
    c = gemm.deterministic_gemm(a_d, b_d)
    assert c.shape == (128, 1024) and c.dtype == torch.bfloat16
    _assert_parity(oracle, c, a, b.t().contiguous(), "config1")
    # sequential-k restatement (the reference's native twin of the contract)
    # (a different fp32 summation order: within 1 bf16 ulp away from near-total cancellation)
    a16, bt = inputs.bits(a[:16]), inputs.bits(b.t().contiguous())
    seq = oracle.det_gemm_seq(a16, bt)
    af, wf = oracle.bf16_to_f32(a16).astype(np.float64), oracle.bf16_to_f32(bt).astype(np.float64)
    clean = np.abs(af @ wf.T) > 2.0**-6 * (np.abs(af) @ np.abs(wf).T)
    seq_ulp = oracle.bf16_ulp_distance(inputs.bits(c[:16]), seq)
    assert clean.mean() > 0.5 and seq_ulp[clean].max() <= 1, "more than 1 bf16 ulp from the sequential-k restatement"
    assert (seq_ulp > 1).mean() < 1e-3
    # rows 0..6 recomputed at M=1 and M=7 must be bit-identical
    c7 = gemm.deterministic_gemm(a_d[:7], b_d)
    assert _same_bits(c7, c[:7])
    for r in range(7):
        assert _same_bits(gemm.deterministic_gemm(a_d[r : r + 1], b_d), c[r : r + 1]), f"row {r} at M=1"


def test_config1_golden_fixture(gemm, oracle):
    """Stored oracle output for config 1 (tests/golden/make_golden.py wrote it)."""
    from pathlib import Path

    data = np.load(Path(__file__).parent / "golden" / "config1_det_gemm.npz")
    a, b = inputs.config1()
    assert int(inputs.bits(a).astype(np.uint64).sum()) == int(data["a_checksum"]), "input generator drifted"
    assert int(inputs.bits(b).astype(np.uint64).sum()) == int(data["b_checksum"]), "input generator drifted"
    c = gemm.deterministic_gemm(a.to(DEV), b.to(DEV))
    ulp = oracle.bf16_ulp_distance(inputs.bits(c), data["expected_bits"])
    assert (ulp <= 1).mean() > 0.999 and ulp.max() <= int(data["max_ulp_allowed"])


# ---------------------------------------------------------------------------
# Run-to-run determinism and configuration neutrality
# ---------------------------------------------------------------------------


def test_run_to_run_bitwise(gemm):
    a = inputs.randn_bf16(11, 300, 1000).to(DEV)
    w = inputs.randn_bf16(12, 520, 1000, 0.02).to(DEV)
    first = gemm.det_gemm_linear(a, w)
    for _ in range(5):
        assert _same_bits(gemm.det_gemm_linear(a, w), first)


@pytest.mark.parametrize("shape", [(200, 300, 264), (1, 129, 65), (7, 1024, 1024), (33, 48, 4096), (300, 520, 72), (4, 65, 129)])
def test_every_tile_configuration_gives_the_same_bits(gemm, oracle, shape):
    from rl_engine import _lib

    m, n, k = shape
    a = inputs.randn_bf16(21, m, k).to(DEV)
    w = inputs.randn_bf16(22, n, k, 0.02).to(DEV)
    base = gemm.mfma_gemm(a, w.t(), config="256x256")
    _assert_parity(oracle, base, a, w, f"{shape}")
    for name, value in _lib.GEMM_CONFIGS.items():
        assert _same_bits(gemm.mfma_gemm(a, w.t(), config=name), base), name
        assert _same_bits(gemm.mfma_gemm(a, w.t(), config=value | _lib.FORCE_STAGED), base), f"{name} staged"


@pytest.mark.parametrize("shape", [(512, 1024, 4096), (300, 520, 256), (64, 64, 64), (1000, 777 * 8, 128), (16, 4096, 12288), (1, 1000, 4096), (8, 72, 64), (9, 40, 1600)])
def test_pingpong_and_staged_main_loops_give_the_same_bits(gemm, shape):
    """K % 64 == 0 shapes take the direct-to-LDS ping-pong loop; forcing the
    register-staged loop must not change a bit, in any tile configuration,
    repeatedly (the ping-pong loop is the one with hand-placed waits)."""
    from rl_engine import _lib

    m, n, k = shape
    a = inputs.randn_bf16(23, m, k).to(DEV)
    w = inputs.randn_bf16(24, n, k, 0.02).to(DEV)
    base = gemm.mfma_gemm(a, w.t(), config=_lib.GEMM_CONFIGS["16x16"])
    for name, value in _lib.GEMM_CONFIGS.items():
        for _ in range(3):
            assert _same_bits(gemm.mfma_gemm(a, w.t(), config=value), base), name
        assert _same_bits(gemm.mfma_gemm(a, w.t(), config=value | _lib.FORCE_STAGED), base), f"{name} staged"


@pytest.mark.parametrize("m", (17, 31, 32, 33, 47, 48, 49, 64))
@pytest.mark.parametrize("nk", ((4096, 12288), (40, 192), (16, 64), (250, 320), (72, 1088)))
def test_streaming_kernel_for_17_to_64_tokens_gives_the_same_bits(gemm, native, m, nk):
    """Two, three and four token tiles, panels past the N edge, stage counts that do not divide K / 64,
    bf16 and fp32 output, against the one-wave 16x16 tile kernel; rows batch invariant."""
    from rl_engine import _lib

    n, k = nk
    a = inputs.randn_bf16(2500 + m, m, k).to(DEV)
    w = inputs.randn_bf16(2501 + n, n, k, 0.02).to(DEV)
    base = gemm.mfma_gemm(a, w.t(), config="16x16")
    got = gemm.mfma_gemm(a, w.t(), config="stream64")
    assert _same_bits(got, base)
    assert _same_bits(gemm.mfma_gemm(a, w.t(), config="stream64"), got)
    f32 = torch.empty((m, n), dtype=torch.float32, device=DEV)
    f32_base = torch.empty_like(f32)
    native.gemm_strided(a, w.t(), f32, config=_lib.GEMM_CONFIGS["stream64"])
    native.gemm_strided(a, w.t(), f32_base, config=_lib.GEMM_CONFIGS["16x16"])
    assert torch.equal(f32.view(torch.int32), f32_base.view(torch.int32))
    one = gemm.mfma_gemm(a[m - 1 :], w.t())
    assert _same_bits(one, got[m - 1 :])


def test_seeded_random_shapes_layouts_and_offsets_match_the_element_loader(gemm):
    """Whatever kernel the picker and the dispatch conditions choose for a shape, alignment and layout,
    the bits are those of the one-wave tile kernel with the element-wise staged loader."""
    from rl_engine import _lib

    rng = np.random.default_rng(2600)
    reference_config = _lib.GEMM_CONFIGS["16x16"] | _lib.FORCE_STAGED
    for case in range(70):
        m = int(rng.choice([1, 3, 8, 16, 17, 40, 64, 65, 130, 257]))
        n = int(rng.choice([8, 16, 24, 72, 128, 200, 520]))
        k = int(rng.choice([8, 64, 72, 128, 192, 320, 1024, 1088]))
        a_layout, b_layout = rng.integers(0, 3, size=2)  # 0 native, 1 other axis contiguous, 2 padded rows + offset
        a_full = inputs.randn_bf16(2601 + case, m + 1, k + 24).to(DEV)
        w_full = inputs.randn_bf16(2801 + case, n + 1, k + 24, 0.05).to(DEV)
        a = a_full[:m, :k] if a_layout != 2 else a_full[1:, 3 : k + 3]
        w = w_full[:n, :k] if b_layout != 2 else w_full[1:, 5 : k + 5]
        if a_layout == 1:
            a = a.t().contiguous().t()  # token-contiguous activations
        if b_layout == 1:
            w = w.t().contiguous().t()  # B[K, N] with N contiguous
        want = gemm.mfma_gemm(a.contiguous(), w.contiguous().t(), config=reference_config)
        got = gemm.mfma_gemm(a, w.t())
        assert _same_bits(got, want), (case, m, n, k, int(a_layout), int(b_layout))


# ---------------------------------------------------------------------------
# Batch invariance (rows, cuts, strided views, chunked prefill, padding)
# ---------------------------------------------------------------------------


def test_rows_are_batch_invariant_for_cuts_and_strided_views(gemm):
    k, n = 4096, 4096
    a = inputs.randn_bf16(31, 512, k).to(DEV)
    w = inputs.randn_bf16(32, n, k, 0.02).to(DEV)
    full = gemm.det_gemm_linear(a, w)
    for rows, start in ((1, 0), (1, 511), (7, 3), (16, 100), (17, 250), (64, 448), (129, 200)):
        part = gemm.det_gemm_linear(a[start : start + rows], w)
        assert _same_bits(part, full[start : start + rows]), (rows, start)
    strided = a[::2]  # row stride 2K, still unit stride along K
    assert _same_bits(gemm.det_gemm_linear(strided, w), full[::2])


def test_chunked_prefill_and_padding(gemm):
    a = inputs.randn_bf16(41, 256, 4096).to(DEV)
    w = inputs.randn_bf16(42, 1024, 4096, 0.02).to(DEV)
    full = gemm.det_gemm_linear(a, w)
    chunked = torch.cat([gemm.det_gemm_linear(a[:100], w), gemm.det_gemm_linear(a[100:], w)])
    assert _same_bits(chunked, full)
    padded = torch.cat([a[:37], torch.zeros((91, 4096), dtype=a.dtype, device=DEV)])
    assert _same_bits(gemm.det_gemm_linear(padded, w)[:37], full[:37])
    left = torch.cat([torch.zeros((91, 4096), dtype=a.dtype, device=DEV), a[:37]])
    assert _same_bits(gemm.det_gemm_linear(left, w)[91:], full[:37])


# ---------------------------------------------------------------------------
# Config 2: Qwen3-8B FFN shapes, every row bit-invariant across T
# ---------------------------------------------------------------------------


@pytest.fixture(scope="module")
def ffn():
    w_gu, w_d = inputs.ffn_weights()
    x, h = inputs.ffn_activations(4096)
    return {"w_gu": w_gu.to(DEV), "w_d": w_d.to(DEV), "x": x.to(DEV), "h": h.to(DEV), "cpu": (w_gu, w_d, x, h)}


def test_config2_rows_are_bit_invariant_across_token_counts(gemm, ffn):
    gu_full = gemm.det_gemm_linear(ffn["x"], ffn["w_gu"])
    dn_full = gemm.det_gemm_linear(ffn["h"], ffn["w_d"])
    assert gu_full.shape == (4096, 24576) and dn_full.shape == (4096, 4096)
    for t in (1, 16, 256):
        assert _same_bits(gemm.det_gemm_linear(ffn["x"][:t], ffn["w_gu"]), gu_full[:t]), f"gate_up T={t}"
        assert _same_bits(gemm.det_gemm_linear(ffn["h"][:t], ffn["w_d"]), dn_full[:t]), f"down T={t}"
    # a row in the middle of the batch, recomputed alone
    assert _same_bits(gemm.det_gemm_linear(ffn["x"][2049:2050], ffn["w_gu"]), gu_full[2049:2050])
    assert _same_bits(gemm.det_gemm_linear(ffn["h"][4095:4096], ffn["w_d"]), dn_full[4095:4096])


def _edge_rows(m: int, seed: int, extra: int = 64) -> torch.Tensor:
    """Rows on both sides of every tile height in use (16 ... 256), the last rows, and `extra` random ones."""
    fixed = [0, 1, 15, 16, 63, 64, 127, 128, 191, 192, 255, 256, 257, 511, 512, m // 2 - 1, m // 2, m - 257, m - 256, m - 2, m - 1]
    rnd = torch.randperm(m, generator=torch.Generator().manual_seed(seed))[:extra].tolist()
    return torch.tensor(sorted({r for r in fixed + rnd if 0 <= r < m}))


def _edge_cols(n: int) -> torch.Tensor:
    """Columns on both sides of the 64 / 192 / 256-wide tile seams, of the last tile and of the gate | up seam."""
    fixed = [0, 15, 16, 63, 64, 191, 192, 255, 256, 383, 384, 511, 512, n // 2 - 1, n // 2, n - 257, n - 256, n - 193, n - 192, n - 65, n - 64, n - 1]
    return torch.tensor(sorted({c for c in fixed if 0 <= c < n}))


def _assert_whole_rows_and_columns(oracle, got, a, w, seed, tag):
    """Every column of the rows at tile edges (plus 64 random rows) and every row of the columns at tile
    edges, against the fp64 oracle on the host: a refill or edge-clamp mistake at a tile seam shows here,
    where bit-equality of the kernel with itself would not."""
    m, n = got.shape
    rows, cols = _edge_rows(m, seed), _edge_cols(n)
    _assert_parity(oracle, got[rows.to(DEV)], a[rows], w, f"{tag} whole rows")
    _assert_parity(oracle, got[:, cols.to(DEV)], a, w[cols], f"{tag} whole columns")


@pytest.mark.parametrize("tokens", [4096, 256])
def test_config2_parity_on_whole_rows_and_columns_at_tile_edges(gemm, oracle, ffn, tokens):
    w_gu, w_d, x, h = ffn["cpu"]
    gu = gemm.det_gemm_linear(ffn["x"][:tokens], ffn["w_gu"])
    dn = gemm.det_gemm_linear(ffn["h"][:tokens], ffn["w_d"])
    _assert_whole_rows_and_columns(oracle, gu, x[:tokens], w_gu, 2101 + tokens, f"gate_up T={tokens}")
    _assert_whole_rows_and_columns(oracle, dn, h[:tokens], w_d, 2102 + tokens, f"down T={tokens}")


def test_config2_small_t_full_parity(gemm, oracle, ffn):
    w_gu, w_d, x, h = ffn["cpu"]
    for t in (1, 16):
        _assert_parity(oracle, gemm.det_gemm_linear(ffn["x"][:t], ffn["w_gu"]), x[:t], w_gu, f"gate_up T={t}")
        _assert_parity(oracle, gemm.det_gemm_linear(ffn["h"][:t], ffn["w_d"]), h[:t], w_d, f"down T={t}")


# ---------------------------------------------------------------------------
# Config 3: attention projections under two ragged packings
# ---------------------------------------------------------------------------


def test_config3_same_token_same_bits_across_packings(gemm, oracle):
    total = 16384
    lengths = inputs.ragged_lengths(total)
    assert sum(lengths) == total and all(1 <= n <= 2048 for n in lengths)
    tokens = inputs.randn_bf16(3001, total, inputs.QWEN3_HIDDEN)
    w_qkv = inputs.randn_bf16(3004, inputs.QWEN3_QKV_OUT, inputs.QWEN3_HIDDEN, 0.02)
    w_o = inputs.randn_bf16(3005, inputs.QWEN3_HIDDEN, inputs.QWEN3_HIDDEN, 0.02)
    map_a = inputs.pack_rows(lengths, inputs.packing_order(len(lengths), 3002))
    map_b = inputs.pack_rows(lengths, inputs.packing_order(len(lengths), 3003))
    assert not torch.equal(map_a, map_b) and torch.equal(map_a.sort().values, torch.arange(total))
    tok_d = tokens.to(DEV)
    for name, w in (("qkv", w_qkv), ("o_proj", w_o)):
        w_d = w.to(DEV)
        out_a = gemm.det_gemm_linear(tok_d[map_a.to(DEV)], w_d)
        out_b = gemm.det_gemm_linear(tok_d[map_b.to(DEV)], w_d)
        canon_a = torch.empty_like(out_a)
        canon_b = torch.empty_like(out_b)
        canon_a[map_a.to(DEV)] = out_a
        canon_b[map_b.to(DEV)] = out_b
        assert _same_bits(canon_a, canon_b), name
        # packing A against the oracle in packed order, so the rows at tile edges are the kernel's own
        _assert_whole_rows_and_columns(oracle, out_a, tokens[map_a], w, 3100, f"{name} packing A")


# ---------------------------------------------------------------------------
# Layouts, ragged K, special values, outputs
# ---------------------------------------------------------------------------


@pytest.mark.parametrize("shape", [(128, 128, 128), (31, 128, 128), (31, 70, 65), (5, 33, 1000)])
def test_operand_layouts_give_the_same_bits(gemm, native, shape):
    m, k, n = shape
    a = inputs.randn_bf16(51, m, k).to(DEV)
    bt = inputs.randn_bf16(52, n, k, 0.02).to(DEV)
    b = bt.t().contiguous()  # [K,N]
    expected = native.det_gemm_fwd(a, b)
    assert expected.is_contiguous() and tuple(expected.shape) == (m, n)
    assert _same_bits(native.det_gemm_fwd_rhs_transposed(a, bt), expected)
    assert _same_bits(gemm.det_gemm_linear(a, bt), expected)
    assert _same_bits(gemm.det_gemm_linear_prepared(a, gemm.prepare_det_gemm_linear_weight(bt)), expected)
    a_colmajor = a.t().contiguous().t()  # unit stride along M
    assert _same_bits(gemm.mfma_gemm(a_colmajor, b), expected)
    unaligned = torch.empty(n * k + 1, dtype=torch.bfloat16, device=DEV)[1:].view(n, k)
    unaligned.copy_(bt)
    assert _same_bits(native.det_gemm_fwd_rhs_transposed(a, unaligned), expected)


@pytest.mark.parametrize("shape", [(512, 1024, 4096), (300, 1000, 192), (1000, 2056, 320), (64, 8, 64), (7, 1024, 1024), (2048, 4096, 1024),
                                   (520, 1024, 200), (264, 520, 1000), (16, 128, 72),  # these three: K % 64 != 0, a zero-filled tail tile
                                   (200, 1000, 1152), (256, 2056, 640), (72, 200, 640)])  # K % 128 == 0 with feature and token edges: the small tiles' direct-to-LDS K-major loop
def test_kmajor_weight_fast_path_gives_the_same_bits(gemm, native, shape):
    """B[K,N] with N contiguous (the `a @ b`, prepared-weight and input-gradient
    form) and token-contiguous activations are read through transposing LDS loads. Each must
    equal the [N,K] path bit for bit, including N edges inside a 256-wide tile, a
    row-padded weight and a weight view whose base is not 16-byte aligned (which
    has to fall back to the element loader)."""
    m, n, k = shape
    a = inputs.randn_bf16(53, m, k).to(DEV)
    bt = inputs.randn_bf16(54, n, k, 0.02).to(DEV)  # [N,K]
    b = bt.t().contiguous()  # [K,N]
    expected = gemm.mfma_gemm(a, bt.t(), config="16x16")
    # (128x128, 128x64 and 64x64 with a K-major weight: the direct-to-LDS loop with a shared stage column when
    # 128 divides K, else the register-staged K-major loop)
    for name in ("auto", "256x256", "256x128", "256x64", "128x128", "128x64", "64x64"):
        for _ in range(2):
            assert _same_bits(gemm.mfma_gemm(a, b, config=name), expected), name
    # the activation as a K-major view (tokens contiguous: the operands of a weight gradient),
    # alone and together with the K-major weight; M % 8 != 0 falls back to the element loader
    a_kmajor = a.t().contiguous().t()
    for name in ("auto", "256x256", "256x128", "256x64"):
        assert _same_bits(gemm.mfma_gemm(a_kmajor, bt.t(), config=name), expected), f"x k-major {name}"
        assert _same_bits(gemm.mfma_gemm(a_kmajor, b, config=name), expected), f"both k-major {name}"
    padded = torch.zeros((k, n + 24), dtype=torch.bfloat16, device=DEV)
    padded[:, 8 : 8 + n] = b
    assert _same_bits(gemm.mfma_gemm(a, padded[:, 8 : 8 + n]), expected)
    shifted = torch.zeros((k, n + 8), dtype=torch.bfloat16, device=DEV)
    shifted[:, 1 : 1 + n] = b
    assert _same_bits(gemm.mfma_gemm(a, shifted[:, 1 : 1 + n]), expected)
    # fp32 output: same accumulator from both layouts, and it rounds to the bf16 result
    acc_kn = native.det_gemm_fwd_out_fp32(a, b)
    acc_nk = native.det_gemm_fwd_out_fp32(a, bt.t())
    assert torch.equal(acc_kn.view(torch.int32), acc_nk.view(torch.int32))
    assert _same_bits(acc_kn.to(torch.bfloat16), expected)


@pytest.mark.parametrize("tokens", (256, 200, 520))
def test_input_gradient_of_the_lm_head_at_full_reduction_length(gemm, oracle, tokens):
    """dX = dZ[T, V] @ W[V, D] at V = 151936, D = 4096: 2374 K tiles against few outputs, the shape the small
    K-major tiles serve (direct-to-LDS loop with a shared stage column: 64 x 64 at up to 256 tokens, 128 x 64 up
    to 512). Every tile shape must give the bits of the 256 x 256 K-major loop, and sampled rows and columns
    (tile edges included) must meet the oracle's bound."""
    v, d = 151936, 4096
    gen = torch.Generator(device=DEV)
    gen.manual_seed(7100 + tokens)
    w = (torch.randn((v, d), generator=gen, device=DEV) * 0.02).to(torch.bfloat16)  # [K, N]: K-major weight
    dz = (torch.randn((tokens, v), generator=gen, device=DEV) * 0.01).to(torch.bfloat16)
    expected = gemm.mfma_gemm(dz, w, config="256x256")
    for name in ("auto", "64x64", "128x64", "128x128", "256x64"):
        assert _same_bits(gemm.mfma_gemm(dz, w, config=name), expected), name
    rows = sorted({0, 63, 64, tokens // 2, tokens - 1})
    cols = sorted({0, 15, 16, 63, 64, 127, 128, 255, 256, 2047, d - 1})
    sub = expected[rows][:, cols]
    _assert_parity(oracle, sub, dz[rows], w[:, cols].t().contiguous(), f"input gradient T={tokens}")


@pytest.mark.parametrize("tokens", (1, 7, 63, 64, 65, 100, 257, 1000, 4095))
def test_weight_gradient_at_any_token_count_keeps_the_bits(gemm, native, oracle, tokens):
    """dW = dY^T @ X reduces over the tokens with both operands K-major. A token count that 64 does not divide
    runs its whole K tiles in the transposing ping-pong loop and the rest in a zero-filled tail step: the bits
    of the element loader (forced 16x16 tile on transposed copies), whatever the tile."""
    n, k = 384, 520
    x = inputs.randn_bf16(71, tokens, k).to(DEV)
    dy = inputs.randn_bf16(72, tokens, n, 0.05).to(DEV)
    expected = gemm.mfma_gemm(dy.t().contiguous(), x.t().contiguous().t(), config="16x16")  # [n, tokens] @ [tokens, k]
    for name in ("auto", "256x256", "256x128"):
        assert _same_bits(gemm.mfma_gemm(dy.t(), x, config=name), expected), name
    assert _same_bits(native.det_gemm_db_transposed(x, dy), expected)
    assert _same_bits(gemm.det_gemm_linear_weight_gradient(x, dy), expected)
    # the mixed pairs need whole 16-byte chunks of the native operand
    if tokens % 8 == 0:
        assert _same_bits(gemm.mfma_gemm(dy.t().contiguous(), x, config="256x256"), expected)
        assert _same_bits(gemm.mfma_gemm(dy.t(), x.t().contiguous().t(), config="256x256"), expected)
    _assert_parity(oracle, expected, dy.t().contiguous().cpu(), x.t().contiguous().cpu(), f"weight gradient, {tokens} tokens")


@pytest.mark.parametrize("tokens", (64, 128, 192, 256))
@pytest.mark.parametrize("rows,feats", ((1000, 520), (4160, 768), (8, 16), (72, 250)))
def test_short_reduction_streaming_kernel_keeps_the_bits(native, tokens, rows, feats):
    """A weight gradient of up to 256 tokens, dW[rows, feats] = dY[tokens, rows]^T @ X[tokens, feats], on the kernel
    that keeps the feature operand in registers and streams the K-major token operand: the bits of the element
    loader (forced 16x16 tile on transposed copies) for bf16 and fp32 results, whole and partial feature blocks
    and token tiles, a native feature operand, and an output whose rows are not 16-byte aligned."""
    from rl_engine import _lib

    shortk = _lib.GEMM_CONFIGS["shortk"]
    reference = _lib.GEMM_CONFIGS["16x16"] | _lib.FORCE_STAGED

    def bits(t):
        return t.contiguous().view(torch.int32 if t.dtype == torch.float32 else torch.int16)

    dy = inputs.randn_bf16(91, tokens, rows, 0.05).to(DEV)
    x = inputs.randn_bf16(92, tokens, feats).to(DEV)
    for dtype in (torch.bfloat16, torch.float32):
        expected = torch.empty((rows, feats), dtype=dtype, device=DEV)
        native.gemm_strided(dy.t().contiguous(), x.t().contiguous().t(), expected, config=reference)
        got = torch.full((rows, feats), 7.0, dtype=dtype, device=DEV)
        native.gemm_strided(dy.t(), x, got, config=shortk)
        assert torch.equal(bits(got), bits(expected)), dtype
        # feature operand in the native layout (its transposed copy)
        got.fill_(7.0)
        native.gemm_strided(dy.t(), x.t().contiguous().t(), got, config=shortk)
        assert torch.equal(bits(got), bits(expected)), ("native feature operand", dtype)
        # rows of the output that start at odd elements: the element-wise stores, nothing written beside them
        wide = torch.full((rows, feats + 3), 7.0, dtype=dtype, device=DEV)
        native.gemm_strided(dy.t(), x, wide[:, 1 : feats + 1], config=shortk)
        assert torch.equal(bits(wide[:, 1 : feats + 1]), bits(expected)), ("unaligned rows", dtype)
        assert bool((wide[:, 0] == 7.0).all()) and bool((wide[:, feats + 1 :] == 7.0).all())
    # the automatic choice and the wrappers of the weight gradient land on the same bits
    expected = torch.empty((rows, feats), dtype=torch.bfloat16, device=DEV)
    native.gemm_strided(dy.t().contiguous(), x.t().contiguous().t(), expected, config=reference)
    auto = torch.empty_like(expected)
    native.gemm_strided(dy.t(), x, auto)
    assert _same_bits(auto, expected)
    assert _same_bits(native.det_gemm_db_transposed(x, dy), expected)


@pytest.mark.parametrize("tokens,rows,feats", ((128, 24576, 4096), (256, 24648, 4136), (64, 40000, 1024), (192, 16392, 520)))
def test_short_reduction_kernel_over_many_token_tiles_per_workgroup(native, tokens, rows, feats):
    """Shapes that give a workgroup of the streaming kernel 6 ... 40 token tiles, so the ring wraps and the
    counted waits reach their steady state: whole chunks (every store a whole line, loads counted past the
    stores), a result with a partial last token tile and a partial last feature block (guarded stores,
    conservative waits), and the automatic choice (which takes this kernel at these sizes) against a forced tile
    kernel."""
    from rl_engine import _lib

    dy = inputs.randn_bf16(93, tokens, rows, 0.05).to(DEV)
    x = inputs.randn_bf16(94, tokens, feats).to(DEV)
    expected = torch.empty((rows, feats), dtype=torch.bfloat16, device=DEV)
    native.gemm_strided(dy.t(), x, expected, config=_lib.GEMM_CONFIGS["256x256"])
    for config in ("shortk", "auto"):
        got = torch.full((rows, feats), 7.0, dtype=torch.bfloat16, device=DEV)
        native.gemm_strided(dy.t(), x, got, config=_lib.GEMM_CONFIGS[config])
        assert _same_bits(got, expected), config
    got32 = torch.empty((rows, feats), dtype=torch.float32, device=DEV)
    want32 = torch.empty((rows, feats), dtype=torch.float32, device=DEV)
    native.gemm_strided(dy.t(), x, got32, config=_lib.GEMM_CONFIGS["shortk"])
    native.gemm_strided(dy.t(), x, want32, config=_lib.GEMM_CONFIGS["256x256"])
    assert torch.equal(got32.view(torch.int32), want32.view(torch.int32))
    assert _same_bits(got32.to(torch.bfloat16), expected)


def test_a_remainder_of_tokens_launched_on_its_own_changes_no_bit(gemm):
    """513 tokens against 32768 features: the three token rows of 256 x 256 tiles would be 384 tiles, a round and
    a half; the automatic choice launches the last token separately on the few-token kernel. Rows are
    independent: every row equals the forced single launch, for the native and the K-major weight."""
    m, n, k = 513, 32768, 1024
    a = inputs.randn_bf16(81, m, k).to(DEV)
    w = inputs.randn_bf16(82, n, k, 0.02).to(DEV)
    whole = gemm.mfma_gemm(a, w.t(), config="256x256")
    assert _same_bits(gemm.mfma_gemm(a, w.t()), whole)
    staging = torch.zeros((m, n + 8), dtype=torch.bfloat16, device=DEV)
    gemm.mfma_gemm(a, w.t(), out=staging[:, :n])
    assert _same_bits(staging[:, :n], whole) and bool((staging[:, n:] == 0).all())
    w_kn = w.t().contiguous()  # [K, N]: the K-major weight
    assert _same_bits(gemm.mfma_gemm(a[:, :], w_kn), whole)
    m2, n2, k2 = 4097, 4096, 4096  # the down-projection case: 272 tiles
    a2 = inputs.randn_bf16(83, m2, k2).to(DEV)
    w2 = inputs.randn_bf16(84, n2, k2, 0.02).to(DEV)
    assert _same_bits(gemm.mfma_gemm(a2, w2.t()), gemm.mfma_gemm(a2, w2.t(), config="256x256"))
    assert _same_bits(gemm.mfma_gemm(a2, w2.t().contiguous()), gemm.mfma_gemm(a2, w2.t(), config="256x256"))


@pytest.mark.parametrize("k", (1, 8, 31, 32, 33, 65, 100, 1000))
def test_ragged_k_equals_zero_padded_k(gemm, k):
    a = inputs.randn_bf16(61, 9, k).to(DEV)
    w = inputs.randn_bf16(62, 40, k, 0.05).to(DEV)
    kp = ((k + 255) // 256) * 256
    a_pad = torch.zeros((9, kp), dtype=a.dtype, device=DEV)
    w_pad = torch.zeros((40, kp), dtype=a.dtype, device=DEV)
    a_pad[:, :k] = a
    w_pad[:, :k] = w
    assert _same_bits(gemm.det_gemm_linear(a, w), gemm.det_gemm_linear(a_pad, w_pad))


SPECIAL_BITS = (0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x807F, 0x0080, 0x8080, 0x3F80, 0xBF80, 0x7F7F, 0xFF7F, 0x7F80, 0xFF80, 0x7F81, 0x7FC1, 0xFF81, 0xFFFF)


def _special(shape, offset=0):
    n = int(np.prod(shape))
    idx = (np.arange(n) + offset) % len(SPECIAL_BITS)
    return inputs.from_bits(np.array(SPECIAL_BITS, dtype=np.uint16)[idx].reshape(shape), DEV)


@pytest.mark.parametrize("k", (1, 8, 31, 32, 33, 65, 4096))
def test_special_values_same_raw_bytes_in_every_configuration(gemm, k):
    """Zeros, denormals, max finite, infinities and NaN payloads: every tile
    configuration and both operand layouts must produce the same raw bytes."""
    from rl_engine import _lib

    a = _special((3, k))
    b = _special((k, 17), offset=7)
    base = gemm.mfma_gemm(a, b, config="16x16")
    for name in _lib.GEMM_CONFIGS:
        assert _same_bits(gemm.mfma_gemm(a, b, config=name), base), name
    assert _same_bits(gemm.mfma_gemm(a, b.t().contiguous().t()), base)
    vals = base.float()
    # an Inf or NaN anywhere in the row/column pair must surface as non-finite
    a_f, b_f = a.float(), b.float()
    poisoned = (~torch.isfinite(a_f)).any(1)[:, None] & torch.ones_like(vals, dtype=torch.bool)
    assert bool((~torch.isfinite(vals))[poisoned].all())


def test_finite_extremes_match_the_oracle(gemm, oracle):
    # no Inf/NaN: denormals, signed zeros, +-1, +-max-finite; checked value-wise vs fp64.
    finite = [b for b in SPECIAL_BITS if (b & 0x7F80) != 0x7F80]
    k, m, n = 64, 5, 11
    rng = np.random.default_rng(3)
    a_bits = rng.choice(np.array(finite, dtype=np.uint16), size=(m, k))
    w_bits = rng.choice(np.array([0x0000, 0x8000, 0x3F80, 0xBF80, 0x0080, 0x0001], dtype=np.uint16), size=(n, k))
    got = gemm.det_gemm_linear(inputs.from_bits(a_bits, DEV), inputs.from_bits(w_bits, DEV))
    exact = oracle.det_gemm_f64(a_bits, w_bits)
    gotf = oracle.bf16_to_f32(inputs.bits(got)).astype(np.float64)
    ok = np.isfinite(gotf)
    # fp32 accumulation may overflow to inf where the exact sum is representable but partial sums are not
    assert np.all(np.abs(gotf[ok] - exact[ok]) <= 2.0**-8 * np.abs(exact[ok]) + k * 2.0**-24 * 3.4e38 * 4)


def test_fp32_output_is_the_unrounded_accumulator(gemm, native, oracle):
    a = inputs.randn_bf16(71, 50, 520).to(DEV)
    b = inputs.randn_bf16(72, 520, 90, 0.02).to(DEV)
    acc = gemm.DetGemmOp().forward_fp32(a, b)
    assert acc.dtype == torch.float32 and acc.shape == (50, 90)
    assert _same_bits(acc.to(torch.bfloat16), native.det_gemm_fwd(a, b))
    exact = oracle.det_gemm_f64(inputs.bits(a), inputs.bits(b.t().contiguous()))
    assert np.abs(acc.cpu().numpy() - exact).max() < 1e-4


def test_out_argument_and_narrowed_staging_view(gemm):
    a = inputs.randn_bf16(81, 40, 256).to(DEV)
    w = inputs.randn_bf16(82, 72, 256, 0.02).to(DEV)
    expected = gemm.det_gemm_linear(a, w)
    staging = torch.full((64, 72), 7.0, dtype=torch.bfloat16, device=DEV)
    view = staging.narrow(0, 0, 40)
    assert gemm.det_gemm_linear(a, w, out=view) is view
    assert _same_bits(view, expected) and bool((staging[40:] == 7.0).all())
    wide = torch.zeros((40, 100), dtype=torch.bfloat16, device=DEV)
    gemm.mfma_gemm(a, w.t(), out=wide[:, :72])
    assert _same_bits(wide[:, :72], expected) and bool((wide[:, 72:] == 0).all())
    with pytest.raises(ValueError, match="output must have shape"):
        gemm.mfma_gemm(a, w.t(), out=torch.empty((40, 71), dtype=torch.bfloat16, device=DEV))
    with pytest.raises(TypeError, match="output must be BF16"):
        gemm.mfma_gemm(a, w.t(), out=torch.empty((40, 72), dtype=torch.float32, device=DEV))
    with pytest.raises(ValueError, match="rows must be contiguous"):
        gemm.mfma_gemm(a, w.t(), out=torch.empty((72, 40), dtype=torch.bfloat16, device=DEV).t())


def test_empty_and_zero_k(gemm):
    w = inputs.randn_bf16(91, 8, 16).to(DEV)
    assert gemm.det_gemm_linear(torch.empty((0, 16), dtype=torch.bfloat16, device=DEV), w).shape == (0, 8)
    out = gemm.mfma_gemm(torch.empty((3, 0), dtype=torch.bfloat16, device=DEV), torch.empty((0, 5), dtype=torch.bfloat16, device=DEV))
    assert out.shape == (3, 5) and bool((out == 0).all())


def test_native_error_strings(native):
    a = torch.zeros((4, 8), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="A must be bf16"):
        native.det_gemm_fwd(a.float(), a)
    with pytest.raises(RuntimeError, match=r"det_gemm_fwd: expect 2D \[M,K\]@\[K,N\]"):
        native.det_gemm_fwd(a[0], a)
    with pytest.raises(RuntimeError, match="det_gemm_fwd: K mismatch"):
        native.det_gemm_fwd(a, a)
    with pytest.raises(RuntimeError, match="det_gemm_da: N mismatch"):
        native.det_gemm_da(a, torch.zeros((5, 9), dtype=torch.bfloat16, device=DEV))
    with pytest.raises(RuntimeError, match="det_gemm_db: M mismatch"):
        native.det_gemm_db(a, torch.zeros((5, 9), dtype=torch.bfloat16, device=DEV))


# ---------------------------------------------------------------------------
# Backward GEMMs and autograd
# ---------------------------------------------------------------------------


def test_backward_entry_points_match_forward_kernel_bits(gemm, native, oracle):
    m, k, n = 96, 160, 72
    a = inputs.randn_bf16(101, m, k).to(DEV)
    b = inputs.randn_bf16(102, k, n, 0.05).to(DEV)
    dc = inputs.randn_bf16(103, m, n).to(DEV)
    da = native.det_gemm_da(dc, b)  # dC @ B^T
    db = native.det_gemm_db(a, dc)  # A^T @ dC
    dbt = native.det_gemm_db_transposed(a, dc)  # dC^T @ A
    assert da.shape == (m, k) and db.shape == (k, n) and dbt.shape == (n, k) and dbt.is_contiguous()
    assert _same_bits(da, native.det_gemm_fwd(dc, b.t().contiguous()))
    assert _same_bits(db, native.det_gemm_fwd(a.t().contiguous(), dc))
    assert _same_bits(dbt, db.t().contiguous())
    _assert_parity(oracle, da, dc.cpu(), b.cpu(), "da")
    _assert_parity(oracle, db, a.t().contiguous().cpu(), dc.t().contiguous().cpu(), "db")


def test_autograd_of_gemm_and_linear(gemm):
    m, k, n = 33, 96, 40
    a = inputs.randn_bf16(111, m, k).to(DEV).requires_grad_(True)
    w = inputs.randn_bf16(112, n, k, 0.05).to(DEV).requires_grad_(True)
    g = inputs.randn_bf16(113, m, n).to(DEV)
    out = gemm.DetGemmOp().linear(a, w)
    out.backward(g)
    assert _same_bits(a.grad, gemm.det_gemm_linear_input_gradient(g, w.detach()))
    assert _same_bits(w.grad, gemm.det_gemm_linear_weight_gradient(a.detach(), g))
    ref_da = (g.float() @ w.detach().float()).cpu()
    ref_dw = (g.float().t() @ a.detach().float()).cpu()
    assert torch.allclose(a.grad.float().cpu(), ref_da, atol=5e-2, rtol=2e-2)
    assert torch.allclose(w.grad.float().cpu(), ref_dw, atol=5e-2, rtol=2e-2)
    a2 = a.detach().clone().requires_grad_(True)
    b2 = w.detach().t().contiguous().requires_grad_(True)
    gemm.deterministic_gemm(a2, b2).backward(g)
    assert _same_bits(a2.grad, a.grad) and _same_bits(b2.grad, w.grad.t().contiguous())
    with pytest.raises(RuntimeError, match="inference-only"):
        gemm.DetGemmOp().linear(a, w, out=torch.empty((m, n), dtype=torch.bfloat16, device=DEV))


def test_weight_transpose_cache_refresh(gemm):
    w = inputs.randn_bf16(121, 24, 32, 0.1).to(DEV)
    a = inputs.randn_bf16(122, 5, 32).to(DEV)
    prepared = gemm.prepare_det_gemm_linear_weight(w)
    before = gemm.det_gemm_linear_prepared(a, prepared)
    w.mul_(2)
    gemm.prepare_det_gemm_linear_weight(w, out=prepared)
    after = gemm.det_gemm_linear_prepared(a, prepared)
    assert _same_bits(after, gemm.det_gemm_linear(a, w)) and not _same_bits(after, before)
    with pytest.raises(ValueError, match="must not alias"):
        gemm.prepare_det_gemm_linear_weight(w, out=w.view(32, 24))
    # refresh_cached_weight_transposes re-copies, in place, every live prepared buffer of a weight that changed
    second = gemm.prepare_det_gemm_linear_weight(w)
    ptrs = (prepared.data_ptr(), second.data_ptr())
    w.add_(0.25)
    other = inputs.randn_bf16(123, 8, 16).to(DEV)  # never prepared: skipped
    assert gemm.refresh_cached_weight_transposes([w, other, "not a tensor", w[0]]) == 1
    assert (prepared.data_ptr(), second.data_ptr()) == ptrs  # addresses captured by a graph stay valid
    assert torch.equal(prepared, w.t()) and torch.equal(second, w.t())
    assert _same_bits(gemm.det_gemm_linear_prepared(a, second), gemm.det_gemm_linear(a, w))
    del prepared, second  # dropped buffers are forgotten
    assert gemm.refresh_cached_weight_transposes([w]) == 0


def test_prepare_writes_only_its_own_output(gemm):
    # a second prepare of a weight that was updated in place leaves the first buffer alone (it may be a snapshot)
    w = inputs.randn_bf16(124, 24, 32, 0.1).to(DEV)
    old_t = gemm.prepare_det_gemm_linear_weight(w)
    old_bits = old_t.clone()
    w.mul_(3)
    new_t = gemm.prepare_det_gemm_linear_weight(w)
    assert torch.equal(old_t, old_bits) and torch.equal(new_t, w.t()) and not torch.equal(new_t, old_t)
    # weights loaded layer by layer through one staging tensor: the allocator hands out the same address and
    # shape again, and the earlier layers' prepared weights must keep their values
    layers, prepared = [], []
    for seed in (125, 126, 127):
        staging = inputs.randn_bf16(seed, 48, 64, 0.1).to(DEV)
        layers.append(staging.clone().t().contiguous())
        prepared.append(gemm.prepare_det_gemm_linear_weight(staging))
        del staging  # freed: the next layer's staging tensor usually reuses the block
    for want, got in zip(layers, prepared):
        assert torch.equal(want, got)
    # the same through one tensor object that is overwritten in place between layers
    staging = torch.empty((48, 64), dtype=torch.bfloat16, device=DEV)
    layers, prepared = [], []
    for seed in (128, 129):
        staging.copy_(inputs.randn_bf16(seed, 48, 64, 0.1).to(DEV))
        layers.append(staging.clone().t().contiguous())
        prepared.append(gemm.prepare_det_gemm_linear_weight(staging))
    for want, got in zip(layers, prepared):
        assert torch.equal(want, got)
    # a source that died is forgotten: a new tensor at its address has no prepared copies
    del staging
    fresh = torch.zeros((48, 64), dtype=torch.bfloat16, device=DEV)
    assert gemm.refresh_cached_weight_transposes([fresh]) == 0
    assert torch.equal(prepared[1], layers[1])


@pytest.mark.parametrize("rows", (16, 48, 300))
def test_hip_graph_capture_replays_bit_identically(gemm, rows):
    # 16 and 48 rows: the streaming kernel (one and three token tiles); 300: a tile kernel
    a = inputs.randn_bf16(131, rows, 4096).to(DEV)
    w = inputs.randn_bf16(132, 4096, 4096, 0.02).to(DEV)
    out = torch.empty((rows, 4096), dtype=torch.bfloat16, device=DEV)
    eager = gemm.det_gemm_linear(a, w)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        gemm.det_gemm_linear(a, w, out=out)  # warm-up outside capture
    torch.cuda.current_stream().wait_stream(stream)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gemm.det_gemm_linear(a, w, out=out)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert _same_bits(out, eager)


def test_host_threads_on_their_own_streams(gemm):
    """Four host threads, each with its own stream and shapes (so each reaches other kernels),
    launch concurrently; every result equals the one the main thread computed alone. The library
    keeps no state between calls except the per-device 'attribute set' flags and a per-thread
    error string."""
    import threading

    from rl_engine.ops import logprob

    shapes = ((5, 1536, 4096), (48, 4096, 4096), (300, 1024, 2048), (1024, 2048, 1024))
    cases = []
    for i, (m, n, k) in enumerate(shapes):
        a = inputs.randn_bf16(141 + i, m, k).to(DEV)
        w = inputs.randn_bf16(151 + i, n, k, 0.02).to(DEV)
        tgt = torch.randint(0, n, (m,), device=DEV, generator=torch.Generator(device=DEV).manual_seed(161 + i))
        cases.append((a, w, tgt, gemm.det_gemm_linear(a, w), logprob.deterministic_linear_logp(a, w, tgt)))
    torch.cuda.synchronize()
    results: list = [None] * len(cases)
    errors: list = []

    def worker(i):
        try:
            a, w, tgt, _, _ = cases[i]
            stream = torch.cuda.Stream()
            got = []
            with torch.cuda.stream(stream):
                for _ in range(20):
                    got.append((gemm.det_gemm_linear(a, w), logprob.deterministic_linear_logp(a, w, tgt)))
            stream.synchronize()
            results[i] = got
        except Exception as exc:  # surfaced in the main thread
            errors.append((i, repr(exc)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(cases))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    for i, (_, _, _, want, (want_logp, want_lse)) in enumerate(cases):
        assert results[i] is not None and len(results[i]) == 20
        for out, (logp, lse) in results[i]:
            assert _same_bits(out, want), i
            assert torch.equal(logp.view(torch.int32), want_logp.view(torch.int32)), i
            assert torch.equal(lse.view(torch.int32), want_lse.view(torch.int32)), i
