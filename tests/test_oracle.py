"""Pins the CPU oracle: every function is checked against something a plausible
mistake (dropped term, wrong sign or index, transposed operand) would break --
closed forms, brute force in fp64, and the known-answer values the reference's
own tests hold for this path. Runs without a GPU."""

from __future__ import annotations

import math

import numpy as np
import pytest


def _bits(oracle, arr):
    return oracle.f32_to_bf16(np.asarray(arr, dtype=np.float32))


# ---------------------------------------------------------------------------
# bf16 conversion
# ---------------------------------------------------------------------------


def test_bf16_known_bit_patterns(oracle):
    cases = {
        1.0: 0x3F80,
        -1.0: 0xBF80,
        0.0: 0x0000,
        2.0: 0x4000,
        0.5: 0x3F00,
        float("inf"): 0x7F80,
        float("-inf"): 0xFF80,
        3.0: 0x4040,
    }
    for value, pattern in cases.items():
        assert int(oracle.f32_to_bf16(np.float32(value)).reshape(-1)[0]) == pattern, value
    assert int(_bits(oracle, [-0.0])[0]) == 0x8000


def test_bf16_round_to_nearest_even_ties(oracle):
    # 1 + 2^-8 lies exactly between 1.0 (even mantissa) and 1 + 2^-7: ties to even -> 1.0.
    assert int(_bits(oracle, [1.0 + 2.0**-8])[0]) == 0x3F80
    # 1 + 3*2^-8 lies between 1+2^-7 (odd) and 1+2^-6 (even): ties to even -> 1 + 2^-6.
    assert int(_bits(oracle, [1.0 + 3 * 2.0**-8])[0]) == 0x3F82
    # Just above the tie rounds up.
    assert int(_bits(oracle, [np.float32(1.0 + 2.0**-8) + np.float32(2.0**-20)])[0]) == 0x3F81
    # Largest finite fp32 rounds to +inf in bf16.
    assert int(_bits(oracle, [np.finfo(np.float32).max])[0]) == 0x7F80
    assert np.isnan(oracle.bf16_to_f32(_bits(oracle, [np.nan])))[0]


def test_bf16_roundtrip_is_identity_on_bf16_values(oracle):
    all_bits = np.arange(0, 1 << 16, dtype=np.uint32).astype(np.uint16)
    f = oracle.bf16_to_f32(all_bits)
    finite = np.isfinite(f)
    assert np.array_equal(oracle.f32_to_bf16(f[finite]), all_bits[finite])


def test_c_and_numpy_bf16_conversion_agree(oracle):
    rng = np.random.default_rng(3)
    x = np.concatenate(
        [rng.standard_normal(4096).astype(np.float32) * 7, np.array([0.0, -0.0, 1e-40, 3e38, np.inf, -np.inf], np.float32)]
    )
    lib = oracle._c()
    import ctypes

    lib.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
    lib.oracle_f32_to_bf16.restype = ctypes.c_uint16
    got = np.array([lib.oracle_f32_to_bf16(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, oracle.f32_to_bf16(x))


# ---------------------------------------------------------------------------
# det_gemm
# ---------------------------------------------------------------------------

GEMMS = ("det_gemm_ref", "det_gemm_seq")


@pytest.mark.parametrize("fn", GEMMS)
def test_gemm_k1_is_the_rounded_exact_product(oracle, fn):
    rng = np.random.default_rng(1)
    a = oracle.randn_bf16(rng, (5, 1))
    bt = oracle.randn_bf16(rng, (7, 1))
    expect = oracle.f32_to_bf16(oracle.bf16_to_f32(a) * oracle.bf16_to_f32(bt).T)
    assert np.array_equal(getattr(oracle, fn)(a, bt), expect)


@pytest.mark.parametrize("fn", GEMMS)
def test_gemm_one_hot_rows_select_weight_columns(oracle, fn):
    # A = one-hot rows -> C[i, :] is column k_i of B exactly; catches a transposed operand.
    rng = np.random.default_rng(2)
    k, n = 48, 9
    bt = oracle.randn_bf16(rng, (n, k))
    picks = [0, 5, 47, 17]
    a = np.zeros((len(picks), k), dtype=np.float32)
    for r, c in enumerate(picks):
        a[r, c] = 1.0
    got = getattr(oracle, fn)(oracle.f32_to_bf16(a), bt)
    assert np.array_equal(got, bt[:, picks].T)


@pytest.mark.parametrize("fn", GEMMS)
def test_gemm_integer_sums_are_exact(oracle, fn):
    # all-ones x powers of two: every partial sum is a small integer, exact in fp32 and bf16.
    k = 96
    a = oracle.f32_to_bf16(np.ones((3, k), np.float32))
    b = np.zeros((4, k), np.float32)
    b[0, :] = 1.0  # sum = 96
    b[1, :64] = 2.0  # sum = 128
    b[2, ::2] = -0.5  # sum = -24
    b[3, :3] = [4.0, -4.0, 0.25]  # sum = 0.25
    got = oracle.bf16_to_f32(getattr(oracle, fn)(a, oracle.f32_to_bf16(b)))
    assert np.array_equal(got, np.tile(np.array([96.0, 128.0, -24.0, 0.25], np.float32), (3, 1)))


@pytest.mark.parametrize("fn", GEMMS)
def test_gemm_matches_fp64_brute_force_within_accumulation_bound(oracle, fn):
    rng = np.random.default_rng(4)
    m, n, k = 33, 29, 1000
    a = oracle.randn_bf16(rng, (m, k))
    bt = oracle.randn_bf16(rng, (n, k), 0.02)
    exact = oracle.det_gemm_f64(a, bt)
    # independent check of the C fp64 loop against numpy
    assert np.allclose(exact, oracle.bf16_to_f32(a).astype(np.float64) @ oracle.bf16_to_f32(bt).astype(np.float64).T, rtol=1e-12, atol=1e-12)
    got = oracle.bf16_to_f32(getattr(oracle, fn)(a, bt)).astype(np.float64)
    abs_sum = np.abs(oracle.bf16_to_f32(a)).astype(np.float64) @ np.abs(oracle.bf16_to_f32(bt)).astype(np.float64).T
    bound = 2.0**-8 * np.abs(got) + k * 2.0**-24 * abs_sum  # half a bf16 ulp (<= 2^-8 |x|) + fp32 summation bound
    assert np.all(np.abs(got - exact) <= bound + 1e-30)


def test_gemm_reference_equality_demand_at_4x16_by_9x16(oracle):
    # The reference requires its sequential kernel to equal (a.float() @ w.float().t()).to(bf16)
    # bit for bit at this shape (tests/test_musa_det_gemm.py:133-140).
    rng = np.random.default_rng(5)
    a = oracle.randn_bf16(rng, (4, 16))
    w = oracle.randn_bf16(rng, (9, 16))
    assert np.array_equal(oracle.det_gemm_seq(a, w), oracle.det_gemm_ref(a, w))


def test_gemm_ref_and_seq_agree_to_one_ulp_on_config1_shape(oracle):
    rng = np.random.default_rng(6)
    a = oracle.randn_bf16(rng, (16, 1024))
    bt = oracle.randn_bf16(rng, (64, 1024), 0.02)
    ref, seq = oracle.det_gemm_ref(a, bt), oracle.det_gemm_seq(a, bt)
    big = np.abs(oracle.bf16_to_f32(ref)) > 0.05  # away from cancellation
    assert oracle.bf16_ulp_distance(ref, seq)[big].max() <= 1


def test_sequential_fp32_gemm_is_pinned(oracle):
    """oracle.det_gemm_seq_f32 (fp32 operands, fp32 result, one fused multiply-add per k): rounded to bf16 it is
    the sequential bf16 GEMM on bf16-valued operands; one-hot rows select columns exactly; integer sums are
    exact; a sum whose order matters (2^24 + 1 + 1 ...) comes out as the ascending chain gives it and not as a
    pairwise or descending sum would; and it stays within the fp32 accumulation bound of the fp64 value on
    general fp32 operands."""
    rng = np.random.default_rng(21)
    a_bits, bt_bits = oracle.randn_bf16(rng, (7, 200)), oracle.randn_bf16(rng, (5, 200), 0.02)
    af, btf = oracle.bf16_to_f32(a_bits), oracle.bf16_to_f32(bt_bits)
    assert np.array_equal(oracle.f32_to_bf16(oracle.det_gemm_seq_f32(af, btf)), oracle.det_gemm_seq(a_bits, bt_bits))
    eye = np.zeros((3, 200), np.float32)
    eye[0, 0] = eye[1, 77] = eye[2, 199] = 1.0
    assert np.array_equal(oracle.det_gemm_seq_f32(eye, btf), btf[:, [0, 77, 199]].T)
    # order: ((2^24 + 1) + 1) + 1 stays 2^24 in an ascending chain (each +1 is lost to rounding to even),
    # while 1 + 1 + 1 + 2^24 (descending k) or a pairwise sum would give 2^24 + 4 / + 2
    col = np.array([[2.0**24, 1.0, 1.0, 1.0]], np.float32)
    ones = np.ones((1, 4), np.float32)
    assert float(oracle.det_gemm_seq_f32(ones, col)[0, 0]) == 2.0**24
    assert float(oracle.det_gemm_seq_f32(ones, col[:, ::-1].copy())[0, 0]) == 2.0**24 + 4.0
    # fused step: a*b + c with a single rounding. (1 + 2^-12)^2 - (1 + 2^-11) = 2^-24 exactly; an unfused
    # product rounds to 1 + 2^-11 first and gives 0
    x = np.float32(1.0 + 2.0**-12)
    got = oracle.det_gemm_seq_f32(np.array([[-(1.0 + 2.0**-11), x]], np.float32), np.array([[1.0, x]], np.float32))
    assert float(got[0, 0]) == 2.0**-24
    a32 = rng.standard_normal((9, 333)).astype(np.float32)
    b32 = rng.standard_normal((4, 333)).astype(np.float32)
    exact = a32.astype(np.float64) @ b32.astype(np.float64).T
    bound = 333 * 2.0**-24 * (np.abs(a32).astype(np.float64) @ np.abs(b32).astype(np.float64).T)
    assert np.all(np.abs(oracle.det_gemm_seq_f32(a32, b32) - exact) <= bound)


# ---------------------------------------------------------------------------
# k-tree contract
# ---------------------------------------------------------------------------


@pytest.mark.parametrize("leaf_space", (False, True))
def test_k_tree_with_one_leaf_is_the_sequential_gemm(oracle, leaf_space):
    rng = np.random.default_rng(7)
    for k in (1, 8, 31, 32):
        a = oracle.randn_bf16(rng, (5, k))
        bt = oracle.randn_bf16(rng, (6, k))
        assert np.array_equal(oracle.k_tree_gemm(a, bt, leaf_space=leaf_space), oracle.det_gemm_seq(a, bt))


def test_k_tree_two_leaves_is_bf16_add_of_leaf_sums(oracle):
    rng = np.random.default_rng(8)
    a = oracle.randn_bf16(rng, (4, 64))
    bt = oracle.randn_bf16(rng, (5, 64))
    left = oracle.bf16_to_f32(oracle.det_gemm_seq(a[:, :32], bt[:, :32]))
    right = oracle.bf16_to_f32(oracle.det_gemm_seq(a[:, 32:], bt[:, 32:]))
    assert np.array_equal(oracle.k_tree_gemm(a, bt), oracle.f32_to_bf16(left + right))


def test_k_tree_element_and_leaf_space_agree_iff_leaf_count_is_power_of_two(oracle):
    rng = np.random.default_rng(9)
    for k in (1024, 4096):
        a = oracle.randn_bf16(rng, (2, k))
        bt = oracle.randn_bf16(rng, (8, k))
        assert np.array_equal(oracle.k_tree_gemm(a, bt), oracle.k_tree_gemm(a, bt, leaf_space=True))
    # K=12288: element space halves down to 24-wide leaves (512 of them,
    # tests/ops/gemm/test_det_gemm.py:282-283), leaf space keeps 384 leaves of 32.
    a = oracle.randn_bf16(rng, (4, 12288))
    bt = oracle.randn_bf16(rng, (32, 12288))
    assert not np.array_equal(oracle.k_tree_gemm(a, bt), oracle.k_tree_gemm(a, bt, leaf_space=True))


def test_k_tree_balanced_k_shards_reproduce_the_full_tree(oracle):
    # The property the contract exists for (tests/ops/gemm/test_det_gemm.py:276-300):
    # a contiguous half-K GEMM is exactly one child of the root.
    rng = np.random.default_rng(10)
    k = 2048
    a = oracle.randn_bf16(rng, (3, k))
    bt = oracle.randn_bf16(rng, (7, k))
    full = oracle.k_tree_gemm(a, bt)
    lo = oracle.bf16_to_f32(oracle.k_tree_gemm(a[:, : k // 2], bt[:, : k // 2]))
    hi = oracle.bf16_to_f32(oracle.k_tree_gemm(a[:, k // 2 :], bt[:, k // 2 :]))
    assert np.array_equal(full, oracle.f32_to_bf16(lo + hi))


# ---------------------------------------------------------------------------
# linear-LogP
# ---------------------------------------------------------------------------


def test_logp_uniform_logits_give_minus_log_v(oracle):
    # Zero hidden states -> all logits 0 -> logp = -log V, lse = log V.
    n, d, v = 6, 32, 1000
    h = np.zeros((n, d), np.uint16)
    w = oracle.randn_bf16(np.random.default_rng(11), (v, d))
    target = np.arange(n) * 7
    for logp, lse in (oracle.linear_logp_chunked(h, w, target)[:2], oracle.linear_logp_dense(h, w, target)):
        assert np.allclose(lse, math.log(v), atol=1e-6)
        assert np.allclose(logp, -math.log(v), atol=1e-6)


def test_logp_bias_only_closed_form(oracle):
    # h = 0, bias = log of a known distribution -> logp of token t is log p_t exactly.
    n, d, v = 4, 16, 50
    rng = np.random.default_rng(12)
    p = rng.random(v) + 0.1
    p = p / p.sum()
    bias = np.log(p).astype(np.float32)
    h = np.zeros((n, d), np.uint16)
    w = oracle.randn_bf16(rng, (v, d))
    target = np.array([0, 13, 49, 7])
    logp, lse = oracle.linear_logp_dense(h, w, target, bias)
    assert np.allclose(logp, np.log(p[target]), atol=2e-6)
    assert np.allclose(lse, 0.0, atol=2e-6)
    logp_c = oracle.linear_logp_chunked(h, w, target, bias, chunk_elems=4 * 16)[0]
    assert np.allclose(logp_c, np.log(p[target]), atol=2e-6)


def test_logp_chunked_dense_and_fp64_agree_and_chunking_is_immaterial(oracle):
    rng = np.random.default_rng(13)
    n, d, v = 37, 96, 3001
    h = oracle.randn_bf16(rng, (n, d))
    w = oracle.randn_bf16(rng, (v, d), 0.1)
    bias = (rng.standard_normal(v) * 0.3).astype(np.float32)
    target = rng.integers(0, v, n)
    exact, exact_lse = oracle.linear_logp_f64(h, w, target, bias)
    dense, dense_lse = oracle.linear_logp_dense(h, w, target, bias)
    assert np.abs(dense - exact).max() < 2e-5 and np.abs(dense_lse - exact_lse).max() < 2e-5
    for chunk_elems in (1 << 24, n * 512, n * 100, n):  # one chunk ... one vocabulary row per chunk
        logp, lse, m, s, zt = oracle.linear_logp_chunked(h, w, target, bias, chunk_elems=chunk_elems)
        assert np.abs(logp - exact).max() < 2e-5, chunk_elems
        assert np.abs(lse - exact_lse).max() < 2e-5
    # the reference's chunk rule at config 4: 2^24 // 8192 = 2048 rows -> 75 chunks, last 384
    chunk = max(1, min(151936, oracle.BWD_CHUNK_ELEMS // 8192))
    assert chunk == 2048 and math.ceil(151936 / chunk) == 75 and 151936 - 74 * chunk == 384


def test_logp_probabilities_sum_to_one_and_target_picks_the_right_column(oracle):
    rng = np.random.default_rng(14)
    n, d, v = 3, 64, 257
    h = oracle.randn_bf16(rng, (n, d))
    w = oracle.randn_bf16(rng, (v, d), 0.2)
    # logp of every column, one call per column id; exp must sum to 1 per row.
    total = np.zeros(n)
    for t in range(v):
        total += np.exp(oracle.linear_logp_chunked(h, w, np.full(n, t), chunk_elems=n * 64)[0].astype(np.float64))
    assert np.allclose(total, 1.0, atol=1e-4)


def test_logp_vocab_start_index_shifts_target_ownership(oracle):
    rng = np.random.default_rng(15)
    n, d, v = 5, 32, 300
    h = oracle.randn_bf16(rng, (n, d))
    w = oracle.randn_bf16(rng, (v, d), 0.2)
    target = rng.integers(0, v, n)
    base = oracle.linear_logp_chunked(h, w, target, chunk_elems=n * 64)[0]
    shifted = oracle.linear_logp_chunked(h, w, target + 1000, vocab_start_index=1000, chunk_elems=n * 64)[0]
    assert np.array_equal(base, shifted)


def test_logp_temperature_and_padding_follow_the_strict_contract(oracle):
    rng = np.random.default_rng(16)
    n, d, v, real = 4, 32, 128, 100
    h = oracle.randn_bf16(rng, (n, d))
    w = oracle.randn_bf16(rng, (v, d), 0.3)
    target = rng.integers(0, real, n)
    temp = np.array([0.5, 1.0, 2.0, 0.7], np.float32)
    logp, lse = oracle.linear_logp_dense(h, w, target, temperature=temp, real_vocab_size=real)
    # padded lanes contribute nothing: same as dropping the rows of W
    logp2, lse2 = oracle.linear_logp_dense(h, w[:real], target, temperature=temp)
    # (to fp32 rounding: the BLAS may order the dot products differently for another N)
    assert np.allclose(logp, logp2, atol=2e-6, rtol=0) and np.allclose(lse, lse2, atol=2e-6, rtol=0)
    # temperature 1 row equals the untempered value
    plain = oracle.linear_logp_dense(h, w[:real], target)[0]
    assert abs(plain[1] - logp[1]) < 2e-6
    exact = oracle.linear_logp_f64(h, w, target, temperature=temp, real_vocab_size=real)[0]
    assert np.abs(logp - exact).max() < 2e-5


# ---------------------------------------------------------------------------
# linear-LogP backward
# ---------------------------------------------------------------------------


def _objective(h, w, b, target, temp, real, g_logp, g_lse):
    """sum_t g_logp[t] * logp[t] + g_lse[t] * lse[t] in fp64 from real-valued operands,
    through scipy's logsumexp (an independent routine, not the oracle's formula)."""
    from scipy.special import logsumexp

    z = (h @ w.T + b) / temp[:, None]
    z = z[:, :real]
    lse = logsumexp(z, axis=-1)
    logp = z[np.arange(h.shape[0]), target] - lse
    return float((g_logp * logp + g_lse * lse).sum()), lse


def test_logp_backward_matches_central_finite_differences(oracle):
    rng = np.random.default_rng(21)
    n, d, v, real = 3, 8, 12, 10
    h_bits = oracle.randn_bf16(rng, (n, d))
    w_bits = oracle.randn_bf16(rng, (v, d), 0.5)
    bias = rng.standard_normal(v).astype(np.float32)
    temp = np.array([0.5, 1.0, 1.75], np.float32)
    target = np.array([0, 9, 4])
    g_logp = rng.standard_normal(n).astype(np.float32)
    g_lse = rng.standard_normal(n).astype(np.float32)
    h = oracle.bf16_to_f32(h_bits).astype(np.float64)
    w = oracle.bf16_to_f32(w_bits).astype(np.float64)
    b = bias.astype(np.float64)
    t64, gl, gs = temp.astype(np.float64), g_logp.astype(np.float64), g_lse.astype(np.float64)
    _, lse = _objective(h, w, b, target, t64, real, gl, gs)
    dz = oracle.linear_logp_dlogits(
        h_bits, w_bits, target, lse, g_logp, g_lse, bias, temperature=temp, real_vocab_size=real, dtype=np.float64
    )
    grad_h, grad_w, grad_b = dz @ w, dz.T @ h, dz.sum(axis=0)
    eps = 1e-6

    def fd(arr, index):
        saved = arr[index]
        arr[index] = saved + eps
        up, _ = _objective(h, w, b, target, t64, real, gl, gs)
        arr[index] = saved - eps
        down, _ = _objective(h, w, b, target, t64, real, gl, gs)
        arr[index] = saved
        return (up - down) / (2 * eps)

    for i in range(n):
        for j in range(d):
            assert abs(fd(h, (i, j)) - grad_h[i, j]) < 1e-7, ("hidden", i, j)
    for i in range(v):
        for j in range(d):
            assert abs(fd(w, (i, j)) - grad_w[i, j]) < 1e-7, ("weight", i, j)
        assert abs(fd(b, i) - grad_b[i]) < 1e-7, ("bias", i)
    # padded vocabulary rows receive no gradient at all
    assert np.all(grad_w[real:] == 0) and np.all(grad_b[real:] == 0)
    # the fp32 restatement and the packaged backward agree with the fp64 anchor
    gh32, gw32, gb32, dz32 = oracle.linear_logp_backward(
        h_bits, w_bits, target, lse, g_logp, g_lse, bias, temperature=temp, real_vocab_size=real,
        round_dlogits_to_bf16=False,
    )  # fmt: skip
    assert np.abs(dz32 - dz).max() < 1e-5
    assert np.abs(gh32 - grad_h).max() < 1e-4 and np.abs(gw32 - grad_w).max() < 1e-4 and np.abs(gb32 - grad_b).max() < 1e-4


def test_logp_backward_closed_forms(oracle):
    rng = np.random.default_rng(22)
    n, d, v = 5, 16, 64
    h_bits = oracle.randn_bf16(rng, (n, d))
    w_bits = oracle.randn_bf16(rng, (v, d), 0.3)
    target = rng.integers(0, v, n)
    temp = np.array([0.5, 1.0, 2.0, 0.7, 1.3], np.float32)
    g_logp = rng.standard_normal(n).astype(np.float32)
    g_lse = rng.standard_normal(n).astype(np.float32)
    _, lse = oracle.linear_logp_f64(h_bits, w_bits, target, temperature=temp)
    dz = oracle.linear_logp_dlogits(h_bits, w_bits, target, lse, g_logp, g_lse, temperature=temp, dtype=np.float64)
    # probabilities sum to one: a row of d(logits) sums to grad_lse / temperature
    assert np.allclose(dz.sum(axis=-1), g_lse.astype(np.float64) / temp.astype(np.float64), atol=1e-12)
    # grad_logp only: the target column gets g * (1 - p_t) / T, every other column -g * p / T
    dz_lp = oracle.linear_logp_dlogits(h_bits, w_bits, target, lse, g_logp, None, temperature=temp, dtype=np.float64)
    rows = np.arange(n)
    assert np.all(np.sign(dz_lp[rows, target]) == np.sign(g_logp))
    others = dz_lp.copy()
    others[rows, target] = 0
    assert np.all(others * g_logp[:, None] <= 0)
    # identical weight rows: logits are constant per token, so logp = -log V whatever hidden is
    same = np.repeat(w_bits[:1], v, axis=0)
    lse_same = oracle.linear_logp_f64(h_bits, same, target)[1]
    gh, gw, gb, _ = oracle.linear_logp_backward(h_bits, same, target, lse_same, g_logp, None, round_dlogits_to_bf16=False)
    assert np.abs(gh).max() < 1e-5
    # ... and the weight gradient of row v is (onehot - 1/V) g h summed over tokens
    hf = oracle.bf16_to_f32(h_bits).astype(np.float64)
    expect = -(g_logp[:, None] * hf).sum(axis=0) / v
    expect_rows = np.tile(expect, (v, 1))
    for t in range(n):
        expect_rows[target[t]] += g_logp[t] * hf[t]
    assert np.abs(gw - expect_rows).max() < 1e-5


def test_logp_backward_bf16_dlogits_stay_within_their_rounding(oracle):
    rng = np.random.default_rng(23)
    n, d, v = 8, 32, 256
    h_bits = oracle.randn_bf16(rng, (n, d))
    w_bits = oracle.randn_bf16(rng, (v, d), 0.3)
    target = rng.integers(0, v, n)
    g = rng.standard_normal(n).astype(np.float32)
    lse = oracle.linear_logp_f64(h_bits, w_bits, target)[1]
    exact = oracle.linear_logp_backward(h_bits, w_bits, target, lse, g, None, round_dlogits_to_bf16=False)
    rounded = oracle.linear_logp_backward(h_bits, w_bits, target, lse, g, None, round_dlogits_to_bf16=True)
    dz = np.abs(exact[3].astype(np.float64))
    w = np.abs(oracle.bf16_to_f32(w_bits).astype(np.float64))
    h = np.abs(oracle.bf16_to_f32(h_bits).astype(np.float64))
    assert np.all(np.abs(rounded[0] - exact[0]) <= 2.0**-8 * (dz @ w) + 1e-12)
    assert np.all(np.abs(rounded[1] - exact[1]) <= 2.0**-8 * (dz.T @ h) + 1e-12)
    assert np.array_equal(rounded[2], exact[2])  # the bias gradient sums the unrounded values


# ---------------------------------------------------------------------------
# log-probabilities from materialised logits
# ---------------------------------------------------------------------------


def test_logits_tile_stats_and_merge_against_scipy(oracle):
    from scipy.special import logsumexp

    rng = np.random.default_rng(31)
    rows, v, start, real = 6, 96, 32, 32 + 70  # global columns 32..127, the last 26 are padding
    z = (rng.standard_normal((rows, v)) * 3).astype(np.float32)
    temp = np.array([0.5, 1.0, 2.0, 0.7, 1.0, 1.3], np.float32)
    target = start + rng.integers(0, 70, rows)
    exact = logsumexp(z[:, :70].astype(np.float64) / temp[:, None], axis=1)
    for tiles in (1, 2, 8, 96):
        m, s = oracle.logits_tile_stats(z, start, real, tiles, temperature=temp)
        assert m.shape == (rows, tiles)
        width = v // tiles
        for t in range(tiles):
            lo, hi = t * width, min((t + 1) * width, 70)
            if hi <= lo:  # all padding: the identity of the merge
                assert np.all(m[:, t] == -np.inf) and np.all(s[:, t] == 0)
            else:
                assert np.array_equal(m[:, t], (z[:, lo:hi] / temp[:, None]).astype(np.float32).max(axis=1))
                assert np.all(s[:, t] >= 1.0) and np.all(s[:, t] <= hi - lo)
        assert np.abs(oracle.merge_tile_partials(m, s) - exact).max() < 2e-6
        logp, lse = oracle.logp_from_logits(z, target, start, real, tiles, temperature=temp)
        zt = z[np.arange(rows), target - start].astype(np.float64) / temp
        assert np.abs(logp - (zt - exact)).max() < 3e-6 and np.abs(lse - exact).max() < 2e-6
    # a target owned by another shard contributes a zero logit
    logp, lse = oracle.logp_from_logits(z, np.full(rows, 5), start, real, 8)
    assert np.array_equal(logp, -lse)


def test_logits_backward_matches_finite_differences(oracle):
    from scipy.special import logsumexp

    rng = np.random.default_rng(32)
    rows, v, real = 3, 10, 8
    z = rng.standard_normal((rows, v))
    temp = np.array([0.5, 1.0, 1.75])
    target = np.array([0, 7, 3])
    g_logp = rng.standard_normal(rows)
    g_lse = rng.standard_normal(rows)

    def objective(arr):
        y = arr[:, :real] / temp[:, None]
        lse = logsumexp(y, axis=1)
        return float((g_logp * (y[np.arange(rows), target] - lse) + g_lse * lse).sum()), lse

    _, lse = objective(z)
    grad = oracle.logits_logp_backward(z, lse, g_logp, g_lse, target, 0, real, temperature=temp, dtype=np.float64)
    eps = 1e-6
    for i in range(rows):
        for j in range(v):
            up, down = z.copy(), z.copy()
            up[i, j] += eps
            down[i, j] -= eps
            fd = (objective(up)[0] - objective(down)[0]) / (2 * eps)
            assert abs(fd - grad[i, j]) < 1e-7, (i, j)
    assert np.all(grad[:, real:] == 0)
    # rows of the gradient sum to coef_lse / temperature; a non-finite lse row gives onehot * coef only
    assert np.allclose(grad.sum(axis=1), g_lse / temp, atol=1e-12)
    dead = oracle.logits_logp_backward(z, np.full(rows, -np.inf), g_logp, None, target, 0, real, dtype=np.float64)
    expect = np.zeros_like(z)
    expect[np.arange(rows), target] = g_logp
    assert np.array_equal(dead, expect)


# ---------------------------------------------------------------------------
# SwiGLU / gated FFN
# ---------------------------------------------------------------------------


def test_swiglu_closed_forms_and_finite_differences(oracle):
    f = lambda arr: oracle.bf16_to_f32(arr).astype(np.float64)  # noqa: E731
    zero = _bits(oracle, [0.0])
    assert f(oracle.swiglu(zero, _bits(oracle, [3.0])))[0] == 0.0
    # tails: silu(x) -> x for large x, -> 0 for very negative x
    assert f(oracle.swiglu(_bits(oracle, [40.0]), _bits(oracle, [1.0])))[0] == 40.0
    assert abs(f(oracle.swiglu(_bits(oracle, [-40.0]), _bits(oracle, [1.0])))[0]) < 1e-15
    # silu(1) * 2 = 2 / (1 + e^-1)
    assert abs(f(oracle.swiglu(_bits(oracle, [1.0]), _bits(oracle, [2.0])))[0] - 2.0 / (1.0 + math.exp(-1.0))) < 2.0**-8 * 1.5
    rng = np.random.default_rng(41)
    g = oracle.randn_bf16(rng, (64,), 2.0)
    u = oracle.randn_bf16(rng, (64,), 1.0)
    dy = oracle.randn_bf16(rng, (64,), 1.0)
    gf, uf, dyf = f(g), f(u), f(dy)
    exact = gf / (1.0 + np.exp(-gf)) * uf
    assert np.all(np.abs(f(oracle.swiglu(g, u)) - exact) <= 2.0**-8 * np.abs(exact) + 1e-30)
    # linear in up: swiglu(g, 2u) = 2 swiglu(g, u) exactly (a power-of-two scale commutes with rounding)
    u2 = _bits(oracle, (2.0 * uf).astype(np.float32))
    assert np.array_equal(f(oracle.swiglu(g, u2)), 2.0 * f(oracle.swiglu(g, u)))
    # backward against central differences of the fp64 formula
    eps = 1e-6
    silu = lambda x: x / (1.0 + np.exp(-x))  # noqa: E731
    d_gate_fd = dyf * uf * (silu(gf + eps) - silu(gf - eps)) / (2 * eps)
    d_up_fd = dyf * silu(gf)
    d_gate, d_up = oracle.swiglu_backward(dy, g, u)
    assert np.all(np.abs(f(d_gate) - d_gate_fd) <= 2.0**-8 * np.abs(d_gate_fd) + 1e-6)
    assert np.all(np.abs(f(d_up) - d_up_fd) <= 2.0**-8 * np.abs(d_up_fd) + 1e-30)
    # packed layout: columns [0, I) gate, [I, 2I) up
    packed = np.concatenate([g.reshape(4, 16), u.reshape(4, 16)], axis=1)
    assert np.array_equal(oracle.swiglu_packed(packed), oracle.swiglu(g, u).reshape(4, 16))


def test_gated_ffn_against_fp64(oracle):
    rng = np.random.default_rng(42)
    t, h, i = 6, 32, 48
    x = oracle.randn_bf16(rng, (t, h))
    w_gu = oracle.randn_bf16(rng, (2 * i, h), 0.2)
    w_d = oracle.randn_bf16(rng, (h, i), 0.2)
    f = lambda arr: oracle.bf16_to_f32(arr).astype(np.float64)  # noqa: E731
    gu = f(x) @ f(w_gu).T
    act = gu[:, :i] / (1.0 + np.exp(-gu[:, :i])) * gu[:, i:]
    exact = act @ f(w_d).T
    got = f(oracle.gated_ffn(x, w_gu, w_d))
    # three roundings to bf16 along the way: gate_up, the activation, the output
    scale = np.abs(act) @ np.abs(f(w_d)).T
    assert np.all(np.abs(got - exact) <= 2.0**-8 * np.abs(exact) + 3 * 2.0**-8 * scale + 1e-6)


# ---------------------------------------------------------------------------
# GRPO
# ---------------------------------------------------------------------------


def test_masked_reductions_reference_known_answers(oracle):
    # tests/reference/test_reference_ops.py:77-84
    values = np.array([[1.0, 100.0], [3.0, 4.0]], np.float32)
    mask = np.array([[True, False], [True, True]])
    assert oracle.masked_mean(values, mask) == pytest.approx(8.0 / 3.0, rel=1e-6)
    assert oracle.masked_mean(values) == pytest.approx(27.0, rel=1e-6)
    assert oracle.masked_mean(values, np.zeros((2, 2), bool)) == 0.0


def test_ratio_and_kl_reference_example(oracle):
    # tests/reference/test_reference_ops.py:88-98: current - old = 0.5 and ref - current = -0.25 everywhere.
    current = np.array([[0.0, -1.0], [-2.0, -3.0]], np.float32)
    old = np.array([[-0.5, -1.5], [-2.5, -3.5]], np.float32)
    ref = np.array([[-0.25, -1.25], [-2.25, -3.25]], np.float32)
    mask = np.array([[True, False], [True, True]])
    ratio = oracle.compute_policy_ratio(current, old, mask)
    kl = oracle.compute_reference_kl(current, ref, mask)
    assert ratio[0, 1] == 0.0 and kl[0, 1] == 0.0
    assert np.allclose(ratio[mask], math.exp(0.5), rtol=1e-6)
    assert np.allclose(kl[mask], math.exp(-0.25) + 0.25 - 1.0, rtol=1e-5)


def test_group_advantages_reference_known_answer(oracle):
    # tests/ops/loss/test_grpo_loss.py:112-119
    got = oracle.group_advantages([1.0, 3.0, 10.0, 20.0, 30.0], group_boundaries=[0, 2, 5])
    g1 = (np.array([10.0, 20.0, 30.0]) - 20.0) / math.sqrt(200.0 / 3.0)
    assert np.allclose(got, np.concatenate([[-1.0, 1.0], g1]), atol=1e-5)
    uniform = oracle.group_advantages([1.0, 3.0, 10.0, 30.0], samples_per_prompt=2)
    assert np.allclose(uniform, [-1, 1, -1, 1], atol=1e-5)
    with pytest.raises(ValueError):
        oracle.group_advantages([1.0, 2.0])


def test_grpo_closed_forms(oracle):
    rng = np.random.default_rng(17)
    logp = -np.abs(rng.standard_normal((3, 8))).astype(np.float32)
    adv = np.array([1.0, -2.0, 0.5], np.float32)
    # old == logp -> ratio exactly 1 -> term = -A; ref == logp -> k3 exactly 0.
    loss, policy, kl, ratio, k3 = oracle.grpo_ratio_kl_loss(logp, logp, logp, adv, beta=0.3)
    assert np.all(ratio == 1.0) and np.all(k3 == 0.0) and kl == 0.0
    assert policy == pytest.approx(-adv.mean(), rel=1e-6) and loss == policy
    # ratio far above 1+eps with A>0 saturates at -(1+eps)A; with A<0 the unclipped branch wins.
    old = logp - 1.0
    _, policy, _, ratio, _ = oracle.grpo_ratio_kl_loss(logp, old, logp, np.array([2.0, 2.0, 2.0], np.float32), clip_eps=0.2)
    assert policy == pytest.approx(-1.2 * 2.0, rel=1e-6)
    _, policy, _, _, _ = oracle.grpo_ratio_kl_loss(logp, old, logp, np.array([-2.0, -2.0, -2.0], np.float32), clip_eps=0.2)
    assert policy == pytest.approx(math.e * 2.0, rel=1e-6)
    # k3 is non-negative and ~ d^2/2 for small d
    _, _, _, _, k3 = oracle.grpo_ratio_kl_loss(logp, logp, logp + np.float32(0.01), adv)
    assert np.all(k3 >= 0) and np.allclose(k3, 0.5e-4, rtol=0.05)


def test_grpo_hand_computed_2x2(oracle):
    logp = np.array([[-1.0, -2.0], [-0.5, -3.0]], np.float32)
    old = np.array([[-1.1, -1.7], [-0.5, -3.3]], np.float32)
    ref = np.array([[-0.9, -2.0], [-0.7, -2.5]], np.float32)
    adv = np.array([1.5, -0.5], np.float32)
    mask = np.array([[1, 1], [0, 1]], bool)
    loss, policy, kl, ratio, k3 = oracle.grpo_ratio_kl_loss(logp, old, ref, adv, mask, clip_eps=0.2, beta=0.01)
    r = [math.exp(0.1), math.exp(-0.3), 0.0, math.exp(0.3)]
    terms = [
        -min(r[0] * 1.5, min(max(r[0], 0.8), 1.2) * 1.5),
        -min(r[1] * 1.5, min(max(r[1], 0.8), 1.2) * 1.5),
        -min(r[3] * -0.5, min(max(r[3], 0.8), 1.2) * -0.5),
    ]
    ks = [math.exp(0.1) - 0.1 - 1, 0.0, math.exp(0.5) - 0.5 - 1]
    assert policy == pytest.approx(sum(terms) / 3, rel=1e-5)
    assert kl == pytest.approx(sum(ks) / 3, rel=1e-4)
    assert loss == pytest.approx(sum(terms) / 3 + 0.01 * sum(ks) / 3, rel=1e-5)
    assert ratio[1, 0] == 0.0 and k3[1, 0] == 0.0


def test_swiglu_values_is_the_unrounded_form_of_the_bf16_functions(oracle):
    rng = np.random.default_rng(77)
    g_bits = oracle.randn_bf16(rng, (9, 40), 2.0)
    u_bits = oracle.randn_bf16(rng, (9, 40))
    dy_bits = oracle.randn_bf16(rng, (9, 40))
    g, u, dy = (oracle.bf16_to_f32(b) for b in (g_bits, u_bits, dy_bits))
    assert np.array_equal(oracle.f32_to_bf16(oracle.swiglu_values(g, u)), oracle.swiglu(g_bits, u_bits))
    d_gate, d_up = oracle.swiglu_values(g, u, dy)
    ref_g, ref_u = oracle.swiglu_backward(dy_bits, g_bits, u_bits)
    assert np.array_equal(oracle.f32_to_bf16(d_gate), ref_g) and np.array_equal(oracle.f32_to_bf16(d_up), ref_u)
    # closed forms: silu(0) = 0, silu'(0) = 1/2, silu(x) -> x for large x
    assert oracle.swiglu_values(np.zeros(3), np.ones(3)).tolist() == [0.0, 0.0, 0.0]
    dg, du = oracle.swiglu_values(np.zeros(2), np.full(2, 3.0), np.full(2, 2.0))
    assert dg.tolist() == [3.0, 3.0] and du.tolist() == [0.0, 0.0]
    assert oracle.swiglu_values(np.full(1, 40.0), np.full(1, 0.5))[0] == 20.0


# ---------------------------------------------------------------------------
# torch forms (what the CPU baseline times)
# ---------------------------------------------------------------------------


def test_torch_forms_agree_with_the_numpy_forms(oracle):
    import torch

    rng = np.random.default_rng(77)
    a_bits = oracle.randn_bf16(rng, (33, 192))
    bt_bits = oracle.randn_bf16(rng, (70, 192), 0.05)
    a = torch.from_numpy(a_bits.view(np.int16)).view(torch.bfloat16)
    bt = torch.from_numpy(bt_bits.view(np.int16)).view(torch.bfloat16)
    want = oracle.det_gemm_ref(a_bits, bt_bits)
    got = oracle.det_gemm_ref_torch(a, bt).view(torch.int16).numpy().view(np.uint16)
    # two fp32 BLAS orders, one rounding each: identical except where the fp32 sums straddle a rounding boundary
    assert (oracle.bf16_ulp_distance(got, want) <= 1).all()
    assert (got == want).mean() > 0.98
    exact = oracle.det_gemm_f64(a_bits, bt_bits)
    native = oracle.native_gemm_torch(a, bt).float().numpy().astype(np.float64)
    scale = np.abs(oracle.bf16_to_f32(a_bits).astype(np.float64)) @ np.abs(oracle.bf16_to_f32(bt_bits).astype(np.float64)).T
    assert (np.abs(native - exact) <= 2.0**-7 * scale).all()  # bf16 matmul: at most bf16-level error of the term sum
    # an order-sensitive transposition check: a @ bt.T is not bt @ a.T
    assert got.shape == (33, 70)

    h_bits = oracle.randn_bf16(rng, (9, 64))
    w_bits = oracle.randn_bf16(rng, (301, 64), 0.3)
    target = rng.integers(0, 301, size=9)
    h = torch.from_numpy(h_bits.view(np.int16)).view(torch.bfloat16)
    w = torch.from_numpy(w_bits.view(np.int16)).view(torch.bfloat16)
    logp_t, lse_t = oracle.linear_logp_chunked_torch(h, w, torch.from_numpy(target), chunk_elems=9 * 50)
    logp_n, lse_n, *_ = oracle.linear_logp_chunked(h_bits, w_bits, target, chunk_elems=9 * 50)
    np.testing.assert_allclose(logp_t.numpy(), logp_n, atol=2e-6, rtol=0)
    np.testing.assert_allclose(lse_t.numpy(), lse_n, atol=2e-6, rtol=0)
    f64_logp, _ = oracle.linear_logp_f64(h_bits, w_bits, target)
    np.testing.assert_allclose(logp_t.numpy(), f64_logp, atol=1e-5, rtol=0)
    assert oracle.cpu_model_string()
