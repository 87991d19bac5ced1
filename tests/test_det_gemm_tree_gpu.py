"""The k-tree GEMM contract on a real MI355X, through the C ABI.

This contract is fully specified (fp32 scalar-FMA leaves of at most 32 K values, bf16
midpoint tree over K; tests/ops/gemm/test_det_gemm.py:156-168 of the reference), so the
bar is bit-exactness against the CPU oracle's restatement, not a tolerance."""

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


def _same_bits(x: torch.Tensor, y: torch.Tensor) -> bool:
    return torch.equal(x.contiguous().view(torch.int16), y.contiguous().view(torch.int16))


def _oracle_tree(oracle, a: torch.Tensor, w_nk: torch.Tensor) -> np.ndarray:
    return oracle.k_tree_gemm(inputs.bits(a), inputs.bits(w_nk))


# (M, K, N); the first three are the shapes of the reference's bitwise test
# (tests/ops/gemm/test_det_gemm.py:510), the rest cover one leaf, uneven leaves
# (K = 33 -> 16 + 17, K = 100 -> 25 x 4, K = 12288 -> 512 leaves of 24) and tile edges.
TREE_SHAPES = [
    (4, 65, 129),
    (8, 4096, 128),
    (4, 12288, 64),
    (1, 1, 1),
    (3, 32, 5),
    (7, 33, 130),
    (70, 100, 200),
    (128, 1024, 1024),
    (65, 1536, 257),
    (16, 6144, 96),
]


@pytest.mark.parametrize("shape", TREE_SHAPES)
def test_tree_gemm_is_bit_exact_against_the_oracle(gemm, oracle, shape):
    m, k, n = shape
    a = inputs.randn_bf16(9100 + k, m, k)
    w = inputs.randn_bf16(9101 + k, n, k, 0.02)  # [N, K]
    want = _oracle_tree(oracle, a, w)
    a_d, w_d = a.to(DEV), w.to(DEV)
    got_linear = gemm.tree_gemm(a_d, w_d.t())  # K-contiguous right-hand side
    got_plain = gemm.tree_gemm(a_d, w_d.t().contiguous())  # B[K, N]
    got_at = gemm.tree_gemm(a_d.t().contiguous().t(), w_d.t())  # A stored [K, M]
    assert np.array_equal(inputs.bits(got_linear), want)
    assert _same_bits(got_plain, got_linear) and _same_bits(got_at, got_linear)
    assert _same_bits(gemm.tree_gemm(a_d, w_d.t()), got_linear)  # run to run


@pytest.mark.parametrize("shape", [(4, 65, 129), (8, 4096, 128), (4, 12288, 64), (1, 1, 1), (3, 32, 5), (7, 33, 130), (70, 100, 200),
                                   (65, 1536, 257), (16, 6144, 96), (130, 1000, 70), (9, 3080, 40)])
def test_leaf_space_tree_is_bit_exact_against_the_oracle(gemm, oracle, shape):
    """The leaf-space split (fixed 32-wide leaves, midpoints counted in leaves: the tree of the reference's
    DetGemmTreeReferenceOp): bit-exact against the oracle's restatement in every operand layout; the same bits as
    the element-space contract exactly when K / 32 is a power of two."""
    m, k, n = shape
    a = inputs.randn_bf16(9150 + k, m, k)
    w = inputs.randn_bf16(9151 + k, n, k, 0.02)  # [N, K]
    want = oracle.k_tree_gemm(inputs.bits(a), inputs.bits(w), leaf_space=True)
    a_d, w_d = a.to(DEV), w.to(DEV)
    got = gemm.tree_gemm(a_d, w_d.t(), leaf_space=True)
    assert np.array_equal(inputs.bits(got), want)
    assert _same_bits(gemm.tree_gemm(a_d, w_d.t().contiguous(), leaf_space=True), got)  # B[K, N]
    assert _same_bits(gemm.tree_gemm(a_d.t().contiguous().t(), w_d.t(), leaf_space=True), got)  # A stored [K, M]
    wide = torch.zeros((m, k + 3), dtype=torch.bfloat16, device=DEV)
    wide[:, :k] = a_d
    assert _same_bits(gemm.tree_gemm(wide[:, :k], w_d.t(), leaf_space=True), got)  # unaligned rows: element loads
    row = m // 2
    assert _same_bits(gemm.tree_gemm(a_d[row : row + 1], w_d.t(), leaf_space=True), got[row : row + 1])  # batch invariant
    element_space = gemm.tree_gemm(a_d, w_d.t())
    leaves = (k + 31) // 32
    if k % 32 == 0 and leaves & (leaves - 1) == 0:
        assert _same_bits(element_space, got)
    elif k > 64 and m * n > 500:
        assert not _same_bits(element_space, got)
    assert gemm.tree_leaf_space_contract_id() != gemm.det_gemm_backend_id()


def test_leaf_space_flag_goes_with_the_tiled_kernels_only():
    from rl_engine import _C, _lib

    a = inputs.randn_bf16(9160, 4, 4096).to(DEV)
    w = inputs.randn_bf16(9161, 64, 4096, 0.02).to(DEV)
    out = torch.empty((4, 64), dtype=torch.bfloat16, device=DEV)
    base = _C.gemm_tree_strided(a, w.t(), out.clone(), _lib.TREE_LEAF_SPACE)
    assert _same_bits(_C.gemm_tree_strided(a, w.t(), out.clone(), _lib.TREE_LEAF_SPACE | 2), base)
    for config in (1, 3, 4):
        with pytest.raises(ValueError, match="LEAF_SPACE"):
            _C.gemm_tree_strided(a, w.t(), out, _lib.TREE_LEAF_SPACE | config)


def test_tree_gemm_differs_from_the_round_once_contract_only_by_rounding(gemm, oracle):
    a = inputs.randn_bf16(9200, 32, 4096).to(DEV)
    w = inputs.randn_bf16(9201, 256, 4096, 0.02).to(DEV)
    tree = gemm.tree_gemm(a, w.t()).float()
    once = gemm.mfma_gemm(a, w.t()).float()
    assert not torch.equal(tree, once)  # two different contracts
    assert float((tree - once).abs().max()) <= 0.05 * float(once.abs().max())  # the reference's reduction atol scale


def test_tree_rows_are_batch_invariant(gemm):
    a = inputs.randn_bf16(9300, 300, 2048).to(DEV)
    w = inputs.randn_bf16(9301, 384, 2048, 0.02).to(DEV)
    full = gemm.tree_gemm(a, w.t())
    for lo, hi in ((0, 1), (37, 38), (0, 7), (100, 229), (299, 300)):
        assert _same_bits(gemm.tree_gemm(a[lo:hi], w.t()), full[lo:hi]), (lo, hi)
    perm = torch.randperm(300, generator=torch.Generator().manual_seed(9302)).to(DEV)
    assert _same_bits(gemm.tree_gemm(a[perm], w.t()), full[perm])


@pytest.mark.parametrize("k", (2048, 12288, 1000))
def test_k_shards_combined_by_bf16_adds_reproduce_the_unsharded_result(gemm, k):
    # The purpose of the contract (tests/ops/gemm/test_det_gemm.py:276-300): a contiguous half of K
    # is exactly one child of the root, a quarter one grandchild.
    a = inputs.randn_bf16(9400 + k, 24, k).to(DEV)
    w = inputs.randn_bf16(9401 + k, 160, k, 0.02).to(DEV)
    full = gemm.tree_gemm(a, w.t())
    h = k // 2
    halves = gemm.tree_gemm(a[:, :h], w[:, :h].t()) + gemm.tree_gemm(a[:, h:], w[:, h:].t())  # torch bf16 add
    assert _same_bits(halves, full)
    q0, q1 = h // 2, h + (k - h) // 2
    cuts = [0, q0, h, q1, k]
    parts = [gemm.tree_gemm(a[:, cuts[i] : cuts[i + 1]], w[:, cuts[i] : cuts[i + 1]].t()) for i in range(4)]
    assert _same_bits((parts[0] + parts[1]) + (parts[2] + parts[3]), full)


def test_simulated_tp_left_fold_differs_and_tp2_is_batch_invariant(gemm):
    # The reference's simulated tensor parallelism (tests/distributed/tp/test_det_gemm_simulated_tp.py:58-102):
    # eight K shards folded left to right are a different parenthesisation from the kernel's tree and must
    # diverge; two shards added once match the unsharded result for a row alone and inside a batch.
    m, k, n = 16, 256, 64
    a = inputs.randn_bf16(9450, m, k).to(DEV)
    b = inputs.randn_bf16(9451, k, n).to(DEV)
    full = gemm.tree_gemm(a, b)
    width = k // 8
    parts = [gemm.tree_gemm(a[:, i * width : (i + 1) * width], b[i * width : (i + 1) * width]) for i in range(8)]
    folded = parts[0]
    for part in parts[1:]:
        folded = folded + part
    assert int((full != folded).sum()) > 0
    balanced = ((parts[0] + parts[1]) + (parts[2] + parts[3])) + ((parts[4] + parts[5]) + (parts[6] + parts[7]))
    assert _same_bits(balanced, full)

    def tp2(x):
        return gemm.tree_gemm(x[:, : k // 2], b[: k // 2]) + gemm.tree_gemm(x[:, k // 2 :], b[k // 2 :])

    big = inputs.randn_bf16(9452, 32, k).to(DEV)
    row = big[:1].clone()
    assert _same_bits(tp2(row)[0], tp2(big)[0]) and _same_bits(tp2(row)[0], gemm.tree_gemm(big, b)[0])


def test_tree_special_values(gemm, oracle):
    # Finite extremes value-exact against the oracle; Inf / NaN surface as Inf / NaN in the same places.
    finite = np.array([0x0000, 0x8000, 0x3F80, 0xBF80, 0x0080, 0x8080, 0x0001, 0x7F7F, 0xFF7F, 0x4000, 0x3F00], dtype=np.uint16)
    rng = np.random.default_rng(9500)
    for k in (1, 31, 32, 33, 64, 200):
        a_bits = rng.choice(finite, size=(5, k))
        w_bits = rng.choice(np.array([0x0000, 0x8000, 0x3F80, 0xBF80, 0x0080, 0x0001], dtype=np.uint16), size=(9, k))
        got = gemm.tree_gemm(inputs.from_bits(a_bits, DEV), inputs.from_bits(w_bits, DEV).t())
        want = oracle.k_tree_gemm(a_bits, w_bits)
        got_bits = inputs.bits(got)
        want_nan = (want & 0x7FFF) > 0x7F80
        got_nan = (got_bits & 0x7FFF) > 0x7F80
        assert np.array_equal(got_nan, want_nan), k
        assert np.array_equal(got_bits[~want_nan], want[~want_nan]), k
    a_bits = rng.choice(finite[:6], size=(4, 96)).astype(np.uint16)
    a_bits[1, 40] = 0x7F80  # +inf
    a_bits[2, 70] = 0x7FC1  # NaN
    w_bits = rng.choice(np.array([0x3F80, 0xBF80, 0x4000], dtype=np.uint16), size=(6, 96))
    got = gemm.tree_gemm(inputs.from_bits(a_bits, DEV), inputs.from_bits(w_bits, DEV).t()).float().cpu()
    assert bool(torch.isfinite(got[0]).all()) and bool(torch.isinf(got[1]).all()) and bool(torch.isnan(got[2]).all())


def test_both_leaf_loops_compute_the_same_bits(oracle):
    # The fp32 matrix-pipe leaf (one v_mfma_f32_16x16x1 per k) against the vector-ALU leaf (one
    # v_fma_f32 per term): every shape of the oracle test, special values (signed zeros, bf16
    # denormals whose products are fp32 denormals, the largest finite values), strided operands.
    from rl_engine import _C

    def run(a_d, b_kn, config):
        out = torch.empty((a_d.size(0), b_kn.size(1)), dtype=torch.bfloat16, device=DEV)
        return _C.gemm_tree_strided(a_d, b_kn, out, config)

    for m, k, n in TREE_SHAPES + [(300, 4096, 384), (130, 12288, 260), (64, 40000, 128)]:
        a = inputs.randn_bf16(9700 + k, m, k).to(DEV)
        w = inputs.randn_bf16(9701 + k, n, k, 0.02).to(DEV)
        for b_kn in (w.t(), w.t().contiguous()):
            valu, mfma = run(a, b_kn, 1), run(a, b_kn, 2)
            assert _same_bits(valu, mfma), (m, k, n)
            assert _same_bits(run(a, b_kn, 0), mfma)
    finite = np.array([0x0000, 0x8000, 0x3F80, 0xBF80, 0x0080, 0x8080, 0x0001, 0x8001, 0x7F7F, 0xFF7F, 0x4000, 0x3F00, 0x0040], dtype=np.uint16)
    small = np.array([0x0000, 0x8000, 0x3F80, 0xBF80, 0x0080, 0x0001, 0x3F00, 0x3E80, 0x0040], dtype=np.uint16)
    rng = np.random.default_rng(9710)
    for k in (1, 31, 32, 33, 64, 200, 4096):
        a_bits = rng.choice(finite, size=(37, k))
        w_bits = rng.choice(small, size=(70, k))
        a_d, w_d = inputs.from_bits(a_bits, DEV), inputs.from_bits(w_bits, DEV)
        valu, mfma = run(a_d, w_d.t(), 1), run(a_d, w_d.t(), 2)
        nan = torch.isnan(valu.float())
        assert torch.equal(nan, torch.isnan(mfma.float())), k
        assert torch.equal(valu.view(torch.int16)[~nan], mfma.view(torch.int16)[~nan]), k
        want = oracle.k_tree_gemm(a_bits, w_bits)
        want_nan = (want & 0x7FFF) > 0x7F80
        assert np.array_equal(inputs.bits(mfma)[~want_nan], want[~want_nan]), k
    with pytest.raises(ValueError, match="unknown configuration"):
        run(a_d, w_d.t(), 9)


def test_skinny_kernel_folds_the_depth_4_nodes_to_the_same_bits(oracle):
    # Up to 16 rows the 16 tree nodes at depth 4 run on 16 waves and are folded in tree order:
    # the same bits as the one-chain-per-output kernels, for every row count and ragged N.
    from rl_engine import _C

    def run(a_d, b_kn, config):
        out = torch.empty((a_d.size(0), b_kn.size(1)), dtype=torch.bfloat16, device=DEV)
        return _C.gemm_tree_strided(a_d, b_kn, out, config)

    for k in (512, 384, 4096, 6144, 12288, 65536):
        for m, n in ((1, 64), (3, 100), (4, 257), (7, 64), (8, 130), (13, 96), (16, 320), (2, 9000), (8, 8200)):  # beyond 8192 columns: whole waves per node
            a = inputs.randn_bf16(9800 + k + m, m, k).to(DEV)
            w = inputs.randn_bf16(9801 + k + m, n, k, 0.02).to(DEV)
            skinny = run(a, w.t(), 3)
            assert _same_bits(skinny, run(a, w.t(), 1)), (m, k, n)
            assert _same_bits(skinny, run(a, w.t(), 2)) and _same_bits(skinny, run(a, w.t(), 0)), (m, k, n)
    a = inputs.randn_bf16(9810, 5, 4096)
    w = inputs.randn_bf16(9811, 70, 4096, 0.02)
    assert np.array_equal(inputs.bits(run(a.to(DEV), w.to(DEV).t(), 3)), _oracle_tree(oracle, a, w))
    # not eligible: more than 16 rows, a tree of fewer than 4 levels, ragged leaves, K-major operand
    a17 = inputs.randn_bf16(9812, 17, 4096).to(DEV)
    w_d = w.to(DEV)
    for bad_a, bad_b in ((a17, w_d.t()), (a17[:4, :256], w_d[:, :256].t()), (a17[:4, :4000], w_d[:, :4000].t()),
                         (a17[:4], w_d.t().contiguous())):
        with pytest.raises(ValueError, match="RLK_TREE_CFG_SKINNY needs"):
            run(bad_a, bad_b, 3)


def test_node_per_wave_kernel_computes_the_same_bits(oracle):
    # 16 rows per workgroup, one depth-3 node per wave on the fp32 matrix pipe: any row count, ragged M and N,
    # leaves of 24 and of 32, against the vector-ALU kernel; one case against the oracle. Narrow problems split
    # a node over the four blocks of the instruction (16 columns per workgroup), problems of 256 and more
    # 64-column groups do not.
    from rl_engine import _C

    def run(a_d, b_kn, config):
        out = torch.empty((a_d.size(0), b_kn.size(1)), dtype=torch.bfloat16, device=DEV)
        return _C.gemm_tree_strided(a_d, b_kn, out, config)

    for k in (512, 384, 4096, 6144, 12288, 32768):
        for m, n in ((1, 64), (16, 100), (17, 257), (50, 64), (64, 130), (200, 96), (333, 320)):
            a = inputs.randn_bf16(9900 + k + m, m, k).to(DEV)
            w = inputs.randn_bf16(9901 + k + m, n, k, 0.02).to(DEV)
            assert _same_bits(run(a, w.t(), 4), run(a, w.t(), 1)), (m, k, n)
    # 258, 257 and 258 groups of 64 columns; then one to eight rows against 257 groups (no split of the blocks)
    for m, n, k in ((40, 5500, 4096), (16, 16400, 2048), (33, 5504, 6144), (1, 16400, 2048), (3, 16448, 4096), (8, 16400, 3072)):
        a = inputs.randn_bf16(9920 + m, m, k).to(DEV)
        w = inputs.randn_bf16(9921 + m, n, k, 0.02).to(DEV)
        assert _same_bits(run(a, w.t(), 4), run(a, w.t(), 1)), (m, k, n)
    a = inputs.randn_bf16(9910, 37, 4096)
    w = inputs.randn_bf16(9911, 70, 4096, 0.02)
    assert np.array_equal(inputs.bits(run(a.to(DEV), w.to(DEV).t(), 4)), _oracle_tree(oracle, a, w))
    # rows that are views into wider storage (row pitch above K), both operands
    a_wide = torch.zeros((37, 4096 + 64), dtype=torch.bfloat16, device=DEV)
    w_wide = torch.zeros((70, 4096 + 8), dtype=torch.bfloat16, device=DEV)
    a_wide[:, :4096], w_wide[:, 8:] = a.to(DEV), w.to(DEV)
    assert np.array_equal(inputs.bits(run(a_wide[:, :4096], w_wide[:, 8:].t(), 4)), _oracle_tree(oracle, a, w))
    assert np.array_equal(inputs.bits(run(a_wide[:, :4096], w_wide[:, 8:].t(), 0)), _oracle_tree(oracle, a, w))
    finite = np.array([0x0000, 0x8000, 0x3F80, 0xBF80, 0x0080, 0x8080, 0x0001, 0x8001, 0x7F7F, 0xFF7F, 0x4000, 0x3F00], dtype=np.uint16)
    rng = np.random.default_rng(9912)
    a_bits, w_bits = rng.choice(finite, size=(40, 1024)), rng.choice(finite[:7], size=(70, 1024))
    a_d, w_d = inputs.from_bits(a_bits, DEV), inputs.from_bits(w_bits, DEV)
    got, want = run(a_d, w_d.t(), 4), run(a_d, w_d.t(), 1)
    nan = torch.isnan(want.float())
    assert torch.equal(nan, torch.isnan(got.float()))
    assert torch.equal(got.view(torch.int16)[~nan], want.view(torch.int16)[~nan])
    with pytest.raises(ValueError, match="RLK_TREE_CFG_NODES"):
        run(a_d[:, :256], w_d[:, :256].t(), 4)  # a tree of three levels


def test_tree_out_argument_empty_shapes_and_errors(gemm):
    a = inputs.randn_bf16(9600, 20, 256).to(DEV)
    w = inputs.randn_bf16(9601, 48, 256, 0.02).to(DEV)
    base = gemm.tree_gemm(a, w.t())
    staging = torch.zeros((20, 64), dtype=torch.bfloat16, device=DEV)
    out = gemm.tree_gemm(a, w.t(), out=staging.narrow(1, 8, 48))
    assert out.data_ptr() == staging.data_ptr() + 16 and _same_bits(out, base)
    assert bool((staging[:, :8] == 0).all()) and bool((staging[:, 56:] == 0).all())
    assert gemm.tree_gemm(a[:0], w.t()).shape == (0, 48)
    zero_k = gemm.tree_gemm(a[:, :0], w[:, :0].t())
    assert zero_k.shape == (20, 48) and bool((zero_k == 0).all())
    with pytest.raises(ValueError):
        gemm.tree_gemm(a, w)  # K mismatch
    with pytest.raises(TypeError):
        gemm.tree_gemm(a.float(), w.t().float())


def test_tree_gradient_forms_are_the_tree_over_their_own_reduction_axis(gemm, oracle):
    # dX = dY @ W reduces over N, dW = dY^T @ X over tokens (tests/ops/gemm/test_det_gemm.py:538-541).
    m, n, k = 96, 160, 192
    x = inputs.randn_bf16(9700, m, k)
    w = inputs.randn_bf16(9701, n, k, 0.05)
    dy = inputs.randn_bf16(9702, m, n)
    dx = gemm.tree_gemm(dy.to(DEV), w.to(DEV))
    dw = gemm.tree_gemm(dy.to(DEV).t(), x.to(DEV))
    assert np.array_equal(inputs.bits(dx), oracle.k_tree_gemm(inputs.bits(dy), inputs.bits(w.t().contiguous())))
    assert np.array_equal(inputs.bits(dw), oracle.k_tree_gemm(inputs.bits(dy.t().contiguous()), inputs.bits(x.t().contiguous())))


def test_tree_contract_id_and_backend_names(gemm):
    from rl_engine import _lib

    lib = _lib.load()
    assert lib.rlk_det_gemm_tree_contract_id().decode() == "rlkernel.det_gemm.hip_ktree32_gfx950.v1"
    assert gemm._resolve_backend_request("tree") == "hip_tree"
    assert gemm._resolve_backend_request("triton_tree") == "hip_tree"
    assert gemm._resolve_backend_request("rocm") == "hip_tree"
    assert gemm._resolve_backend_request("triton_mfma") == "hip_mfma"
    assert gemm._resolve_backend_request("auto") == "auto"
    with pytest.raises(RuntimeError):
        gemm._resolve_backend_request("cublas")


def test_tree_backend_routes_the_whole_facade(gemm, oracle, monkeypatch):
    # RL_KERNEL_DET_GEMM_BACKEND is read at import; switching the resolved request exercises the same routing.
    monkeypatch.setattr(gemm, "_REQUESTED_BACKEND", "hip_tree")
    assert gemm.det_gemm_backend() == "hip_tree"
    assert gemm.det_gemm_backend_id() == "rlkernel.det_gemm.hip_ktree32_gfx950.v1"
    m, n, k = 40, 72, 320
    x = inputs.randn_bf16(9800, m, k)
    w = inputs.randn_bf16(9801, n, k, 0.05)
    dy = inputs.randn_bf16(9802, m, n)
    want = oracle.k_tree_gemm(inputs.bits(x), inputs.bits(w))
    xd = x.to(DEV).requires_grad_(True)
    wd = w.to(DEV).requires_grad_(True)
    op = gemm.DetGemmOp()
    y = op.linear(xd, wd)
    assert np.array_equal(inputs.bits(y.detach()), want)
    assert np.array_equal(inputs.bits(gemm.det_gemm_linear(x.to(DEV), w.to(DEV))), want)
    assert np.array_equal(inputs.bits(gemm.deterministic_gemm(x.to(DEV), w.to(DEV).t())), want)
    y.backward(dy.to(DEV))
    want_dx = oracle.k_tree_gemm(inputs.bits(dy), inputs.bits(w.t().contiguous()))
    want_dw = oracle.k_tree_gemm(inputs.bits(dy.t().contiguous()), inputs.bits(x.t().contiguous()))
    assert np.array_equal(inputs.bits(xd.grad), want_dx) and np.array_equal(inputs.bits(wd.grad), want_dw)
    a2 = x.to(DEV).requires_grad_(True)
    b2 = w.to(DEV).t().contiguous().requires_grad_(True)  # [K, N]
    gemm.deterministic_gemm(a2, b2).backward(dy.to(DEV))
    assert np.array_equal(inputs.bits(a2.grad), want_dx)
    assert np.array_equal(inputs.bits(b2.grad), oracle.k_tree_gemm(inputs.bits(x.t().contiguous()), inputs.bits(dy.t().contiguous())))
    monkeypatch.setattr(gemm, "_REQUESTED_BACKEND", "auto")
    assert gemm.det_gemm_backend() == "hip_mfma"


@pytest.mark.parametrize("shape", [(1, 1, 1), (5, 9, 31), (64, 128, 32), (65, 129, 33), (70, 200, 1000), (130, 40, 4096), (3, 300, 97),
                                   (129, 257, 77), (300, 130, 3), (200, 64, 515), (257, 1, 36),
                                   (300, 200, 96), (1030, 260, 33)])
def test_sequential_fp32_gemm_equals_the_oracle_bit_for_bit(oracle, shape):
    """rlk_det_gemm_seq: one fused multiply-add per k, ascending. Fully specified, so bit-exact against the
    oracle: bf16 and fp32 operands in every combination, both output types, strided views."""
    from rl_engine import _C

    m, n, k = shape
    g = torch.Generator().manual_seed(9700 + m + n + k)
    a32 = torch.randn((m, k), generator=g)
    b32 = torch.randn((n, k), generator=g) * 0.1  # [N, K]
    a16, b16 = a32.to(torch.bfloat16), b32.to(torch.bfloat16)
    for a, b in ((a16, b16), (a32, b32), (a16, b32), (a32, b16)):
        want = oracle.det_gemm_seq_f32(a.float().numpy(), b.float().numpy())
        got = _C.det_gemm_fwd_fp32(a.to(DEV), b.to(DEV).t())
        assert got.dtype == torch.float32 and np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32)), (a.dtype, b.dtype)
        # K-major right-hand side ([K, N] contiguous) and a row-strided left-hand side: same chain, same bits
        got_kn = _C.det_gemm_fwd_fp32(a.to(DEV), b.to(DEV).t().contiguous())
        wide = torch.zeros((m, 2 * k), dtype=a.dtype, device=DEV)
        wide[:, ::2] = a.to(DEV)
        got_strided = _C.det_gemm_fwd_fp32(wide[:, ::2], b.to(DEV).t())
        assert torch.equal(got_kn.view(torch.int32), got.view(torch.int32)) and torch.equal(got_strided.view(torch.int32), got.view(torch.int32))
    # rounded once to the dtype of A
    want16 = oracle.f32_to_bf16(oracle.det_gemm_seq_f32(a16.float().numpy(), b16.float().numpy()))
    got16 = _C.det_gemm_accum_fwd_fp32(a16.to(DEV), b16.to(DEV).t())
    assert got16.dtype == torch.bfloat16 and np.array_equal(inputs.bits(got16), want16)
    assert np.array_equal(want16, oracle.det_gemm_seq(inputs.bits(a16), inputs.bits(b16)))  # the bf16 sequential GEMM
    # a row alone has the bits it has in the batch
    row = m // 2
    alone = _C.det_gemm_fwd_fp32(a32[row : row + 1].to(DEV), b32.to(DEV).t())
    full = _C.det_gemm_fwd_fp32(a32.to(DEV), b32.to(DEV).t())
    assert torch.equal(alone.view(torch.int32), full[row : row + 1].view(torch.int32))


def test_sequential_fp32_gemm_special_values_equal_the_oracle(oracle):
    """The chain runs as one reduction-length-one fp32 MFMA per k. That instruction must behave as the fused
    multiply-add of the oracle (the CPU's fmaf) on every kind of value: signed zeros, fp32 and bf16 denormals, the
    largest finite values, infinities (NaN results compare as NaN), through both loaders."""
    from rl_engine import _C

    g = torch.Generator().manual_seed(9790)
    specials = torch.tensor([0.0, -0.0, 1e-39, -3e-40, 2.0**-126, 3.0e38, -3.0e38, float("inf"), -float("inf"), 1.0, -1.0, 2.0**-133])
    for m, n, k in ((200, 96, 70), (130, 136, 64)):  # element loads with a K tail; 16-byte loads
        a = torch.randn((m, k), generator=g)
        b = torch.randn((n, k), generator=g)
        a.view(-1)[torch.randperm(a.numel(), generator=g)[:900]] = specials[torch.randint(0, len(specials), (900,), generator=g)]
        b.view(-1)[torch.randperm(b.numel(), generator=g)[:500]] = specials[torch.randint(0, len(specials), (500,), generator=g)]
        a[7] = 0.0  # a row of zeros against everything: +0 / NaN only
        a[9] = -0.0
        for lhs, rhs in ((a, b), (a.to(torch.bfloat16), b.to(torch.bfloat16)), (a, b.to(torch.bfloat16))):
            with np.errstate(all="ignore"):
                want = torch.from_numpy(oracle.det_gemm_seq_f32(lhs.float().numpy(), rhs.float().numpy()))
            got = _C.det_gemm_fwd_fp32(lhs.to(DEV), rhs.to(DEV).t()).cpu()
            both_nan = torch.isnan(want) & torch.isnan(got)
            assert torch.equal(torch.where(both_nan, 0, want.view(torch.int32)), torch.where(both_nan, 0, got.view(torch.int32))), (m, lhs.dtype, rhs.dtype)
            assert bool(torch.isnan(got).any()) and bool(torch.isinf(got).any()) and bool((got == 0).any())


def test_sequential_fp32_gemm_order_and_fused_step_known_answers():
    from rl_engine import _C

    ones = torch.ones((1, 4), device=DEV)
    col = torch.tensor([[2.0**24], [1.0], [1.0], [1.0]], device=DEV)
    assert float(_C.det_gemm_fwd_fp32(ones, col)) == 2.0**24  # ascending: every +1 is rounded away
    assert float(_C.det_gemm_fwd_fp32(ones, col.flip(0))) == 2.0**24 + 4.0
    x = 1.0 + 2.0**-12
    a = torch.tensor([[-(1.0 + 2.0**-11), x]], device=DEV)
    b = torch.tensor([[1.0], [x]], device=DEV)
    assert float(_C.det_gemm_fwd_fp32(a, b)) == 2.0**-24  # the step is fused: one rounding per term
    assert _C.det_gemm_fwd_fp32(torch.empty((3, 0), device=DEV), torch.empty((0, 5), device=DEV)).abs().sum().item() == 0.0
    with pytest.raises(RuntimeError, match="K mismatch"):
        _C.det_gemm_fwd_fp32(torch.ones((2, 3), device=DEV), torch.ones((4, 2), device=DEV))
    with pytest.raises(RuntimeError, match="bf16 or fp32"):
        _C.det_gemm_fwd_fp32(torch.ones((2, 3), device=DEV, dtype=torch.float16), torch.ones((3, 2), device=DEV))


def test_fp32_result_paths_never_mix_contracts(gemm, oracle, monkeypatch):
    """DetGemmOp.forward_fp32 / forward_accum_fp32: the MFMA accumulator under the MFMA backend, the sequential
    fp32 chain under the k-tree backend and for any fp32 operand; the reported id says which."""
    a = inputs.randn_bf16(9710, 33, 264)
    b = inputs.randn_bf16(9711, 264, 70, 0.05)  # [K, N]
    seq = oracle.det_gemm_seq_f32(a.float().numpy(), b.t().contiguous().float().numpy())
    op = gemm.DetGemmOp()
    mfma = op.forward_fp32(a.to(DEV), b.to(DEV))
    assert gemm.det_gemm_fp32_backend_id() == "rlkernel.det_gemm.hip_mfma16x16x32_gfx950.v1"
    assert _same_bits(mfma.to(torch.bfloat16), gemm.mfma_gemm(a.to(DEV), b.to(DEV)))
    assert _same_bits(op.forward_accum_fp32(a.to(DEV), b.to(DEV)), gemm.mfma_gemm(a.to(DEV), b.to(DEV)))
    # fp32 operands: accepted, as in the reference, and always the sequential chain
    got32 = op.forward_accum_fp32(a.float().to(DEV), b.float().to(DEV))
    assert got32.dtype == torch.float32 and np.array_equal(got32.cpu().numpy().view(np.uint32), seq.view(np.uint32))
    assert gemm.det_gemm_fp32_backend_id(torch.float32, torch.float32) == "rlkernel.det_gemm.hip_seqfma32_gfx950.v1"
    with pytest.raises(TypeError, match="BF16 or FP32"):
        op.forward_accum_fp32(a.to(DEV).half(), b.to(DEV).half())
    monkeypatch.setattr(gemm, "_REQUESTED_BACKEND", "hip_tree")
    assert gemm.det_gemm_fp32_backend_id() == "rlkernel.det_gemm.hip_seqfma32_gfx950.v1"
    tree32 = op.forward_fp32(a.to(DEV), b.to(DEV))
    assert np.array_equal(tree32.cpu().numpy().view(np.uint32), seq.view(np.uint32))
    assert np.array_equal(inputs.bits(op.forward_accum_fp32(a.to(DEV), b.to(DEV))), oracle.f32_to_bf16(seq))
    monkeypatch.setattr(gemm, "_REQUESTED_BACKEND", "auto")


def test_tree_gemm_is_graph_capturable(gemm):
    a = inputs.randn_bf16(9900, 40, 1024).to(DEV)
    w = inputs.randn_bf16(9901, 200, 1024, 0.02).to(DEV)
    out = torch.empty((40, 200), dtype=torch.bfloat16, device=DEV)
    eager = gemm.tree_gemm(a, w.t())
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        gemm.tree_gemm(a, w.t(), out=out)  # warm-up outside capture
    torch.cuda.current_stream().wait_stream(stream)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gemm.tree_gemm(a, w.t(), out=out)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert _same_bits(out, eager)
