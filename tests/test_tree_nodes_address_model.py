"""A CPU model of the lane addresses of det_gemm_tree_nodes_kernel (csrc/det_gemm_tree.hip): for launch grids the
picker can produce - ragged row and column counts, leaves of 24 and of 32, both block layouts - every global
address a lane forms lies inside its operand, every 16-byte granule of a wave's leaf is loaded exactly once for the
columns and rows that exist, and every LDS access stays inside the wave's own staging region. The model restates the
kernel's index arithmetic; it guards that arithmetic's bounds (what a GPU run can only show by faulting), not the
kernel's values, which the GPU tests compare with the oracle."""

from __future__ import annotations

import itertools

import pytest

NODE_SPLIT, NODE_WAVES, NODE_LEVELS, LEAF = 3, 8, 7, 32


def tree_depth(k: int) -> int:
    depth, size = 0, k
    while size > LEAF:
        size -= size // 2
        depth += 1
    return depth


def eligible(m: int, n: int, k: int) -> tuple[bool, bool, int, int]:
    """(nodes_ok, split_blocks, depth, leaf length) as det_gemm_tree_launch decides them for K-contiguous rows."""
    depth = tree_depth(k)
    leaf = k >> depth
    uniform = depth >= 1 and k % (1 << depth) == 0 and k % (8 << depth) == 0
    ok = uniform and NODE_SPLIT < depth <= NODE_SPLIT + NODE_LEVELS and leaf in (24, 32)
    wide_groups = -(-n // 64) * -(-m // 16)
    return ok, ok and wide_groups < 256 and depth > NODE_SPLIT + 2, depth, leaf


def swizzle(pair: int, chunks: int) -> int:
    return (pair >> 2) & 3 if chunks == 4 else 0


def model(m: int, n: int, k: int, a_pitch: int, b_pitch: int) -> None:
    ok, split, depth, leaf = eligible(m, n, k)
    assert ok
    kb, chunks = (4 if split else 1), leaf // 8
    cols = 16 if kb == 4 else 64
    row_groups = -(-m // 16)
    node_depth = NODE_SPLIT + (2 if kb == 4 else 0)
    leaves = 1 << (depth - node_depth)
    assert leaves >= 2 and leaves % 2 == 0
    block_k = leaves * leaf
    a_bytes = 1024 if kb == 1 else 0
    w_bytes = 1024 * chunks
    leaf_bytes = a_bytes + w_bytes
    a_elems, b_elems = (m - 1) * a_pitch + k, (n - 1) * b_pitch + k  # extent of each operand in elements
    groups = -(-n // cols) * row_groups
    # the corners of the grid and a few groups in the middle
    picked = sorted({0, 1, row_groups - 1, groups - 1, groups - row_groups, groups // 2} & set(range(groups)))
    for gid, wave in itertools.product(picked, (0, NODE_WAVES - 1, 3)):
        n0, m0 = (gid // row_groups) * cols, (gid % row_groups) * 16
        assert n0 < n and m0 < m
        wave_k = (4 * wave if kb == 4 else wave) * block_k
        w_base, a_base = n0 * b_pitch + wave_k, m0 * a_pitch + wave_k
        for leaf_index in (0, 1, leaves - 1):
            lo = leaf_index * leaf
            seen = set()
            for j, lane in itertools.product(range(chunks), range(64)):
                g = 64 * j + lane
                pair, chunk = g // chunks, (g % chunks) ^ swizzle(g // chunks, chunks)
                col = pair & 15 if kb == 4 else pair
                col_in = col if n0 + col < n else n - 1 - n0
                off = col_in * b_pitch + ((pair >> 4) * block_k if kb == 4 else 0) + 8 * chunk
                assert 0 <= 2 * off < 2**32
                first = w_base + lo + off
                assert 0 <= first and first + 8 <= b_elems, (m, n, k, gid, wave, leaf_index, j, lane)
                assert 1024 * j + 16 * lane + 16 <= w_bytes  # where the hardware puts the lane's 16 bytes
                if n0 + col < n:
                    key = (col, (pair >> 4) if kb == 4 else 0, chunk)
                    assert key not in seen
                    seen.add(key)
            assert len(seen) == min(cols, n - n0) * kb * chunks
            for lane in range(64):
                if kb == 1:
                    g = lane if lane < 16 * chunks else 16 * chunks - 1
                    row = g // chunks
                    row_in = row if m0 + row < m else m - 1 - m0
                    off = row_in * a_pitch + 8 * ((g % chunks) ^ swizzle(row, chunks))
                    span = 8
                else:
                    row = lane & 15
                    row_in = row if m0 + row < m else m - 1 - m0
                    off = row_in * a_pitch + (lane >> 4) * block_k
                    span = leaf  # the lane reads its leaf's chunks at off, off + 8, ...
                assert 0 <= 2 * off < 2**32
                first = a_base + lo + off
                assert 0 <= first and first + span <= a_elems, (m, n, k, gid, wave, leaf_index, lane)
        # LDS: a lane's reads of both stages lie inside the wave's region
        for lane, c, stage in itertools.product(range(64), range(chunks), (0, 1)):
            at = lane * 16 * chunks + 16 * (c ^ swizzle(lane, chunks)) + stage * leaf_bytes
            assert at + a_bytes + 16 <= 2 * leaf_bytes  # the weight read, behind the rows
            assert at + 16 <= 2 * leaf_bytes  # the row read (lanes past 15 read inside the region, unused)
    assert NODE_WAVES * 2 * leaf_bytes <= 80 * 1024  # two workgroups per CU


SHAPES = [
    (1, 64, 512), (1, 24576, 4096), (16, 100, 384), (17, 257, 4096), (50, 64, 6144), (64, 130, 12288),
    (200, 96, 32768), (333, 320, 512), (40, 5500, 4096), (16, 16400, 2048), (33, 5504, 6144), (8, 16400, 3072),
    (4096, 24576, 4096), (4096, 4096, 12288), (5, 151936, 4096), (64, 4096, 12288), (1000, 16, 768),
]  # fmt: skip


@pytest.mark.parametrize("shape", SHAPES)
def test_every_lane_address_lies_inside_its_operand(shape):
    m, n, k = shape
    model(m, n, k, k, k)
    model(m, n, k, k + 64, k + 8)  # rows that are views into wider storage


def test_the_model_rejects_what_the_launcher_rejects():
    assert not eligible(16, 64, 256)[0]  # a tree of three levels: one leaf per node
    assert not eligible(16, 64, 4000)[0]  # ragged leaves
    assert not eligible(16, 64, 65536)[0]  # eleven levels
    assert eligible(64, 4096, 12288)[:2] == (True, False) and eligible(16, 4096, 12288)[:2] == (True, True)
