"""A CPU model of the lane addresses of the native-layout direct-to-LDS loader (DmaLoader in csrc/det_gemm_tile.h):
its row maps, chunk swizzle and edge clamping, with the widths the kernel computes in (64-bit pointers, 32-bit lane
offsets), and of its K-major weight form. Walks launch grids of the GEMM, the gated projection and the stream-group LogP kernel - including the
workgroups whose origin lies past the last vocabulary row - and asserts that every lane reads 16 bytes inside its
operand, at the row and K position the stage layout expects. As a control, the same walk with the edge path's row
distance computed in 32 bits (a form that once faulted the GPU) must leave the operand."""

from __future__ import annotations

import itertools

import pytest

U32 = 1 << 32


def plain_block_offset(b: int, tn: int) -> int:
    wave_rows, r0 = 16 * tn, b * 8
    return (r0 // wave_rows) * wave_rows + ((r0 % wave_rows) // 16) * 4


def strided_block_offset(b: int, stride: int) -> int:
    r0 = b * 8
    return (r0 // 64) * stride + ((r0 % 64) // 16) * 4


def gated_block_offset(b: int) -> int:
    r0 = b * 8
    return (r0 // 64) * 32 + (((r0 % 64) // 16) & 1) * 4


def gated_block_half(b: int) -> int:
    return ((b * 8 % 64) // 16) >> 1


def lane_offset(parity: int, rib: int, run: int) -> int:
    i = parity * 8 + rib
    return (i >> 2) * run + (i & 3)


def weight_addresses(kind: str, bn: int, n0: int, n_rows: int, ld: int, k0: int, narrow_edge: bool):
    """(block, lane) -> (element address relative to W.ptr, the row the stage layout expects there, k)."""
    tn = bn // 64
    run = 8 if kind == "gated" else 4 * tn
    for b, lane in itertools.product(range(bn // 8), range(64)):
        rib, parity = lane >> 3, b & 1
        chunk_elems = ((lane & 7) ^ rib) * 8
        if kind == "plain":
            row0, half = plain_block_offset(b, tn), 0
        elif kind == "gated":
            row0, half = gated_block_offset(b), gated_block_half(b)
        else:
            row0, half = strided_block_offset(b, 256), 0
        lane_row = lane_offset(parity, rib, run)
        base = n0 * ld + half * n_rows * ld  # 64-bit: w_base + half
        if n0 + row0 + lane_offset(parity, 7, run) < n_rows:
            lane_off = (lane_row * ld) % U32 + chunk_elems  # w_lane_off: 32 bits
            addr = base + row0 * ld + k0 + lane_off % U32
            want_row = n0 + row0 + lane_row
        else:
            g = min(n0 + row0 + lane_row, n_rows - 1)
            dist = (g - n0) * ld
            if narrow_edge:
                dist = dist % U32  # the variant that faulted: a negative distance wraps to +4 GB
            addr = base + dist + k0 + chunk_elems
            want_row = g
        yield b, lane, addr, half * n_rows + want_row, k0 + chunk_elems


def check(kind: str, bn: int, origins, n_rows: int, total_rows: int, ld: int, k: int, narrow_edge: bool = False) -> int:
    bad = 0
    for n0, k0 in itertools.product(origins, (0, k - 64)):
        for b, lane, addr, row, kk in weight_addresses(kind, bn, n0, n_rows, ld, k0, narrow_edge):
            inside = 0 <= addr and addr + 8 <= (total_rows - 1) * ld + k
            bad += not (inside and addr == row * ld + kk and 0 <= row < total_rows)
    return bad


GEMM_GRIDS = [  # (tile features, N, K, row pitch)
    (256, 24576, 4096, 4096), (256, 4099, 4096, 4104), (192, 1000, 512, 512), (128, 130, 128, 192), (64, 70, 64, 64),
    (256, 151936, 4096, 4096), (128, 8, 64, 1 << 23),
]  # fmt: skip


@pytest.mark.parametrize("bn,n,k,ld", GEMM_GRIDS)
def test_gemm_tiles_read_inside_the_weight(bn, n, k, ld):
    origins = sorted({0, (n - 1) // bn * bn, ((n - 1) // bn // 2) * bn})
    assert check("plain", bn, origins, n, n, ld, k) == 0
    # every row of an interior tile appears exactly once per 16-byte chunk position
    if n >= bn:
        rows = sorted(row for _, _, _, row, kk in weight_addresses("plain", bn, 0, n, ld, 0, False) if kk == 0)
        assert rows == list(range(bn))


@pytest.mark.parametrize("inter,k", [(12288, 4096), (1000, 512), (130, 64)])
def test_gated_tiles_read_gate_and_up_rows_of_the_same_features(inter, k):
    origins = sorted({0, (inter - 1) // 128 * 128})
    assert check("gated", 256, origins, inter, 2 * inter, k, k) == 0
    rows = sorted(row for _, _, _, row, kk in weight_addresses("gated", 256, 0, inter, k, 0, False) if kk == 0)
    if inter >= 128:
        assert rows == list(range(128)) + list(range(inter, inter + 128))


@pytest.mark.parametrize("vocab", [4099, 151936, 1024, 1030, 65])
def test_stream_group_workgroups_past_the_last_vocabulary_row_stay_inside(vocab):
    k, ld = 256, 264
    splits = -(-vocab // 1024)
    origins = [split * 1024 + sg * 64 for split in (0, splits - 1) for sg in range(4)]
    assert any(n0 >= vocab for n0 in origins) or vocab % 1024 == 0 or vocab > 100000
    assert check("strided", 256, origins, vocab, vocab, ld, k) == 0


def test_the_model_catches_the_edge_distance_computed_in_32_bits():
    # V = 4099: the last split's groups start at 4096 + 64 g; for g >= 1 the origin lies past the last row
    origins = [4 * 1024 + sg * 64 for sg in range(4)]
    assert check("strided", 256, origins, 4099, 4099, 264, 256) == 0
    assert check("strided", 256, origins, 4099, 4099, 264, 256, narrow_edge=True) > 0


def test_lane_offsets_fit_32_bits_below_the_pitch_the_launchers_admit():
    for tn in (1, 2, 3, 4):
        rows = max(lane_offset(p, r, 4 * tn) for p in (0, 1) for r in range(8))
        assert rows < 64 and rows * ((1 << 24) - 8) + 56 < U32


def kmajor_weight_addresses(bn: int, n0: int, rows: int, ld: int, k0: int):
    """K-major weight w[k * ld + n]: (block, lane) -> (element address relative to W.ptr, K row, first feature)."""
    for b, lane in itertools.product(range(bn // 8), range(64)):
        rib = lane >> 3
        lane_chunk = (lane & 7) ^ (4 * ((rib >> 1) & 1))  # kmajor_swizzle_of_row_in_block
        col, kblk = b >> 3, b & 7
        chunk = lane_chunk ^ (2 * ((kblk ^ (kblk >> 1)) & 1))  # kmajor_swizzle_of_block
        at = col * 64 + chunk * 8
        if n0 + col * 64 + 64 > rows:
            at = min(at, rows - 8 - n0)
        lane_off = (rib * ld) % U32  # 32 bits
        yield b, lane, n0 + (k0 + kblk * 8) * ld + lane_off + at, k0 + kblk * 8 + rib, n0 + at


@pytest.mark.parametrize("bn,n,k,ld", [(256, 4096, 151936, 4096), (256, 4104, 128, 4104), (128, 72, 64, 80), (64, 8, 64, 8), (256, 24576, 4096, 24576)])
def test_kmajor_weight_tiles_read_inside_the_weight(bn, n, k, ld):
    for n0 in sorted({0, (n - 1) // bn * bn}):
        for k0 in (0, k - 64):
            seen = set()
            for b, lane, addr, k_row, feat in kmajor_weight_addresses(bn, n0, n, ld, k0):
                assert 0 <= addr and addr + 8 <= (k - 1) * ld + n, (n0, k0, b, lane)
                assert addr == k_row * ld + feat and k0 <= k_row < k0 + 64 and n0 <= feat <= n - 8
                seen.add((k_row, feat))
            if n0 + bn <= n:  # an interior tile: every 8-feature chunk of every K row exactly once
                assert len(seen) == 64 * (bn // 8)
