"""The fp16 GEMM moves its operands with direct global -> LDS loads, whose addresses nothing checks on the device: the
library computes, on the host, the last byte those loads reach in each operand buffer and refuses a launch that would
pass one.  These tests run that arithmetic (no GPU call) over the shape space - ragged row counts, last column tiles of
both widths, K not a multiple of 32 - and compare it with a lane-by-lane enumeration of the kernels' addressing rule
written out here: lane p of a 64-lane load fetches 16 bytes at row p // 4, 8-element chunk (p % 4) ^ ((p // 16) % 4) of
a 16-row block; a scale load fetches 4 bytes per lane, 64 lanes per wavefront, 4 wavefronts from the tile's first
column on."""
import itertools

import numpy as np
import pytest

from deepj_amd import HipNative

TILES = [(128, 256), (128, 192), (64, 256), (64, 192)]


def enumerate_reach(m, k, n, tile_rows, tile_cols):
    kp = (k + 31) // 32 * 32
    pitch, steps = kp + 64, kp // 32
    m_pad, n_pad = (m + 127) // 128 * 128, (n + 767) // 768 * 768
    m_tiles, n_tiles = -(-m // tile_rows), -(-n // tile_cols)
    lanes = np.arange(64)
    prow = lanes // 4
    pchunk = (lanes % 4) ^ ((prow // 4) % 4)
    lane_elems = prow * pitch + pchunk * 8                      # fp16 elements from a 16-row block's origin
    last_step = (steps - 1) * 32
    x_end = w_end = s_end = 0
    for mt in range(m_tiles):
        for plane in range(2):
            for rb in range(tile_rows // 16):
                origin = plane * m_pad * pitch + (mt * tile_rows + rb * 16) * pitch
                x_end = max(x_end, int((origin + lane_elems + last_step + 8).max()) * 2)
    for nt in range(n_tiles):
        for rb in range(tile_cols // 16):
            origin = (nt * tile_cols + rb * 16) * pitch
            w_end = max(w_end, int((origin + lane_elems + last_step + 8).max()) * 2)
        for wave in range(4):
            s_end = max(s_end, int(((steps - 1) * n_pad + nt * tile_cols + wave * 64 + lanes + 1).max()) * 4)
    return [x_end, w_end, s_end]


@pytest.mark.parametrize("tile", TILES)
def test_reach_matches_a_lane_by_lane_enumeration(tile):
    for m, k, n in [(256, 64, 256), (300, 100, 516), (257, 2048, 2052), (512, 96, 1540), (384, 70, 764), (1000, 33, 772)]:
        ok, reach, size = HipNative.q8GemmF16Extents(m, k, n, *tile)
        assert ok == 1, (m, k, n, tile, reach, size)
        assert reach == enumerate_reach(m, k, n, *tile), (m, k, n, tile)


def test_every_load_stays_inside_over_the_shape_space():
    ms = [16, 17, 63, 64, 65, 100, 128, 129, 192, 255, 256, 257, 300, 319, 320, 384, 448, 511, 512, 513, 1000, 1024, 2048, 4096]
    ks = [64, 65, 96, 100, 2048, 2080, 4096, 5632, 11008]
    ns = [4, 64, 188, 192, 196, 252, 256, 260, 764, 768, 772, 1536, 2048, 2052, 3072, 4096, 5632, 6144, 11008, 11264, 32000]
    checked = 0
    for m, k, n in itertools.product(ms, ks, ns):
        for tile in TILES + [(0, 0)]:
            ok, reach, size = HipNative.q8GemmF16Extents(m, k, n, *tile)
            if tile == (0, 0) and ok == -1:
                continue                                        # the library keeps this shape on its other kernels
            assert ok == 1, (m, k, n, tile, reach, size)
            assert all(r <= s for r, s in zip(reach, size))
            checked += 1
    assert checked > 3 * len(ms) * len(ks) * len(ns)


def test_buffer_sizes_agree_with_the_prepared_weight_and_workspace_queries():
    for m, k, n in [(512, 2048, 2048), (300, 100, 516), (1000, 5632, 2048), (256, 2048, 11264)]:
        ok, reach, size = HipNative.q8GemmF16Extents(m, k, n)
        if ok == -1:
            continue
        kp = (k + 31) // 32 * 32
        n_pad = (n + 767) // 768 * 768
        prepared_bytes = HipNative.q8PreparedFloats(k, n) * 4
        # fp16 rows, then the scales: both parts lie inside the prepared buffer
        assert size[1] <= 2 * n_pad * (kp + 64)
        assert 2 * n_pad * (kp + 64) + size[2] <= prepared_bytes + 256


def test_tiles_the_kernels_do_not_have_and_single_rows_are_not_answered():
    assert HipNative.q8GemmF16Extents(512, 2048, 2048, 64, 192)[0] == 1
    assert HipNative.q8GemmF16Extents(512, 2048, 2048, 96, 256)[0] == -1
    assert HipNative.q8GemmF16Extents(512, 2048, 2048, 128, 128)[0] == -1
    assert HipNative.q8GemmF16Extents(1, 2048, 2048)[0] == -1
