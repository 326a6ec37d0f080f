"""The block-index decode of the tiled kernels on the host: a block index is split into (channel block, tile
column, tile row, image) with multiply-high divisions that are exact only while dividend * divisor < 2^32.  The
launchers refuse a layer outside that; these tests run the same host arithmetic (no GPU call) on the grids of the
reference's extreme conformance shapes (verif/conformance/tosa_ext_profile_ops_info.json:2508-2560: axes of 65535
and 65536) and on grids at the edge of the guard."""
import ctypes

import numpy as np
import pytest

from reference_model_amd import capi


def decode(grid, n_ocb, tiles_x, tiles_y, block):
    lib = capi.load_library()
    out = (ctypes.c_int32 * 4)()
    ok = lib.tmi_debug_tile_decode(grid, n_ocb, tiles_x, tiles_y, block, out)
    return ok, tuple(out)


def want(n_ocb, tiles_x, tiles_y, block):
    tile, ocb = divmod(block, n_ocb)
    trow, tx = divmod(tile, tiles_x)
    n, ty = divmod(trow, tiles_y)
    return (ocb, tx, ty, n)


def tiles(extent, tile):
    return (extent + tile - 1) // tile


# (N, OH, OW, OC) of a layer and the (TH, TW) tile a launcher may pick
LAYERS = [
    ((8, 56, 56, 64), (8, 32)), ((32, 56, 56, 64), (16, 16)),                     # the benchmark layer
    ((1, 65535, 3, 64), (64, 4)), ((1, 65535, 3, 64), (4, 4)), ((1, 2, 65536, 64), (2, 128)),
    ((1, 2, 65536, 64), (1, 8)), ((3, 49, 14, 128), (7, 14)), ((1, 11, 44, 192), (11, 22)),
    ((64, 2, 65536, 64), (2, 64)), ((255, 4, 16384, 128), (4, 32)),
]


@pytest.mark.parametrize("layer,tile", LAYERS)
def test_admitted_grids_decode_every_probed_block_exactly(layer, tile):
    n, oh, ow, oc = layer
    n_ocb, tiles_y, tiles_x = tiles(oc, 64), tiles(oh, tile[0]), tiles(ow, tile[1])
    grid = n * tiles_y * tiles_x * n_ocb
    ok, _ = decode(grid, n_ocb, tiles_x, tiles_y, 0)
    assert ok == 1
    rng = np.random.default_rng(grid & 0xFFFF)
    blocks = {0, grid - 1, grid // 2, tiles_x * n_ocb - 1, tiles_x * n_ocb, tiles_x * tiles_y * n_ocb - 1}
    blocks |= {int(b) for b in rng.integers(0, grid, 2000)}
    # the blocks just under a multiple of a divisor are where an inexact quotient first shows
    blocks |= {grid - 1 - k * tiles_x * n_ocb for k in range(min(64, n * tiles_y))}
    for b in blocks:
        if 0 <= b < grid:
            assert decode(grid, n_ocb, tiles_x, tiles_y, b)[1] == want(n_ocb, tiles_x, tiles_y, b), b


def test_grids_outside_the_exact_range_are_refused():
    # 64 images of [2, 65536] pixels in 1 x 8 tiles: tile index * tiles_x reaches 2^33
    n_ocb, tiles_y, tiles_x = 1, 2, 8192
    grid = 64 * tiles_y * tiles_x
    assert decode(grid, n_ocb, tiles_x, tiles_y, 0)[0] == 0
    # and the decode of the last block by the inexact quotient really is wrong there, which is what the guard is for
    bad = [b for b in range(grid - 1, grid - 1 - 8192 * 40, -8192)
           if decode(grid, n_ocb, tiles_x, tiles_y, b)[1] != want(n_ocb, tiles_x, tiles_y, b)]
    assert bad
    # the last admitted and the first refused grid for one divisor: max_bid * n_ocb < 2^32
    assert decode((1 << 32) // 16, 16, 1, 1, 0)[0] == 1
    assert decode((1 << 32) // 16 + 2, 16, 1, 1, 0)[0] == 0
    # grids that do not fit a launch at all, and zero divisors
    assert decode(1 << 31, 1, 1, 1, 0)[0] == 0 and decode(0, 1, 1, 1, 0)[0] == 0 and decode(8, 0, 1, 1, 0)[0] == 0


def test_exhaustive_decode_of_a_small_odd_grid():
    n_ocb, tiles_x, tiles_y, n = 3, 7, 5, 11
    grid = n * tiles_y * tiles_x * n_ocb
    assert decode(grid, n_ocb, tiles_x, tiles_y, 0)[0] == 1
    for b in range(grid):
        assert decode(grid, n_ocb, tiles_x, tiles_y, b)[1] == want(n_ocb, tiles_x, tiles_y, b)
