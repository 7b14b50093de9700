"""The order in which workgroups take the tiles of a GEMM grid (host arithmetic of the kernel library, prepared as
multiply-and-shift constants per launch): every tile exactly once, and the order the definition gives -- XCD x owns a
contiguous range of tile numbers, which walk the grid in 32-tile blocks or, where the grid does not divide into
blocks, in groups of tile rows column by column."""
import ctypes

import pytest

from plaidml_amd import hipkernels as hk


def definition(bid, tiles_m, tiles_n):
    n = tiles_m * tiles_n
    per, rem = divmod(n, 8)
    x = bid % 8
    t = x * per + min(x, rem) + bid // 8
    if rem == 0 and per % 32 == 0:
        for th, tw in ((4, 8), (8, 4), (16, 2), (2, 16)):
            if tiles_m % th == 0 and tiles_n % tw == 0:
                blk, inside = divmod(t, 32)
                blocks_n = tiles_n // tw
                return (blk // blocks_n) * th + inside // tw, (blk % blocks_n) * tw + inside % tw
    tw = min(tiles_n, 8)
    th = 32 // tw
    group = th * tiles_n
    first_m = (t // group) * th
    rows = min(tiles_m - first_m, th)
    inside = t % group
    return first_m + inside % rows, inside // rows


GRIDS = [(1, 1), (1, 7), (7, 1), (16, 16), (32, 16), (181, 6), (3136, 2), (784, 4), (49, 16), (13, 5), (100, 3), (64, 64),
         (5, 40), (33, 9), (8, 4), (6272, 1), (2, 16), (17, 17), (361, 12), (250, 31)]


@pytest.mark.parametrize('tiles_m,tiles_n', GRIDS)
def test_every_tile_once_and_in_the_defined_order(tiles_m, tiles_n):
    L = hk.lib()
    tm, tn = ctypes.c_int(), ctypes.c_int()
    seen = set()
    for bid in range(tiles_m * tiles_n):
        assert L.pml_hip_tile_of_workgroup(tiles_m, tiles_n, bid, ctypes.byref(tm), ctypes.byref(tn)) == 0
        assert (tm.value, tn.value) == definition(bid, tiles_m, tiles_n), (bid, tiles_m, tiles_n)
        assert 0 <= tm.value < tiles_m and 0 <= tn.value < tiles_n
        seen.add((tm.value, tn.value))
    assert len(seen) == tiles_m * tiles_n


def test_bad_arguments_are_refused():
    L = hk.lib()
    tm, tn = ctypes.c_int(), ctypes.c_int()
    assert L.pml_hip_tile_of_workgroup(4, 4, 16, ctypes.byref(tm), ctypes.byref(tn)) != 0
    assert L.pml_hip_tile_of_workgroup(0, 4, 0, ctypes.byref(tm), ctypes.byref(tn)) != 0
    assert L.pml_hip_tile_of_workgroup(4, 4, 0, None, ctypes.byref(tn)) != 0
