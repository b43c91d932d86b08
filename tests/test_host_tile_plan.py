"""The tile arithmetic of the GEMM launches (`csrc/km_tile_plan.h`, compiled with g++): which tile
a work-group id computes, and how many tile columns a two-shape launch gives to its large tiles.
Checked by what the arithmetic must guarantee, on every small grid and on the benchmark grids:
each tile handed out exactly once, work-groups dealt to the eight XCDs in contiguous runs, whole
rounds never exceeded."""

import ctypes

import numpy as np
import pytest

from kohakumosstrainer_amd import build as km_build

XCDS = 8


@pytest.fixture(scope="module")
def host():
    lib = ctypes.CDLL(str(km_build.build_hostcheck()))
    lib.km_host_tiles_of.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.km_host_tiles_of.restype = None
    lib.km_host_whole_round_columns.argtypes = [ctypes.c_int] * 3
    return lib


def tiles_of(lib, tiles_m, tiles_n, group_m):
    out = np.empty((tiles_m * tiles_n, 2), dtype=np.int32)
    lib.km_host_tiles_of(tiles_m, tiles_n, group_m, out.ctypes.data)
    return out


BANDS = (8, 4)  # tile rows per band: the fp8 / int8 GEMMs, the weight-only GEMMs


GRIDS = [(m, n) for m in range(1, 20) for n in range(1, 14)] + [(64, 36), (32, 48), (32, 12), (16, 12), (274, 1), (1, 300), (33, 17)]


def test_every_tile_is_computed_exactly_once(host):
    for tiles_m, tiles_n, band in [(m, n, b) for m, n in GRIDS for b in BANDS]:
        t = tiles_of(host, tiles_m, tiles_n, band)
        assert t[:, 0].min() >= 0 and t[:, 0].max() < tiles_m and t[:, 1].min() >= 0 and t[:, 1].max() < tiles_n
        flat = t[:, 0].astype(np.int64) * tiles_n + t[:, 1]
        assert np.array_equal(np.sort(flat), np.arange(tiles_m * tiles_n)), (tiles_m, tiles_n)


def test_an_xcd_walks_a_contiguous_run_of_the_band_order(host):
    """Work-group ids go round-robin over the XCDs. The tiles of one XCD, in the order it gets them,
    must be a contiguous stretch of the band order (bands of eight or four tile rows, column by column
    within a band, rows fastest), so that neighbours in time share operand rows in that XCD's L2."""
    for tiles_m, tiles_n, band in [(m, n, b) for m, n in [(64, 36), (32, 12), (33, 17), (5, 3), (8, 8)] for b in BANDS]:
        t = tiles_of(host, tiles_m, tiles_n, band)
        order = {}
        p = 0
        for first in range(0, tiles_m, band):
            rows = min(band, tiles_m - first)
            for tn in range(tiles_n):
                for r in range(rows):
                    order[(first + r, tn)] = p
                    p += 1
        runs = []
        for xcd in range(XCDS):
            mine = [order[tuple(x)] for x in t[xcd::XCDS]]
            assert mine == list(range(mine[0], mine[0] + len(mine))) if mine else True, (tiles_m, tiles_n, xcd)
            runs.append(len(mine))
        assert max(runs) - min(runs) <= 1


def test_whole_round_columns(host):
    f = host.km_host_whole_round_columns
    assert f(32, 12, 256) == 8  # 8192 x 3072 outputs: 256 of the 384 large tiles are one round
    assert f(32, 48, 256) == 48 and f(64, 36, 256) == 36  # whole rounds already
    assert f(16, 12, 256) == 0  # fewer tiles than compute units: no whole round
    assert f(17, 17, 256) == 15  # 289 tiles: 15 columns = 255 tiles fit the one whole round
    assert f(0, 5, 256) == 5 and f(5, 0, 256) == 0 and f(3, 3, 0) == 3
    for tiles_m in range(1, 40):
        for tiles_n in range(1, 40):
            for units in (1, 7, 64, 256, 304):
                cols = f(tiles_m, tiles_n, units)
                total = tiles_m * tiles_n
                assert 0 <= cols <= tiles_n
                if total % units == 0:
                    assert cols == tiles_n
                else:
                    whole = total // units * units
                    assert cols * tiles_m <= whole < (cols + 1) * tiles_m
