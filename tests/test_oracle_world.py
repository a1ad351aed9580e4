"""The oracle's chare-by-chare execution of a fused stencil group (halo pack and delivery, local
and received fragments, aligned cells, one kernel per cell, SET_REGION copy) against NumPy on the
global array. A wrong direction, offset, stride or cell origin anywhere in the planner shows up as
a wrong value here; the message and cell counts are the ones upstream's design implies."""
import numpy as np
import pytest

from charmnumeric_amd import _lib as L
from tests import helpers as H


def _sweep2d(w, coef=0.25):
    out = w.copy()
    out[1:-1, 1:-1] = coef * (((w[:-2, 1:-1] + w[2:, 1:-1]) + w[1:-1, :-2]) + w[1:-1, 2:])
    return out


def _sweep3d(w, c=0.16666666666666666):
    out = w.copy()
    out[1:-1, 1:-1, 1:-1] = c * (((((w[:-2, 1:-1, 1:-1] + w[2:, 1:-1, 1:-1]) + w[1:-1, :-2, 1:-1])
                                   + w[1:-1, 2:, 1:-1]) + w[1:-1, 1:-1, :-2]) + w[1:-1, 1:-1, 2:])
    return out


@pytest.mark.parametrize("n,tile,threads", [(64, 16, 1), (70, 16, 3), (37, 64, 1), (48, 8, 4)])
def test_jacobi2d_through_the_chare_path_matches_numpy(orc, n, tile, threads):
    w = H.np_uniform(n * n, 21, 0, -1.0, 1.0).reshape(n, n)
    tiles = orc.split_tiles(w, tile)
    ast = H.ast_jacobi2d(n)
    for sweep in range(3):
        rc, st = orc.world_group(ast, L.F64, (n, n), tile, tiles, threads)
        assert rc == 0
        w = _sweep2d(w)
        assert np.array_equal(orc.join_tiles(tiles, (n, n), tile), w)
    g = (n + tile - 1) // tile
    # one message per direction across every edge between neighbouring tiles (4 shifted views,
    # each contributing exactly one direction); at most 3x3 aligned cells per chare
    assert st["messages"] == 2 * 2 * g * (g - 1)
    assert st["max_cells"] <= 9 and st["kernels"] >= g * g
    if g >= 3:
        assert st["max_cells"] == 9


@pytest.mark.parametrize("n,tile,threads", [(20, 8, 2), (16, 16, 1), (19, 4, 4)])
def test_jacobi3d_through_the_chare_path_matches_numpy(orc, n, tile, threads):
    w = H.np_uniform(n ** 3, 22, 0, 0.0, 1.0).reshape(n, n, n)
    tiles = orc.split_tiles(w, tile)
    ast = H.ast_jacobi3d(n)
    for sweep in range(2):
        rc, st = orc.world_group(ast, L.F64, (n, n, n), tile, tiles, threads)
        assert rc == 0
        w = _sweep3d(w)
        assert np.array_equal(orc.join_tiles(tiles, (n, n, n), tile), w)
    g = (n + tile - 1) // tile
    assert st["messages"] == 2 * 3 * g * g * (g - 1)      # 6 views, one direction each
    assert st["max_cells"] <= 27


def test_upstream_known_answer_through_the_chare_path(orc):
    """4^3 grid with unit faces: all 8 interior points become 0.5 (upstream's integration test),
    here on 2^3 chares of 2^3."""
    n = 4
    w = np.zeros((n, n, n))
    w[0], w[-1] = 1.0, 1.0
    w[:, 0], w[:, -1] = 1.0, 1.0
    w[:, :, 0], w[:, :, -1] = 1.0, 1.0
    tiles = orc.split_tiles(w, 2)
    rc, st = orc.world_group(H.ast_jacobi3d(n, coef=1.0 / 6.0), L.F64, (n, n, n), 2, tiles, 1)
    assert rc == 0
    got = orc.join_tiles(tiles, (n, n, n), 2)
    assert np.allclose(got[1:-1, 1:-1, 1:-1], 0.5) and np.array_equal(got[0], w[0])
