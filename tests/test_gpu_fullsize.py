"""The stencil configurations at their full size, bit for bit against NumPy: what the small-shape
tests cannot reach (workgroups whose whole window lies inside a tile, wavefront lane exchange,
ordering groups of neighbouring tiles, 64-partition grids)."""
import numpy as np
import pytest

import charmnumeric_amd as cnp
from charmnumeric_amd import _lib as L
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _connect(odf, flat_rank3=True):
    cnp.reset()
    it = cnp.CharmNumericInterface(device=0)
    it.set_layout(flat_rank3)
    it.connect(odf=odf)
    return it


def test_jacobi2d_8192_two_sweeps_match_numpy():
    n = 8192
    itf = _connect(16)
    try:
        u = cnp.random.uniform((n, n), seed=3, stream=0, low=0.0, high=1.0)
        w = H.np_uniform(n * n, 3, 0, 0.0, 1.0).reshape(n, n)
        for _ in range(2):
            u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
            nxt = w.copy()
            nxt[1:-1, 1:-1] = 0.25 * (w[:-2, 1:-1] + w[2:, 1:-1] + w[1:-1, :-2] + w[1:-1, 2:])
            w = nxt
        got = u.get(itf)
        assert itf.array_info(u.name)["tile"] == 2048
        bad = np.count_nonzero(got != w)
        assert bad == 0, f"{bad} elements differ"
        del u
    finally:
        cnp.reset()
        itf.close()


@pytest.mark.parametrize("flat_rank3", [True, False], ids=["one-block", "buffer-per-partition"])
def test_jacobi3d_512_two_sweeps_match_numpy(flat_rank3):
    n = 512
    itf = _connect(64, flat_rank3)
    try:
        u = cnp.random.uniform((n, n, n), seed=1, stream=0, low=0.0, high=1.0)
        w = H.np_uniform(n * n * n, 1, 0, 0.0, 1.0).reshape(n, n, n)
        c = 0.16666666666666666
        for _ in range(2):
            u[1:-1, 1:-1, 1:-1] = c * (u[:-2, 1:-1, 1:-1] + u[2:, 1:-1, 1:-1] + u[1:-1, :-2, 1:-1]
                                       + u[1:-1, 2:, 1:-1] + u[1:-1, 1:-1, :-2] + u[1:-1, 1:-1, 2:])
            nxt = w.copy()
            nxt[1:-1, 1:-1, 1:-1] = c * (w[:-2, 1:-1, 1:-1] + w[2:, 1:-1, 1:-1] + w[1:-1, :-2, 1:-1]
                                         + w[1:-1, 2:, 1:-1] + w[1:-1, 1:-1, :-2] + w[1:-1, 1:-1, 2:])
            w = nxt
        got = u.get(itf)
        assert itf.array_info(u.name)["tile"] == 128
        bad = np.count_nonzero(got != w)
        assert bad == 0, f"{bad} elements differ"
        del u
    finally:
        cnp.reset()
        itf.close()


@pytest.mark.parametrize("flat_rank3", [True, False], ids=["one-block", "buffer-per-partition"])
@pytest.mark.parametrize("tx,ry,rz", [(16, 2, 4), (16, 1, 2), (32, 4, 1)])
def test_small_workgroup_footprints_reach_the_interior_paths(tx, ry, rz, flat_rank3):
    """Narrow workgroups make interior workgroups, lane exchange at row ends inside a wavefront
    and ordering groups occur on small arrays too (256^3 in 8 tiles of 128^3, 700^2 in 4 tiles)."""
    for name, v in (("direct_tx", tx), ("direct_ry", ry), ("direct_rz", rz)):
        L.check(L.lib.cnh_set_option(name.encode(), v))
    itf = _connect(8, flat_rank3)
    try:
        n = 256
        u = cnp.random.uniform((n, n, n), seed=7, stream=0, low=-1.0, high=1.0)
        w = H.np_uniform(n ** 3, 7, 0, -1.0, 1.0).reshape(n, n, n)
        c = 0.16666666666666666
        u[1:-1, 1:-1, 1:-1] = c * (u[:-2, 1:-1, 1:-1] + u[2:, 1:-1, 1:-1] + u[1:-1, :-2, 1:-1]
                                   + u[1:-1, 2:, 1:-1] + u[1:-1, 1:-1, :-2] + u[1:-1, 1:-1, 2:])
        nxt = w.copy()
        nxt[1:-1, 1:-1, 1:-1] = c * (w[:-2, 1:-1, 1:-1] + w[2:, 1:-1, 1:-1] + w[1:-1, :-2, 1:-1]
                                     + w[1:-1, 2:, 1:-1] + w[1:-1, 1:-1, :-2] + w[1:-1, 1:-1, 2:])
        assert np.array_equal(u.get(itf), nxt)
        assert itf.array_info(u.name)["tile"] == 128
        m = 700
        v2 = cnp.random.uniform((m, m), seed=8, stream=0, low=-1.0, high=1.0)
        h2 = H.np_uniform(m * m, 8, 0, -1.0, 1.0).reshape(m, m)
        v2[1:-1, 1:-1] = 0.25 * (v2[:-2, 1:-1] + v2[2:, 1:-1] + v2[1:-1, :-2] + v2[1:-1, 2:])
        n2 = h2.copy()
        n2[1:-1, 1:-1] = 0.25 * (h2[:-2, 1:-1] + h2[2:, 1:-1] + h2[1:-1, :-2] + h2[1:-1, 2:])
        assert np.array_equal(v2.get(itf), n2)
        del u, v2
    finally:
        for name in ("direct_tx", "direct_ry", "direct_rz"):
            L.check(L.lib.cnh_set_option(name.encode(), 0))
        cnp.reset()
        itf.close()
