"""The dense CG configuration at its full size (n = 16384, A in 2 x 2 tiles of 8192^2): the tiled
matvec against the oracle's tile matvec + partial accumulate, and 50 CG iterations in the order of
examples/cg.py:40-52 upstream against the same iterations on the oracle's kernels."""
import ctypes as C
import os

import numpy as np
import pytest

import bench
from charmnumeric_amd import _lib as L
from oracle import cn_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

N = 16384
THREADS = min(os.cpu_count() or 1, 16)


@pytest.fixture(scope="module")
def cpu_system():
    """Matrix tiles and right-hand side on the host (oracle generator, seed 2)."""
    return bench.cpu_cg_setup(N)


def test_gemv_tiles_n16384_matches_oracle_tile_matvec(dev, cpu_system):
    orc, tile, g, tiles, b = cpu_system
    assert (tile, g) == (8192, 2)
    lib = orc.lib
    bufs = []
    for i in range(g):
        for j in range(g):
            t = tiles[i][j]
            buf = bench.Buf(L, t.nbytes)
            # generated on the device, as the benchmark does; must equal the host tile bit for bit
            L.check(L.lib.cnh_fill_cg_matrix(buf.ptr, N, i * tile, t.shape[0], j * tile, t.shape[1],
                                             t.shape[1], 2, None))
            bufs.append(buf)
    sample = bufs[1].get(np.float64, count=4096)
    assert np.array_equal(sample, tiles[0][1].reshape(-1)[:4096])
    x = orc.uniform(N, 9, 0, -1.0, 1.0)
    dx, dy = dev.array(x), dev.empty((N,), np.float64)
    L.check(L.lib.cnh_gemv_tiles(L.F64, N, N, tile, L.vparr([t.ptr for t in bufs]), dx.ptr, dy.ptr, None))
    got = dy.get()
    want = np.zeros(N)
    bound = np.zeros(N)
    part = np.zeros(tile)
    for i in range(g):
        seg = want[i * tile:(i + 1) * tile]
        for j in range(g):
            t = tiles[i][j]
            xs = x[j * tile:(j + 1) * tile]
            lib.orc_gemv_sub_mt(O.F64, O.ptr(t), t.shape[1], 0, 0, t.shape[0], t.shape[1], O.ptr(xs),
                                O.ptr(part), THREADS)
            if j == 0:
                seg[:] = part
            else:
                lib.orc_axpy1(O.F64, tile, O.ptr(part), O.ptr(seg))
            bound[i * tile:(i + 1) * tile] += np.abs(t) @ np.abs(xs)
    assert np.all(np.abs(got - want) <= 1e-12 * bound), float(np.max(np.abs(got - want) / bound))
    for t in bufs:
        t.free()
    dev.free_all()


def test_cg_50_iterations_n16384_match_oracle(cpu_system):
    iters = 50
    cg = bench.run_cg(L, N, iters, 0, trace_iters=iters)
    _, xc, rtr_c, cpu_trace = bench.cpu_cg(cpu_system, N, iters, THREADS, keep_x_at=iters)
    par = bench.cg_parity(cg["trace"], cpu_trace, cpu_trace["rtr0"])
    # final solutions: || x_gpu - x_cpu ||_inf <= 1e-10 || x_cpu ||_inf
    assert par["x_max_rel_diff"] <= 1e-10, par
    # the timed pass repeats the traced one on the same system: same bits
    assert np.array_equal(cg["x"], cg["trace"]["x"])
    # alpha, beta and r.r while r.r is above 1e-24 of its start (four iterations on this system;
    # from the sixth on the recursion runs on rounding noise and any two summation orders differ
    # by factors): quotients of dots that each hold the 1e-12 bound
    assert par["scalar_iterations"] >= 4, par
    assert par["alpha_max_rel_dev"] <= 1e-10, par
    assert par["beta_max_rel_dev"] <= 1e-10, par
    assert par["rtr_max_rel_dev"] <= 1e-10, par
    # r.r decreases monotonically on a symmetric positive definite system
    r = cg["trace"]["rtr"]
    assert all(r[i + 1] < r[i] for i in range(par["scalar_iterations"])), r[:8]
