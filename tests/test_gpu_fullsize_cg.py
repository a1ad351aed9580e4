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
def cpu_system(cpu_cg_system):
    """Matrix tiles and right-hand side on the host (oracle generator, seed 2)."""
    return cpu_cg_system


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


def test_fused_matvec_forms_its_vector_and_leaves_the_dot(dev, cpu_system):
    """cnh_gemv_tiles_fused against the separate steps: the vector xa + (S / den) xb bit for bit
    (S summed in the kernel's stated order), y the bits cnh_gemv_tiles gives for that vector, the
    per-workgroup partial sums of x . y bit for bit in their stated order."""
    orc, tile, g, tiles, b = cpu_system
    bufs = []
    for i in range(g):
        for j in range(g):
            t = tiles[i][j]
            buf = bench.Buf(L, t.nbytes)
            L.check(L.lib.cnh_fill_cg_matrix(buf.ptr, N, i * tile, t.shape[0], j * tile, t.shape[1],
                                             t.shape[1], 2, None))
            bufs.append(buf)
    tp = L.vparr([t.ptr for t in bufs])
    xa = orc.uniform(N, 9, 1, -1.0, 1.0)
    xb = orc.uniform(N, 9, 2, -1.0, 1.0)
    num = orc.uniform(128, 9, 3, 0.0, 1.0)
    den = np.array([3.25])
    dxa, dxb, dnum, dden = dev.array(xa), dev.array(xb), dev.array(num), dev.array(den)
    dx, dy, dy2 = dev.empty((N,), np.float64), dev.empty((N,), np.float64), dev.empty((N,), np.float64)
    dfold, dpart = dev.empty((1,), np.float64), dev.empty((N // 64,), np.float64)
    dquot = dev.array(np.array([np.nan, 5.0]))
    f = L.GemvFusion(dxa.ptr, dxb.ptr, dnum.ptr, 128, dden.ptr, dfold.ptr, dx.ptr, dpart.ptr, N // 64, dquot.ptr)
    npart = C.c_int64()
    L.check(L.lib.cnh_gemv_tiles_fused(N, N, tile, tp, dx.ptr, dy.ptr, C.byref(f), C.byref(npart), None))
    assert npart.value == N // 64
    # S: lane l adds num[l], num[l + 64], ... in order, then the halving tree over the 64 lanes
    lanes = num[:64] + num[64:128]
    for off in (32, 16, 8, 4, 2, 1):
        lanes[:off] = lanes[:off] + lanes[off:2 * off]
    S = lanes[0]
    assert dfold.get()[0] == S
    want_x = xa + (S / den[0]) * xb
    assert dquot.get()[0] == S / den[0] and dquot.get()[1] == 5.0
    got_x = dx.get()
    assert got_x.tobytes() == want_x.tobytes()
    L.check(L.lib.cnh_gemv_tiles(L.F64, N, N, tile, tp, dx.ptr, dy2.ptr, None))
    y = dy.get()
    assert y.tobytes() == dy2.get().tobytes()
    # partial b: its 8 wavefronts' 8 rows each in order, then the wavefronts in order
    prod = (got_x * y).reshape(N // 64, 8, 8)
    wave = np.zeros((N // 64, 8))
    for q in range(8):
        wave = wave + prod[:, :, q]
    part = wave[:, 0].copy()
    for w in range(1, 8):
        part = part + wave[:, w]
    assert dpart.get().tobytes() == part.tobytes()
    # the plain product with the dot alone (first CG iteration): x is read as given
    f2 = L.GemvFusion(None, None, None, 0, None, None, dx.ptr, dpart.ptr, N // 64)
    L.check(L.lib.cnh_memset0(dy.ptr, N * 8, None))
    L.check(L.lib.cnh_gemv_tiles_fused(N, N, tile, tp, dx.ptr, dy.ptr, C.byref(f2), None, None))
    assert dy.get().tobytes() == y.tobytes() and dpart.get().tobytes() == part.tobytes()
    assert dx.get().tobytes() == want_x.tobytes()
    # refused where it does not apply
    assert L.lib.cnh_gemv_tiles_fused(4096, 4096, 2048, tp, dx.ptr, dy.ptr, C.byref(f2), None, None) == -3
    f3 = L.GemvFusion(dx.ptr, dxb.ptr, dnum.ptr, 128, dden.ptr, None, None, None, 0)
    assert L.lib.cnh_gemv_tiles_fused(N, N, tile, tp, dx.ptr, dy.ptr, C.byref(f3), None, None) == -2
    # y may not be one of the vectors other workgroups still read
    for alias in (dx.ptr, dxa.ptr, dxb.ptr):
        assert L.lib.cnh_gemv_tiles_fused(N, N, tile, tp, dx.ptr, alias, C.byref(f), None, None) == -2
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
