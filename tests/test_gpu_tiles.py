"""GPU parity: shifted-slice groups over tiles resident on one device (stencils, slice copies)."""
import numpy as np
import pytest

from charmnumeric_amd import _lib as L
from charmnumeric_amd.astbuild import AstBuilder
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["direct", "slide", "slide-march2d", "gather"])
def stencil_path(request):
    """Run the stencil tests through the register-window kernel, the LDS sliding-window kernel
    (both rank-2 mappings) and the general gather kernel."""
    mode = {"gather": 0, "slide": 1, "slide-march2d": 1, "direct": 2}[request.param]
    L.check(L.lib.cnh_set_option(b"stencil_mode", mode))
    L.check(L.lib.cnh_set_option(b"slide2d_march", 1 if request.param == "slide-march2d" else 0))
    yield request.param
    L.check(L.lib.cnh_set_option(b"stencil_mode", 2))
    L.check(L.lib.cnh_set_option(b"slide2d_march", 1))


def _sweeps(dev, u0, tile, ast, nd, nsweeps, np_step):
    k = H.compile_group(ast, L.F64, nd)
    a = H.TiledArray(dev, u0, tile)
    b = H.TiledArray(dev, np.zeros_like(u0), tile)
    ref = u0.copy()
    for _ in range(nsweeps):
        H.launch_tiles(k, [a] * 2 * nd, [], a, b)
        a, b = b, a
        ref = np_step(ref)
    dev.sync()
    got = a.gather()
    dev.free_all()
    return got, ref


@pytest.mark.parametrize("n,tile", [(64, 16), (70, 32), (33, 64), (1030, 256), (300, 4)])
def test_jacobi2d_tiles_bit_exact(dev, stencil_path, n, tile):
    u0 = np.zeros((n, n))
    u0[0, :] = 1.0
    got, ref = _sweeps(dev, u0, tile, H.ast_jacobi2d(n), 2, 7, H.np_jacobi2d)
    assert np.array_equal(got.view(np.int64), ref.view(np.int64))
    # hot top row: after k sweeps only rows <= k are non-zero; row 1 interior after sweep 1 = 0.25
    assert np.all(got[8:, :] == 0.0)
    one = H.np_jacobi2d(u0)
    assert np.all(one[1, 1:-1] == 0.25)


@pytest.mark.parametrize("n,tile", [(32, 16), (20, 8), (70, 32), (37, 16)])
def test_jacobi3d_tiles_bit_exact(dev, orc, stencil_path, n, tile):
    u0 = orc.uniform(n ** 3, 1, 0, 0.0, 1.0).reshape(n, n, n)
    u0[0], u0[-1], u0[:, 0], u0[:, -1], u0[:, :, 0], u0[:, :, -1] = 0, 0, 0, 0, 0, 0
    got, ref = _sweeps(dev, u0, tile, H.ast_jacobi3d(n), 3, 4, H.np_jacobi3d)
    assert np.array_equal(got.view(np.int64), ref.view(np.int64))


@pytest.mark.parametrize("nd,n,tile", [(2, 64, 16), (2, 70, 32), (2, 1030, 256), (2, 512, 256), (3, 20, 8),
                                       (3, 36, 16), (3, 128, 128)])
def test_sweep_with_source_term_in_a_second_array(dev, orc, stencil_path, nd, n, tile):
    """u[1:-1,..] = c*((neighbours)+f[1:-1,..]): the register-window kernel reads the second array
    at the element's own position; the other stencil modes take the general gather. Bit for bit
    against NumPy on every path."""
    shape = (n,) * nd
    u0 = orc.uniform(n ** nd, 3, 0, -1.0, 1.0).reshape(shape)
    f0 = orc.uniform(n ** nd, 4, 0, -1.0, 1.0).reshape(shape)
    coef = 0.25 if nd == 2 else 1.0 / 6.0
    ast = H.ast_poisson2d(n, coef=coef) if nd == 2 else H.ast_poisson3d(n, coef=coef)
    k = H.compile_group(ast, L.F64, nd)
    a, b = H.TiledArray(dev, u0, tile), H.TiledArray(dev, np.zeros_like(u0), tile)
    f = H.TiledArray(dev, f0, tile)
    ref = u0.copy()
    for _ in range(3):
        H.launch_tiles(k, [a] * (2 * nd) + [f], [], a, b)
        a, b = b, a
        ref = H.np_poisson(ref, f0, coef)
    dev.sync()
    got = a.gather()
    took_direct = L.lib.cnh_kernel_variants_loaded(k, b"direct") > 0
    dev.free_all()
    assert np.array_equal(got.view(np.int64), ref.view(np.int64))
    assert took_direct == (stencil_path == "direct")


def test_source_term_at_a_shifted_position_takes_the_general_gather(dev):
    """f read one column off the element's position is not something the register window holds."""
    n, tile = 64, 16
    rng = np.random.default_rng(2)
    u0, f0 = rng.standard_normal((n, n)), rng.standard_normal((n, n))
    b = AstBuilder(L.F64, 2)
    u, f = b.leaf(0), b.leaf(1)
    mid = ((1, 1), (n - 1, n - 1), (1, 1))
    t1 = b.binary(L.OP_ADD, 100, u, u, ((0, 1), (n - 2, n - 1), (1, 1)), ((2, 1), (n, n - 1), (1, 1)))
    t2 = b.binary(L.OP_ADD, 101, t1, f, None, ((1, 0), (n - 1, n - 2), (1, 1)))
    b.set_region(102, u, t2, mid)
    k = H.compile_group(b.finish(), L.F64, 2)
    a, c, ft = H.TiledArray(dev, u0, tile), H.TiledArray(dev, np.zeros_like(u0), tile), H.TiledArray(dev, f0, tile)
    H.launch_tiles(k, [a, a, ft], [], a, c)
    dev.sync()
    got = c.gather()
    took_direct = L.lib.cnh_kernel_variants_loaded(k, b"direct") > 0
    dev.free_all()
    want = u0.copy()
    want[1:-1, 1:-1] = (u0[:-2, 1:-1] + u0[2:, 1:-1]) + f0[1:-1, :-2]
    assert np.array_equal(got, want) and not took_direct


def _pitched_views(dev, host, tile):
    """One row-major block on the device and a descriptor whose tiles are views into it."""
    import ctypes as C
    nd, n = host.ndim, host.shape[0]
    block = dev.array(host)
    g = (n + tile - 1) // tile
    ptrs = (C.c_void_p * (g ** nd))()
    for i, idx in enumerate(np.ndindex(*([g] * nd))):
        off = 0
        for d in range(nd):
            off = off * n + idx[d] * tile
        ptrs[i] = block.ptr + off * 8
    d = L.Tiled()
    d.ndims, d.tile = nd, tile
    for k in range(nd):
        d.offset[k], d.shape[k], d.grid_lo[k], d.grid[k] = 0, n, 0, g
        d.pitch[k] = n ** (nd - 1 - k)
    d.tiles = C.cast(ptrs, C.POINTER(C.c_void_p))
    return block, ptrs, d


@pytest.mark.parametrize("nd,n,tile,source", [(2, 70, 32, False), (2, 256, 128, True), (3, 36, 16, False),
                                               (3, 64, 32, True)])
def test_tiles_as_pitched_views_into_one_block(dev, nd, n, tile, source):
    """The register-window kernels take tiles that are views into one row-major block (common row
    and plane pitches): an array stored whole, addressed through the same tile grid. Bit for bit
    against NumPy; other kernels refuse such descriptors."""
    import ctypes as C
    rng = np.random.default_rng(n + nd)
    u0, f0 = rng.standard_normal((n,) * nd), rng.standard_normal((n,) * nd)
    coef = 0.25 if nd == 2 else 1.0 / 6.0
    if source:
        ast = H.ast_poisson2d(n, coef=coef) if nd == 2 else H.ast_poisson3d(n, coef=coef)
    else:
        ast = H.ast_jacobi2d(n, coef=coef) if nd == 2 else H.ast_jacobi3d(n, coef=coef)
    k = H.compile_group(ast, L.F64, nd)
    ba, _pa, da = _pitched_views(dev, u0, tile)
    bb, _pb, db = _pitched_views(dev, np.zeros_like(u0), tile)
    bf, _pf, df = _pitched_views(dev, f0, tile)
    nleaf = 2 * nd + (1 if source else 0)
    ref = u0.copy()
    for _ in range(3):
        descs = (L.Tiled * nleaf)(*([da] * (2 * nd) + ([df] if source else [])))
        L.check(L.lib.cnh_launch_group_tiles(k, nleaf, descs, 0, None, 0, C.byref(da), C.byref(db), None))
        da, db, ba, bb = db, da, bb, ba
        ref = H.np_poisson(ref, f0, coef) if source else (H.np_jacobi2d(ref, coef) if nd == 2 else H.np_jacobi3d(ref, coef))
    dev.sync()
    got = ba.get().reshape(u0.shape)
    assert np.array_equal(got, ref)
    assert L.lib.cnh_kernel_variants_loaded(k, b"direct") == 1
    # the general gather addresses tiles through their own extents: pitched views are refused
    L.check(L.lib.cnh_set_option(b"stencil_mode", 0))
    try:
        descs = (L.Tiled * nleaf)(*([da] * (2 * nd) + ([df] if source else [])))
        assert L.lib.cnh_launch_group_tiles(k, nleaf, descs, 0, None, 0, C.byref(da), C.byref(db), None) != 0
    finally:
        L.check(L.lib.cnh_set_option(b"stencil_mode", 2))
    dev.free_all()


@pytest.mark.parametrize("nd,n,tile", [(2, 64, 16), (2, 70, 32), (2, 2048 // 8, 128), (3, 36, 16), (3, 128, 128)])
@pytest.mark.parametrize("dt,npdt", [(L.F32, np.float32), (L.I32, np.int32)])
def test_four_byte_elements_on_every_stencil_path(dev, stencil_path, nd, n, tile, dt, npdt):
    """upstream's jacobi2d example is a float32 grid: the register-window kernel works on pairs of
    4-byte elements as well (8-byte accesses). Bit for bit against NumPy in the same type."""
    rng = np.random.default_rng(n * nd)
    if npdt == np.float32:
        u0 = rng.standard_normal((n,) * nd).astype(npdt)
        coef = npdt(0.25 if nd == 2 else 1.0 / 6.0)
    else:
        u0 = rng.integers(-1000, 1000, (n,) * nd).astype(npdt)
        coef = npdt(3)
    ast = H.ast_jacobi2d(n, dtype=dt, coef=float(coef)) if nd == 2 else H.ast_jacobi3d(n, dtype=dt, coef=float(coef))
    k = H.compile_group(ast, dt, nd)
    a, b = H.TiledArray(dev, u0, tile), H.TiledArray(dev, np.zeros_like(u0), tile)
    ref = u0.copy()
    for _ in range(3):
        H.launch_tiles(k, [a] * (2 * nd), [], a, b)
        a, b = b, a
        with np.errstate(over="ignore"):
            ref = (H.np_jacobi2d(ref, coef) if nd == 2 else H.np_jacobi3d(ref, coef)).astype(npdt)
    dev.sync()
    got = a.gather()
    took_direct = L.lib.cnh_kernel_variants_loaded(k, b"direct") > 0
    dev.free_all()
    assert got.dtype == npdt and np.array_equal(got, ref)
    assert took_direct == (stencil_path == "direct")


def test_bad_pitches_are_refused(dev):
    import ctypes as C
    n, tile = 64, 32
    u0 = np.zeros((n, n))
    k = H.compile_group(H.ast_jacobi2d(n), L.F64, 2)
    ba, _pa, da = _pitched_views(dev, u0, tile)
    bb, _pb, db = _pitched_views(dev, u0, tile)

    def launch(src, dst):
        descs = (L.Tiled * 4)(*([src] * 4))
        return L.lib.cnh_launch_group_tiles(k, 4, descs, 0, None, 0, C.byref(src), C.byref(dst), None)

    assert launch(da, db) == 0
    for bad in ((0, 1), (n, 2), (tile - 2, 1), (-n, 1)):     # one missing, step along rows, too short, negative
        da.pitch[0], da.pitch[1] = bad
        assert launch(da, db) != 0, bad
        assert b"pitch" in L.lib.cnh_last_error()
    da.pitch[0], da.pitch[1] = n, 1
    db.pitch[0], db.pitch[1] = 0, 0                          # source pitched, destination not
    assert launch(da, db) != 0
    dev.sync()
    dev.free_all()


def test_reference_jacobi3d_known_answer(dev, stencil_path):
    """4^3 grid, faces 1.0: every interior point becomes (1/6)*3 = 0.5 (upstream test)."""
    u0 = np.zeros((4, 4, 4))
    u0[0], u0[-1], u0[:, 0], u0[:, -1], u0[:, :, 0], u0[:, :, -1] = 1, 1, 1, 1, 1, 1
    got, _ = _sweeps(dev, u0, 2, H.ast_jacobi3d(4, coef=1.0 / 6.0), 3, 1,
                     lambda u: H.np_jacobi3d(u, 1.0 / 6.0))
    assert np.allclose(got[1:-1, 1:-1, 1:-1], 0.5, rtol=0, atol=1e-15)
    assert np.all(got[0] == 1.0)


def test_shifted_slice_sum_with_offset_decomposition(dev):
    """src[100:300] + src[150:350] on arange(512): the result lives in a decomposition whose
    offset (150) lines its tiles up with the second operand (upstream solver test vector)."""
    src = np.arange(512, dtype=np.float64)
    b = AstBuilder(L.F64, 1)
    s = b.leaf(0)
    b.binary(L.OP_ADD, 2, s, s, ((100,), (300,), (1,)), ((150,), (350,), (1,)), is_temp=False)
    k = H.compile_group(b.finish(), L.F64, 1)
    a = H.TiledArray(dev, src, 64)
    out = H.TiledArray(dev, np.zeros(200), 64, offset=(150,))
    H.launch_tiles(k, [a, a], [], None, out)
    assert np.array_equal(out.gather(), src[100:300] + src[150:350])
    dev.free_all()


def test_strided_slice_assignment_between_arrays(dev):
    """coarse[1:-1,1:-1] = fine[2:-2:2,2:-2:2] for n=17 (upstream integration test)."""
    n, cn = 17, 9
    fine = np.arange(n * n, dtype=np.float64).reshape(n, n)
    coarse = np.full((cn, cn), -1.0)
    b = AstBuilder(L.F64, 2)
    tgt, src = b.leaf(0), b.leaf(1)
    b.set_region(5, tgt, src, ((1, 1), (cn - 1, cn - 1), (1, 1)),
                 rhs_region=((2, 2), (n - 2, n - 2), (2, 2)))
    k = H.compile_group(b.finish(), L.F64, 2)
    f = H.TiledArray(dev, fine, 8)
    c = H.TiledArray(dev, coarse, 4)
    H.launch_tiles(k, [f], [], c, c)  # in place: the target is not an input
    want = coarse.copy()
    want[1:-1, 1:-1] = fine[2:-2:2, 2:-2:2]
    assert np.array_equal(c.gather(), want)
    dev.free_all()


def test_strided_target_region(dev):
    """fine[2:-2:2] = 3*coarse[1:-1] leaves the odd points untouched."""
    n, cn = 33, 17
    fine = np.arange(n, dtype=np.float64)
    coarse = np.arange(cn, dtype=np.float64) * 10
    b = AstBuilder(L.F64, 1)
    tgt, src = b.leaf(0), b.leaf(1)
    t = b.binary(L.OP_MUL, 100, b.scalar(3.0), src, None, ((1,), (cn - 1,), (1,)))
    b.set_region(5, tgt, t, ((2,), (n - 2,), (2,)))
    k = H.compile_group(b.finish(), L.F64, 1)
    f = H.TiledArray(dev, fine, 8)
    f2 = H.TiledArray(dev, np.zeros(n), 8)
    c = H.TiledArray(dev, coarse, 8)
    H.launch_tiles(k, [c], [], f, f2)
    want = fine.copy()
    want[2:-2:2] = 3.0 * coarse[1:-1]
    assert np.array_equal(f2.gather(), want)
    dev.free_all()


def test_tiles_rejects_bad_descriptors(dev):
    n = 64
    k = H.compile_group(H.ast_jacobi2d(n), L.F64, 2)
    a = H.TiledArray(dev, np.zeros((n, n)), 16)
    small = H.TiledArray(dev, np.zeros((32, 32)), 16)
    with pytest.raises(L.CnhError):
        H.launch_tiles(k, [small] * 4, [], a, a)      # input regions leave the 32x32 array
    with pytest.raises(L.CnhError):
        H.launch_tiles(k, [a] * 3, [], a, a)          # wrong number of inputs
    dev.free_all()
