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


def _pitched_views(dev, host, tile, pad=(0, 0)):
    """One row-major block on the device and a descriptor whose tiles are views into it. `pad`
    = extra elements per row and extra rows per plane between the array's own."""
    import ctypes as C
    nd, shape = host.ndim, host.shape
    padded = list(shape)
    padded[-1] += pad[0]
    if nd == 3:
        padded[1] += pad[1]
    store = np.full(padded, -777.0, dtype=host.dtype)
    store[tuple(slice(0, s) for s in shape)] = host
    block = dev.array(store)
    pitch = [1] * nd
    for k in range(nd - 2, -1, -1):
        pitch[k] = pitch[k + 1] * padded[k + 1]
    grid = [(s + tile - 1) // tile for s in shape]
    ptrs = (C.c_void_p * int(np.prod(grid)))()
    for i, idx in enumerate(np.ndindex(*grid)):
        ptrs[i] = block.ptr + sum(idx[k] * tile * pitch[k] for k in range(nd)) * host.dtype.itemsize
    d = L.Tiled()
    d.ndims, d.tile = nd, tile
    for k in range(nd):
        d.offset[k], d.shape[k], d.grid_lo[k], d.grid[k] = 0, shape[k], 0, grid[k]
        d.pitch[k] = pitch[k]
    d.tiles = C.cast(ptrs, C.POINTER(C.c_void_p))
    block.view = lambda: block.get()[tuple(slice(0, s) for s in shape)]
    block.padding_untouched = lambda: bool(np.all(block.get()[..., shape[-1]:] == -777.0))
    return block, ptrs, d


@pytest.mark.parametrize("flat", [1, 0])
@pytest.mark.parametrize("nd,n,tile,source", [(2, 70, 32, False), (2, 256, 128, True), (3, 36, 16, False),
                                               (3, 64, 32, True)])
def test_tiles_as_pitched_views_into_one_block(dev, nd, n, tile, source, flat):
    """Tiles that are views into one row-major block (common row and plane pitches): an array
    stored whole, addressed through the same tile grid. With direct_flat the whole-array kernel
    runs, without it the per-tile register-window kernels with pitches; the general gather takes
    such views too. Bit for bit against NumPy."""
    import ctypes as C
    rng = np.random.default_rng(n + nd)
    u0, f0 = rng.standard_normal((n,) * nd), rng.standard_normal((n,) * nd)
    coef = 0.25 if nd == 2 else 1.0 / 6.0
    if source:
        ast = H.ast_poisson2d(n, coef=coef) if nd == 2 else H.ast_poisson3d(n, coef=coef)
    else:
        ast = H.ast_jacobi2d(n, coef=coef) if nd == 2 else H.ast_jacobi3d(n, coef=coef)
    step = (lambda r: H.np_poisson(r, f0, coef)) if source else (
        (lambda r: H.np_jacobi2d(r, coef)) if nd == 2 else (lambda r: H.np_jacobi3d(r, coef)))
    k = H.compile_group(ast, L.F64, nd)
    ba, _pa, da = _pitched_views(dev, u0, tile)
    bb, _pb, db = _pitched_views(dev, np.zeros_like(u0), tile)
    bf, _pf, df = _pitched_views(dev, f0, tile)
    nleaf = 2 * nd + (1 if source else 0)
    ref = u0.copy()
    L.check(L.lib.cnh_set_option(b"direct_flat", flat))
    try:
        for _ in range(3):
            descs = (L.Tiled * nleaf)(*([da] * (2 * nd) + ([df] if source else [])))
            L.check(L.lib.cnh_launch_group_tiles(k, nleaf, descs, 0, None, 0, C.byref(da), C.byref(db), None))
            da, db, ba, bb = db, da, bb, ba
            ref = step(ref)
        dev.sync()
        assert np.array_equal(ba.view(), ref)
        assert L.lib.cnh_kernel_variants_loaded(k, b"direct") == 1
        # one more sweep through the general gather
        L.check(L.lib.cnh_set_option(b"stencil_mode", 0))
        descs = (L.Tiled * nleaf)(*([da] * (2 * nd) + ([df] if source else [])))
        L.check(L.lib.cnh_launch_group_tiles(k, nleaf, descs, 0, None, 0, C.byref(da), C.byref(db), None))
        dev.sync()
        assert np.array_equal(bb.view(), step(ref))
        assert L.lib.cnh_kernel_variants_loaded(k, b"tiles") == 1
    finally:
        L.check(L.lib.cnh_set_option(b"stencil_mode", 2))
        L.check(L.lib.cnh_set_option(b"direct_flat", 1))
    dev.free_all()


def _ast_star(shape, dtype=L.F64, coef=0.125, source=False, target=0, window=0):
    """target[1:-1,..] = coef * (sum of the 2*nd face neighbours of `window` [+ f[1:-1,..]]) on an
    array of any extents (array names: window, target, f = 9)."""
    nd = len(shape)
    b = AstBuilder(dtype, nd)
    w = b.leaf(window)
    tgt = w if target == window else b.leaf(target)

    def reg(shift):
        return (tuple(shift), tuple(s + e - 2 for s, e in zip(shift, shape)), (1,) * nd)

    shifts = []
    for d in range(nd):
        lo, hi = [1] * nd, [1] * nd
        lo[d], hi[d] = 0, 2
        shifts += [reg(lo), reg(hi)]
    t = b.binary(L.OP_ADD, 100, w, w, shifts[0], shifts[1])
    for i, r in enumerate(shifts[2:]):
        t = b.binary(L.OP_ADD, 101 + i, t, w, None, r)
    if source:
        t = b.binary(L.OP_ADD, 119, t, b.leaf(9), None, reg([1] * nd))
    t = b.binary(L.OP_MUL, 120, b.scalar(coef), t)
    b.set_region(121, tgt, t, reg([1] * nd))
    return b.finish()


def _np_star(u, coef, f=None):
    nd = u.ndim
    mid = (slice(1, -1),) * nd
    acc = None
    for d in range(nd):
        for sl in (slice(0, -2), slice(2, None)):
            idx = tuple(sl if k == d else slice(1, -1) for k in range(nd))
            acc = u[idx] if acc is None else acc + u[idx]
    if f is not None:
        acc = acc + f[mid]
    return mid, coef * acc


@pytest.mark.parametrize("shape,tile,pad,ob", [
    ((9, 17, 130), 8, (0, 0), None), ((9, 17, 130), 16, (6, 1), (8, 16, 128)), ((33, 40, 258), 32, (2, 0), (16, 32, 256)),
    ((50, 300), 64, (0, 0), None), ((37, 128), 32, (4, 0), (0, 16, 128)), ((5, 9, 2), 4, (0, 0), None),
    ((130, 1026), 128, (0, 0), (0, 64, 512)), ((64, 72, 384), 64, (0, 0), None)])
@pytest.mark.parametrize("source", [False, True])
def test_whole_array_kernel_on_ragged_blocks(dev, shape, tile, pad, ob, source):
    """The whole-array register-window kernel on extents that are no multiple of a wavefront's
    128 columns, of a workgroup's rows and planes or of the ordering block, with padded rows and
    planes: bit for bit against NumPy, and nothing written between the rows."""
    import ctypes as C
    nd = len(shape)
    rng = np.random.default_rng(sum(shape))
    u0, f0 = rng.standard_normal(shape), rng.standard_normal(shape)
    k = H.compile_group(_ast_star(shape, source=source), L.F64, nd)
    ba, _pa, da = _pitched_views(dev, u0, tile, pad)
    bb, _pb, db = _pitched_views(dev, np.zeros_like(u0), tile, pad)
    bf, _pf, df = _pitched_views(dev, f0, tile, pad)
    nleaf = 2 * nd + (1 if source else 0)
    for name, v in zip((b"flat_obz", b"flat_oby", b"flat_obx"), ob or (0, 0, 0)):
        L.check(L.lib.cnh_set_option(name, v))
    try:
        ref = u0.copy()
        for _ in range(2):
            descs = (L.Tiled * nleaf)(*([da] * (2 * nd) + ([df] if source else [])))
            L.check(L.lib.cnh_launch_group_tiles(k, nleaf, descs, 0, None, 0, C.byref(da), C.byref(db), None))
            da, db, ba, bb = db, da, bb, ba
            mid, val = _np_star(ref, 0.125, f0 if source else None)
            ref = ref.copy()
            ref[mid] = val
        dev.sync()
        assert np.array_equal(ba.view(), ref)
        assert ba.padding_untouched() and bb.padding_untouched()
        assert L.lib.cnh_kernel_variants_loaded(k, b"direct") == 1
    finally:
        for name in (b"flat_obz", b"flat_oby", b"flat_obx"):
            L.check(L.lib.cnh_set_option(name, 0))
    dev.free_all()


def test_whole_array_kernel_from_one_array_into_another(dev):
    """unew[interior] = f(u shifted): the window array is not the assigned one; only assigned
    elements of the target are written."""
    import ctypes as C
    shape, tile = (20, 24, 260), 16
    rng = np.random.default_rng(4)
    u0, t0 = rng.standard_normal(shape), rng.standard_normal(shape)
    k = H.compile_group(_ast_star(shape, target=1, window=0), L.F64, 3)
    bu, _pu, du = _pitched_views(dev, u0, tile)
    bt, _pt, dt = _pitched_views(dev, t0, tile)
    descs = (L.Tiled * 6)(*([du] * 6))
    L.check(L.lib.cnh_launch_group_tiles(k, 6, descs, 0, None, 0, C.byref(dt), C.byref(dt), None))
    dev.sync()
    mid, val = _np_star(u0, 0.125)
    want = t0.copy()
    want[mid] = val
    assert np.array_equal(bt.view(), want)
    assert np.array_equal(bu.view(), u0)
    assert L.lib.cnh_kernel_variants_loaded(k, b"direct") == 1
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


# ---- sweeps that also reduce what they change ----

def _residual_cases():
    # (shape, tile, one block?) — ragged tiles, tiles narrower and wider than a wavefront's 128 columns
    return [((70, 70), 32, False), ((256, 512), 128, False), ((36, 36, 36), 16, False),
            ((24, 40, 256), 128, False), ((50, 300), 64, True), ((33, 40, 258), 32, True),
            ((9, 17, 130), 8, True), ((128, 128, 128), 128, True)]


@pytest.mark.parametrize("mode", [0, 1], ids=["sumsq", "maxabs"])
@pytest.mark.parametrize("shape,tile,block", _residual_cases())
def test_sweep_with_residual_matches_the_separate_pass(dev, shape, tile, block, mode):
    """cnh_launch_group_tiles_residual: the new contents bit for bit, the maximum of |new - old|
    exactly and the sum of (new - old)^2 within 1e-12 of what the separate reduction kernels give
    over the same two buffers; the same bits on a second run."""
    import ctypes as C
    nd = len(shape)
    rng = np.random.default_rng(sum(shape) + tile)
    u0 = rng.standard_normal(shape)
    k = H.compile_group(_ast_star(shape), L.F64, nd)
    if block:
        ba, _pa, da = _pitched_views(dev, u0, tile)
        bb, _pb, db = _pitched_views(dev, np.zeros_like(u0), tile)
        new = lambda: bb.view()
        chunks = ([bb.ptr], [ba.ptr], [int(np.prod(shape))])
    else:
        ta, tb = H.TiledArray(dev, u0, tile), H.TiledArray(dev, np.zeros_like(u0), tile)
        da, db = ta.desc(), tb.desc()
        new = lambda: tb.gather()
        chunks = ([b.ptr for b in tb.bufs], [b.ptr for b in ta.bufs], [int(np.prod(b.shape)) for b in ta.bufs])
    out = dev.array(np.full(3, -1.0))
    descs = (L.Tiled * (2 * nd))(*([da] * (2 * nd)))
    for slot in (0, 1):
        L.check(L.lib.cnh_launch_group_tiles_residual(k, 2 * nd, descs, 0, None, 0, C.byref(da), C.byref(db),
                                                      mode, out.ptr + 8 * slot, None))
    fn = L.lib.cnh_sumsq_diff_tiles if mode == 0 else L.lib.cnh_maxabs_diff_tiles
    L.check(fn(len(chunks[2]), L.vparr(chunks[0]), L.vparr(chunks[1]), L.i64arr(chunks[2]), out.ptr + 16, None))
    dev.sync()
    mid, val = _np_star(u0, 0.125)
    want = u0.copy()
    want[mid] = val
    assert np.array_equal(new(), want)
    got = out.get()
    assert got.view(np.int64)[0] == got.view(np.int64)[1]            # run to run
    d = want - u0
    if mode == 1:
        assert got[0] == got[2] == np.max(np.abs(d))
    else:
        ref = float(np.sum(d.astype(np.longdouble) ** 2))
        assert abs(got[0] - ref) <= 1e-12 * ref and abs(got[0] - got[2]) <= 1e-12 * ref
    dev.free_all()


def test_residual_refuses_what_it_cannot_do(dev):
    import ctypes as C
    shape, tile = (64, 64), 32
    k = H.compile_group(_ast_star(shape), L.F64, 2)
    ta = H.TiledArray(dev, np.zeros(shape), tile)
    da = ta.desc()
    out = dev.array(np.zeros(1))
    descs = (L.Tiled * 4)(*([da] * 4))
    # in place: the old contents would be gone
    assert L.lib.cnh_launch_group_tiles_residual(k, 4, descs, 0, None, 0, C.byref(da), C.byref(da), 0,
                                                 out.ptr, None) == -4
    tb = H.TiledArray(dev, np.zeros(shape), tile)
    db = tb.desc()
    assert L.lib.cnh_launch_group_tiles_residual(k, 4, descs, 0, None, 0, C.byref(da), C.byref(db), 2,
                                                 out.ptr, None) == -2
    k32 = H.compile_group(_ast_star(shape, dtype=L.F32), L.F32, 2)
    assert L.lib.cnh_launch_group_tiles_residual(k32, 4, descs, 0, None, 0, C.byref(da), C.byref(db), 0,
                                                 out.ptr, None) == -2
    dev.free_all()
