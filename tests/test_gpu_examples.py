"""The programs of upstream's self-checking example scripts that the other frontend tests do not
already hold, written against this frontend and compared with NumPy running the same statements:
red-black Gauss-Seidel by strided slices (examples/gauss_seidel.py), matvec and matmatmul on sliced
and dimension-dropped operands (examples/matvec_slice.py, examples/matmatmul.py), the pieces and a
whole V-cycle of the 2-D multigrid solver (examples/multigrid2d.py, with its weighted Jacobi smoother
and residual), numpy.diag both ways (examples/diag.py) and the Jacobi iteration x += D^-1 (b - A x)
built from diag and matvec (examples/jacobi_iteration.py). Element-wise statements must match NumPy
bit for bit; products are held to 1e-12 of the sum of absolute products."""
import os

import numpy as np
import pytest

import charmnumeric_amd as cnp

pytestmark = pytest.mark.gpu


@pytest.fixture
def itf():
    cnp.reset()
    it = cnp.CharmNumericInterface(device=0)
    it.connect(odf=4)
    it.set_min_tile(1, 64)
    it.set_min_tile(2, 16)
    it.set_min_tile(3, 8)
    yield it
    cnp.reset()
    it.close()


# ---- red-black Gauss-Seidel ----

def _red_black_sweep(phi, f, h2):
    for r0, c0 in ((1, 1), (2, 2), (1, 2), (2, 1)):          # red, red, black, black
        rows, cols = slice(r0, -1, 2), slice(c0, -1, 2)
        up, down = slice(r0 - 1, -2, 2), slice(r0 + 1, None, 2)
        left, right = slice(c0 - 1, -2, 2), slice(c0 + 1, None, 2)
        phi[rows, cols] = 0.25 * (phi[up, cols] + phi[down, cols] + phi[rows, left] + phi[rows, right]
                                  - h2 * f[rows, cols])


@pytest.mark.parametrize("n", [33, 64])
def test_red_black_gauss_seidel(itf, n):
    h2 = (1.0 / (n - 1)) ** 2
    rng = np.random.default_rng(n)
    f_host = rng.standard_normal((n, n))
    phi_host = np.zeros((n, n))
    phi, f = cnp.zeros((n, n)), cnp.array(f_host)
    for _ in range(5):
        _red_black_sweep(phi, f, h2)
        _red_black_sweep(phi_host, f_host, h2)
    got = phi.get(itf)
    assert np.array_equal(got, phi_host)
    assert np.abs(got).max() > 0


@pytest.mark.parametrize("fusion", [True, False], ids=["paired", "one-by-one"])
@pytest.mark.parametrize("shape", [(33, 33), (64, 64), (70, 131), (129, 258), (200, 64), (18, 20, 22), (17, 19, 33)])
def test_red_black_sweeps_on_lattices(itf, shape, fusion):
    """The two lattices of a colour go out as one sweep in place (arrays laid out as one block on
    the way); one by one, or paired, the result is NumPy's bit for bit. Rank 3: the colours of a
    red-black sweep are four lattices each, paired two by two."""
    itf.set_fusion(fusion)
    itf.set_trace()
    rng = np.random.default_rng(sum(shape))
    f_host = rng.standard_normal(shape)
    phi_host = rng.standard_normal(shape)
    phi, f = cnp.array(phi_host), cnp.array(f_host)
    h2 = 0.37

    def sweep2(p, g):
        _red_black_sweep(p, g, h2)

    def sweep3(p, g):
        starts = [(a, b, c) for a in (1, 2) for b in (1, 2) for c in (1, 2)]
        for colour in (0, 1):
            for s in [t for t in starts if sum(t) % 2 == (1 + colour) % 2]:
                me = tuple(slice(q, -1, 2) for q in s)
                def sh(d, delta):
                    k = list(me)
                    k[d] = slice(s[d] + delta, -2 if delta < 0 else None, 2)
                    return tuple(k)
                p[me] = (1.0 / 6.0) * (p[sh(0, -1)] + p[sh(0, 1)] + p[sh(1, -1)] + p[sh(1, 1)]
                                       + p[sh(2, -1)] + p[sh(2, 1)] - h2 * g[me])

    sweep = sweep2 if len(shape) == 2 else sweep3
    for _ in range(3):
        sweep(phi, f)
        sweep(phi_host, f_host)
    got = phi.get(itf)
    assert np.array_equal(got, phi_host)
    tr = itf.trace()
    paired = [ln for ln in tr if "path=lattices" in ln]
    planning = os.environ.get("CHARMNUMERIC_SOLVER", "0") not in ("", "0")
    if fusion and not planning:
        assert len(paired) == 3 * (2 if len(shape) == 2 else 4), tr
    else:
        assert not paired


# ---- products on slices ----

def _close_product(got, a, b):
    want = a @ b
    assert got.shape == want.shape
    assert np.all(np.abs(got - want) <= 1e-12 * (np.abs(a) @ np.abs(b)))


@pytest.mark.parametrize("rows,cols", [
    (slice(None), slice(None)), (slice(0, 32), slice(None)), (slice(None), slice(16, 48)),
    (slice(8, 40), slice(10, 50)), (slice(3, 37), slice(5, 47))])
def test_matvec_on_slices(itf, rows, cols):
    rng = np.random.default_rng(5)
    a_host, x_host = rng.standard_normal((128, 128)), np.arange(1.0, 129.0)
    A, x = cnp.array(a_host), cnp.arange(1, 129, dtype=np.float64)
    y = A[rows, cols].matvec(x[cols])
    cnp.execute(itf)
    _close_product(y.get(itf).reshape(-1), a_host[rows, cols], x_host[cols])


def test_matvec_on_a_plane_of_a_rank3_array(itf):
    rng = np.random.default_rng(6)
    a_host, x_host = rng.standard_normal((2, 96, 128)), rng.standard_normal(128)
    A3, x = cnp.array(a_host), cnp.array(x_host)
    for plane in (0, 1):
        y = A3[plane, :, :].matvec(x)
        _close_product(y.get(itf).reshape(-1), a_host[plane], x_host)


@pytest.mark.parametrize("ra,ca,cb", [
    (slice(None), slice(None), slice(None)), (slice(0, 32), slice(None), slice(None)),
    (slice(None), slice(None), slice(16, 48)), (slice(8, 40), slice(10, 50), slice(5, 45)),
    (slice(3, 37), slice(5, 47), slice(7, 39))])
def test_matmatmul_on_slices(itf, ra, ca, cb):
    rng = np.random.default_rng(7)
    a_host, b_host = rng.standard_normal((128, 128)), rng.standard_normal((128, 128))
    A, B = cnp.array(a_host), cnp.array(b_host)
    C = A[ra, ca] @ B[ca, cb]
    cnp.execute(itf)
    _close_product(C.get(itf), a_host[ra, ca], b_host[ca, cb])


def test_matmatmul_shapes_chain_and_dropped_dimension(itf):
    rng = np.random.default_rng(8)
    a_host, b_host = rng.standard_normal((128, 64)), rng.standard_normal((64, 256))
    _close_product((cnp.array(a_host) @ cnp.array(b_host)).get(itf), a_host, b_host)
    # (A @ B) @ x
    sq_a, sq_b, x_host = rng.standard_normal((96, 96)), rng.standard_normal((96, 96)), rng.standard_normal(96)
    y = (cnp.array(sq_a) @ cnp.array(sq_b)).matvec(cnp.array(x_host))
    want = (sq_a @ sq_b) @ x_host
    got = y.get(itf).reshape(-1)
    assert np.all(np.abs(got - want) <= 1e-11 * (np.abs(sq_a) @ np.abs(sq_b) @ np.abs(x_host)))
    # A3[0] @ B
    a3_host = rng.standard_normal((2, 96, 64))
    C = cnp.array(a3_host)[0, :, :] @ cnp.array(b_host)
    _close_product(C.get(itf), a3_host[0], b_host)


# ---- diag ----

@pytest.mark.parametrize("k", [0, 1, -1, 37, -70])
@pytest.mark.parametrize("dtype", [np.float64, np.int32])
def test_diag_builds_and_extracts(itf, k, dtype):
    """numpy.diag both ways (examples/diag.py upstream), on tiles the diagonal enters off-corner."""
    v_host = (np.arange(100) * 3 - 50).astype(dtype)
    m_host = np.arange(96 * 150).reshape(96, 150).astype(dtype)
    D = cnp.diag(cnp.array(v_host), k=k)
    got = D.get(itf)
    assert got.dtype == dtype and np.array_equal(got, np.diag(v_host, k=k))
    assert np.array_equal(cnp.diag(D, k).get(itf), v_host)
    assert np.array_equal(cnp.diag(cnp.array(m_host), k).get(itf), np.diag(m_host, k))
    assert np.array_equal(cnp.diag(cnp.array(m_host.T.copy()), k).get(itf), np.diag(m_host.T, k))
    assert np.array_equal(cnp.diag(cnp.array(m_host)[3:80, 5:121], k).get(itf), np.diag(m_host[3:80, 5:121], k))


def test_jacobi_iteration_with_diag_and_matvec(itf):
    """A = ones + 2N I assembled with diag, its diagonal read back with diag, 50 steps of
    x += D^-1 (b - A x): converges to the direct solution (upstream checks atol 1e-6)."""
    n = 128
    A = cnp.ones((n, n)) + cnp.diag(cnp.full((n,), 2.0 * n))
    d = cnp.diag(A).get(itf)
    assert np.array_equal(d, np.full(n, 2.0 * n + 1.0))
    b, x = cnp.ones((n,)), cnp.zeros((n,))
    d_inv = cnp.full((n,), 1.0 / (2.0 * n + 1.0))
    a_host = np.ones((n, n)) + 2.0 * n * np.eye(n)
    x_host = np.zeros(n)
    for _ in range(50):
        x = x + d_inv * (b - A @ x)
        x_host = x_host + (1.0 / (2.0 * n + 1.0)) * (1.0 - a_host @ x_host)
    got = x.get(itf)
    assert np.allclose(got, np.linalg.solve(a_host, np.ones(n)), atol=1e-6)
    assert np.allclose(got, x_host, rtol=1e-12, atol=0)


# ---- multigrid pieces ----

def _pattern(n):
    """Fills that cross tile boundaries and both parities: whole, interior, the four parity classes,
    a block, two strided boxes, a small centre box."""
    q, tq, e, te, se, mid = n // 4, 3 * n // 4 + 1, n // 8, 3 * n // 8, 7 * n // 8 + 1, n // 2
    s = slice
    return [((s(None), s(None)), 0.0), ((s(1, n - 1), s(1, n - 1)), 1.0),
            ((s(1, n - 1, 2), s(1, n - 1, 2)), 2.0), ((s(2, n - 2, 2), s(1, n - 1, 2)), -1.0),
            ((s(1, n - 1, 2), s(2, n - 2, 2)), 0.5), ((s(2, n - 2, 2), s(2, n - 2, 2)), -0.25),
            ((s(q, tq), s(q, tq)), 3.0), ((s(te, se, 2), s(e, 5 * n // 8 + 1, 2)), -2.0),
            ((s(e, se, 4), s(5 * n // 16, 15 * n // 16, 2)), 0.75),
            ((s(mid - 2, mid + 3), s(mid - 2, mid + 3)), -4.0)]


def _fill_pattern(arr):
    for key, value in _pattern(arr.shape[0]):
        arr[key] = float(value)


def _smooth(u, f, h2, sweeps, omega=2.0 / 3.0):
    for _ in range(sweeps):
        upd = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:] + h2 * f[1:-1, 1:-1])
        u[1:-1, 1:-1] = (1.0 - omega) * u[1:-1, 1:-1] + omega * upd


def _residual(xp, u, f, h2):
    r = xp.zeros(u.shape, dtype=np.float64)
    r[1:-1, 1:-1] = f[1:-1, 1:-1] - (1.0 / h2) * (4.0 * u[1:-1, 1:-1] - u[:-2, 1:-1] - u[2:, 1:-1]
                                                   - u[1:-1, :-2] - u[1:-1, 2:])
    return r


def _restrict(fine, coarse):
    c, lo, hi = slice(2, -2, 2), slice(1, -3, 2), slice(3, -1, 2)
    coarse[:, :] = 0.0
    coarse[1:-1, 1:-1] = (0.25 * fine[c, c]
                          + 0.125 * (fine[lo, c] + fine[hi, c] + fine[c, lo] + fine[c, hi])
                          + 0.0625 * (fine[lo, lo] + fine[lo, hi] + fine[hi, lo] + fine[hi, hi]))


def _prolong_and_correct(xp, e_coarse, u_fine):
    n = u_fine.shape[0]
    e = xp.zeros((n, n), dtype=np.float64)
    e[2:-2:2, 2:-2:2] = e_coarse[1:-1, 1:-1]
    e[1:-1:2, 2:-2:2] = 0.5 * (e_coarse[:-1, 1:-1] + e_coarse[1:, 1:-1])
    e[2:-2:2, 1:-1:2] = 0.5 * (e_coarse[1:-1, :-1] + e_coarse[1:-1, 1:])
    e[1:-1:2, 1:-1:2] = 0.25 * (e_coarse[:-1, :-1] + e_coarse[1:, :-1] + e_coarse[:-1, 1:] + e_coarse[1:, 1:])
    u_fine[1:-1, 1:-1] = u_fine[1:-1, 1:-1] + e[1:-1, 1:-1]


def _vcycle(xp, u, f, h, pre, post, coarse_sweeps):
    n, h2 = u.shape[0], h * h
    if n <= 5:
        _smooth(u, f, h2, coarse_sweeps)
        return
    _smooth(u, f, h2, pre)
    r = _residual(xp, u, f, h2)
    nc = (n - 1) // 2 + 1
    rc = xp.zeros((nc, nc), dtype=np.float64)
    _restrict(r, rc)
    ec = xp.zeros((nc, nc), dtype=np.float64)
    _vcycle(xp, ec, rc, 2.0 * h, pre, post, coarse_sweeps)
    _prolong_and_correct(xp, ec, u)
    _smooth(u, f, h2, post)


@pytest.mark.parametrize("n", [33, 65])
def test_strided_fill_pattern(itf, n):
    host = np.zeros((n, n))
    dev = cnp.zeros((n, n))
    _fill_pattern(host)
    _fill_pattern(dev)
    assert np.array_equal(dev.get(itf), host)


@pytest.mark.parametrize("n", [33, 65])
def test_full_weighting_restriction(itf, n):
    nc = (n - 1) // 2 + 1
    fine_host, coarse_host = np.zeros((n, n)), np.full((nc, nc), 9.0)
    fine, coarse = cnp.zeros((n, n)), cnp.full((nc, nc), 9.0)
    _fill_pattern(fine_host)
    _fill_pattern(fine)
    _restrict(fine_host, coarse_host)
    _restrict(fine, coarse)
    assert np.array_equal(coarse.get(itf), coarse_host)


@pytest.mark.parametrize("n", [33, 65])
def test_bilinear_prolongation(itf, n):
    nc = (n - 1) // 2 + 1
    ec_host, u_host = np.zeros((nc, nc)), np.zeros((n, n))
    ec, u = cnp.zeros((nc, nc)), cnp.zeros((n, n))
    _fill_pattern(ec_host)
    _fill_pattern(ec)
    _prolong_and_correct(np, ec_host, u_host)
    _prolong_and_correct(cnp, ec, u)
    assert np.array_equal(u.get(itf), u_host)


def _interpolate(fine, coarse):
    """Linear interpolation onto a grid of 2 c - 1 points per dimension, one statement per parity
    pattern of the fine index (4 statements in 2-D, 8 in 3-D), boundary points left alone."""
    nd = coarse.ndim
    for bits in np.ndindex(*([2] * nd)):
        target = tuple(slice(1, -1, 2) if b else slice(2, -2, 2) for b in bits)
        total, terms = None, 0
        for side in np.ndindex(*[2 if b else 1 for b in bits]):
            src = tuple((slice(None, -1) if s == 0 else slice(1, None)) if b else slice(1, -1)
                        for b, s in zip(bits, side))
            total = coarse[src] if total is None else total + coarse[src]
            terms += 1
        fine[target] = total if terms == 1 else (1.0 / terms) * total


@pytest.mark.parametrize("fusion", [True, False], ids=["one-launch", "one-by-one"])
@pytest.mark.parametrize("cshape", [(3, 3), (17, 33), (65, 64), (130, 257), (5, 9, 33), (12, 10, 70)])
def test_interleaved_lattices_are_assigned_by_one_scatter(itf, cshape, fusion):
    """The statements of a prolongation assign interleaved lattices of the fine array and read only
    the coarse one: up to four of them are one launch. Same bits as NumPy and as one by one."""
    rng = np.random.default_rng(sum(cshape))
    fshape = tuple(2 * c - 1 for c in cshape)
    c_host, f_host = rng.standard_normal(cshape), rng.standard_normal(fshape)
    itf.set_fusion(fusion)
    itf.set_trace()
    c, f = cnp.array(c_host), cnp.array(f_host)
    for _ in range(2):
        _interpolate(f, c)
        _interpolate(f_host, c_host)
        c[...] = c * 0.5 + 1.0
        c_host[...] = c_host * 0.5 + 1.0
    assert np.array_equal(f.get(itf), f_host)
    launches = [ln for ln in itf.trace() if "path=scatter" in ln]
    planning = os.environ.get("CHARMNUMERIC_SOLVER", "0") not in ("", "0")
    if fusion and not planning and min(cshape) > 3:
        assert len(launches) == 2 * (1 << len(cshape)) // 4 and all("roots=4" in ln for ln in launches)
    if not fusion:
        assert not launches


@pytest.mark.parametrize("width", [40, 41, 130, 131])
@pytest.mark.parametrize("longer", ["left", "right", "equal"])
def test_lattices_side_by_side_are_stored_as_pairs_whichever_is_longer(itf, width, longer):
    """Two statements that assign the odd and the even columns of the same rows (step 2) from other
    arrays are one scatter launch whose lanes store both values as one pair; where one lattice has a
    point more than the other at the end of a row, that point is stored alone. Rows of even and
    odd length (pairs aligned and not)."""
    rows = 9
    rng = np.random.default_rng(width)
    # left lattice: columns 1, 3, ...; right lattice: columns 2, 4, ... of the rows 1, 3, 5, 7
    stop_left, stop_right = {"left": (width, width - 2), "right": (width - 3, width),
                             "equal": (width - 2, width - 1)}[longer]
    left, right = slice(1, stop_left, 2), slice(2, stop_right, 2)
    nl, nr = len(range(width)[left]), len(range(width)[right])
    a_host, b_host = rng.standard_normal((4, nl)), rng.standard_normal((4, nr))
    e_host = rng.standard_normal((rows, width))
    itf.set_trace()
    a, b, e = cnp.array(a_host), cnp.array(b_host), cnp.array(e_host)
    for xp_e, xp_a, xp_b in ((e, a, b), (e_host, a_host, b_host)):
        xp_e[1:-1:2, left] = xp_a * 2.0
        xp_e[1:-1:2, right] = xp_b + 1.0
    assert np.array_equal(e.get(itf), e_host)
    if os.environ.get("CHARMNUMERIC_SOLVER", "0") in ("", "0"):
        assert sum("path=scatter roots=2" in ln for ln in itf.trace()) == 1


def test_weighted_jacobi_and_residual(itf):
    n = 65
    h2 = (1.0 / (n - 1)) ** 2
    u_host, f_host = np.zeros((n, n)), np.zeros((n, n))
    u, f = cnp.zeros((n, n)), cnp.zeros((n, n))
    for arr in (u_host, f_host, u, f):
        _fill_pattern(arr)
    _smooth(u_host, f_host, h2, 3)
    _smooth(u, f, h2, 3)
    assert np.array_equal(u.get(itf), u_host)
    assert np.array_equal(_residual(cnp, u, f, h2).get(itf), _residual(np, u_host, f_host, h2))


@pytest.mark.parametrize("auto_flush", [0, 24])
def test_multigrid_v_cycles(itf, auto_flush):
    """Two V-cycles from 65x65 down to 5x5 for -lap(u) = 2 pi^2 sin(pi x) sin(pi y): every level's
    arrays, strided transfers between levels and temporaries, bit for bit against NumPy; and the
    error against the continuous solution drops."""
    n, h = 65, 1.0 / 64
    xs = np.linspace(0.0, 1.0, n)
    exact = np.outer(np.sin(np.pi * xs), np.sin(np.pi * xs))
    f_host = 2.0 * np.pi ** 2 * exact
    u_host = np.zeros((n, n))
    if auto_flush:
        cnp.set_auto_flush(itf, auto_flush)
    try:
        u, f = cnp.zeros((n, n)), cnp.array(f_host)
        errs = []
        for _ in range(2):
            _vcycle(np, u_host, f_host, h, 2, 2, 40)
            _vcycle(cnp, u, f, h, 2, 2, 40)
            got = u.get(itf)
            assert np.array_equal(got, u_host)
            errs.append(np.abs(got - exact).max())
    finally:
        cnp.reset()
    assert errs[1] < 0.2 * errs[0] < 0.1


# ---- 1-D Jacobi through a named temporary (examples/jacobi.py upstream) ----

@pytest.mark.parametrize("n,dtype", [(128, np.float32), (1000, np.float64)])
def test_jacobi_1d_with_a_temporary(itf, n, dtype):
    u = cnp.zeros((n,), dtype=dtype)
    hu = np.zeros((n,), dtype=dtype)
    u[0] = 1.0
    u[-1] = 1.0
    hu[0] = hu[-1] = 1.0
    for _ in range(3):
        t = 0.5 * (u[:-2] + u[2:])
        u[1:-1] = t
        ht = 0.5 * (hu[:-2] + hu[2:])
        hu[1:-1] = ht
    got = u.get(itf)
    assert got.dtype == dtype and np.array_equal(got, hu)
    assert got[1] == 0.625 and got[2] == 0.25 and got[3] == 0.125   # three sweeps from the ends


# ---- products and dots read unit-step windows in place ----

def _creates(itf):
    return [ln for ln in itf.trace() if ln.startswith("create")]


@pytest.mark.parametrize("r0,r1,c0,c1", [(0, 70, 0, 50), (3, 61, 5, 47), (16, 48, 16, 32), (17, 18, 1, 50)])
def test_windows_of_matrices_and_vectors_in_place(itf, r0, r1, c0, c1):
    rng = np.random.default_rng(r0 + c1)
    hA, hB, hv = rng.standard_normal((70, 50)), rng.standard_normal((50, 70)), rng.standard_normal(90)
    A, B, v = cnp.array(hA), cnp.array(hB), cnp.array(hv)
    A.get(itf), B.get(itf), v.get(itf)
    itf.set_trace()
    k = c1 - c0
    y = A[r0:r1, c0:c1] @ v[7:7 + k]
    P = A[r0:r1, c0:c1] @ B[c0:c1, 2:60]
    d = v[3:3 + k] @ v[11:11 + k]
    got_y, got_P, got_d = y.get(itf), P.get(itf), d.get(itf)
    assert len(_creates(itf)) == 3                      # the three results, no copies of operands
    wa = hA[r0:r1, c0:c1]
    assert np.abs(got_y - wa @ hv[7:7 + k]).max() <= 1e-12 * (np.abs(wa) @ np.abs(hv[7:7 + k])).max()
    wb = hB[c0:c1, 2:60]
    assert np.all(np.abs(got_P - wa @ wb) <= 1e-12 * (np.abs(wa) @ np.abs(wb)))
    want_d = hv[3:3 + k] @ hv[11:11 + k]
    assert abs(got_d.reshape(-1)[0] - want_d) <= 1e-12 * (np.abs(hv[3:3 + k]) @ np.abs(hv[11:11 + k]))


def test_planes_of_a_rank3_array_in_place(itf):
    rng = np.random.default_rng(77)
    hX, hW, hv = rng.standard_normal((5, 40, 36)), rng.standard_normal((36, 20)), rng.standard_normal(36)
    X, W, v = cnp.array(hX), cnp.array(hW), cnp.array(hv)
    X.get(itf), W.get(itf), v.get(itf)
    itf.set_trace()
    got = [(X[2] @ W).get(itf), (X[3, 4:30, :] @ W).get(itf), (X[4] @ v).get(itf),
           (X[:, 7, :] @ W).get(itf), (X[1:4, 9, 2:36] @ v[0:34]).get(itf)]
    assert len(_creates(itf)) == 5
    want = [hX[2] @ hW, hX[3, 4:30, :] @ hW, hX[4] @ hv, hX[:, 7, :] @ hW, hX[1:4, 9, 2:36] @ hv[0:34]]
    for g, w in zip(got, want):
        assert g.shape == w.shape and np.allclose(g, w, rtol=1e-12, atol=1e-12)
    # dropping the last dimension leaves rows that are not contiguous: copied out first
    g = (X[:, 0:36, 5] @ W).get(itf)
    assert len(_creates(itf)) == 2
    assert np.allclose(g, hX[:, 0:36, 5] @ hW, rtol=1e-12, atol=1e-12)
    # strided windows are copied out too
    g = (X[2, ::2, :] @ W).get(itf)
    assert len(_creates(itf)) == 2
    assert np.allclose(g, hX[2, ::2, :] @ hW, rtol=1e-12, atol=1e-12)


def test_column_operand_becomes_a_vector(itf):
    """A @ c with c of shape (N, 1): upstream copies the column into a 1-D temporary and returns
    the 1-D matvec result (charmnumeric.py:528-531 upstream)."""
    rng = np.random.default_rng(12)
    hA, hc = rng.standard_normal((70, 50)), rng.standard_normal((50, 1))
    A, c = cnp.array(hA), cnp.array(hc)
    got = (A @ c).get(itf)
    want = hA @ hc[:, 0]
    assert got.shape == (70,)
    assert np.abs(got - want).max() <= 1e-12 * (np.abs(hA) @ np.abs(hc[:, 0])).max()
    # a column cut out of a matrix
    hM = rng.standard_normal((50, 9))
    M = cnp.array(hM)
    got = A.matvec(M[:, 4:5]).get(itf)
    assert np.abs(got - hA @ hM[:, 4]).max() <= 1e-12 * (np.abs(hA) @ np.abs(hM[:, 4])).max()
    v = cnp.zeros((50,))
    v[:] = c                                  # the assignment itself, bit for bit
    assert np.array_equal(v.get(itf), hc[:, 0])


# ---- stencils that read one array and assign another ----

def _kernels(itf):
    return [ln.rsplit("kernel=", 1)[1] for ln in itf.trace() if ln.startswith("group") and "kernel=" in ln]


@pytest.mark.parametrize("nd,n,dtype", [(2, 96, np.float64), (2, 50, np.float32), (3, 40, np.float64)])
def test_two_array_sweeps_take_the_register_window_kernel(itf, nd, n, dtype):
    rng = np.random.default_rng(nd * n)
    hu = rng.standard_normal((n,) * nd).astype(dtype)
    hv = rng.standard_normal((n,) * nd).astype(dtype)
    hf = rng.standard_normal((n,) * nd).astype(dtype)
    u, v, f = cnp.array(hu), cnp.array(hv), cnp.array(hf)
    u.get(itf), v.get(itf), f.get(itf)
    inner = (slice(1, -1),) * nd

    def neighbours(x):
        out = None
        for d in range(nd):
            for s in (slice(0, -2), slice(2, None)):
                key = list(inner)
                key[d] = s
                out = x[tuple(key)] if out is None else out + x[tuple(key)]
        return out

    itf.set_trace()
    c = 1.0 / (2 * nd)
    for _ in range(4):                                   # unew = sweep(u); swap
        v[inner] = c * neighbours(u)
        hv[inner] = c * neighbours(hu)
        u, v, hu, hv = v, u, hv, hu
    r = cnp.zeros((n,) * nd, dtype=dtype)
    hr = np.zeros((n,) * nd, dtype=dtype)
    r[inner] = f[inner] - (2.0 * nd * u[inner] - neighbours(u))        # residual: three arrays
    hr[inner] = hf[inner] - (2.0 * nd * hu[inner] - neighbours(hu))
    v[inner] = v[inner] + 0.125 * neighbours(u)                        # the target at its own position
    hv[inner] = hv[inner] + 0.125 * neighbours(hu)
    got_u, got_v, got_r = u.get(itf), v.get(itf), r.get(itf)
    assert np.array_equal(got_u, hu) and np.array_equal(got_v, hv) and np.array_equal(got_r, hr)
    kernels = _kernels(itf)
    assert len(kernels) == 6 and all(k == "direct" for k in kernels), kernels


def test_two_shifted_arrays_fall_back_to_the_gather(itf):
    rng = np.random.default_rng(5)
    hu, hw = rng.standard_normal((64, 64)), rng.standard_normal((64, 64))
    u, w = cnp.array(hu), cnp.array(hw)
    v = cnp.zeros((64, 64))
    hv = np.zeros((64, 64))
    u.get(itf), w.get(itf), v.get(itf)
    itf.set_trace()
    v[1:-1, 1:-1] = u[:-2, 1:-1] + w[2:, 1:-1]
    hv[1:-1, 1:-1] = hu[:-2, 1:-1] + hw[2:, 1:-1]
    assert np.array_equal(v.get(itf), hv)
    assert _kernels(itf) == ["gather"]


# ---- both register-window kernels in both ranks ----

@pytest.mark.parametrize("lean", [0, 1])
@pytest.mark.parametrize("shape,tile", [((20, 40, 384), 128), ((300, 512), 128)])
def test_stencil_kernels_with_and_without_lane_exchange(itf, shape, tile, lean):
    """The wavefront-level kernel (neighbours in x by lane exchange, the pairs beyond the
    wavefront's 128 columns gathered by one load) and the general one give the same bits; the first
    is the default, here each rank runs both."""
    from charmnumeric_amd import _lib as L
    nd = len(shape)
    itf.set_min_tile(nd, tile)
    L.check(L.lib.cnh_set_option(b"direct_lean", lean))
    try:
        rng = np.random.default_rng(lean + nd)
        hu, hf = rng.standard_normal(shape), rng.standard_normal(shape)
        u, f = cnp.array(hu), cnp.array(hf)
        inner = (slice(1, -1),) * nd

        def neighbours(x):
            out = None
            for d in range(nd):
                for s in (slice(0, -2), slice(2, None)):
                    key = list(inner)
                    key[d] = s
                    out = x[tuple(key)] if out is None else out + x[tuple(key)]
            return out

        itf.set_trace()
        for _ in range(3):
            u[inner] = (1.0 / (2 * nd)) * (neighbours(u) + f[inner])
            hu[inner] = (1.0 / (2 * nd)) * (neighbours(hu) + hf[inner])
        assert np.array_equal(u.get(itf), hu)
        assert _kernels(itf) == ["direct"] * 3
    finally:
        L.check(L.lib.cnh_set_option(b"direct_lean", -1))


# ---- 2^k + 1 grids wider than a wavefront's 128 columns ----

@pytest.mark.parametrize("tail", [1, 0], ids=["folded", "own-workgroups"])
@pytest.mark.parametrize("shape", [(37, 257), (21, 129), (20, 385), (70, 258), (9, 10, 257), (6, 9, 129), (40, 130)])
def test_last_column_of_a_2k_plus_1_grid(itf, shape, tail):
    """A row of 128 k + 1 elements: the boundary column beyond the k-th wavefront is copied by that
    wavefront's last lane instead of by workgroups of its own. Same bits either way and as NumPy;
    a two-wide stencil (whose last two columns are boundary) covers 128 k + 2."""
    from charmnumeric_amd import _lib as L
    nd = len(shape)
    L.check(L.lib.cnh_set_option(b"flat_tail", tail))
    try:
        rng = np.random.default_rng(shape[-1] + nd)
        hu, hf = rng.standard_normal(shape), rng.standard_normal(shape)
        u, f = cnp.array(hu), cnp.array(hf)
        wide = shape[-1] % 128 == 2
        h = 2 if wide else 1
        inner = (slice(h, -h),) * nd

        def neighbours(x):
            out = None
            for d in range(nd):
                for s in (slice(0, -2 * h), slice(2 * h, None)):
                    key = list(inner)
                    key[d] = s
                    out = x[tuple(key)] if out is None else out + x[tuple(key)]
            return out

        itf.set_trace()
        for _ in range(3):
            u[inner] = (1.0 / (2 * nd)) * (neighbours(u) + f[inner])
            hu[inner] = (1.0 / (2 * nd)) * (neighbours(hu) + hf[inner])
        r = cnp.zeros(shape)
        hr = np.zeros(shape)
        r[inner] = f[inner] - neighbours(u)              # into another array: its boundary stays 0
        hr[inner] = hf[inner] - neighbours(hu)
        assert np.array_equal(u.get(itf), hu)
        assert np.array_equal(r.get(itf), hr)
        assert _kernels(itf) == ["direct"] * 4
    finally:
        L.check(L.lib.cnh_set_option(b"flat_tail", 1))


def test_large_tiled_arrays_of_a_gather_statement_are_laid_out_as_one_block(itf):
    """A strided statement on large rank-2 arrays that have a buffer per tile runs through the
    gather over tile tables once; the arrays are then one block each and its next occurrences (and
    every other kind of statement on them) give NumPy's bits as before."""
    n = 2048
    rng = np.random.default_rng(12)
    hr, hw = rng.standard_normal((n, n)), rng.standard_normal((n, n))
    hc, hv = np.zeros((n // 2, n // 2)), np.zeros((n, n))
    itf.set_min_tile(2, 512)
    r, w = cnp.array(hr), cnp.array(hw)
    c, v = cnp.zeros((n // 2, n // 2)), cnp.zeros((n, n))
    mid, lo, hi = slice(2, -2, 2), slice(1, -3, 2), slice(3, -1, 2)
    itf.set_trace()
    for _ in range(3):
        c[1:-1, 1:-1] = 0.25 * r[mid, mid] + 0.125 * (r[lo, mid] + r[hi, mid] + r[mid, lo] + r[mid, hi])
        hc[1:-1, 1:-1] = 0.25 * hr[mid, mid] + 0.125 * (hr[lo, mid] + hr[hi, mid] + hr[mid, lo] + hr[mid, hi])
        v[1:-1, 1:-1] = r[:-2, 1:-1] * w[2:, 1:-1] + r[1:-1, 2:] * w[1:-1, :-2]          # two shifted arrays
        hv[1:-1, 1:-1] = hr[:-2, 1:-1] * hw[2:, 1:-1] + hr[1:-1, 2:] * hw[1:-1, :-2]
        r[1:-1, 1:-1] = 0.25 * (r[:-2, 1:-1] + r[2:, 1:-1] + r[1:-1, :-2] + r[1:-1, 2:])  # an aligned sweep
        hr[1:-1, 1:-1] = 0.25 * (hr[:-2, 1:-1] + hr[2:, 1:-1] + hr[1:-1, :-2] + hr[1:-1, 2:])
        cnp.execute(itf)
    y = r @ w[:, 0:1]                                          # a product on the arrays laid out anew
    assert np.array_equal(c.get(itf), hc) and np.array_equal(v.get(itf), hv) and np.array_equal(r.get(itf), hr)
    want = hr @ hw[:, 0]
    assert np.all(np.abs(y.get(itf) - want) <= 1e-12 * (np.abs(hr) @ np.abs(hw[:, 0])))
    planning = os.environ.get("CHARMNUMERIC_SOLVER", "0") not in ("", "0")
    if not planning:
        blocks = [ln for ln in itf.trace() if ln.startswith("block ")]
        assert len(blocks) == 4 and all("tiles=16" in ln or "tiles=4" in ln for ln in blocks), blocks


@pytest.mark.parametrize("route", ["windows", "gather-pairs", "gather-single-elements"])
@pytest.mark.parametrize("shape", [(37, 129), (40, 131), (6, 200), (150, 258), (17, 19, 33), (9, 10, 130), (12, 9, 257)])
def test_shifted_reads_of_two_arrays_over_one_block_arrays(itf, shape, route):
    """out[interior] = f(u shifted one way, w shifted another) on arrays stored as one block: the
    whole-array register-window kernel keeps a window per array; with the stencil kernels switched
    off the same statements run as the gather, by pairs of neighbouring elements or one by one.
    Rows of odd and even length, rows sharing a workgroup, more than one wavefront per row. NumPy's
    bits on every route."""
    from charmnumeric_amd import _lib as L
    nd = len(shape)
    L.check(L.lib.cnh_set_option(b"stencil_mode", 2 if route == "windows" else 0))
    L.check(L.lib.cnh_set_option(b"block_pairs", 0 if route == "gather-single-elements" else 1))
    try:
        rng = np.random.default_rng(sum(shape))
        hu, hw = rng.standard_normal(shape), rng.standard_normal(shape)
        hv = np.zeros(shape)
        u, w, v = cnp.array(hu), cnp.array(hw), cnp.zeros(shape)
        inner = (slice(1, -1),) * nd
        up = (slice(0, -2),) + inner[1:]
        down = (slice(2, None),) + inner[1:]
        right = inner[:-1] + (slice(2, None),)
        left = inner[:-1] + (slice(0, -2),)
        itf.set_trace()
        for _ in range(2):
            v[inner] = u[up] * w[right] + u[right] * w[left] - 0.5 * v[inner]
            hv[inner] = hu[up] * hw[right] + hu[right] * hw[left] - 0.5 * hv[inner]
            u[inner] = u[inner] + 0.25 * v[left]                 # in place, reading another array shifted
            hu[inner] = hu[inner] + 0.25 * hv[left]
            w[inner] = 0.5 * (w[down] + w[left]) * u[up] + v[right]   # the target and two others, all shifted
            hw[inner] = 0.5 * (hw[down] + hw[left]) * hu[up] + hv[right]
        assert np.array_equal(v.get(itf), hv) and np.array_equal(u.get(itf), hu) and np.array_equal(w.get(itf), hw)
        planning = os.environ.get("CHARMNUMERIC_SOLVER", "0") not in ("", "0")
        if not planning:
            assert set(_kernels(itf)) == {"direct" if route == "windows" else "gather"}
    finally:
        L.check(L.lib.cnh_set_option(b"stencil_mode", 2))
        L.check(L.lib.cnh_set_option(b"block_pairs", 1))
