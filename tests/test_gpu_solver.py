"""Arrays laid out by the decomposition solver (tile edges and offsets planned per DAG message):
every statement gives the values NumPy gives, bit for bit for element-wise work and to 1e-12 for
products, whichever way the tiles of its operands happen to be cut. The programs are chosen so
that each consumer of a tiled array meets one whose tile grid does not start at element 0:
fills, gets and uploads, the per-tile and the gathering launch, stencils over temporaries kept as
arrays, dots and differences of differently cut vectors, products (which work on a copy), diag
and tile."""
import numpy as np
import pytest

import charmnumeric_amd as cnp
from charmnumeric_amd import lazy

pytestmark = pytest.mark.gpu


@pytest.fixture
def itf():
    cnp.reset()
    it = cnp.CharmNumericInterface(device=0)
    it.connect(odf=4)
    it.set_min_tile(1, 64)
    it.set_min_tile(2, 16)
    it.set_min_tile(3, 8)
    it.set_solver(True)
    yield it
    cnp.reset()
    it.close()


def info(itf, arr):
    lazy.execute(itf)
    return itf.array_info(arr.name)


def test_shifted_and_strided_copies_take_their_offsets(itf):
    host = np.arange(512, dtype=np.float64) * 0.5 - 7
    a = cnp.array(host)
    b = a[150:350] + 1.0
    c = b * b
    d = b[0:100] - a[150:250]
    e = a[2:202:2] * 2.0
    assert info(itf, b)["offset"] == (150,) and info(itf, b)["tile"] == 64
    assert info(itf, c)["offset"] == (150,)
    assert info(itf, e)["offset"] == (1,) and info(itf, e)["tile"] == 64
    hb = host[150:350] + 1.0
    assert np.array_equal(b.get(itf), hb)
    assert np.array_equal(c.get(itf), hb * hb)
    assert np.array_equal(d.get(itf), hb[0:100] - host[150:250])
    assert np.array_equal(e.get(itf), host[2:202:2] * 2.0)


def test_fill_upload_and_get_of_an_offset_array(itf):
    rng = np.random.default_rng(3)
    host = rng.standard_normal((70, 90))
    a = cnp.array(host)
    b = a[5:60, 7:80] * 1.0                 # offset (5, 7), tiles 16
    assert info(itf, b)["offset"] == (5, 7)
    hb = host[5:60, 7:80] * 1.0
    b[3:50:4, 10:-2:3] = 2.5
    hb[3:50:4, 10:-2:3] = 2.5
    assert np.array_equal(b.get(itf), hb)
    b[:, :] = 0.125
    hb[:, :] = 0.125
    assert np.array_equal(b.get(itf), hb)


@pytest.mark.parametrize("nd,n", [(1, 200), (2, 70), (3, 21)])
def test_jacobi_with_temporaries_kept_as_arrays(itf, nd, n):
    rng = np.random.default_rng(nd)
    hu, hf = rng.standard_normal((n,) * nd), rng.standard_normal((n,) * nd)
    u, f = cnp.array(hu), cnp.array(hf)
    inner = (slice(1, -1),) * nd

    def shifted(x):
        out = []
        for d in range(nd):
            for s in (slice(0, -2), slice(2, None)):
                key = list(inner)
                key[d] = s
                out.append(x[tuple(key)])
        return out

    for _ in range(3):
        parts = shifted(u)
        upd = parts[0]
        for p in parts[1:]:
            upd = upd + p
        upd = (upd + f[inner]) * (1.0 / (2 * nd))
        lazy.execute(itf)                    # upd becomes an array of its own, offset (1,..,1)
        assert itf.array_info(upd.name)["offset"] == (1,) * nd
        w = u[inner] * (1.0 / 3.0) + upd * (2.0 / 3.0)
        lazy.execute(itf)
        u[inner] = w
        hparts = shifted(hu)
        hupd = hparts[0]
        for p in hparts[1:]:
            hupd = hupd + p
        hupd = (hupd + hf[inner]) * (1.0 / (2 * nd))
        hu[inner] = hu[inner] * (1.0 / 3.0) + hupd * (2.0 / 3.0)
    assert np.array_equal(u.get(itf), hu)


def test_dot_and_differences_of_differently_cut_vectors(itf):
    rng = np.random.default_rng(5)
    host = rng.standard_normal(1000)
    a = cnp.array(host)
    x = a[37:637] * 1.0                     # offset 37
    y = a[300:900] * 1.0                    # offset 300
    hx, hy = host[37:637] * 1.0, host[300:900] * 1.0
    assert info(itf, x)["offset"] == (37,) and info(itf, y)["offset"] == (300,)
    got = float((x @ y).get(itf).reshape(-1)[0])
    assert abs(got - float(hx @ hy)) <= 1e-12 * float(np.abs(hx) @ np.abs(hy))
    want = float(((hx - hy) ** 2).sum())
    assert abs(float(cnp.sumsq_diff(x, y).get(itf).reshape(-1)[0]) - want) <= 1e-12 * want
    assert float(cnp.maxabs_diff(y, x).get(itf).reshape(-1)[0]) == np.abs(hx - hy).max()
    # rank 2: the second operand is brought onto the first one's tiles
    hm = rng.standard_normal((90, 90))
    m = cnp.array(hm)
    p, q = m[3:73, 5:75] * 1.0, m[20:90, 1:71] * 1.0
    hp, hq = hm[3:73, 5:75] * 1.0, hm[20:90, 1:71] * 1.0
    want = float(((hp - hq) ** 2).sum())
    assert abs(float(cnp.sumsq_diff(p, q).get(itf).reshape(-1)[0]) - want) <= 1e-12 * want


def test_products_of_offset_operands_work_on_a_copy(itf):
    rng = np.random.default_rng(7)
    hA, hv = rng.standard_normal((100, 90)), rng.standard_normal(200)
    A, v = cnp.array(hA), cnp.array(hv)
    B = A[3:83, 5:85] * 1.0                 # (80, 80), offset (3, 5)
    x = v[11:91] * 1.0                      # offset 11
    assert info(itf, B)["offset"] == (3, 5)
    itf.set_trace()
    y = B @ x
    C2 = B @ B
    hB, hx = hA[3:83, 5:85] * 1.0, hv[11:91] * 1.0
    got_y, got_C = y.get(itf), C2.get(itf)
    log = itf.trace()
    assert sum(ln.startswith("relayout") for ln in log) == 3
    assert np.abs(got_y - hB @ hx).max() <= 1e-12 * (np.abs(hB) @ np.abs(hx)).max()
    assert np.abs(got_C - hB @ hB).max() <= 1e-12 * (np.abs(hB) @ np.abs(hB)).max()
    assert itf.array_info(y.name)["offset"] == (0,)
    assert itf.array_info(C2.name)["offset"] == (0, 0)


def test_diag_and_tile_of_offset_arrays(itf):
    rng = np.random.default_rng(9)
    hM, hv = rng.standard_normal((60, 60)), rng.standard_normal(100)
    M, v = cnp.array(hM), cnp.array(hv)
    S = M[7:47, 9:49] * 1.0                 # offset (7, 9)
    w = v[13:53] * 1.0                      # offset 13
    hS, hw = hM[7:47, 9:49] * 1.0, hv[13:53] * 1.0
    for k in (0, 3, -5):
        assert np.array_equal(cnp.diag(S, k).get(itf), np.diag(hS, k))
        assert np.array_equal(cnp.diag(w, k).get(itf), np.diag(hw, k))
    assert np.array_equal(cnp.tile(w, (3, 2)).get(itf), np.tile(hw, (3, 2)))
    assert np.array_equal(cnp.tile(S, (2, 3)).get(itf), np.tile(hS, (2, 3)))


def test_multigrid_transfers_under_the_solver(itf):
    """Restriction by strided reads and prolongation by strided assignments between a 65^2 and a
    33^2 grid: the coarse arrays take half the fine tile where they are strided copies."""
    rng = np.random.default_rng(11)
    hf = rng.standard_normal((65, 65))
    fine = cnp.array(hf)
    coarse = fine[0::2, 0::2] * 1.0
    inj = 0.25 * (fine[1:-1:2, 1:-1:2] + fine[2::2, 2::2]) + 0.5 * fine[0:-2:2, 0:-2:2]
    hc = hf[0::2, 0::2] * 1.0
    hinj = 0.25 * (hf[1:-1:2, 1:-1:2] + hf[2::2, 2::2]) + 0.5 * hf[0:-2:2, 0:-2:2]
    assert np.array_equal(coarse.get(itf), hc)
    assert np.array_equal(inj.get(itf), hinj)
    out = cnp.zeros((65, 65))
    ho = np.zeros((65, 65))
    out[0::2, 0::2] = coarse
    out[1:-1:2, 1:-1:2] = inj
    ho[0::2, 0::2] = hc
    ho[1:-1:2, 1:-1:2] = hinj
    assert np.array_equal(out.get(itf), ho)
