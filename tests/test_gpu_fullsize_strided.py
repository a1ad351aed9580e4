"""The strided and odd-sized programs of upstream's multigrid and Gauss-Seidel examples at the sizes
the benchmark times them at, through the frontend, against NumPy running the same statements: bit
for bit. At these sizes the executor picks what the small example tests never reach: the whole-array
register-window kernel on element-aligned pairs with 32 wavefronts per row of 4097 (the boundary
column copied by the last lane), two wavefronts per row of 257 in 3-D, the two lattices of a colour
swept in place over 8192^2, the one-block gather with XCD-contiguous rows and the four-lattice
scatter of a prolongation."""
import os

import numpy as np
import pytest

import charmnumeric_amd as cnp

pytestmark = pytest.mark.gpu


def _connect(odf=4, fusion=True):
    cnp.reset()
    it = cnp.CharmNumericInterface(device=0)
    it.connect(odf=odf)
    it.set_fusion(fusion)
    return it


def _smooth(u, f, h2, omega):
    upd = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:] + h2 * f[1:-1, 1:-1])
    u[1:-1, 1:-1] = (1.0 - omega) * u[1:-1, 1:-1] + omega * upd


def _residual(r, u, f, h2):
    r[1:-1, 1:-1] = f[1:-1, 1:-1] - (1.0 / h2) * (4.0 * u[1:-1, 1:-1] - u[:-2, 1:-1] - u[2:, 1:-1]
                                                   - u[1:-1, :-2] - u[1:-1, 2:])


def _restrict(coarse, r):
    c, lo, hi = slice(2, -2, 2), slice(1, -3, 2), slice(3, -1, 2)
    coarse[1:-1, 1:-1] = (0.25 * r[c, c]
                          + 0.125 * (r[lo, c] + r[hi, c] + r[c, lo] + r[c, hi])
                          + 0.0625 * (r[lo, lo] + r[lo, hi] + r[hi, lo] + r[hi, hi]))


def _prolong(e, coarse):
    e[2:-2:2, 2:-2:2] = coarse[1:-1, 1:-1]
    e[1:-1:2, 2:-2:2] = 0.5 * (coarse[:-1, 1:-1] + coarse[1:, 1:-1])
    e[2:-2:2, 1:-1:2] = 0.5 * (coarse[1:-1, :-1] + coarse[1:-1, 1:])
    e[1:-1:2, 1:-1:2] = 0.25 * (coarse[:-1, :-1] + coarse[1:, :-1] + coarse[:-1, 1:] + coarse[1:, 1:])


@pytest.mark.parametrize("fusion", [True, False], ids=["merged", "node-by-node"])
def test_multigrid_pieces_on_4097_squared(fusion):
    """examples/multigrid2d.py upstream on the 2^12 + 1 grid: two smoothing sweeps, the residual,
    its restriction to 2049^2, a smoothing sweep there, and the prolongation back."""
    n = 4097
    nc = (n - 1) // 2 + 1
    rng = np.random.default_rng(41)
    hu, hf = rng.uniform(0.0, 1.0, (n, n)), rng.uniform(-1.0, 1.0, (n, n))
    hr, he, hc = np.zeros((n, n)), np.zeros((n, n)), np.zeros((nc, nc))
    h2, omega = (1.0 / (n - 1)) ** 2, 2.0 / 3.0
    itf = _connect(4, fusion)
    try:
        itf.set_trace()
        u, f = cnp.array(hu), cnp.array(hf)
        r, e, c = cnp.zeros((n, n)), cnp.zeros((n, n)), cnp.zeros((nc, nc))
        for xp_u, xp_f, xp_r, xp_e, xp_c in ((u, f, r, e, c), (hu, hf, hr, he, hc)):
            for _ in range(2):
                _smooth(xp_u, xp_f, h2, omega)
            _residual(xp_r, xp_u, xp_f, h2)
            _restrict(xp_c, xp_r)
            xp_c[1:-1, 1:-1] = 0.5 * xp_c[1:-1, 1:-1] + 0.125 * (xp_c[:-2, 1:-1] + xp_c[2:, 1:-1]
                                                                + xp_c[1:-1, :-2] + xp_c[1:-1, 2:])
            _prolong(xp_e, xp_c)
            xp_u[1:-1, 1:-1] = xp_u[1:-1, 1:-1] + xp_e[1:-1, 1:-1]
        for name, dev, host in (("u", u, hu), ("r", r, hr), ("coarse", c, hc), ("e", e, he)):
            assert np.array_equal(dev.get(itf), host), name
        trace = itf.trace()
        planning = os.environ.get("CHARMNUMERIC_SOLVER", "0") not in ("", "0")
        if fusion and not planning:
            assert sum("path=scatter roots=4" in ln for ln in trace) == 1
        if not planning:
            assert sum("kernel=direct" in ln for ln in trace) >= 4
    finally:
        cnp.reset()
        itf.close()


@pytest.mark.parametrize("fusion", [True, False], ids=["paired", "one-by-one"])
def test_red_black_sweeps_on_8192_squared(fusion):
    """examples/gauss_seidel.py upstream at 8192^2: two sweeps of four statements."""
    n = 8192
    rng = np.random.default_rng(42)
    hg = rng.uniform(-1.0, 1.0, (n, n))
    hphi = np.zeros((n, n))
    h2 = (1.0 / (n - 1)) ** 2
    itf = _connect(4, fusion)
    try:
        itf.set_trace()
        phi, g = cnp.zeros((n, n)), cnp.array(hg)
        for xp_phi, xp_g in ((phi, g), (hphi, hg)):
            for _ in range(2):
                for r0, c0 in ((1, 1), (2, 2), (1, 2), (2, 1)):
                    rows, cols = slice(r0, -1, 2), slice(c0, -1, 2)
                    up, down = slice(r0 - 1, -2, 2), slice(r0 + 1, None, 2)
                    left, right = slice(c0 - 1, -2, 2), slice(c0 + 1, None, 2)
                    xp_phi[rows, cols] = 0.25 * (xp_phi[up, cols] + xp_phi[down, cols] + xp_phi[rows, left]
                                                 + xp_phi[rows, right] - h2 * xp_g[rows, cols])
        assert np.array_equal(phi.get(itf), hphi)
        planning = os.environ.get("CHARMNUMERIC_SOLVER", "0") not in ("", "0")
        if fusion and not planning:
            assert sum("path=lattices roots=2" in ln for ln in itf.trace()) == 4
    finally:
        cnp.reset()
        itf.close()


def test_poisson_sweeps_on_257_cubed():
    """A seven-point sweep with a source term on the 2^8 + 1 grid in 3-D, three sweeps."""
    n = 257
    rng = np.random.default_rng(43)
    hv, hq = rng.uniform(0.0, 1.0, (n, n, n)), rng.uniform(-1.0, 1.0, (n, n, n))
    c6, h2 = 0.16666666666666666, (1.0 / (n - 1)) ** 2
    itf = _connect(64)
    try:
        itf.set_trace()
        v, q = cnp.array(hv), cnp.array(hq)
        for xp_v, xp_q in ((v, q), (hv, hq)):
            for _ in range(3):
                xp_v[1:-1, 1:-1, 1:-1] = c6 * (xp_v[:-2, 1:-1, 1:-1] + xp_v[2:, 1:-1, 1:-1] + xp_v[1:-1, :-2, 1:-1]
                                               + xp_v[1:-1, 2:, 1:-1] + xp_v[1:-1, 1:-1, :-2] + xp_v[1:-1, 1:-1, 2:]
                                               + h2 * xp_q[1:-1, 1:-1, 1:-1])
        assert np.array_equal(v.get(itf), hv)
        if os.environ.get("CHARMNUMERIC_SOLVER", "0") in ("", "0"):
            assert sum("kernel=direct" in ln for ln in itf.trace()) == 3
    finally:
        cnp.reset()
        itf.close()
