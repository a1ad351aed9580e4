"""Programs written against the NumPy-like frontend, run through the DAG message, the host executor
and the HIP kernels, and compared with NumPy evaluating the same statements in the same order.
The first block restates the cases of upstream's integration tests
(tests/test_backend_integration.py upstream) and of its self-checking example scripts."""
import os

import numpy as np
import pytest

import charmnumeric_amd as cnp
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture
def itf():
    cnp.reset()
    it = cnp.CharmNumericInterface(device=0)
    it.connect(odf=4)
    yield it
    cnp.reset()
    it.close()


@pytest.fixture
def small_tiles(itf):
    """Minimum tiles as in upstream's own test builds (64), so small arrays span several tiles."""
    itf.set_min_tile(1, 64)
    itf.set_min_tile(2, 16)
    itf.set_min_tile(3, 8)
    return itf


# ---- upstream's integration cases ----

def test_elementwise_expression_known_answer(itf):
    a = cnp.create_array((32,), dtype=np.float32)
    b = cnp.create_array((32,), dtype=np.float32)
    a[:] = 1.5
    b[:] = -0.5
    got = (2.0 * (a + b + 3.0)).get(itf)
    assert got.dtype == np.float32 and np.array_equal(got, np.full(32, 8.0, np.float32))


@pytest.mark.parametrize("shape", [(8,), (4, 4), (4, 4, 4)])
def test_add_on_every_rank(itf, shape):
    lhs = cnp.create_array(shape, dtype=np.float32)
    rhs = cnp.create_array(shape, dtype=np.float32)
    lhs[...] = 1.0
    rhs[...] = 1.0
    got = (lhs + rhs).get(itf)
    assert got.shape == shape and np.array_equal(got, np.full(shape, 2.0, np.float32))


@pytest.mark.parametrize("shape", [(1000,), (40, 50), (10, 12, 20)])
def test_mixed_element_types_promote_like_numpy(small_tiles, shape):
    """Upstream labels such results with np.result_type (charmnumeric.py:369-373); NumPy evaluating
    the same statements is the answer the label promises."""
    itf = small_tiles
    rng = np.random.default_rng(21)
    hi32 = rng.integers(-1000, 1000, shape).astype(np.int32)
    hi64 = rng.integers(-10**12, 10**12, shape).astype(np.int64)
    hf32 = rng.uniform(-3, 3, shape).astype(np.float32)
    hf64 = rng.uniform(-3, 3, shape)
    i32, i64, f32, f64 = (cnp.array(h) for h in (hi32, hi64, hf32, hf64))
    for got, want in (((i32 + f32) * 2, (hi32 + hf32) * 2), (i64 - i32, hi64 - hi32),
                      (f64 * f32 + i32, hf64 * hf32 + hi32), (f32 / i64, hf32 / hi64),
                      (i32.astype(np.float32) + f32, hi32.astype(np.float32) + hf32),
                      (f64.astype(np.int64), hf64.astype(np.int64)),
                      (i64.astype(np.float32), hi64.astype(np.float32))):
        g = got.get(itf)
        assert g.dtype == want.dtype and g.tobytes() == want.tobytes()
    # a slice of one type into a region of another: the target's type wins, as in NumPy
    sl = tuple(slice(1, s - 1) for s in shape)
    tgt = cnp.array(hi32)
    tgt[sl] = f64[sl] * 100.0
    hw = hi32.copy()
    hw[sl] = hf64[sl] * 100.0
    assert np.array_equal(tgt.get(itf), hw)
    if len(shape) == 1:
        assert (i32 @ f64).get(itf)[0] == pytest.approx(float(hi32 @ hf64), rel=1e-12)
    if len(shape) == 2:
        v = cnp.array(rng.uniform(-1, 1, shape[1]))
        np.testing.assert_allclose((i32 @ v).get(itf), hi32 @ v.get(itf), rtol=1e-12, atol=1e-9)
        m = cnp.array(rng.integers(-5, 5, (shape[1], 7)).astype(np.int32))
        np.testing.assert_allclose((f32 @ m).get(itf), hf32.astype(np.float64) @ m.get(itf), rtol=1e-12, atol=1e-9)


def test_dot_with_ones_gives_the_bits_of_the_dot(small_tiles):
    """`z @ ones` is recorded as a sum (one array read instead of two): the same bits as the dot
    with an array that merely holds ones, for every element type."""
    itf = small_tiles
    rng = np.random.default_rng(8)
    for dt in (np.float64, np.float32, np.int32, np.int64):
        h = (rng.uniform(-3, 3, 70001) * 100).astype(dt)
        z = cnp.array(h)
        ones = cnp.ones((70001,), dtype=dt)
        held = cnp.array(np.ones(70001, dt))          # uploaded: not known to be ones
        a, b = (z @ ones).get(itf), (z @ held).get(itf)
        assert a.dtype == dt and a.tobytes() == b.tobytes()
        assert (ones @ z).get(itf).tobytes() == b.tobytes()
        ones[3] = 2                                   # assigned into: a dot again
        got = (z @ ones).get(itf)[0]
        with np.errstate(over="ignore"):
            want = b[0] + h[3]
        assert got == want if np.issubdtype(dt, np.integer) else got == pytest.approx(want, rel=1e-5)


def test_a_coefficient_that_changes_every_step_compiles_once(small_tiles):
    """u = u + c_k * v and a stencil with a changing weight, 12 steps with 12 different Python
    floats: NumPy's bits, and after the first step no further code object is compiled."""
    from charmnumeric_amd import _lib as L
    itf = small_tiles
    rng = np.random.default_rng(4)
    hu, hv = rng.standard_normal((70, 90)), rng.standard_normal((70, 90))
    u, v = cnp.array(hu), cnp.array(hv)
    counts = []
    for k in range(12):
        c = 0.1 + 0.0137 * k
        w = 1.0 / (3.5 + k)
        u = u + c * v
        hu = hu + c * hv
        u[1:-1, 1:-1] = w * (u[:-2, 1:-1] + u[2:, 1:-1]) + (c * u[1:-1, :-2] - u[1:-1, 2:])
        hu[1:-1, 1:-1] = w * (hu[:-2, 1:-1] + hu[2:, 1:-1]) + (c * hu[1:-1, :-2] - hu[1:-1, 2:])
        assert np.array_equal(u.get(itf), hu)
        counts.append(L.lib.cnh_code_objects())
    assert counts[-1] == counts[0], counts


def test_shifted_slices_of_arange(small_tiles):
    src = cnp.arange(512, dtype=np.float32)
    got = (src[100:300] + src[150:350]).get(small_tiles)
    host = np.arange(512, dtype=np.float32)
    assert np.array_equal(got, host[100:300] + host[150:350])


def test_strided_slice_assignment_17_to_9(small_tiles):
    n, cn = 17, 9
    coarse = cnp.create_array((cn, cn), dtype=np.float64)
    fine = cnp.create_array((n, n), dtype=np.float64)
    coarse[:, :] = 0.0
    fine[:, :] = 1.0
    coarse[1:-1, 1:-1] = fine[2:-2:2, 2:-2:2]
    want = np.zeros((cn, cn))
    want[1:-1, 1:-1] = np.ones((n, n))[2:-2:2, 2:-2:2]
    assert np.array_equal(coarse.get(small_tiles), want)


def _faces(u, v):
    u[0, :, :] = v
    u[-1, :, :] = v
    u[:, 0, :] = v
    u[:, -1, :] = v
    u[:, :, 0] = v
    u[:, :, -1] = v


def test_jacobi3d_single_step_on_4_cubed(itf):
    u = cnp.create_array((4, 4, 4), dtype=np.float32)
    _faces(u, 1.0)
    u[1:-1, 1:-1, 1:-1] = (1.0 / 6.0) * (u[:-2, 1:-1, 1:-1] + u[2:, 1:-1, 1:-1] + u[1:-1, :-2, 1:-1]
                                          + u[1:-1, 2:, 1:-1] + u[1:-1, 1:-1, :-2] + u[1:-1, 1:-1, 2:])
    w = np.zeros((4, 4, 4), np.float32)
    _faces(w, 1.0)
    c = np.float32(1.0 / 6.0)
    w[1:-1, 1:-1, 1:-1] = c * (w[:-2, 1:-1, 1:-1] + w[2:, 1:-1, 1:-1] + w[1:-1, :-2, 1:-1]
                               + w[1:-1, 2:, 1:-1] + w[1:-1, 1:-1, :-2] + w[1:-1, 1:-1, 2:])
    got = u.get(itf)
    assert np.array_equal(got, w)
    assert np.allclose(got[1:-1, 1:-1, 1:-1], 0.5)


# ---- upstream's example scripts ----

def test_simple_example_with_overlapping_self_assignment(small_tiles):
    """x = 2*(a+b+3); x[:50] = x[70:120] + 1 (examples/simple.py upstream)."""
    a = cnp.zeros((128,), dtype=cnp.float32)
    b = cnp.zeros((128,), dtype=cnp.float32)
    x = 2 * (a + b + 3)
    x[:50] = x[70:120] + 1
    want = np.full(128, 6.0, np.float32)
    want[:50] = want[70:120] + 1
    assert np.array_equal(x.get(small_tiles), want)


def test_reduction_example(itf):
    """res = x @ x; x = x / res (examples/reduction.py upstream): ones(64) -> 1/64 everywhere."""
    x = cnp.ones((64,), dtype=cnp.float32)
    res = x @ x
    x = x / res
    assert np.array_equal(x.get(itf), np.full(64, 1.0 / 64.0, np.float32))
    assert res.get(itf).item() == 64.0


def test_matvec_closed_form(small_tiles):
    """A[i,j] = i + j, x = 1: y_i = N*i + N(N-1)/2, exact in fp64 (examples/matvec.py upstream)."""
    n = 96
    host = np.add.outer(np.arange(n), np.arange(n)).astype(np.float64)
    A = cnp.array(host)
    x = cnp.ones((n,))
    y = (A @ x).get(small_tiles)
    assert np.array_equal(y, n * np.arange(n) + n * (n - 1) / 2)


def test_matmatmul_of_ones_and_against_numpy(small_tiles):
    A = cnp.ones((48, 80))
    B = cnp.ones((80, 40))
    assert np.array_equal((A @ B).get(small_tiles), np.full((48, 40), 80.0))
    rng = np.random.default_rng(3)
    ha, hb = rng.standard_normal((50, 70)), rng.standard_normal((70, 33))
    got = (cnp.array(ha) @ cnp.array(hb)).get(small_tiles)
    bound = 1e-12 * (np.abs(ha) @ np.abs(hb))
    assert np.all(np.abs(got - ha @ hb) <= bound)


def test_matmatmul_result_is_not_zero_filled_first(itf):
    """fp64 products overwrite their result: a buffer taken back from the free list with other
    contents must not leak into it."""
    rng = np.random.default_rng(8)
    ha, hb = rng.standard_normal((96, 200)), rng.standard_normal((200, 80))
    A, B = cnp.array(ha), cnp.array(hb)
    junk = cnp.array(np.full((96, 80), np.nan))
    junk.get(itf)
    del junk                               # its buffer (same size as the product's) is free again
    got = (A @ B).get(itf)
    want = (ha.astype(np.longdouble) @ hb.astype(np.longdouble)).astype(np.float64)
    assert np.all(np.abs(got - want) <= 1e-12 * (np.abs(ha) @ np.abs(hb)))
    assert itf.stats()["reuses"] >= 1


def test_cg_example_against_the_closed_form(small_tiles):
    """A = N*I + 1 1^T, b = 1..N: x = (b - sum(b)/(2N))/N; CG reaches it in two iterations
    (examples/cg.py upstream)."""
    itf = small_tiles
    n = 128
    A = cnp.ones((n, n), dtype=cnp.float64)
    for i in range(n):
        A[i, i] = n + 1.0
    b = cnp.arange(1, n + 1, dtype=cnp.float64)
    x = cnp.zeros((n,), dtype=cnp.float64)
    r = b.copy()
    p = b.copy()
    rtr = r @ r
    history = []
    for k in range(3):
        Ap = A @ p
        pAp = p @ Ap
        alpha = rtr / pAp
        x = x + alpha * p
        r = r - alpha * Ap
        rtr_new = r @ r
        beta = rtr_new / rtr
        p = r + beta * p
        rtr = rtr_new
        history.append(rtr.get(itf).item())
    bn = np.arange(1, n + 1, dtype=np.float64)
    want = (bn - bn.sum() / (2 * n)) / n
    got = x.get(itf)
    assert np.allclose(got, want, rtol=1e-11, atol=0)
    assert history[0] > history[1] and history[1] < 1e-12 * history[0]
    st = itf.stats()
    assert st["reuses"] > 0


# ---- sweeps, multi-tile, ragged ----

def test_jacobi2d_sweeps_match_numpy_bit_for_bit(small_tiles):
    n = 70                                        # ragged against the tile edge
    u = cnp.zeros((n, n), dtype=cnp.float64)
    u[0, :] = 1.0
    u[:, -1] = 0.5
    w = np.zeros((n, n))
    w[0, :] = 1.0
    w[:, -1] = 0.5
    for _ in range(7):
        u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
        w[1:-1, 1:-1] = 0.25 * (w[:-2, 1:-1] + w[2:, 1:-1] + w[1:-1, :-2] + w[1:-1, 2:])
    got = u.get(small_tiles)
    assert np.array_equal(got, w)
    assert small_tiles.array_info(u.name)["tile"] < n
    st = small_tiles.stats()
    assert st["compiled"] <= 4 and st["cache_hits"] >= 6


def test_jacobi3d_sweeps_with_residual(small_tiles, rank3_layout):
    n = 20
    u = cnp.random.uniform((n, n, n), seed=1, stream=0, low=0.0, high=1.0)
    _faces(u, 0.0)
    w = H.np_uniform(n * n * n, 1, 0, 0.0, 1.0).reshape(n, n, n)
    _faces(w, 0.0)
    c = 0.16666666666666666
    for it in range(4):
        old = u.copy()
        u[1:-1, 1:-1, 1:-1] = c * (u[:-2, 1:-1, 1:-1] + u[2:, 1:-1, 1:-1] + u[1:-1, :-2, 1:-1]
                                   + u[1:-1, 2:, 1:-1] + u[1:-1, 1:-1, :-2] + u[1:-1, 1:-1, 2:])
        wold = w.copy()
        w[1:-1, 1:-1, 1:-1] = c * (w[:-2, 1:-1, 1:-1] + w[2:, 1:-1, 1:-1] + w[1:-1, :-2, 1:-1]
                                   + w[1:-1, 2:, 1:-1] + w[1:-1, 1:-1, :-2] + w[1:-1, 1:-1, 2:])
        d = cnp.maxabs_diff(u, old).get(small_tiles).item()
        assert d == np.max(np.abs(w - wold))
        s = cnp.sumsq_diff(u, old).get(small_tiles).item()
        ref = np.sum((w - wold) ** 2)
        assert abs(s - ref) <= 1e-12 * ref
    assert np.array_equal(u.get(small_tiles), w)


def test_c1_statement_and_reductions(itf):
    n = 1 << 20
    x = cnp.random.uniform((n,), seed=0, stream=0, low=-1.0, high=1.0)
    y = cnp.random.uniform((n,), seed=0, stream=1, low=-1.0, high=1.0)
    z = ((2.5 * x) - (0.5 * y)) + (x * y)
    hx, hy = H.np_uniform(n, 0, 0, -1.0, 1.0), H.np_uniform(n, 0, 1, -1.0, 1.0)
    hz = ((2.5 * hx) - (0.5 * hy)) + (hx * hy)
    assert np.array_equal(z.get(itf), hz)
    s = cnp.sum(z).get(itf).item()
    zz = (z @ z).get(itf).item()
    import math
    assert abs(s - math.fsum(hz)) <= 1e-12 * np.sum(np.abs(hz))
    assert abs(zz - math.fsum(hz * hz)) <= 1e-12 * np.sum(hz * hz)


def test_put_get_roundtrip_on_ragged_tiles(small_tiles, rank3_layout):
    rng = np.random.default_rng(11)
    for shape, dt in [((200,), np.float64), ((37, 53), np.float32), ((9, 14, 21), np.int64),
                      ((70, 70), np.int32)]:
        host = (rng.standard_normal(shape) * 100).astype(dt)
        a = cnp.array(host)
        got = a.get(small_tiles)
        assert got.dtype == dt and np.array_equal(got, host)
        # and a strided view of it, copied out
        key = tuple(slice(1, None, 2) for _ in shape)
        assert np.array_equal(a[key].get(small_tiles), host[key])


def test_integer_arithmetic_wraps_and_truncates(small_tiles):
    host = np.array([7, -7, 2**31 - 1, -2**31, 5, -5, 0, 1] * 20, dtype=np.int32)
    a = cnp.array(host)
    with np.errstate(over="ignore"):
        want = (host * np.int32(3) + np.int32(11))
    assert np.array_equal((a * 3 + 11).get(small_tiles), want)
    q = (a / 2).get(small_tiles)
    assert np.array_equal(q, np.trunc(host / 2).astype(np.int32))


def test_sigmoid_and_tanh_statement(itf):
    n = 4096
    hx = H.np_uniform(n, 9, 0, -8.0, 8.0)
    x = cnp.array(hx)
    s = 1.0 / (1.0 + cnp.exp(-x))
    t = cnp.tanh(x)
    import math
    ws = np.array([1.0 / (1.0 + math.exp(v * -1)) for v in hx])
    wt = np.array([math.tanh(v) for v in hx])
    ds, dt = H.ulp_distance(s.get(itf), ws), H.ulp_distance(t.get(itf), wt)
    lim = 0 if H.host_libm_is_the_restated_one() else 4
    assert ds <= lim and dt <= min(lim, 1)


def test_pending_reader_sees_the_old_contents(itf):
    u = cnp.full((32,), 2.0)
    t = u + 1.0
    u[...] = 5.0
    v = u + 1.0
    assert np.array_equal(t.get(itf), np.full(32, 3.0))
    assert np.array_equal(v.get(itf), np.full(32, 6.0))


def test_view_of_view_assignment_and_inplace_update(small_tiles):
    host = np.arange(400, dtype=np.float64).reshape(20, 20)
    a = cnp.array(host)
    v = a[2:18, 1:19][::2, 3:15:3]
    v[1:, :] = 7.0
    host[2:18, 1:19][::2, 3:15:3][1:, :] = 7.0
    a[5, :] += a[6, :] * 2.0
    host[5, :] += host[6, :] * 2.0
    assert np.array_equal(a.get(small_tiles), host)


def test_assignment_through_a_strided_view_whose_extent_is_no_multiple_of_the_step(small_tiles):
    ha = np.zeros(10)
    a = cnp.zeros(10)
    a[::4][:] = 1.0
    ha[::4][:] = 1.0
    hu = np.arange(11, dtype=np.float64)
    u = cnp.array(hu)
    u[::3].fill(2.0)
    hu[::3].fill(2.0)
    hb = np.arange(3, dtype=np.float64) + 1.0
    b = cnp.array(hb)
    a[::4][0:3] = b + b
    ha[::4][0:3] = hb + hb
    hm = np.arange(150, dtype=np.float64).reshape(10, 15)
    m = cnp.array(hm)
    m[1::4, ::7][:, 1:] = m[1::4, ::7][:, 1:] * 3.0
    hm[1::4, ::7][:, 1:] = hm[1::4, ::7][:, 1:] * 3.0
    assert np.array_equal(a.get(small_tiles), ha)
    assert np.array_equal(u.get(small_tiles), hu)
    assert np.array_equal(m.get(small_tiles), hm)


# ---- the LSTM forward pass of upstream's example, statement for statement ----

def _lstm_numpy(X, h0, W, n, b, d, word):
    import math
    sig = np.vectorize(lambda v: 1.0 / (1.0 + math.exp(v * -1)))
    tanh = np.vectorize(math.tanh)
    Hin = np.zeros((n, b, word + d))
    Hout = np.zeros((n, b, d))
    IFOG = np.zeros((n, b, 4 * d))
    IFOGf = np.zeros((n, b, 4 * d))
    Cc = np.zeros((n, b, d))
    Ct = np.zeros((n, b, d))
    for t in range(n):
        prev = np.tile(h0, (b, 1)) if t == 0 else Hout[t - 1]
        Hin[t, :, :word] = X[t]
        Hin[t, :, word:] = prev
        IFOG[t] = Hin[t].dot(W)
        IFOGf[t, :, :3 * d] = sig(IFOG[t, :, :3 * d])
        IFOGf[t, :, 3 * d:] = tanh(IFOG[t, :, 3 * d:])
        Cc[t] = IFOGf[t, :, :d] * IFOGf[t, :, 3 * d:]
        if t > 0:
            Cc[t] += IFOGf[t, :, d:2 * d] * Cc[t - 1]
        Ct[t] = tanh(Cc[t])
        Hout[t] = IFOGf[t, :, 2 * d:3 * d] * Ct[t]
    return Hout, Cc, IFOG


@pytest.fixture(params=[True, False], ids=["one-block", "buffer-per-partition"])
def rank3_layout(request, itf):
    """Both storage forms of rank-3 arrays."""
    itf.set_layout(request.param)
    return request.param


@pytest.mark.parametrize("n,b,d,word,small", [(4, 32, 10, 10, False), (3, 48, 40, 24, True)])
def test_lstm_forward_example(itf, rank3_layout, n, b, d, word, small):
    """examples/lstm_forward.py upstream: 3-D state arrays, one time step per leading index, a
    dimension-dropped matmul per step, tile() for the first hidden state, in-place cell update."""
    if small:
        itf.set_min_tile(2, 16)
        itf.set_min_tile(3, 8)
    rng = np.random.default_rng(5)
    hX = rng.uniform(-1, 1, (n, b, word))
    hh0 = rng.uniform(-1, 1, (1, d))
    hW = rng.uniform(-1, 1, (word + d, 4 * d)) / np.sqrt(word + d)
    X, h0, WLSTM = cnp.array(hX), cnp.array(hh0), cnp.array(hW)
    xphpb = word + d
    Hin = cnp.zeros((n, b, xphpb))
    Hout = cnp.zeros((n, b, d))
    IFOG = cnp.zeros((n, b, d * 4))
    IFOGf = cnp.zeros((n, b, d * 4))
    Cs = cnp.zeros((n, b, d))
    Ct = cnp.zeros((n, b, d))
    for t in range(n):
        prev = cnp.tile(h0, (b, 1)) if t == 0 else Hout[t - 1]
        Hin[t, :, :word] = X[t]
        Hin[t, :, word:] = prev
        IFOG[t] = Hin[t].dot(WLSTM)
        IFOGf[t, :, : 3 * d] = 1.0 / (1.0 + cnp.exp(-IFOG[t, :, : 3 * d]))
        IFOGf[t, :, 3 * d:] = cnp.tanh(IFOG[t, :, 3 * d:])
        Cs[t] = IFOGf[t, :, :d] * IFOGf[t, :, 3 * d:]
        if t > 0:
            Cs[t] += IFOGf[t, :, d: 2 * d] * Cs[t - 1]
        Ct[t] = cnp.tanh(Cs[t])
        Hout[t] = IFOGf[t, :, 2 * d: 3 * d] * Ct[t]
    wH, wC, wI = _lstm_numpy(hX, hh0, hW, n, b, d, word)
    gI = IFOG.get(itf)
    bound = 1e-12 * (np.abs(np.concatenate([hX[0], np.tile(hh0, (b, 1))], axis=1)) @ np.abs(hW))
    assert np.all(np.abs(gI[0] - wI[0]) <= bound)
    assert np.allclose(Cs.get(itf), wC, rtol=1e-11, atol=1e-13)
    assert np.allclose(Hout.get(itf), wH, rtol=1e-11, atol=1e-13)


def test_pipelined_executor_gives_the_same_results(small_tiles):
    """Asynchronous mode: messages queue up for the executor's own thread while Python records;
    reads wait for the queue. Same statements, same bits."""
    itf = small_tiles
    itf.set_pipeline(True)
    cnp.set_auto_flush(itf, 8)
    n = 70
    rng = np.random.default_rng(12)
    host = rng.standard_normal((n, n))
    u = cnp.array(host)
    w = cnp.array(rng.standard_normal((n,)))
    x = cnp.ones((n,))
    for _ in range(12):
        u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
        host[1:-1, 1:-1] = 0.25 * (host[:-2, 1:-1] + host[2:, 1:-1] + host[1:-1, :-2] + host[1:-1, 2:])
        x = x + 0.5 * w
    assert np.array_equal(u.get(itf), host)
    y = (u @ x).get(itf)
    hx = np.ones(n)
    for _ in range(12):
        hx = hx + 0.5 * w.get(itf)
    assert np.array_equal(x.get(itf), hx)
    assert np.all(np.abs(y - host @ hx) <= 1e-12 * (np.abs(host) @ np.abs(hx)))
    # an executor error is reported by the next call, and the interface works afterwards
    itf.send_dag(99, b"not a dag message")
    with pytest.raises(RuntimeError):
        itf.sync()
    assert np.array_equal(x.get(itf), hx)


def test_tile_matches_numpy(small_tiles, rank3_layout):
    host = np.arange(12, dtype=np.float64).reshape(3, 4)
    a = cnp.array(host)
    for reps in [(2, 3), (1, 1), 2, (2, 1, 2), (5, 1)]:
        assert np.array_equal(cnp.tile(a, reps).get(small_tiles), np.tile(host, reps))
    row = cnp.array(np.arange(7, dtype=np.float64).reshape(1, 7))
    assert np.array_equal(cnp.tile(row, (40, 1)).get(small_tiles), np.tile(np.arange(7.0).reshape(1, 7), (40, 1)))
    v = cnp.arange(5, dtype=np.float64)
    assert np.array_equal(cnp.tile(v, (3, 2)).get(small_tiles), np.tile(np.arange(5.0), (3, 2)))


def test_disjoint_self_reference_updates_in_place(itf):
    """C[t] = f(C[t-1]) reads and writes disjoint slabs of one array: no second buffer is needed,
    and the values are those of the sequential program."""
    n, b, d = 5, 8, 16
    host = np.random.default_rng(1).standard_normal((n, b, d))
    Cs = cnp.array(host)
    itf.set_trace()
    for t in range(1, n):
        Cs[t] = Cs[t] * 0.5 + Cs[t - 1]
        host[t] = host[t] * 0.5 + host[t - 1]
    got = Cs.get(itf)
    assert np.array_equal(got, host)
    groups = [ln for ln in itf.trace() if ln.startswith("group")]
    # merged into runs of statements (one launch, the chained slab handed on in registers) or run
    # one by one in place; never through a second buffer
    assert all("inplace" in g or "path=statements" in g for g in groups)
    counted = sum(int(g.split("count=")[1].split()[0]) if "count=" in g else 1 for g in groups)
    assert counted == n - 1


@pytest.mark.parametrize("fusion", [True, False], ids=["merged", "one-by-one"])
def test_statement_runs_give_what_the_statements_give_one_by_one(itf, fusion, rank3_layout):
    """Runs of same-extent assignments (merged into one launch by default) against NumPy executing
    the same statements in order: register forwarding through an assigned box, a store dropped
    because a later statement assigns the same box, other slabs of the assigned array, lower-rank
    values into slabs, and the hazards that must end a run."""
    itf.set_fusion(fusion)
    rng = np.random.default_rng(8)
    n, b, d = 5, 12, 20
    hA, hC, hH = rng.standard_normal((n, b, 2 * d)), rng.standard_normal((n, b, d)), rng.standard_normal((n, b, d))
    hW = rng.standard_normal((d, 2 * d))
    hM = rng.standard_normal((b, d))
    A, C, H, W, M = (cnp.array(x) for x in (hA, hC, hH, hW, hM))
    for t in range(1, n):
        A[t] = H[t - 1].dot(W)
        hA[t] = hH[t - 1] @ hW
        C[t] = A[t, :, :d] * A[t, :, d:]
        hC[t] = hA[t, :, :d] * hA[t, :, d:]
        C[t] += A[t, :, :d] * C[t - 1]
        hC[t] += hA[t, :, :d] * hC[t - 1]
        H[t] = cnp.tanh(C[t]) * 0.25
        hH[t] = np.tanh(hC[t]) * 0.25
        H[t - 1] = M * 0.5                    # assigns a slab an earlier statement of the run read
        hH[t - 1] = hM * 0.5
    assert np.allclose(A.get(itf), hA, rtol=1e-12, atol=1e-12)
    assert np.allclose(C.get(itf), hC, rtol=1e-12, atol=1e-12)
    assert np.allclose(H.get(itf), hH, rtol=1e-12, atol=1e-12)
    # chains through one array, bit for bit
    hx = rng.standard_normal((40, 6))
    x = cnp.array(hx)
    for t in range(1, 40):
        x[t] = x[t - 1] * 0.5 + x[t]
        hx[t] = hx[t - 1] * 0.5 + hx[t]
    assert np.array_equal(x.get(itf), hx)
    # hazards: shifted read of what the previous statement assigned, and assigning over what it read
    hu, hv = rng.standard_normal(64), rng.standard_normal(64)
    u, v = cnp.array(hu), cnp.array(hv)
    v[0:32] = u[1:33] * 2.0
    hv[0:32] = hu[1:33] * 2.0
    u[2:34] = v[2:34] + 1.0
    hu[2:34] = hv[2:34] + 1.0
    v[4:36] = u[3:35] - v[4:36]
    hv[4:36] = hu[3:35] - hv[4:36]
    u[4:36] = u[4:36] * v[4:36]
    hu[4:36] = hu[4:36] * hv[4:36]
    assert np.array_equal(u.get(itf), hu) and np.array_equal(v.get(itf), hv)


@pytest.mark.parametrize("fusion", [True, False], ids=["merged", "one-by-one"])
def test_wider_assignments_are_cut_to_join_their_run(itf, fusion, rank3_layout):
    """An assignment two to four times as wide as the statements next to it is cut into pieces that
    join their run: the wide one first (an LSTM step's sigmoid over three gates' columns), the wide
    one last, its pieces read from registers by later statements, and one that updates its own
    box. Only + - * here, so NumPy running the statements in order gives the same bits."""
    itf.set_fusion(fusion)
    rng = np.random.default_rng(21)
    n, b, d = 4, 12, 10
    hI, hF = rng.standard_normal((n, b, 4 * d)), np.zeros((n, b, 4 * d))
    hC, hH = rng.standard_normal((n, b, d)), np.zeros((n, b, d))
    hP = rng.standard_normal((n, b, 2 * d))
    I, F, C, H, P = (cnp.array(x) for x in (hI, hF, hC, hH, hP))
    itf.set_trace()
    for t in range(n):
        F[t, :, : 3 * d] = I[t, :, : 3 * d] * 0.5 - 1.0             # three times as wide, first
        hF[t, :, : 3 * d] = hI[t, :, : 3 * d] * 0.5 - 1.0
        F[t, :, 3 * d:] = I[t, :, 3 * d:] * I[t, :, 3 * d:]
        hF[t, :, 3 * d:] = hI[t, :, 3 * d:] * hI[t, :, 3 * d:]
        C[t] = F[t, :, :d] * F[t, :, 3 * d:] + F[t, :, d: 2 * d] * C[t]
        hC[t] = hF[t, :, :d] * hF[t, :, 3 * d:] + hF[t, :, d: 2 * d] * hC[t]
        H[t] = F[t, :, 2 * d: 3 * d] * C[t]
        hH[t] = hF[t, :, 2 * d: 3 * d] * hC[t]
        P[t] = P[t] * 0.25 + F[t, :, d: 3 * d]                       # twice as wide, last, in place
        hP[t] = hP[t] * 0.25 + hF[t, :, d: 3 * d]
    for dev, host in ((F, hF), (C, hC), (H, hH), (P, hP)):
        assert np.array_equal(dev.get(itf), host)
    runs = [ln for ln in itf.trace() if ln.startswith("group") and "path=statements" in ln]
    if fusion and runs:      # (layouts chosen by the decomposition solver may leave nothing to merge)
        # per step one launch: 3 pieces + 3 statements + 2 pieces
        assert any("count=8" in ln for ln in runs), runs


@pytest.mark.parametrize("m", [2, 3, 4, 5])
@pytest.mark.parametrize("along", [0, 1])
def test_cut_assignments_along_either_dimension(itf, m, along):
    """A whole-window assignment m times as long as the statements that follow along rows or along
    columns (m = 5 is beyond what is cut and runs on its own); the pieces are read back from
    registers by the statements on the m blocks, one of which updates its block in place."""
    rng = np.random.default_rng(10 * m + along)
    b, d = 6, 8
    shape = (m * b, d) if along == 0 else (b, m * d)
    hS, hA = rng.standard_normal(shape), np.zeros(shape)
    hR = [rng.standard_normal((b, d)) for _ in range(m)]
    S, A = cnp.array(hS), cnp.array(hA)
    R = [cnp.array(x) for x in hR]
    block = (lambda k: (slice(k * b, (k + 1) * b), slice(None))) if along == 0 else \
            (lambda k: (slice(None), slice(k * d, (k + 1) * d)))
    for rounds in range(3):
        A[:, :] = S * 0.5 - A                      # m blocks wide
        hA[:, :] = hS * 0.5 - hA
        for k in range(m):
            R[k][:, :] = R[k] * 0.25 + A[block(k)]
            hR[k][:, :] = hR[k] * 0.25 + hA[block(k)]
        A[block(m - 1)] = A[block(m - 1)] * R[0]   # a block of the wide target, in place
        hA[block(m - 1)] = hA[block(m - 1)] * hR[0]
    assert np.array_equal(A.get(itf), hA)
    for k in range(m):
        assert np.array_equal(R[k].get(itf), hR[k])


@pytest.mark.parametrize("fusion", [True, False], ids=["fused", "node-by-node"])
@pytest.mark.parametrize("shape", [(100000,), (300, 70), (20, 30, 40)])
def test_reductions_fused_into_their_producer(itf, small_tiles, fusion, shape):
    """z = f(x, y) followed by reductions of z: one launch with reducing roots by default. The
    stored array is the same bit for bit either way; sums agree with NumPy to summation order and
    the maximum exactly."""
    itf.set_fusion(fusion)
    rng = np.random.default_rng(len(shape))
    hx, hy = rng.standard_normal(shape), rng.standard_normal(shape)
    x, y = cnp.array(hx), cnp.array(hy)
    x.get(itf)
    itf.set_trace()
    z = 2.5 * x - 0.5 * y + x * y
    hz = 2.5 * hx - 0.5 * hy + hx * hy
    total = cnp.sum(z)
    ssd = cnp.sumsq_diff(z, y)
    top = cnp.maxabs_diff(x, z)
    dot = z @ x if len(shape) == 1 else None
    assert np.array_equal(z.get(itf), hz)
    close = lambda got, terms: abs(got - terms.sum()) <= 1e-13 * np.abs(terms).sum()
    assert close(total.get(itf).item(), hz)
    assert close(ssd.get(itf).item(), (hz - hy) ** 2)
    assert top.get(itf).item() == np.max(np.abs(hx - hz))
    if dot is not None:
        assert close(dot.get(itf).item(), hz * hx)
    fused = [ln for ln in itf.trace() if "path=dense+reduce" in ln]
    # with decomposition planning forced on (CHARMNUMERIC_SOLVER=1) nodes run one by one
    planning = os.environ.get("CHARMNUMERIC_SOLVER", "0") not in ("", "0")
    assert len(fused) == (1 if fusion and not planning else 0)


def test_slices_of_another_rank_are_assigned_through_a_copy(itf):
    """`A[2] = u[0:16]` (a slice of a 1-D array into a row of a matrix) and a column slice into a
    vector: the slice is copied out, then assigned like a whole array of that rank."""
    rng = np.random.default_rng(12)
    hA, hu, hB = rng.standard_normal((6, 16)), rng.standard_normal(40), rng.standard_normal((16, 5))
    A, u, B = cnp.array(hA), cnp.array(hu), cnp.array(hB)
    A[2] = u[3:19]
    hA[2] = hu[3:19]
    v = cnp.zeros(16)
    hv = np.zeros(16)
    v[:] = B[:, 1:2]
    hv[:] = hB[:, 1]
    A[4, 2:10] = u[30:38] * 2.0
    hA[4, 2:10] = hu[30:38] * 2.0
    assert np.array_equal(A.get(itf), hA) and np.array_equal(v.get(itf), hv)


def test_code_objects_from_the_disk_cache_run(tmp_path):
    """A second process loads the code objects the first one compiled (CHARMNUMERIC_KERNEL_CACHE)
    and computes the same bits with them."""
    import subprocess
    import sys

    prog = (
        "import numpy as np\n"
        "import charmnumeric_amd as cnp\n"
        "from charmnumeric_amd import _lib as L\n"
        "itf = cnp.CharmNumericInterface(device=0); itf.connect(odf=4)\n"
        "h = np.arange(4096.0).reshape(64, 64) / 7.0\n"
        "u = cnp.array(h)\n"
        "u[1:-1, 1:-1] = 0.3 * (u[:-2, 1:-1] + u[2:, 1:-1]) + cnp.tanh(u[1:-1, :-2] * 0.01)\n"
        "s = (u @ cnp.ones((64,))).get(itf)\n"
        "print(L.lib.cnh_code_objects(), L.lib.cnh_code_objects_from_disk(), s.tobytes().hex())\n"
        "itf.close()\n"
    )
    env = dict(os.environ, CHARMNUMERIC_KERNEL_CACHE=str(tmp_path), PYTHONPATH=os.getcwd())
    run = lambda: subprocess.run([sys.executable, "-c", prog], env=env, capture_output=True, text=True,
                                 check=True, timeout=150).stdout.split()
    first, second = run(), run()
    assert int(first[0]) >= 1 and first[1] == "0"
    assert second[0] == first[0] and second[1] == first[0]       # every code object came from disk
    assert second[2] == first[2]


# ---- dense statements, scalar statements and reductions as one launch; partial sums that wait ----

@pytest.mark.parametrize("fusion", [True, False], ids=["merged", "node-by-node"])
@pytest.mark.parametrize("shape", [(300,), (2000,), (5000,), (40, 50), (12, 20, 30)])
def test_vector_updates_with_the_scalars_between_them(itf, fusion, shape, rank3_layout):
    """alpha = s / t; x2 = x + alpha p; r2 = r - alpha q; rr = sum-type reductions of r2; beta = rr / s;
    p2 = r2 + beta p: element-wise results and the scalars formed from stored values are NumPy's bit
    for bit whichever way the nodes are launched; values that depend on a reduction agree to the
    order of summation."""
    itf.set_fusion(fusion)
    rng = np.random.default_rng(sum(shape))
    hx, hp, hq, hr = (rng.standard_normal(shape) for _ in range(4))
    x, p, q, r = cnp.array(hx), cnp.array(hp), cnp.array(hq), cnp.array(hr)
    s, t = cnp.array(np.array([1.75])), cnp.array(np.array([-0.6]))
    x.get(itf)
    itf.set_trace()
    alpha = s / t
    x2 = x + alpha * p
    r2 = r - alpha * q
    rr = cnp.sum(r2 * r2) if len(shape) > 1 else r2 @ r2
    top = cnp.maxabs_diff(r2, r)
    beta = rr / s
    p2 = r2 + beta * p
    gamma = beta * alpha + 1.0
    ha = np.float64(1.75) / np.float64(-0.6)
    assert alpha.get(itf).item() == ha
    assert np.array_equal(x2.get(itf), hx + ha * hp)
    hr2 = hr - ha * hq
    assert np.array_equal(r2.get(itf), hr2)
    assert top.get(itf).item() == np.max(np.abs(hr2 - hr))
    grr = rr.get(itf).item()
    assert abs(grr - np.sum(hr2 * hr2)) <= 1e-13 * np.sum(hr2 * hr2)
    gb = beta.get(itf).item()
    assert gb == grr / 1.75                                   # from the stored sum: one IEEE division
    assert np.array_equal(p2.get(itf), hr2 + gb * hp)
    assert gamma.get(itf).item() == gb * ha + 1.0
    runs = [ln for ln in itf.trace() if "path=run" in ln]
    planning = os.environ.get("CHARMNUMERIC_SOLVER", "0") not in ("", "0")
    if fusion and not planning:
        assert len(runs) == 2 and "scalars_formed=1" in runs[0] and "scalars_formed=2" in runs[1]
        if len(shape) == 1:
            assert "statements=3 scalars_formed=1 reductions=2" in runs[0]
            assert ("sums_taken=1" in runs[1]) == (int(np.prod(shape)) > 512)
    if not fusion:
        assert not runs


def test_a_pending_sum_is_folded_for_whoever_else_reads_it(itf):
    """r.r left as partial sums by the launch that made r: read back, used by a statement on a
    slice, used as an operand of a product-free reduction. Same values as node by node."""
    n = 3000
    rng = np.random.default_rng(4)
    hr, hq = rng.standard_normal(n), rng.standard_normal(n)

    def program():
        r, q = cnp.array(hr), cnp.array(hq)
        r2 = r - 0.5 * q
        w = r2 * 2.0
        rr = r2 @ r2
        y = cnp.zeros((8,))
        y[0:3] = q[0:3] * rr                   # a statement run reads it as a kernel scalar
        z = w + rr                             # a dense statement reads it: folded on the way in
        return rr.get(itf).item(), y.get(itf), z.get(itf)

    itf.set_fusion(True)
    itf.set_trace()
    a = program()
    tr = itf.trace()
    # with decomposition planning forced on (CHARMNUMERIC_SOLVER=1) nodes run one by one
    if os.environ.get("CHARMNUMERIC_SOLVER", "0") in ("", "0"):
        assert any("path=run" in ln and "reductions=1" in ln for ln in tr)
        assert any(ln.startswith("fold") and "partials=6" in ln for ln in tr)
    itf.set_fusion(False)
    b = program()
    hr2 = hr - 0.5 * hq
    assert abs(a[0] - np.sum(hr2 * hr2)) <= 1e-13 * np.sum(hr2 * hr2)
    assert abs(a[0] - b[0]) <= 1e-13 * abs(b[0])
    for got in (a, b):
        want_y = np.zeros(8)
        want_y[0:3] = hq[0:3] * got[0]
        assert np.array_equal(got[1], want_y)
        assert np.array_equal(got[2], hr2 * 2.0 + got[0])


def test_cg_on_a_small_system_with_merged_launches(small_tiles):
    """The CG example with vectors longer than a workgroup's share (sums pending between launches):
    converges to the closed-form solution as the node-by-node run does."""
    itf = small_tiles
    itf.set_min_tile(1, 4096)
    n = 1200
    A = cnp.ones((n, n), dtype=cnp.float64)
    for i in range(n):
        A[i, i] = n + 1.0
    b = cnp.arange(1, n + 1, dtype=cnp.float64)
    x = cnp.zeros((n,), dtype=cnp.float64)
    r = b.copy()
    p = b.copy()
    rtr = r @ r
    history = []
    for k in range(3):
        Ap = A @ p
        pAp = p @ Ap
        alpha = rtr / pAp
        x = x + alpha * p
        r = r - alpha * Ap
        rtr_new = r @ r
        beta = rtr_new / rtr
        p = r + beta * p
        rtr = rtr_new
        if k == 1:
            history.append(rtr.get(itf).item())
    bn = np.arange(1, n + 1, dtype=np.float64)
    want = (bn - bn.sum() / (2 * n)) / n
    assert np.allclose(x.get(itf), want, rtol=1e-10, atol=0)
    assert history[0] < 1e-12 * float(bn @ bn)


# ---- a product and the statements that read it ----

def _product_program(xp, A, B, C, out1, out2, blocks, variant):
    """C[...] = A @ B and statements on C's column blocks; `variant` picks what makes the executor
    keep the product and the statements apart (or nothing)."""
    n = C.shape[1] // blocks
    C[:, :] = A @ B
    if variant == "blocks":
        out1[:, :] = C[:, :n] * 2.0 + out2[:, :]
        if blocks > 1:
            out2[:, :] = C[:, (blocks - 1) * n:] - C[:, :n]
    elif variant == "assigns-left-operand":
        out1[:, :] = C[:, :n] * 2.0
        A[:, :n] = C[:, :n] * 0.5
    elif variant == "off-block-read":
        out1[:, :] = C[:, 8:8 + n] * 2.0
        out2[:, :] = C[:, :n] + 1.0
    elif variant == "assigns-into-product":
        out1[:, :] = C[:, :n] * 2.0
        C[:, :n] = out1[:, :] + 1.0


@pytest.mark.parametrize("blocks", [1, 2, 4])
@pytest.mark.parametrize("variant", ["blocks", "assigns-left-operand", "off-block-read", "assigns-into-product"])
def test_statements_behind_a_product(itf, blocks, variant):
    """Statements that read a product's box block by block ride on the product's launch; a statement
    that assigns where the product reads or writes, or reads the box across blocks, keeps it a launch
    of its own (the trace says why). NumPy runs the same statements; products agree to 1e-12 of
    sum |a||b|, everything else follows from them."""
    if variant == "off-block-read" and blocks == 1:
        pytest.skip("a single block has no other offset of its width")
    M, K, N = 128, 256, 256
    n = N // blocks
    rng = np.random.default_rng(50 + blocks)
    hA, hB = rng.uniform(-1, 1, (M, K)), rng.uniform(-1, 1, (K, N))
    h1, h2 = np.zeros((M, n)), rng.uniform(-1, 1, (M, n))
    hC = np.zeros((M, N))
    itf.set_trace()
    A, B, C, o1, o2 = cnp.array(hA), cnp.array(hB), cnp.zeros((M, N)), cnp.zeros((M, n)), cnp.array(h2)
    _product_program(cnp, A, B, C, o1, o2, blocks, variant)
    _product_program(np, hA, hB, hC, h1, h2, blocks, variant)
    tol = 1e-12 * K
    for name, dev, host in (("C", C, hC), ("out1", o1, h1), ("out2", o2, h2), ("A", A, hA)):
        assert np.allclose(dev.get(itf), host, rtol=0, atol=4 * tol), name
    if os.environ.get("CHARMNUMERIC_SOLVER", "0") in ("", "0"):
        trace = itf.trace()
        taken = sum(" with_statements" in ln for ln in trace)
        refused = [ln for ln in trace if "statements_not_taken" in ln]
        if variant == "blocks":
            assert taken == 1 and not refused, trace
        else:
            assert taken == 0 and len(refused) == 1, trace
