"""Pins the oracle's numerics (CPU only): fused groups vs NumPy in the same operand order,
fill/copy vs NumPy slicing, dot/matvec/matmatmul closed forms from the upstream examples, the
generator vs an independent NumPy restatement."""
import ctypes as C
import math

import numpy as np
import pytest

from charmnumeric_amd import _lib as L
from charmnumeric_amd.astbuild import AstBuilder
from oracle import cn_oracle as O
from tests import helpers as H


def test_generator_matches_numpy_restatement(orc):
    for seed, stream, first in [(0, 0, 0), (0, 1, 0), (1, 0, 12345), (5, 2, 1 << 40)]:
        got = orc.uniform(1000, seed, stream, -1.0, 1.0, first=first)
        assert np.array_equal(got, H.np_uniform(1000, seed, stream, -1.0, 1.0, first=first))
    u = orc.uniform(100000, 3, 0, 0.0, 1.0)
    assert u.min() >= 0.0 and u.max() < 1.0 and abs(u.mean() - 0.5) < 0.01
    # the CG matrix: symmetric, diagonal 2.0, off-diagonal in [0, 1/n), blocks agree with the whole
    n = 96
    A = orc.cg_matrix(n, 0, n, 0, n, 2)
    assert np.array_equal(A, A.T) and np.all(np.diag(A) == 2.0)
    off = A[~np.eye(n, dtype=bool)]
    assert off.min() >= 0.0 and off.max() < 1.0 / n
    assert np.array_equal(orc.cg_matrix(n, 32, 40, 8, 50, 2), A[32:72, 8:58])
    i, j = 5, 77
    want = (H.np_u01(2, 0, [i * n + j])[0] + H.np_u01(2, 0, [j * n + i])[0]) / (2.0 * n)
    assert A[i, j] == want
    assert np.all(np.linalg.eigvalsh(A) > 0)  # diagonally dominant, hence SPD


def test_c1_group_is_numpy_in_ast_order(orc):
    x = orc.uniform(10007, 0, 0, -1, 1)
    y = orc.uniform(10007, 0, 1, -1, 1)
    ast = H.ast_c1(L.F64)
    out = np.empty_like(x)
    assert orc.eval_group(ast, L.F64, 1, [x, y, x, y], [], [out]) == 0
    assert np.array_equal(out, ((2.5 * x) - (0.5 * y)) + (x * y))
    # an FMA-contracted or re-associated evaluation differs in some elements
    fused = np.array([math.fsum([2.5 * a, -0.5 * b, a * b]) for a, b in zip(x[:2000], y[:2000])])
    assert not np.array_equal(out[:2000], fused)
    # float32: scalars are cast to the element type first
    xf, yf = x.astype(np.float32), y.astype(np.float32)
    outf = np.empty_like(xf)
    assert orc.eval_group(H.ast_c1(L.F32), L.F32, 1, [xf, yf, xf, yf], [], [outf]) == 0
    want = ((np.float32(2.5) * xf) - (np.float32(0.5) * yf)) + (xf * yf)
    assert np.array_equal(outf, want)


@pytest.mark.parametrize("dt,npdt", [(L.I32, np.int32), (L.I64, np.int64)])
def test_integer_groups_wrap_and_truncate(orc, dt, npdt):
    rng = np.random.default_rng(0)
    info = np.iinfo(npdt)
    a = rng.integers(info.min, info.max, 5000, dtype=npdt)
    b = rng.integers(-1000, 1000, 5000).astype(npdt)
    b[b == 0] = 7
    bld = AstBuilder(dt, 1)
    la, lb = bld.leaf(0), bld.leaf(1)
    t1 = bld.binary(L.OP_MUL, 100, la, lb)
    t2 = bld.binary(L.OP_ADD, 101, t1, bld.scalar(3.9))   # scalar cast through int64: 3
    bld.binary(L.OP_DIV, 2, t2, lb, is_temp=False)
    out = np.empty_like(a)
    assert orc.eval_group(bld.finish(), dt, 1, [a, b, b], [], [out]) == 0  # one memref per leaf use
    with np.errstate(over="ignore"):
        t = a * b + npdt(3)
    want = np.trunc(t.astype(np.float64) / b.astype(np.float64)) if npdt == np.int32 else None
    # exact reference with Python integers: two's-complement wrap, division truncating toward zero
    bits = info.bits

    def wrap(v):
        v &= (1 << bits) - 1
        return v - (1 << bits) if v >> (bits - 1) else v

    exact = []
    for ai, bi in zip(a.tolist(), b.tolist()):
        tt = wrap(wrap(ai * bi) + 3)
        q = abs(tt) // abs(bi)
        exact.append(wrap(q if (tt >= 0) == (bi > 0) else -q))
    assert out.tolist() == exact
    if want is not None:
        assert np.array_equal(out, want.astype(npdt))


def test_uncompilable_groups_are_refused(orc):
    bld = AstBuilder(L.I32, 1)
    bld.unary(L.OP_TANH, 2, bld.leaf(0), is_temp=False)
    a = np.zeros(4, np.int32)
    assert orc.eval_group(bld.finish(), L.I32, 1, [a], [], [a.copy()]) < 0


def test_exp_tanh_are_host_libm(orc):
    xs = np.linspace(-30, 30, 20001)
    for opc, fn in ((L.OP_EXP, math.exp), (L.OP_TANH, math.tanh)):
        bld = AstBuilder(L.F64, 1)
        bld.unary(opc, 2, bld.leaf(0), is_temp=False)
        out = np.empty_like(xs)
        assert orc.eval_group(bld.finish(), L.F64, 1, [xs], [], [out]) == 0
        assert np.array_equal(out, np.array([fn(v) for v in xs]))  # CPython calls the same libm


def test_strided_memrefs_and_set_region_root(orc):
    """Stencil group on strided views == NumPy slicing; the SET_REGION root yields the value."""
    n = 40
    u = orc.uniform(n * n, 3, 0, 0, 1).reshape(n, n)
    ast = H.ast_jacobi2d(n)
    out = np.zeros((n - 2, n - 2))
    ins = [u[:-2, 1:-1], u[2:, 1:-1], u[1:-1, :-2], u[1:-1, 2:]]
    assert orc.eval_group(ast, L.F64, 2, ins, [], [out]) == 0
    assert np.array_equal(out, H.np_jacobi2d(u)[1:-1, 1:-1])
    n3 = 12
    v = orc.uniform(n3 ** 3, 3, 1, 0, 1).reshape(n3, n3, n3)
    ins = [v[:-2, 1:-1, 1:-1], v[2:, 1:-1, 1:-1], v[1:-1, :-2, 1:-1], v[1:-1, 2:, 1:-1],
           v[1:-1, 1:-1, :-2], v[1:-1, 1:-1, 2:]]
    out = np.zeros((n3 - 2,) * 3)
    assert orc.eval_group(H.ast_jacobi3d(n3), L.F64, 3, ins, [], [out]) == 0
    assert np.array_equal(out, H.np_jacobi3d(v)[1:-1, 1:-1, 1:-1])


def test_reference_known_answers(orc):
    # 2*(a+b+3) = 8 in f32 (upstream tests/test_backend_integration.py:13-23)
    b = AstBuilder(L.F32, 1)
    t1 = b.binary(L.OP_ADD, 100, b.leaf(0), b.leaf(1))
    t2 = b.binary(L.OP_ADD, 101, t1, b.scalar(3.0))
    b.binary(L.OP_MUL, 2, b.scalar(2.0), t2, is_temp=False)
    out = np.zeros(32, np.float32)
    assert orc.eval_group(b.finish(), L.F32, 1, [np.full(32, 1.5, np.float32),
                                                  np.full(32, -0.5, np.float32)], [], [out]) == 0
    assert np.all(out == 8.0)
    # 4^3 grid with faces 1.0: every interior point becomes (1/6)*3 = 0.5 (:68-105)
    u = np.zeros((4, 4, 4))
    u[0], u[-1], u[:, 0], u[:, -1], u[:, :, 0], u[:, :, -1] = 1, 1, 1, 1, 1, 1
    ins = [u[:-2, 1:-1, 1:-1], u[2:, 1:-1, 1:-1], u[1:-1, :-2, 1:-1], u[1:-1, 2:, 1:-1],
           u[1:-1, 1:-1, :-2], u[1:-1, 1:-1, 2:]]
    out = np.zeros((2, 2, 2))
    assert orc.eval_group(H.ast_jacobi3d(4, coef=1.0 / 6.0), L.F64, 3, ins, [], [out]) == 0
    assert np.allclose(out, 0.5, rtol=0, atol=1e-15)


def test_fill_and_copy_region_are_numpy_slicing(orc):
    lib = orc.lib
    rng = np.random.default_rng(2)
    fine = rng.standard_normal((17, 17))
    coarse = np.zeros((9, 9))
    keep = []

    def i64(v):
        arr = L.i64arr(v)
        keep.append(arr)  # ctypes arrays must outlive the call that receives their address
        return C.addressof(arr)

    lib.orc_copy_region(2, 8, O.ptr(coarse), i64([9, 1]), i64([1, 1]), i64([1, 1]), O.ptr(fine),
                        i64([17, 1]), i64([2, 2]), i64([2, 2]), i64([7, 7]))
    want = np.zeros((9, 9))
    want[1:-1, 1:-1] = fine[2:-2:2, 2:-2:2]    # upstream strided-assignment test, n = 17
    assert np.array_equal(coarse, want)
    a = np.zeros((6, 7, 30), np.int32)
    five = np.array([5], np.int32)
    lib.orc_fill_region(3, 4, O.ptr(a), i64([210, 30, 1]), i64([1, 0, 3]), i64([2, 3, 1]),
                        i64([3, 3, 20]), O.ptr(five))
    want = np.zeros((6, 7, 30), np.int32)
    want[1:6:2, 0:7:3, 3:23] = 5
    assert np.array_equal(a, want)
    buf = np.zeros(1, np.int64)
    lib.orc_scalar_to_dtype(L.I32, -3.9, O.ptr(buf))
    assert buf.view(np.int32)[0] == -3


def test_dot_gemv_gemm_closed_forms(orc):
    # ones . ones = N (upstream examples/reduction.py)
    assert orc.dot(np.ones(64, np.float32), np.ones(64, np.float32)) == 64.0
    # A[i,j] = i + j, x = 1 -> y_i = N*i + N(N-1)/2 exactly (upstream examples/matvec.py)
    n = 128
    A = np.add.outer(np.arange(n, dtype=np.float64), np.arange(n, dtype=np.float64))
    assert np.array_equal(orc.gemv(A, np.ones(n)), n * np.arange(n) + n * (n - 1) / 2)
    # ones(M,N) @ arange(1..N) = N(N+1)/2 (upstream examples/matvec_slice.py)
    assert np.array_equal(orc.gemv(np.ones((7, 100)), np.arange(1, 101, dtype=np.float64)),
                          np.full(7, 5050.0))
    # ones(M,K) @ ones(K,N) = K exactly (upstream examples/matmatmul.py)
    Cm = orc.gemm_acc(np.ones((9, 40)), np.ones((40, 13)), np.zeros((9, 13)))
    assert np.all(Cm == 40.0)
    # brute force on tiny inputs + long-double reference; accumulation on top of C
    rng = np.random.default_rng(3)
    A, B, C0 = rng.standard_normal((5, 7)), rng.standard_normal((7, 4)), rng.standard_normal((5, 4))
    got = orc.gemm_acc(A, B, C0.copy(), threads=3)
    brute = C0.copy()
    for i in range(5):
        for j in range(4):
            for k in range(7):
                brute[i, j] += A[i, k] * B[k, j]
    assert np.array_equal(got, brute)
    # dot: left-to-right order, and within 1e-12 of the exact sum relative to sum |terms|
    a, b = orc.uniform(100000, 0, 0, -1, 1), orc.uniform(100000, 0, 1, -1, 1)
    acc = 0.0
    for p in (a[:1000] * b[:1000]).tolist():
        acc += p
    assert orc.dot(a[:1000], b[:1000]) == acc
    assert abs(orc.dot(a, b) - math.fsum((a * b).tolist())) <= 1e-12 * math.fsum(np.abs(a * b).tolist())
    # sub-matrix view with offsets (eigen_gemv_sub arguments)
    full = rng.standard_normal((10, 12))
    x = rng.standard_normal(5)
    res = np.zeros(4)
    orc.lib.orc_gemv_sub(L.F64, O.ptr(full), 12, 3, 6, 4, 5, O.ptr(x), O.ptr(res))
    assert np.allclose(res, full[3:7, 6:11] @ x, rtol=1e-14, atol=1e-14)
    # reduce_partials: sequential a += b like the upstream reducer
    p = np.array([1e16, 1.0, -1e16, 3.0])
    out = np.zeros(1)
    orc.lib.orc_reduce_partials(L.F64, 4, O.ptr(p), O.ptr(out))
    assert out[0] == ((1e16 + 1.0) + -1e16) + 3.0


def test_cg_closed_form_system(orc):
    """A = N*I + 11^T, b = 1..N  =>  x = (b - sum(b)/(2N))/N (upstream examples/cg.py:14-22,66-73).
    CG in exact arithmetic needs 2 iterations for this 2-eigenvalue matrix."""
    n = 128
    A = np.ones((n, n)) + n * np.eye(n)
    b = np.arange(1, n + 1, dtype=np.float64)
    x = np.zeros(n)
    r, p = b.copy(), b.copy()
    rtr = orc.dot(r, r)
    for _ in range(3):
        Ap = orc.gemv(A, p)
        alpha = rtr / orc.dot(p, Ap)
        x = x + alpha * p
        r = r - alpha * Ap
        rtr_new = orc.dot(r, r)
        p = r + (rtr_new / rtr) * p
        rtr = rtr_new
    want = (b - b.sum() / (2 * n)) / n
    assert np.allclose(x, want, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("dt,npdt", [(L.F32, np.float32), (L.F64, np.float64), (L.I32, np.int32),
                                     (L.I64, np.int64)])
def test_axpy1_is_one_ieee_or_wrapping_add_per_element(orc, dt, npdt):
    """The 1-D accumulate of matvec partials: res[i] += partial[i], nothing else."""
    rng = np.random.default_rng(11)
    n = 4099
    if np.issubdtype(npdt, np.integer):
        info = np.iinfo(npdt)
        res = rng.integers(info.min, info.max, n, dtype=npdt)
        part = rng.integers(info.min, info.max, n, dtype=npdt)
        res[:2], part[:2] = [info.max, info.min], [1, -1]          # wrap both ways
        bits = info.bits
        want = [((int(a) + int(b) + (1 << (bits - 1))) % (1 << bits)) - (1 << (bits - 1))
                for a, b in zip(res, part)]                        # Python big integers
        want = np.array(want, dtype=npdt)
    else:
        res = (rng.standard_normal(n) * 10.0 ** rng.integers(-8, 8, n)).astype(npdt)
        part = (rng.standard_normal(n) * 10.0 ** rng.integers(-8, 8, n)).astype(npdt)
        want = res + part
    untouched = part.copy()
    assert orc.lib.orc_axpy1(dt, n, O.ptr(part), O.ptr(res)) == 0
    assert np.array_equal(res, want) and np.array_equal(part, untouched)
    # n = 0 touches nothing
    before = res.copy()
    assert orc.lib.orc_axpy1(dt, 0, O.ptr(part), O.ptr(res)) == 0 and np.array_equal(res, before)
    assert orc.lib.orc_axpy1(9, 1, O.ptr(part), O.ptr(res)) == -1


def test_threaded_matvec_and_product_are_the_single_thread_bits(orc):
    """Rows are split over threads, a row's sum is not: any thread count gives the same bits, and
    those are within 1e-12 * sum|a||x| of the exactly rounded row dots."""
    rng = np.random.default_rng(12)
    rows, cols, ld = 301, 257, 300
    M = rng.uniform(-1, 1, (rows + 7, ld))
    x = rng.uniform(-1, 1, cols)
    row_off, col_off = 5, 31

    def run(threads):
        y = np.full(rows, np.nan)
        assert orc.lib.orc_gemv_sub_mt(L.F64, O.ptr(M), ld, row_off, col_off, rows, cols, O.ptr(x),
                                       O.ptr(y), threads) == 0
        return y

    one = run(1)
    for threads in (2, 5, 16, 1000):
        assert np.array_equal(run(threads), one)
    sub = M[row_off:row_off + rows, col_off:col_off + cols]
    exact = np.array([math.fsum(sub[i] * x) for i in range(rows)])
    assert np.all(np.abs(one - exact) <= 1e-12 * (np.abs(sub) @ np.abs(x)))
    # left-to-right order, the one the single-thread pins fix
    lr = np.zeros(rows)
    for j in range(cols):
        lr += sub[:, j] * x[j]
    assert np.array_equal(one, lr)
    # products: C += A.B with rows split over threads
    A, B = rng.uniform(-1, 1, (37, 29)), rng.uniform(-1, 1, (29, 23))
    C0 = rng.uniform(-1, 1, (37, 23))
    ref = orc.gemm_acc(A, B, C0.copy(), threads=1)
    for threads in (2, 5, 16):
        assert np.array_equal(orc.gemm_acc(A, B, C0.copy(), threads=threads), ref)
    exact = np.array([[math.fsum([C0[i, j]] + list(A[i] * B[:, j])) for j in range(23)] for i in range(37)])
    assert np.all(np.abs(ref - exact) <= 1e-12 * (np.abs(C0) + np.abs(A) @ np.abs(B)))


def test_sum_and_difference_reductions(orc):
    """sum: one accumulator, index order (floats: Python's left-to-right sum of the same doubles;
    integers wrap). sumsq_diff: sum of (a-b)*(a-b), same order. maxabs_diff: exact, any order."""
    rng = np.random.default_rng(13)
    n = 5003
    a = rng.uniform(-1, 1, n) * 10.0 ** rng.integers(-3, 3, n)
    b = rng.uniform(-1, 1, n)
    out = np.zeros(1)
    assert orc.lib.orc_sum(L.F64, n, O.ptr(a), O.ptr(out)) == 0
    acc = 0.0
    for v in a.tolist():
        acc += v
    assert out[0] == acc and abs(out[0] - math.fsum(a)) <= 1e-12 * np.abs(a).sum()
    af = a.astype(np.float32)
    outf = np.zeros(1, np.float32)
    assert orc.lib.orc_sum(L.F32, n, O.ptr(af), O.ptr(outf)) == 0
    accf = np.float32(0)
    for v in af:
        accf = np.float32(accf + v)
    assert outf[0] == accf
    for dt, npdt in ((L.I32, np.int32), (L.I64, np.int64)):
        info = np.iinfo(npdt)
        v = rng.integers(info.min, info.max, 777, dtype=npdt)
        o = np.zeros(1, npdt)
        assert orc.lib.orc_sum(dt, v.size, O.ptr(v), O.ptr(o)) == 0
        total = sum(int(t) for t in v)
        assert int(o[0]) == ((total + (1 << (info.bits - 1))) % (1 << info.bits)) - (1 << (info.bits - 1))
    # closed forms: arange, ones (examples/reduction.py:3-6 upstream)
    ar = np.arange(1.0, 1001.0)
    assert orc.lib.orc_sum(L.F64, 1000, O.ptr(ar), O.ptr(out)) == 0 and out[0] == 500500.0
    # sum of squared differences
    assert orc.lib.orc_sumsq_diff(n, O.ptr(a), O.ptr(b), O.ptr(out)) == 0
    acc = 0.0
    for p, q in zip(a.tolist(), b.tolist()):
        d = p - q
        acc += d * d
    assert out[0] == acc
    assert abs(out[0] - math.fsum((a - b) ** 2)) <= 1e-12 * ((a - b) ** 2).sum()
    assert orc.lib.orc_sumsq_diff(n, O.ptr(a), O.ptr(a), O.ptr(out)) == 0 and out[0] == 0.0
    # a sign error (a + b) or a missing square would fail these
    three, one = np.full(10, 3.0), np.ones(10)
    assert orc.lib.orc_sumsq_diff(10, O.ptr(three), O.ptr(one), O.ptr(out)) == 0 and out[0] == 40.0
    # largest absolute difference
    assert orc.lib.orc_maxabs_diff(n, O.ptr(a), O.ptr(b), O.ptr(out)) == 0
    assert out[0] == np.abs(a - b).max() == max(abs(p - q) for p, q in zip(a.tolist(), b.tolist()))
    assert orc.lib.orc_maxabs_diff(n, O.ptr(b), O.ptr(a), O.ptr(out)) == 0 and out[0] == np.abs(a - b).max()
    neg = -three
    assert orc.lib.orc_maxabs_diff(10, O.ptr(neg), O.ptr(one), O.ptr(out)) == 0 and out[0] == 4.0
    assert orc.lib.orc_maxabs_diff(0, O.ptr(a), O.ptr(b), O.ptr(out)) == 0 and out[0] == 0.0
