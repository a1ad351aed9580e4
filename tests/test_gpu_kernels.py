"""GPU parity for the non-JIT seams: fill/copy, reductions, matvec, matmatmul, generators."""
import ctypes as C
import math

import numpy as np
import pytest

from charmnumeric_amd import _lib as L
from tests import helpers as H

pytestmark = pytest.mark.gpu

REL = 1e-12  # reductions, matvec and matmatmul: |got - ref| <= 1e-12 * sum |terms|


def test_generators_match_oracle_and_numpy(dev, orc):
    n = 100003
    d = dev.empty((n,), np.float64)
    L.check(L.lib.cnh_fill_uniform(d.ptr, n, 0, 1, 5, -1.0, 1.0, None))
    got = d.get()
    want = orc.uniform(n, 0, 1, -1.0, 1.0, first=5)
    assert np.array_equal(got, want)
    assert np.array_equal(got, H.np_uniform(n, 0, 1, -1.0, 1.0, first=5))
    m = dev.empty((96, 160), np.float64)
    L.check(L.lib.cnh_fill_cg_matrix(m.ptr, 512, 64, 96, 32, 160, 160, 2, None))
    got = m.get()
    want = orc.cg_matrix(512, 64, 96, 32, 160, 2)
    assert np.array_equal(got, want)
    full = orc.cg_matrix(512, 0, 512, 0, 512, 2)
    assert np.array_equal(full, full.T) and np.all(np.diag(full) == 2.0)
    dev.free_all()


@pytest.mark.parametrize("esz,npdt", [(8, np.float64), (4, np.int32)])
def test_fill_and_copy_region_bit_exact(dev, esz, npdt):
    rng = np.random.default_rng(1)
    # strided 17 -> 9 assignment held by the upstream tests: coarse[1:-1,1:-1] = fine[2:-2:2,2:-2:2]
    n, cn = 17, 9
    fine = rng.integers(-99, 99, (n, n)).astype(npdt)
    coarse = np.zeros((cn, cn), npdt)
    dfine, dcoarse = dev.array(fine), dev.array(coarse)
    L.check(L.lib.cnh_copy_region(2, esz, dcoarse.ptr, H.L.i64arr([cn, 1]), H.L.i64arr([1, 1]),
                                  H.L.i64arr([1, 1]), dfine.ptr, H.L.i64arr([n, 1]),
                                  H.L.i64arr([2, 2]), H.L.i64arr([2, 2]), H.L.i64arr([7, 7]), None))
    want = coarse.copy()
    want[1:-1, 1:-1] = fine[2:-2:2, 2:-2:2]
    assert np.array_equal(dcoarse.get(), want)
    # 3-D fill of a strided box
    a = rng.integers(-9, 9, (6, 7, 300)).astype(npdt)
    da = dev.array(a)
    val = np.array([5], dtype=npdt)
    buf8 = np.zeros(8, np.uint8)
    buf8[:esz] = val.view(np.uint8)
    L.check(L.lib.cnh_fill_region(3, esz, da.ptr, H.L.i64arr([2100, 300, 1]), H.L.i64arr([1, 0, 3]),
                                  H.L.i64arr([2, 3, 1]), H.L.i64arr([3, 3, 290]),
                                  buf8.ctypes.data, None))
    want = a.copy()
    want[1:6:2, 0:7:3, 3:293] = 5
    assert np.array_equal(da.get(), want)
    # 1-D halo-style pack
    v = rng.integers(-9, 9, 5000).astype(npdt)
    dv = dev.array(v)
    pk = dev.empty((1200,), npdt)
    L.check(L.lib.cnh_copy_region(1, esz, pk.ptr, H.L.i64arr([1]), H.L.i64arr([0]),
                                  H.L.i64arr([1]), dv.ptr, H.L.i64arr([1]), H.L.i64arr([100]),
                                  H.L.i64arr([4]), H.L.i64arr([1200]), None))
    assert np.array_equal(pk.get(), v[100:4900:4])
    # empty region is a no-op
    L.check(L.lib.cnh_copy_region(1, esz, pk.ptr, H.L.i64arr([1]), H.L.i64arr([0]),
                                  H.L.i64arr([1]), dv.ptr, H.L.i64arr([1]), H.L.i64arr([0]),
                                  H.L.i64arr([1]), H.L.i64arr([0]), None))
    dev.free_all()


def test_convert_region_is_numpy_astype(dev):
    """Every pair of element types, whole and strided: bit-exact against ndarray.astype (round to
    nearest even into floating point, truncation into integers; values kept inside the range of
    every integer type, beyond it C leaves the result open)."""
    rng = np.random.default_rng(5)
    types = ((L.F32, np.float32), (L.F64, np.float64), (L.I32, np.int32), (L.I64, np.int64))
    n = 70001
    for sdt, snp in types:
        if np.issubdtype(snp, np.floating):
            src = (rng.uniform(-2.0e9, 2.0e9, n) * rng.choice([1.0, 1e-3, 1e-9], n)).astype(snp)
            src[:6] = np.array([0.5, -0.5, 1.5, 2.5, -0.0, 16777217.0]).astype(snp)
        else:
            hi = 2**31 - 1 if snp is np.int32 else 2**62
            src = rng.integers(-hi, hi, n).astype(snp)
            src[:4] = np.array([16777217, -16777217, 2**31 - 1, 0]).astype(snp)   # ties of float32
        dsrc = dev.array(src)
        for ddt, dnp in types:
            if np.issubdtype(snp, np.floating) and dnp is np.int32:
                use = np.clip(src, -2.0e9, 2.0e9).astype(snp)
                dsrc.put(use)
            elif snp is np.int64 and dnp is np.int32:
                use = (src >> 33).astype(snp)
                dsrc.put(use)
            else:
                use = src
                dsrc.put(use)
            out = dev.empty((n,), dnp)
            L.check(L.lib.cnh_convert_region(1, ddt, out.ptr, H.L.i64arr([1]), H.L.i64arr([0]), H.L.i64arr([1]),
                                             sdt, dsrc.ptr, H.L.i64arr([1]), H.L.i64arr([0]), H.L.i64arr([1]),
                                             H.L.i64arr([n]), None))
            with np.errstate(all="ignore"):
                want = use.astype(dnp)
            assert out.get().tobytes() == want.tobytes(), (snp, dnp)
    # strided 2-D window into a window of another type
    a = rng.integers(-1000, 1000, (40, 50)).astype(np.int32)
    da = dev.array(a)
    b = np.full((30, 64), -1.0)
    db = dev.array(b)
    L.check(L.lib.cnh_convert_region(2, L.F64, db.ptr, H.L.i64arr([64, 1]), H.L.i64arr([2, 5]), H.L.i64arr([1, 3]),
                                     L.I32, da.ptr, H.L.i64arr([50, 1]), H.L.i64arr([1, 0]), H.L.i64arr([2, 1]),
                                     H.L.i64arr([19, 17]), None))
    b[2:21, 5:56:3] = a[1:39:2, 0:17]
    assert np.array_equal(db.get(), b)
    assert L.lib.cnh_convert_region(1, 7, db.ptr, H.L.i64arr([1]), H.L.i64arr([0]), H.L.i64arr([1]), L.I32, da.ptr,
                                    H.L.i64arr([1]), H.L.i64arr([0]), H.L.i64arr([1]), H.L.i64arr([4]), None) == -2
    dev.free_all()


def test_d2h_region_gathers_tiles(dev):
    g = np.arange(40 * 56, dtype=np.float64).reshape(40, 56)
    out = np.zeros_like(g)
    for i in range(0, 40, 16):
        for j in range(0, 56, 16):
            t = np.ascontiguousarray(g[i:i + 16, j:j + 16])
            dt = dev.array(t)
            L.check(L.lib.cnh_d2h_region(2, 8, out.ctypes.data, H.L.i64arr([56, 1]),
                                         H.L.i64arr([i, j]), dt.ptr, H.L.i64arr([t.shape[1], 1]),
                                         H.L.i64arr([0, 0]), H.L.i64arr(list(t.shape)), None))
    assert np.array_equal(out, g)
    dev.free_all()


def _tiles(dev, arr, parts):
    bounds = np.linspace(0, arr.size, parts + 1).astype(np.int64)
    bufs = [dev.array(arr[bounds[i]:bounds[i + 1]]) for i in range(parts)]
    return bufs, [int(bounds[i + 1] - bounds[i]) for i in range(parts)]


@pytest.mark.parametrize("n,parts", [(1 << 24, 4), (1 << 22, 4), (16384, 1), (100003, 3), (5, 1), (70000, 1)])
def test_dot_and_sum_fp64(dev, orc, n, parts):
    """(2^24, 4) is the elementwise configuration's size: 4 partitions of 4 194 304."""
    a = orc.uniform(n, 0, 0, -1, 1)
    b = orc.uniform(n, 0, 1, -1, 1)
    ab, lens = _tiles(dev, a, parts)
    bb, _ = _tiles(dev, b, parts)
    out = dev.empty((1,), np.float64)
    L.check(L.lib.cnh_dot_tiles(L.F64, parts, L.vparr([x.ptr for x in ab]),
                                L.vparr([x.ptr for x in bb]), L.i64arr(lens), out.ptr, None))
    got = out.get()[0]
    ref = math.fsum((a * b).tolist())
    denom = math.fsum(np.abs(a * b).tolist())
    assert abs(got - ref) <= REL * denom
    assert abs(orc.dot(a, b) - ref) <= REL * denom
    # determinism: same launch twice gives the same bits
    out2 = dev.empty((1,), np.float64)
    L.check(L.lib.cnh_dot_tiles(L.F64, parts, L.vparr([x.ptr for x in ab]),
                                L.vparr([x.ptr for x in bb]), L.i64arr(lens), out2.ptr, None))
    assert out2.get()[0].tobytes() == np.float64(got).tobytes()
    L.check(L.lib.cnh_sum_tiles(L.F64, parts, L.vparr([x.ptr for x in ab]), L.i64arr(lens),
                                out.ptr, None))
    got = out.get()[0]
    assert abs(got - math.fsum(a.tolist())) <= REL * math.fsum(np.abs(a).tolist())
    osum = np.zeros(1)
    assert orc.lib.orc_sum(L.F64, n, a.ctypes.data, osum.ctypes.data) == 0
    assert abs(got - osum[0]) <= 2 * REL * math.fsum(np.abs(a).tolist())
    dev.free_all()


def test_dot_closed_forms_and_ints(dev):
    # ones . ones = N (upstream examples/reduction.py)
    for n in (64, 1 << 20):
        o = dev.array(np.ones(n, np.float32))
        out = dev.empty((1,), np.float32)
        L.check(L.lib.cnh_dot_partial(L.F32, n, o.ptr, o.ptr, out.ptr, None))
        assert out.get()[0] == np.float32(n)
    # integer dot wraps modulo 2^32 / 2^64: bit-exact whatever the order
    rng = np.random.default_rng(0)
    for dt, npdt in ((L.I32, np.int32), (L.I64, np.int64)):
        a = rng.integers(-2**30, 2**30, 300001).astype(npdt)
        b = rng.integers(-2**30, 2**30, 300001).astype(npdt)
        da, db = dev.array(a), dev.array(b)
        out = dev.empty((1,), npdt)
        L.check(L.lib.cnh_dot_partial(dt, a.size, da.ptr, db.ptr, out.ptr, None))
        with np.errstate(over="ignore"):
            want = np.sum(a * b, dtype=npdt)
        assert out.get()[0] == want
    # arange sum
    n = 100000
    ar = dev.array(np.arange(n, dtype=np.float64))
    out = dev.empty((1,), np.float64)
    L.check(L.lib.cnh_sum_tiles(L.F64, 1, L.vparr([ar.ptr]), L.i64arr([n]), out.ptr, None))
    assert out.get()[0] == n * (n - 1) / 2
    dev.free_all()


def test_reduce_final_sequential(dev, orc):
    p = np.array([1e16, 1.0, -1e16, 3.0])
    dp = dev.array(p)
    out = dev.empty((1,), np.float64)
    L.check(L.lib.cnh_reduce_final(L.F64, 4, dp.ptr, out.ptr, None))
    assert out.get()[0] == ((1e16 + 1.0) + -1e16) + 3.0  # left-to-right, like the upstream reducer


def test_sumsq_and_maxabs_diff(dev, orc):
    n = 300007
    a = orc.uniform(n, 4, 0, 0, 1)
    b = orc.uniform(n, 4, 1, 0, 1)
    ab, lens = _tiles(dev, a, 3)
    bb, _ = _tiles(dev, b, 3)
    out = dev.empty((1,), np.float64)
    L.check(L.lib.cnh_sumsq_diff_tiles(3, L.vparr([x.ptr for x in ab]),
                                       L.vparr([x.ptr for x in bb]), L.i64arr(lens), out.ptr, None))
    ref = math.fsum(((a - b) ** 2).tolist())
    assert abs(out.get()[0] - ref) <= REL * ref
    L.check(L.lib.cnh_maxabs_diff_tiles(3, L.vparr([x.ptr for x in ab]),
                                        L.vparr([x.ptr for x in bb]), L.i64arr(lens), out.ptr, None))
    assert out.get()[0] == np.max(np.abs(a - b))  # exact, order-independent
    # and the oracle's own forms of the two
    o = np.zeros(1)
    assert orc.lib.orc_maxabs_diff(n, a.ctypes.data, b.ctypes.data, o.ctypes.data) == 0
    assert out.get()[0] == o[0]
    assert orc.lib.orc_sumsq_diff(n, a.ctypes.data, b.ctypes.data, o.ctypes.data) == 0
    assert abs(o[0] - ref) <= REL * ref
    dev.free_all()


@pytest.mark.parametrize("dt,npdt", [(L.F64, np.float64), (L.F32, np.float32), (L.I64, np.int64), (L.I32, np.int32)])
def test_reductions_count_every_element_once(dev, dt, npdt):
    """Small integer values make sums and dots exact in any order of additions, so an element that a
    slice boundary, a ragged end or a misaligned start drops or takes twice changes the result.
    Tile lengths sit on and around the slice sizes (512, 8192 per workgroup, 65536 for the one-launch
    form); every tile also runs from a start that is not 16-byte aligned."""
    rng = np.random.default_rng(11)
    esz = np.dtype(npdt).itemsize
    lens = [1, 2, 3, 511, 512, 513, 1023, 1025, 8191, 8192, 8193, 12289, 65535, 65536, 65537,
            65536 + 8192, 100003, 3 * 8192 + 7, 1 << 20, (1 << 20) + 1]
    hi = 3 if npdt == np.float32 else 50          # float32 sums stay below 2^24
    for shift in (0, 1):
        host_a = [rng.integers(-hi, hi + 1, n + shift).astype(npdt) for n in lens]
        host_b = [rng.integers(-hi, hi + 1, n + shift).astype(npdt) for n in lens]
        da = [dev.array(x) for x in host_a]
        db = [dev.array(x) for x in host_b]
        out = dev.empty((1,), npdt)
        for i, n in enumerate(lens):           # tiles one at a time
            a, b = host_a[i][shift:], host_b[i][shift:]
            pa, pb = da[i].ptr + shift * esz, db[i].ptr + shift * esz
            L.check(L.lib.cnh_dot_partial(dt, n, pa, pb, out.ptr, None))
            assert out.get()[0] == np.sum(a.astype(np.int64) * b.astype(np.int64)), (n, shift, "dot")
            L.check(L.lib.cnh_sum_tiles(dt, 1, L.vparr([pa]), L.i64arr([n]), out.ptr, None))
            assert out.get()[0] == np.sum(a.astype(np.int64)), (n, shift, "sum")
        # all tiles in one call
        pas = [d.ptr + shift * esz for d in da]
        pbs = [d.ptr + shift * esz for d in db]
        L.check(L.lib.cnh_dot_tiles(dt, len(lens), L.vparr(pas), L.vparr(pbs), L.i64arr(lens), out.ptr, None))
        want = sum(int(np.sum(a[shift:].astype(np.int64) * b[shift:].astype(np.int64)))
                   for a, b in zip(host_a, host_b))
        assert out.get()[0] == want, (shift, "dot over all tiles")
        L.check(L.lib.cnh_sum_tiles(dt, len(lens), L.vparr(pas), L.i64arr(lens), out.ptr, None))
        assert out.get()[0] == sum(int(np.sum(a[shift:].astype(np.int64))) for a in host_a)
        if npdt == np.float64:
            o64 = dev.empty((1,), np.float64)
            L.check(L.lib.cnh_sumsq_diff_tiles(len(lens), L.vparr(pas), L.vparr(pbs), L.i64arr(lens),
                                               o64.ptr, None))
            assert o64.get()[0] == sum(float(np.sum((a[shift:] - b[shift:]) ** 2))
                                       for a, b in zip(host_a, host_b))
            L.check(L.lib.cnh_maxabs_diff_tiles(len(lens), L.vparr(pas), L.vparr(pbs), L.i64arr(lens),
                                                o64.ptr, None))
            assert o64.get()[0] == max(float(np.max(np.abs(a[shift:] - b[shift:])))
                                       for a, b in zip(host_a, host_b))
        dev.free_all()


def _check_matvec(got, A, x):
    ref = np.array([math.fsum((A[i] * x).tolist()) for i in range(A.shape[0])])
    denom = np.abs(A) @ np.abs(x)
    assert np.all(np.abs(got - ref) <= REL * denom + 1e-300)


def test_gemv_closed_forms(dev):
    # A[i,j] = i + j, x = 1  =>  y_i = N*i + N(N-1)/2 exactly (upstream examples/matvec.py)
    n = 512
    A = np.add.outer(np.arange(n, dtype=np.float64), np.arange(n, dtype=np.float64))
    dA, dx, dy = dev.array(A), dev.array(np.ones(n)), dev.empty((n,), np.float64)
    L.check(L.lib.cnh_gemv(L.F64, n, n, dA.ptr, n, dx.ptr, dy.ptr, 0, None))
    assert np.array_equal(dy.get(), n * np.arange(n) + n * (n - 1) / 2)
    # ones(M,N) @ arange(1..N) = N(N+1)/2 (upstream examples/matvec_slice.py)
    M, N = 96, 1000
    dA = dev.array(np.ones((M, N)))
    dx = dev.array(np.arange(1, N + 1, dtype=np.float64))
    dy = dev.empty((M,), np.float64)
    L.check(L.lib.cnh_gemv(L.F64, M, N, dA.ptr, N, dx.ptr, dy.ptr, 0, None))
    assert np.array_equal(dy.get(), np.full(M, N * (N + 1) / 2))
    dev.free_all()


@pytest.mark.parametrize("rows,cols,lda", [(300, 257, 257), (128, 4096, 4100), (1000, 33, 40)])
def test_gemv_sub_matrix_views(dev, orc, rows, cols, lda):
    rng = np.random.default_rng(2)
    full = rng.standard_normal((rows, lda))
    x = rng.standard_normal(cols)
    y0 = rng.standard_normal(rows)
    dA, dx, dy = dev.array(full), dev.array(x), dev.array(y0)
    L.check(L.lib.cnh_gemv(L.F64, rows, cols, dA.ptr, lda, dx.ptr, dy.ptr, 0, None))
    _check_matvec(dy.get(), full[:, :cols], x)
    # beta = 1 accumulates on top of y, then axpy1 adds a partial
    dy.put(y0)
    L.check(L.lib.cnh_gemv(L.F64, rows, cols, dA.ptr, lda, dx.ptr, dy.ptr, 1, None))
    got = dy.get()
    ref = y0 + full[:, :cols] @ x
    assert np.allclose(got, ref, rtol=1e-12, atol=1e-12)
    part = dev.array(y0)
    L.check(L.lib.cnh_axpy1(L.F64, rows, part.ptr, dy.ptr, None))
    assert np.array_equal(dy.get(), got + y0)
    dev.free_all()


def test_gemv_tiles_matches_oracle_tiling(dev, orc):
    """2x2 (ragged) tile grid; partials added in column-tile order like the 1-D accumulate."""
    rows, cols, tile = 700, 900, 512
    A = orc.cg_matrix(1024, 0, rows, 0, cols, 2)
    x = orc.uniform(cols, 2, 1, -1, 1)
    gr, gc = 2, 2
    bufs = []
    for i in range(gr):
        for j in range(gc):
            bufs.append(dev.array(np.ascontiguousarray(A[i * tile:(i + 1) * tile,
                                                         j * tile:(j + 1) * tile])))
    dx, dy = dev.array(x), dev.empty((rows,), np.float64)
    L.check(L.lib.cnh_gemv_tiles(L.F64, rows, cols, tile, L.vparr([b.ptr for b in bufs]), dx.ptr,
                                 dy.ptr, None))
    got = dy.get()
    _check_matvec(got, A, x)
    # oracle: per-tile gemv then sequential accumulate of the partials
    want = np.zeros(rows)
    for i in range(gr):
        acc = None
        for j in range(gc):
            t = np.ascontiguousarray(A[i * tile:(i + 1) * tile, j * tile:(j + 1) * tile])
            part = orc.gemv(t, np.ascontiguousarray(x[j * tile:(j + 1) * tile]))
            acc = part if acc is None else acc + part
        want[i * tile:i * tile + acc.size] = acc
    denom = np.abs(A) @ np.abs(x)
    assert np.all(np.abs(got - want) <= REL * denom)
    dev.free_all()


@pytest.mark.parametrize("M,N,K", [(64, 64, 16), (128, 192, 64), (70, 50, 33), (256, 512, 256),
                                   (1, 1, 1), (17, 130, 5)])
def test_gemm_acc_fp64_mfma(dev, orc, M, N, K):
    rng = np.random.default_rng(M * 1000 + N + K)
    A = rng.standard_normal((M, K))
    B = rng.standard_normal((K, N))
    C0 = rng.standard_normal((M, N))
    dA, dB, dC = dev.array(A), dev.array(B), dev.array(C0)
    L.check(L.lib.cnh_gemm_acc(L.F64, M, N, K, dA.ptr, K, dB.ptr, N, dC.ptr, N, None))
    got = dC.get()
    want = orc.gemm_acc(A, B, C0.copy())
    denom = np.abs(A) @ np.abs(B) + np.abs(C0)
    assert np.all(np.abs(got - want) <= REL * denom)
    # independent pin: long double accumulation
    ref = (A.astype(np.longdouble) @ B.astype(np.longdouble) + C0).astype(np.float64)
    assert np.all(np.abs(got - ref) <= REL * denom)
    dev.free_all()


def test_gemm_ones_closed_form_and_strided_panels(dev, orc):
    # ones(M,K) @ ones(K,N) = K exactly (upstream examples/matmatmul.py), C zeroed first
    M, N, K = 96, 160, 200
    dA, dB = dev.array(np.ones((M, K))), dev.array(np.ones((K, N)))
    dC = dev.array(np.zeros((M, N)))
    L.check(L.lib.cnh_gemm_acc(L.F64, M, N, K, dA.ptr, K, dB.ptr, N, dC.ptr, N, None))
    assert np.array_equal(dC.get(), np.full((M, N), float(K)))
    # panels inside larger buffers (row strides > extents), accumulated twice
    rng = np.random.default_rng(11)
    Af, Bf, Cf = rng.standard_normal((64, 100)), rng.standard_normal((48, 90)), np.zeros((64, 80))
    dA, dB, dC = dev.array(Af), dev.array(Bf), dev.array(Cf)
    for _ in range(2):
        L.check(L.lib.cnh_gemm_acc(L.F64, 64, 70, 48, dA.ptr + 8 * 4, 100, dB.ptr + 8 * 6, 90,
                                   dC.ptr + 8 * 2, 80, None))
    want = Cf.copy()
    want[:, 2:72] = 2 * (Af[:, 4:52] @ Bf[:, 6:76])
    assert np.allclose(dC.get(), want, rtol=1e-12, atol=1e-12)
    dev.free_all()


@pytest.mark.parametrize("dt,npdt", [(L.F64, np.float64), (L.I64, np.int64)])
@pytest.mark.parametrize("aligned", [True, False])
def test_gemm_batch_is_the_jobs_one_after_another(dev, orc, dt, npdt, aligned):
    """A matmatmul cut into tiles: several C blocks, each fed by several K pieces from panels inside
    larger buffers. One batched launch must give what the same jobs give one call at a time: exactly
    for integers; within the 1e-12 bar for fp64, where a workgroup adds the pieces of its block in
    list order either way, but carries one running sum across them instead of adding per-piece sums."""
    rng = np.random.default_rng(21)
    M, N, K = (128, 192, 160) if aligned else (100, 150, 77)
    kcuts = [0, 64, 96, K] if aligned else [0, 30, 31, K]
    ncuts = [0, 128, N] if aligned else [0, 70, N]
    mcuts = [0, 64, M] if aligned else [0, 33, M]
    if npdt == np.float64:
        A, B = rng.standard_normal((M, K)), rng.standard_normal((K, N))
    else:
        A, B = rng.integers(-9, 9, (M, K)).astype(npdt), rng.integers(-9, 9, (K, N)).astype(npdt)
    C0 = np.zeros((M, N), npdt)
    dA, dB, dC, dC1 = dev.array(A), dev.array(B), dev.array(C0), dev.array(C0)
    esz = A.itemsize
    jobs = []
    for mi in range(len(mcuts) - 1):
        for ni in range(len(ncuts) - 1):
            for ki in range(len(kcuts) - 1):
                m0, m1, n0, n1, k0, k1 = mcuts[mi], mcuts[mi + 1], ncuts[ni], ncuts[ni + 1], kcuts[ki], kcuts[ki + 1]
                jobs.append((m1 - m0, n1 - n0, k1 - k0, (m0 * K + k0) * esz, (k0 * N + n0) * esz, (m0 * N + n0) * esz))
    jobs.append((0, 5, 5, 0, 0, 0))                  # an empty job is skipped
    arr = (L.GemmJob * len(jobs))()
    for j, (m, n, k, oa, ob, oc) in zip(arr, jobs):
        j.M, j.N, j.K, j.A, j.lda, j.B, j.ldb, j.C, j.ldc = m, n, k, dA.ptr + oa, K, dB.ptr + ob, N, dC.ptr + oc, N
    L.check(L.lib.cnh_gemm_acc_batch(dt, len(jobs), arr, None))
    for (m, n, k, oa, ob, oc) in jobs:
        L.check(L.lib.cnh_gemm_acc(dt, m, n, k, dA.ptr + oa, K, dB.ptr + ob, N, dC1.ptr + oc, N, None))
    got, one_by_one = dC.get(), dC1.get()
    if npdt == np.float64:
        bound = REL * (np.abs(A) @ np.abs(B))
        assert np.all(np.abs(got - one_by_one) <= bound)
        assert np.all(np.abs(got - (A.astype(np.longdouble) @ B.astype(np.longdouble)).astype(np.float64)) <= bound)
    else:
        assert np.array_equal(got, one_by_one) and np.array_equal(got, A @ B)
    dev.free_all()


@pytest.mark.parametrize("M,N,K", [(128, 192, 160), (100, 150, 77)])
def test_gemm_batch_overwrites_without_reading(dev, M, N, K):
    """overwrite = 1: C becomes the product whatever it held (NaNs included), two K pieces per block."""
    rng = np.random.default_rng(M + K)
    A, B = rng.standard_normal((M, K)), rng.standard_normal((K, N))
    C0 = np.full((M, N), np.nan)
    dA, dB, dC = dev.array(A), dev.array(B), dev.array(C0)
    kc = K // 2
    arr = (L.GemmJob * 2)()
    for j, (k0, k1) in zip(arr, ((0, kc), (kc, K))):
        j.M, j.N, j.K, j.A, j.lda, j.B, j.ldb, j.C, j.ldc = M, N, k1 - k0, dA.ptr + 8 * k0, K, dB.ptr + 8 * k0 * N, N, dC.ptr, N
    L.check(L.lib.cnh_gemm_batch(L.F64, 2, arr, 1, None))
    got = dC.get()
    # aligned products fetch through buffer descriptors by default; plain global loads give the same bits
    L.check(L.lib.cnh_set_option(b"gemm_buffer_loads", 0))
    try:
        dC.put(C0)
        L.check(L.lib.cnh_gemm_batch(L.F64, 2, arr, 1, None))
        assert dC.get().tobytes() == got.tobytes()
    finally:
        L.check(L.lib.cnh_set_option(b"gemm_buffer_loads", 1))
    bound = REL * (np.abs(A) @ np.abs(B))
    assert np.all(np.abs(got - (A.astype(np.longdouble) @ B.astype(np.longdouble)).astype(np.float64)) <= bound)
    # accumulate on top of it
    L.check(L.lib.cnh_gemm_batch(L.F64, 2, arr, 0, None))
    assert np.all(np.abs(dC.get() - 2 * got) <= 2 * bound)
    assert L.lib.cnh_gemm_batch(L.I64, 2, arr, 1, None) != 0          # overwriting is fp64 only
    dev.free_all()


@pytest.mark.parametrize("M,N,Ks,overwrite", [(256, 1024, (512,), 1), (128, 512, (64, 96, 32), 0),
                                              (64, 64, (32,), 1), (256, 4096, (2048,), 1)])
def test_gemm_with_the_k_steps_split_over_two_sets_of_wavefronts(dev, M, N, Ks, overwrite):
    """Grids of at most one workgroup per CU whose K pieces are multiples of 32 run with two sets of
    wavefronts per workgroup, each taking every other K step (option gemm_ksplit, on by default).
    Small integer values make every sum exact, so both forms and NumPy must give the same bits; with
    real values both stay within the bound and the split form gives the same bits on every run."""
    rng = np.random.default_rng(M + N + sum(Ks))
    K = sum(Ks)
    for integers in (True, False):
        if integers:
            A = rng.integers(-4, 5, (M, K)).astype(np.float64)
            B = rng.integers(-4, 5, (K, N)).astype(np.float64)
            C0 = rng.integers(-9, 10, (M, N)).astype(np.float64)
        else:
            A, B, C0 = rng.standard_normal((M, K)), rng.standard_normal((K, N)), rng.standard_normal((M, N))
        dA, dB, dC = dev.array(A), dev.array(B), dev.array(C0)
        arr = (L.GemmJob * len(Ks))()
        k0 = 0
        for j, kk in zip(arr, Ks):
            j.M, j.N, j.K, j.A, j.lda, j.B, j.ldb, j.C, j.ldc = M, N, kk, dA.ptr + 8 * k0, K, dB.ptr + 8 * k0 * N, N, dC.ptr, N
            k0 += kk
        results = {}
        try:
            for split in (1, 0, 1):
                L.check(L.lib.cnh_set_option(b"gemm_ksplit", split))
                dC.put(C0)
                L.check(L.lib.cnh_gemm_batch(L.F64, len(Ks), arr, overwrite, None))
                got = dC.get()
                if split in results:
                    assert got.tobytes() == results[split].tobytes()       # run to run
                results[split] = got
        finally:
            L.check(L.lib.cnh_set_option(b"gemm_ksplit", 1))
        if integers or M * N * K > 10 ** 8:      # exact in fp64 / the bound is 1e4 roundings wide
            want = A @ B + (0 if overwrite else C0)
        else:
            want = (A.astype(np.longdouble) @ B.astype(np.longdouble)).astype(np.float64) + (0 if overwrite else C0)
        if integers:
            assert results[1].tobytes() == want.tobytes() and results[0].tobytes() == want.tobytes()
        else:
            bound = REL * (np.abs(A) @ np.abs(B) + np.abs(C0))
            assert np.all(np.abs(results[1] - want) <= bound) and np.all(np.abs(results[0] - want) <= bound)
            assert results[1].tobytes() != results[0].tobytes() or K <= 32     # the split form did run
        dev.free_all()


@pytest.mark.parametrize("dt,npdt", [(L.F64, np.float64), (L.I32, np.int32)])
def test_gemv_over_a_window_of_tiles(dev, dt, npdt):
    """A 100 x 90 matrix in 32 x 32 tiles; the window rows 5..77, columns 9..70 against x."""
    rng = np.random.default_rng(31)
    M, N, T = 100, 90, 32
    A = (rng.standard_normal((M, N)) if npdt == np.float64 else rng.integers(-99, 99, (M, N))).astype(npdt)
    x = (rng.standard_normal(80) if npdt == np.float64 else rng.integers(-99, 99, 80)).astype(npdt)
    r0, r1, c0, c1 = 5, 77, 9, 70
    tiles = {}
    for ti in range((M + T - 1) // T):
        for tj in range((N + T - 1) // T):
            tiles[ti, tj] = dev.array(np.ascontiguousarray(A[ti * T:(ti + 1) * T, tj * T:(tj + 1) * T]))
    pr0, pr1, pc0, pc1 = r0 // T, (r1 - 1) // T, c0 // T, (c1 - 1) // T
    panels = (L.GemvPanel * ((pr1 - pr0 + 1) * (pc1 - pc0 + 1)))()
    i = 0
    for pr in range(pr0, pr1 + 1):
        for pc in range(pc0, pc1 + 1):
            width = min(T, N - pc * T)
            first = max(pc * T, c0)
            panels[i].base = tiles[pr, pc].ptr + (first - pc * T) * A.itemsize
            panels[i].ld, panels[i].ncols, panels[i].xoff = width, min((pc + 1) * T, c1) - first, first - c0
            i += 1
    dx, dy = dev.array(x), dev.array(np.zeros(r1 - r0, npdt))
    L.check(L.lib.cnh_gemv_panels(dt, r1 - r0, pc1 - pc0 + 1, T, r0 - pr0 * T, len(panels), panels,
                                  dx.ptr + 3 * A.itemsize, dy.ptr, None))
    want = A[r0:r1, c0:c1] @ x[3:3 + c1 - c0]
    if npdt == np.float64:
        assert np.abs(dy.get() - want).max() <= REL * (np.abs(A[r0:r1, c0:c1]) @ np.abs(x[3:3 + c1 - c0])).max()
    else:
        assert np.array_equal(dy.get(), want)
    assert L.lib.cnh_gemv_panels(dt, r1 - r0, pc1 - pc0 + 1, T, T, len(panels), panels, dx.ptr, dy.ptr, None) != 0
    assert L.lib.cnh_gemv_panels(dt, r1 - r0, pc1 - pc0 + 1, T, 0, len(panels) - 1, panels, dx.ptr, dy.ptr, None) != 0
    dev.free_all()


def test_descriptor_table_outlives_the_stream_it_was_uploaded_on(dev):
    """The same job list (hence the same descriptor table) on a stream, then on a second stream after
    the first was destroyed: the cached table must be usable without touching the dead stream."""
    rng = np.random.default_rng(31)
    A, B = rng.standard_normal((64, 48)), rng.standard_normal((48, 64))
    dA, dB, dC = dev.array(A), dev.array(B), dev.array(np.zeros((64, 64)))
    arr = (L.GemmJob * 2)()
    for j, (k0, k1) in zip(arr, ((0, 16), (16, 48))):
        j.M, j.N, j.K, j.A, j.lda, j.B, j.ldb, j.C, j.ldc = 64, 64, k1 - k0, dA.ptr + k0 * 8, 48, dB.ptr + k0 * 64 * 8, 64, dC.ptr, 64
    for _ in range(2):
        st = C.c_void_p()
        L.check(L.lib.cnh_stream_create(C.byref(st)))
        L.check(L.lib.cnh_gemm_acc_batch(L.F64, 2, arr, st))
        L.check(L.lib.cnh_stream_sync(st))
        L.check(L.lib.cnh_stream_destroy(st))
    L.check(L.lib.cnh_gemm_acc_batch(L.F64, 2, arr, None))
    L.check(L.lib.cnh_device_sync())
    assert np.all(np.abs(dC.get() - 3 * (A @ B)) <= 3 * REL * (np.abs(A) @ np.abs(B)))
    dev.free_all()


def test_gemm_batch_refuses_bad_jobs(dev):
    arr = (L.GemmJob * 1)()
    arr[0].M, arr[0].N, arr[0].K, arr[0].lda, arr[0].ldb, arr[0].ldc = 4, 4, 4, 2, 4, 4
    arr[0].A = arr[0].B = arr[0].C = 256
    assert L.lib.cnh_gemm_acc_batch(L.F64, 1, arr, None) != 0      # row stride shorter than the row
    assert L.lib.cnh_gemm_acc_batch(L.F64, -1, arr, None) != 0
    assert L.lib.cnh_gemm_acc_batch(L.F64, 0, None, None) == 0


@pytest.mark.parametrize("dt,npdt", [(L.F32, np.float32), (L.I32, np.int32), (L.I64, np.int64)])
def test_gemm_other_dtypes(dev, orc, dt, npdt):
    rng = np.random.default_rng(4)
    M, N, K = 37, 45, 29
    if npdt == np.float32:
        A, B = rng.standard_normal((M, K)).astype(npdt), rng.standard_normal((K, N)).astype(npdt)
    else:
        A = rng.integers(-50, 50, (M, K)).astype(npdt)
        B = rng.integers(-50, 50, (K, N)).astype(npdt)
    C0 = np.zeros((M, N), npdt)
    dA, dB, dC = dev.array(A), dev.array(B), dev.array(C0)
    L.check(L.lib.cnh_gemm_acc(dt, M, N, K, dA.ptr, K, dB.ptr, N, dC.ptr, N, None))
    want = orc.gemm_acc(A, B, C0.copy())
    if npdt == np.float32:
        assert np.allclose(dC.get(), want, rtol=1e-5, atol=1e-5)
    else:
        assert np.array_equal(dC.get(), want)
    dev.free_all()


def test_stream_event_and_callback(dev):
    s = C.c_void_p()
    L.check(L.lib.cnh_stream_create(C.byref(s)))
    e0, e1 = C.c_void_p(), C.c_void_p()
    L.check(L.lib.cnh_event_create(C.byref(e0)))
    L.check(L.lib.cnh_event_create(C.byref(e1)))
    d = dev.empty((1 << 20,), np.float64)
    L.check(L.lib.cnh_event_record(e0, s))
    L.check(L.lib.cnh_fill_uniform(d.ptr, 1 << 20, 1, 2, 0, 0.0, 1.0, s))
    L.check(L.lib.cnh_event_record(e1, s))
    hit = []
    CB = C.CFUNCTYPE(None, C.c_void_p)
    cb = CB(lambda _: hit.append(1))
    L.check(L.lib.cnh_stream_callback(s, C.cast(cb, C.c_void_p), None))
    L.check(L.lib.cnh_stream_sync(s))
    ms = C.c_float()
    L.check(L.lib.cnh_event_elapsed_ms(e0, e1, C.byref(ms)))
    assert ms.value >= 0 and hit == [1]
    L.check(L.lib.cnh_event_destroy(e0))
    L.check(L.lib.cnh_event_destroy(e1))
    L.check(L.lib.cnh_stream_destroy(s))
    dev.free_all()


@pytest.mark.parametrize("rows,widths,dt", [(16400, (2048, 1000), np.float64), (8200, (2048, 1024, 520), np.float64),
                                             (16384, (3000,), np.float32)])
def test_large_matvec_with_x_staged_in_lds(dev, orc, rows, widths, dt):
    """Matvecs of 8192 rows or more keep the vector in LDS, 32 or 64 rows per workgroup. The result
    has the bits of the one-wavefront-per-row kernel (same elements meet in the same order) and
    agrees with a float64 NumPy product to the summation bound. Ragged column panels, a row count
    that is no multiple of the rows per workgroup, two panel rows."""
    rng = np.random.default_rng(rows)
    cols = sum(widths)
    tile_rows = 8192 if rows > 8192 else rows
    hA = rng.standard_normal((rows, cols)).astype(dt)
    hx = rng.standard_normal(cols).astype(dt)
    panels, keep, xoff = [], [], 0
    n_panel_rows = (rows + tile_rows - 1) // tile_rows
    for pr in range(n_panel_rows):
        r0, r1 = pr * tile_rows, min(rows, (pr + 1) * tile_rows)
        xoff = 0
        for w in widths:
            b = dev.array(np.ascontiguousarray(hA[r0:r1, xoff:xoff + w]))
            keep.append(b)
            panels.append((b.ptr, w, w, xoff))
            xoff += w
    arr = (L.GemvPanel * len(panels))(*[L.GemvPanel(*p) for p in panels])
    x = dev.array(hx)
    out = {}
    for mode in (1, 0):
        y = dev.array(np.full(rows, -7.0, dtype=dt))
        L.check(L.lib.cnh_set_option(b"gemv_xlds", mode))
        try:
            L.check(L.lib.cnh_gemv_panels(H.DT[np.dtype(dt)], rows, len(widths), tile_rows, 0, len(panels), arr,
                                          x.ptr, y.ptr, None))
        finally:
            L.check(L.lib.cnh_set_option(b"gemv_xlds", 1))
        out[mode] = y.get()
    assert np.array_equal(out[0], out[1])
    exact = hA.astype(np.float64) @ hx.astype(np.float64)
    bound = (np.abs(hA).astype(np.float64) @ np.abs(hx).astype(np.float64)) * (1e-12 if dt == np.float64 else 2e-5)
    assert np.all(np.abs(out[1] - exact) <= bound)
    dev.free_all()
