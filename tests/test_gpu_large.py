"""Arrays of more than 2^31 elements (a 288 GB device holds many): element indices, workgroup
counts and region arithmetic must be 64-bit all the way. int32 values, so every check is exact
(sums wrap modulo 2^32, as the wire type does)."""
import ctypes as C

import numpy as np
import pytest

from charmnumeric_amd import _lib as L
from charmnumeric_amd.astbuild import AstBuilder
from tests import helpers as H

pytestmark = pytest.mark.gpu

N = (1 << 31) + 4100          # past 2^31, not a multiple of any vector or workgroup width


def _alloc(nbytes):
    p = C.c_void_p()
    L.check(L.lib.cnh_alloc(nbytes, 0, C.byref(p)))
    return p


def _fill(ptr, start, count, value):
    v = np.zeros(8, np.uint8)
    v[:4] = np.array([value], np.int32).view(np.uint8)
    L.check(L.lib.cnh_fill_region(1, 4, ptr, L.i64arr([1]), L.i64arr([start]), L.i64arr([1]),
                                  L.i64arr([count]), v.ctypes.data, None))


def _read(ptr, start, count):
    out = np.empty(count, np.int32)
    L.check(L.lib.cnh_d2h(out.ctypes.data, ptr.value + 4 * start, 4 * count, None))
    return out


def _wrap(v):
    return int(np.array([v & 0xFFFFFFFF], np.uint64).astype(np.uint32).view(np.int32)[0])


def test_fill_group_reductions_and_conversion_past_2_to_31(dev):
    a, b, c = _alloc(4 * N), _alloc(4 * N), _alloc(4 * N)
    try:
        _fill(a, 0, N, 3)
        _fill(b, 0, N, 4)
        _fill(a, N - 5, 5, -7)                         # a region that starts beyond 2^31
        _fill(b, (1 << 31) - 2, 4, 10)                 # and one that straddles it
        # c = a * b + a over the whole length, one dense partition
        bld = AstBuilder(L.I32, 1)
        t = bld.binary(L.OP_MUL, 100, bld.leaf(0), bld.leaf(1))
        bld.binary(L.OP_ADD, 10, t, bld.leaf(0), is_temp=False)
        k = H.compile_group(bld.finish(), L.I32, 1)
        ma, mb, mc = (L.Memref.dense(p.value, (N,)) for p in (a, b, c))
        H.launch_batched(k, 1, [[ma, mb, ma]], [], [[mc]])
        dev.sync()
        assert np.array_equal(_read(c, 0, 8), np.full(8, 15, np.int32))
        assert np.array_equal(_read(c, (1 << 31) - 4, 8), np.array([15, 15, 33, 33, 33, 33, 15, 15], np.int32))
        assert np.array_equal(_read(c, N - 8, 8), np.array([15, 15, 15, -35, -35, -35, -35, -35], np.int32))
        want_sum = 15 * (N - 9) + 4 * 33 + 5 * (-35)
        out = dev.empty((2,), np.int32)
        L.check(L.lib.cnh_sum_tiles(L.I32, 1, L.vparr([c.value]), L.i64arr([N]), out.ptr, None))
        # dot of a with b: 12 everywhere but the two patches
        L.check(L.lib.cnh_dot_partial(L.I32, N, a, b, out.ptr + 4, None))
        got = out.get()
        assert int(got[0]) == _wrap(want_sum)
        assert int(got[1]) == _wrap(12 * (N - 9) + 4 * 30 + 5 * (-28))
        # converting copy of the tail (source and destination offsets beyond 2^31 elements)
        d = dev.empty((16,), np.float64)
        L.check(L.lib.cnh_convert_region(1, L.F64, d.ptr, L.i64arr([1]), L.i64arr([0]), L.i64arr([1]),
                                         L.I32, c, L.i64arr([1]), L.i64arr([N - 16]), L.i64arr([1]),
                                         L.i64arr([16]), None))
        assert np.array_equal(d.get(), _read(c, N - 16, 16).astype(np.float64))
        # strided copy that walks the whole length: every 2^20-th element
        cnt = (N + (1 << 20) - 1) >> 20
        e = dev.empty((cnt,), np.int32)
        L.check(L.lib.cnh_copy_region(1, 4, e.ptr, L.i64arr([1]), L.i64arr([0]), L.i64arr([1]), c,
                                      L.i64arr([1]), L.i64arr([0]), L.i64arr([1 << 20]), L.i64arr([cnt]), None))
        want = np.full(cnt, 15, np.int32)
        want[2048] = 33                                 # element 2^31 lies in the straddling patch
        assert np.array_equal(e.get(), want)
        L.check(L.lib.cnh_kernel_release(k))
    finally:
        for p in (a, b, c):
            L.check(L.lib.cnh_free(p))
        dev.free_all()


def test_rank3_block_and_rank2_tiles_past_2_to_31_elements_through_the_frontend():
    """A rank-3 array of 1300^3 doubles is one block of 2.2e9 elements: fills of slabs, one
    seven-point sweep and the read-back of its far corner all address beyond 2^31 elements.
    A rank-2 int32 array of 46400^2 elements is cut into tiles; its sum wraps modulo 2^32."""
    import charmnumeric_amd as cnp

    cnp.reset()
    itf = cnp.CharmNumericInterface(device=0)
    itf.connect(odf=4)
    try:
        n = 1300
        u = cnp.zeros((n, n, n))
        u[n - 12:n] = 5.0
        u[:, n - 9:n, :] = 2.0
        u[:, :, n - 7:n] = -3.0
        u[n - 3, n - 4, n - 5] = 100.0
        u[1:-1, 1:-1, 1:-1] = 0.16666666666666666 * (((((u[:-2, 1:-1, 1:-1] + u[2:, 1:-1, 1:-1])
                                                       + u[1:-1, :-2, 1:-1]) + u[1:-1, 2:, 1:-1])
                                                      + u[1:-1, 1:-1, :-2]) + u[1:-1, 1:-1, 2:])
        m = 24                                           # the far corner, halo included
        got = u[n - m:n, n - m:n, n - m:n].get(itf)
        h = np.zeros((m + 1, m + 1, m + 1))             # one more layer towards the origin
        o = n - m - 1                                   # global index of h[0]
        h[n - 12 - o:] = 5.0
        h[:, n - 9 - o:, :] = 2.0
        h[:, :, n - 7 - o:] = -3.0
        h[n - 3 - o, n - 4 - o, n - 5 - o] = 100.0
        w = h.copy()
        w[1:-1, 1:-1, 1:-1] = 0.16666666666666666 * (((((h[:-2, 1:-1, 1:-1] + h[2:, 1:-1, 1:-1])
                                                       + h[1:-1, :-2, 1:-1]) + h[1:-1, 2:, 1:-1])
                                                      + h[1:-1, 1:-1, :-2]) + h[1:-1, 1:-1, 2:])
        assert got.tobytes() == w[1:, 1:, 1:].tobytes()
        # the near corner too (offsets near zero): untouched zeros and the first interior cells
        assert not u[0:4, 0:4, 0:4].get(itf).any()
        del u
        k = 46400
        a = cnp.ones((k, k), dtype=np.int32)
        a[k - 3:, k - 2:] = 7
        b = a * 3 + a
        s = cnp.sum(b).get(itf)
        want = 4 * (k * k - 6) + 28 * 6
        assert int(s[0]) == _wrap(want)
        assert np.array_equal(b[k - 4:, k - 3:].get(itf),
                              np.array([[4, 4, 4], [4, 28, 28], [4, 28, 28], [4, 28, 28]], np.int32))
    finally:
        cnp.reset()
        itf.close()
