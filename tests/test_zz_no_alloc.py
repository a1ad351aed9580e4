"""The dot entry point that allocates nothing, against cnh_dot_partial (same bits), through the C ABI.

Collected last on purpose: the array behind the entry point is shared by every call on the device,
and this file must pass both alone in a fresh process and after all other GPU tests.
"""
import ctypes as C

import numpy as np
import pytest

from charmnumeric_amd import _lib as L
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _both(dev, dtype, a, b):
    """(bits of cnh_dot_partial, bits of cnh_dot_partial_noalloc) for the same operands."""
    n = a.shape[0]
    da, db = dev.array(a), dev.array(b)
    out = dev.array(np.full(2, -77, dtype=a.dtype))        # stale values both calls must overwrite
    esz = a.dtype.itemsize
    L.check(L.lib.cnh_dot_partial(dtype, n, da.ptr, db.ptr, out.ptr, None))
    L.check(L.lib.cnh_dot_partial_noalloc(dtype, n, da.ptr, db.ptr, out.ptr + esz, None))
    got = out.get()
    it = np.int64 if esz == 8 else np.int32
    return got.view(it)[0], got.view(it)[1], got


def test_two_calls_in_a_row_second_smaller(dev):
    # first call: 3.3 M elements (403 stage-1 slices); second: 300 001 (37 slices, ragged, odd
    # length) — stale partials of the first call lie beyond the slots the second one reads
    rng = np.random.default_rng(11)
    for n in (3_300_007, 300_001):
        a = rng.uniform(-1, 1, n)
        b = rng.uniform(-1, 1, n)
        want, got, vals = _both(dev, L.F64, a, b)
        assert want == got, (n, vals)
        ref = float(np.dot(a.astype(np.longdouble), b.astype(np.longdouble)))
        assert abs(vals[1] - ref) <= 1e-12 * float(np.abs(a) @ np.abs(b))
    dev.free_all()


@pytest.mark.parametrize("dtype,npdt", [(L.F32, np.float32), (L.I32, np.int32), (L.I64, np.int64)])
def test_other_dtypes_and_short_vectors(dev, dtype, npdt):
    rng = np.random.default_rng(5)
    for n in (1_000_003, 70_001, 4097, 1, 0):
        if np.issubdtype(npdt, np.integer):
            a = rng.integers(-1000, 1000, n).astype(npdt)
            b = rng.integers(-1000, 1000, n).astype(npdt)
        else:
            a = rng.uniform(-1, 1, n).astype(npdt)
            b = rng.uniform(-1, 1, n).astype(npdt)
        if n == 0:
            a, b = np.zeros(0, npdt), np.zeros(0, npdt)
        want, got, vals = _both(dev, dtype, a, b)
        assert want == got, (n, vals)
    dev.free_all()


def test_same_operand_twice_and_own_stream(dev):
    rng = np.random.default_rng(3)
    a = rng.uniform(-1, 1, 2_000_000)
    da = dev.array(a)
    out = dev.array(np.zeros(2))
    st = C.c_void_p()
    L.check(L.lib.cnh_stream_create(C.byref(st)))
    L.check(L.lib.cnh_dot_partial(L.F64, a.size, da.ptr, da.ptr, out.ptr, st))
    L.check(L.lib.cnh_dot_partial_noalloc(L.F64, a.size, da.ptr, da.ptr, out.ptr + 8, st))
    L.check(L.lib.cnh_stream_sync(st))
    got = out.get()
    assert got.view(np.int64)[0] == got.view(np.int64)[1]
    L.check(L.lib.cnh_stream_destroy(st))
    dev.free_all()


def test_the_call_allocates_and_uploads_nothing(dev):
    """The property the entry point exists for: no device or pinned allocation, no descriptor copy,
    no workspace growth across the call, for a size that makes the ordinary entry point do all
    three on a fresh stream."""
    rng = np.random.default_rng(9)
    n = 5_000_011
    a, b = rng.uniform(-1, 1, n), rng.uniform(-1, 1, n)
    da, db = dev.array(a), dev.array(b)
    out = dev.array(np.zeros(2))
    st = C.c_void_p()
    L.check(L.lib.cnh_stream_create(C.byref(st)))
    before = L.lib.cnh_allocation_count()
    L.check(L.lib.cnh_dot_partial_noalloc(L.F64, n, da.ptr, db.ptr, out.ptr, st))
    L.check(L.lib.cnh_dot_partial_noalloc(L.F64, n // 3, da.ptr, db.ptr, out.ptr + 8, st))
    assert L.lib.cnh_allocation_count() == before
    L.check(L.lib.cnh_dot_partial(L.F64, n, da.ptr, db.ptr, out.ptr + 8, st))     # a workspace for this stream
    assert L.lib.cnh_allocation_count() > before
    L.check(L.lib.cnh_stream_sync(st))
    got = out.get()
    assert got.view(np.int64)[0] == got.view(np.int64)[1]
    # the zero-fill of an allocation queued on the caller's stream
    p = C.c_void_p()
    L.check(L.lib.cnh_alloc_on(1 << 20, 1, st, C.byref(p)))
    host = np.ones(1 << 17)
    L.check(L.lib.cnh_d2h(host.ctypes.data_as(C.c_void_p), p, 1 << 20, st))
    assert not host.any()
    L.check(L.lib.cnh_free(p))
    L.check(L.lib.cnh_stream_destroy(st))
    dev.free_all()


def test_sizes_beyond_the_array_are_refused(dev):
    out = dev.array(np.zeros(1))
    rc = L.lib.cnh_dot_partial_noalloc(L.F64, (1 << 28) + 1, out.ptr, out.ptr, out.ptr, None)
    assert rc == -3
    assert b"exceed the maximum" in L.lib.cnh_last_error()
    rc = L.lib.cnh_dot_partial_noalloc(L.F64, 10, None, out.ptr, out.ptr, None)
    assert rc == -2
    dev.free_all()
