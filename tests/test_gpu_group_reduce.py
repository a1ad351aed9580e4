"""Reducing roots of a fused group (CNH_OP_SUM_OF / CNH_OP_MAXABS_OF): the values a group produces
are summed (or their largest magnitude taken) by the launch that produces them. Checked against
NumPy on the same inputs: the stored output bit for bit, maxima exactly, sums to rounding of the
summation order (and exactly where every partial sum is an integer)."""
import ctypes as C

import numpy as np
import pytest

from charmnumeric_amd import _lib as L
from charmnumeric_amd.astbuild import AstBuilder
from tests import helpers as H

pytestmark = pytest.mark.gpu


def ast_c1_reduced():
    """z = 2.5x - 0.5y + xy stored (name 10); 20 = sum(z * w), 21 = sum(z * z), 22 = max|z - x|.
    Leaves: x = 0, y = 1, w = 2."""
    b = AstBuilder(L.F64, 1)
    x, y, w = b.leaf(0), b.leaf(1), b.leaf(2)
    t1 = b.binary(L.OP_MUL, 100, b.scalar(2.5), x)
    t2 = b.binary(L.OP_MUL, 101, b.scalar(0.5), y)
    t3 = b.binary(L.OP_SUB, 102, t1, t2)
    t4 = b.binary(L.OP_MUL, 103, x, y)
    z = b.binary(L.OP_ADD, 10, t3, t4, is_temp=False)
    zw = b.binary(L.OP_MUL, 104, z, w)
    b.unary(L.OP_SUM_OF, 20, zw, is_temp=False)
    zz = b.binary(L.OP_MUL, 105, z, z)
    b.unary(L.OP_SUM_OF, 21, zz, is_temp=False)
    d = b.binary(L.OP_SUB, 106, z, x)
    b.unary(L.OP_MAXABS_OF, 22, d, is_temp=False)
    return b.finish()


def bind(k, ins, outs):
    """Memrefs in the kernel's argument order, from dictionaries by array name."""
    n_in, n_sc, n_out = C.c_int(), C.c_int(), C.c_int()
    L.check(L.lib.cnh_kernel_signature(k, C.byref(n_in), C.byref(n_sc), C.byref(n_out)))
    name, has, tgt, sr = C.c_int(), C.c_int(), C.c_int(), C.c_int()
    reg = L.Region()
    a, b = [], []
    for i in range(n_in.value):
        L.check(L.lib.cnh_kernel_input(k, i, C.byref(name), C.byref(has), C.byref(reg)))
        a.append(ins[name.value])
    for i in range(n_out.value):
        L.check(L.lib.cnh_kernel_output(k, i, C.byref(name), C.byref(tgt), C.byref(sr), C.byref(reg)))
        b.append(outs[name.value])
    return a, b


@pytest.mark.parametrize("n,parts,shift", [(1, 1, 0), (77, 1, 0), (1000, 3, 0), (4099, 2, 1),
                                           ((1 << 20) + 3, 1, 0), ((1 << 22) + 517, 4, 0)])
def test_group_with_reducing_roots(dev, n, parts, shift):
    rng = np.random.default_rng(n)
    k = H.compile_group(ast_c1_reduced(), L.F64, 1)
    hx, hy, hw = (rng.standard_normal(n + shift) for _ in range(3))
    x, y, w = dev.array(hx), dev.array(hy), dev.array(hw)
    z = dev.empty((n + shift,), np.float64)
    res = dev.array(np.full(3, np.nan))
    cuts = [shift + (n * q) // parts for q in range(parts + 1)]
    pin, pout = [], []
    for q in range(parts):
        lo, cnt = cuts[q], cuts[q + 1] - cuts[q]
        view = lambda buf: L.Memref.dense(buf.ptr + 8 * lo, (cnt,))
        scalar = lambda i: L.Memref.dense(res.ptr + 8 * i, (1,))
        a, b = bind(k, {0: view(x), 1: view(y), 2: view(w)},
                    {10: view(z), 20: scalar(0), 21: scalar(1), 22: scalar(2)})
        pin.append(a)
        pout.append(b)
    H.launch_batched(k, 1, pin, [], pout)
    ex, ey, ew = hx[shift:], hy[shift:], hw[shift:]
    ez = ((2.5 * ex) - (0.5 * ey)) + (ex * ey)
    assert np.array_equal(z.get()[shift:], ez)
    got = res.get()
    for value, terms in ((got[0], ez * ew), (got[1], ez * ez)):
        assert abs(value - np.sum(terms)) <= 1e-13 * np.sum(np.abs(terms)) + 1e-300
    assert got[2] == np.max(np.abs(ez - ex))
    dev.free_all()


def test_sums_of_integers_are_exact(dev):
    """Every partial sum is an integer below 2^53: whatever the order, the result is the closed form."""
    n = (1 << 21) + 11
    b = AstBuilder(L.F64, 1)
    v = b.binary(L.OP_ADD, 10, b.leaf(0), b.scalar(1.0), is_temp=False)
    b.unary(L.OP_SUM_OF, 20, v, is_temp=False)
    sq = b.binary(L.OP_MUL, 100, v, v)
    b.unary(L.OP_SUM_OF, 21, sq, is_temp=False)
    k = H.compile_group(b.finish(), L.F64, 1)
    x = dev.array(np.arange(n, dtype=np.float64) % 1000)
    out = dev.empty((n,), np.float64)
    res = dev.array(np.zeros(2))
    a, o = bind(k, {0: x.memref()}, {10: out.memref(), 20: L.Memref.dense(res.ptr, (1,)),
                                      21: L.Memref.dense(res.ptr + 8, (1,))})
    for _ in range(2):                      # the partials of a launch do not leak into the next
        H.launch_batched(k, 1, [a], [], [o])
    v = (np.arange(n) % 1000 + 1).astype(np.int64)
    got = res.get()
    assert got[0] == float(v.sum()) and got[1] == float((v * v).sum())
    dev.free_all()


def test_reducing_roots_need_dense_operands(dev):
    b = AstBuilder(L.F64, 2)
    v = b.binary(L.OP_MUL, 10, b.leaf(0), b.scalar(2.0), is_temp=False)
    b.unary(L.OP_SUM_OF, 20, v, is_temp=False)
    k = H.compile_group(b.finish(), L.F64, 2)
    x = dev.array(np.ones((8, 16)))
    out = dev.empty((8, 16), np.float64)
    res = dev.array(np.zeros(1))
    strided = L.Memref.strided(x.ptr, (8, 8), (16, 1))          # every other half row
    a, o = bind(k, {0: strided}, {10: L.Memref.strided(out.ptr, (8, 8), (16, 1)),
                                  20: L.Memref.dense(res.ptr, (1,))})
    with pytest.raises(L.CnhError, match="dense"):
        H.launch_batched(k, 2, [a], [], [o])
    # a reducing root is never a temporary, and there is no integer form
    bad = AstBuilder(L.I32, 1)
    bad.unary(L.OP_SUM_OF, 20, bad.binary(L.OP_ADD, 10, bad.leaf(0), bad.scalar(1), is_temp=False), is_temp=False)
    with pytest.raises(L.CnhError):
        H.compile_group(bad.finish(), L.I32, 1)
    dev.free_all()


def test_partials_left_by_one_launch_are_summed_by_the_next(dev):
    """A reducing output with room for many elements keeps the launch's partial results; a later
    launch takes their sum as a run-time scalar, stores it, and computes with it."""
    n, room = 5000, 256
    rng = np.random.default_rng(3)
    hx, hy = rng.standard_normal(n), rng.standard_normal(n)
    p = AstBuilder(L.F64, 1)
    z = p.binary(L.OP_MUL, 10, p.leaf(0), p.scalar(2.0), is_temp=False)
    p.unary(L.OP_SUM_OF, 20, p.binary(L.OP_MUL, 100, z, z), is_temp=False)
    kp = H.compile_group(p.finish(), L.F64, 1)
    c = AstBuilder(L.F64, 1)
    t = c.binary(L.OP_MUL, 100, c.leaf(0), c.broadcast(5))
    c.binary(L.OP_ADD, 10, t, c.broadcast(6), is_temp=False)
    kc = H.compile_group(c.finish(), L.F64, 1)

    x, y = dev.array(hx), dev.array(hy)
    zb, ob = dev.empty((n,), np.float64), dev.empty((n,), np.float64)
    partials = dev.array(np.zeros(room))
    sc = dev.array(np.array([np.nan, 0.75]))                   # [folded sum, a plain scalar]
    a, o = bind(kp, {0: x.memref()}, {10: zb.memref(), 20: L.Memref.dense(partials.ptr, (room,))})
    H.launch_batched(kp, 1, [a], [], [o])
    hz = hx * 2.0
    got = partials.get()
    used = (n + 511) // 512                                   # one partial per workgroup of 512 elements
    assert np.all(got[used:] == 0.0) and np.count_nonzero(got[:used]) > used // 2
    assert abs(got.sum() - np.sum(hz * hz)) <= 1e-13 * np.sum(hz * hz)

    # the consumer: out = y * sum(partials) + sc[1]
    n_in, n_sc, n_out = C.c_int(), C.c_int(), C.c_int()
    L.check(L.lib.cnh_kernel_signature(kc, C.byref(n_in), C.byref(n_sc), C.byref(n_out)))
    assert (n_in.value, n_sc.value, n_out.value) == (1, 2, 1)
    sums = (L.ScalarSum * 2)()
    name = C.c_int()
    for i in range(2):
        L.check(L.lib.cnh_kernel_scalar(kc, i, C.byref(name)))
        if name.value == 5:
            sums[i].ptr, sums[i].count, sums[i].folded = partials.ptr, room, sc.ptr
        else:
            sums[i].ptr, sums[i].count, sums[i].folded = sc.ptr + 8, 1, None
    ins = (L.Memref * 1)(y.memref())
    outs = (L.Memref * 1)(ob.memref())
    L.check(L.lib.cnh_launch_group_sums(kc, 1, 1, ins, 2, sums, 1, outs, None))
    folded = sc.get()[0]
    assert abs(folded - got.sum()) <= 4e-16 * got.sum() * 8
    assert np.array_equal(ob.get(), hy * folded + 0.75)        # every workgroup used the same bits
    # too little room for the partial results of a launch is refused
    small = dev.array(np.zeros(8))
    a, o = bind(kp, {0: x.memref()}, {10: zb.memref(), 20: L.Memref.dense(small.ptr, (8,))})
    with pytest.raises(L.CnhError, match="room"):
        H.launch_batched(kp, 1, [a], [], [o])
    dev.free_all()


def test_fold_sums_adds_in_the_order_a_consuming_launch_uses(dev):
    """cnh_fold_sums is the value a launch would have formed from the same partial sums: the same
    bits as the `folded` store of cnh_launch_group_sums, for counts on every side of the lane and
    workgroup boundaries."""
    rng = np.random.default_rng(17)
    c = AstBuilder(L.F64, 1)
    c.binary(L.OP_MUL, 10, c.leaf(0), c.broadcast(5), is_temp=False)
    kc = H.compile_group(c.finish(), L.F64, 1)
    y, ob = dev.array(np.ones(100)), dev.empty((100,), np.float64)
    for count in (1, 2, 63, 64, 65, 255, 256, 257, 1000, 1024, 4097):
        hp = rng.standard_normal(count) * 10.0 ** rng.integers(-3, 4, count)
        partials = dev.array(hp)
        out = dev.array(np.array([np.nan, np.nan]))
        L.check(L.lib.cnh_fold_sums(partials.ptr, count, out.ptr, None))
        sums = (L.ScalarSum * 1)()
        sums[0].ptr, sums[0].count, sums[0].folded = partials.ptr, count, out.ptr + 8
        ins, outs = (L.Memref * 1)(y.memref()), (L.Memref * 1)(ob.memref())
        L.check(L.lib.cnh_launch_group_sums(kc, 1, 1, ins, 1, sums, 1, outs, None))
        got = out.get()
        if count > 1:
            assert got[0].tobytes() == got[1].tobytes(), count
        import math
        assert abs(got[0] - math.fsum(hp)) <= 1e-12 * np.abs(hp).sum(), count
        assert np.all(ob.get() == got[0])
    assert L.lib.cnh_fold_sums(None, 4, y.ptr, None) == -2
    assert L.lib.cnh_fold_sums(y.ptr, 0, y.ptr, None) == -2
    dev.free_all()


@pytest.mark.parametrize("n", [1, 5, 512, 513, 100003])
def test_a_scalar_statement_rides_on_the_launch_that_uses_it(dev, n):
    """CNH_OP_SCALAR_OF: alpha = s5 / s6 formed in registers by every lane, stored once; x2 = x + alpha p,
    r2 = r - alpha q and the partial sums of r2 . r2 from the same launch. Checked against NumPy in
    the same operand order, bit for bit (the sum to 1e-12)."""
    rng = np.random.default_rng(n)
    b = AstBuilder(L.F64, 1)
    alpha = b.binary(L.OP_DIV, 100, b.broadcast(5), b.broadcast(6))
    b.unary(L.OP_SCALAR_OF, 20, alpha, is_temp=False)
    t1 = b.binary(L.OP_MUL, 101, alpha, b.leaf(1))
    b.binary(L.OP_ADD, 7, b.leaf(2), t1, is_temp=False)
    t2 = b.binary(L.OP_MUL, 102, alpha, b.leaf(3))
    r_new = b.binary(L.OP_SUB, 8, b.leaf(4), t2, is_temp=False)
    b.unary(L.OP_SUM_OF, 9, b.binary(L.OP_MUL, 103, r_new, r_new), is_temp=False)
    k = H.compile_group(b.finish(), L.F64, 1)
    hp, hx, hq, hr = (rng.standard_normal(n) for _ in range(4))
    p, x, q, r = dev.array(hp), dev.array(hx), dev.array(hq), dev.array(hr)
    x2, r2 = dev.empty((n,), np.float64), dev.empty((n,), np.float64)
    # s5 as 37 partial sums, s6 a plain value
    h5 = rng.uniform(0.5, 1.5, 37)
    s5, s6 = dev.array(h5), dev.array(np.array([1.75]))
    folded = dev.array(np.array([np.nan]))
    alpha_out = dev.array(np.array([np.nan, 7.0, 7.0]))          # one element is written, no more
    rr = dev.array(np.array([np.nan]))
    ins, outs = bind(k, {1: p.memref(), 2: x.memref(), 3: q.memref(), 4: r.memref()},
                     {20: L.Memref.dense(alpha_out.ptr, (1,)), 7: x2.memref(), 8: r2.memref(),
                      9: L.Memref.dense(rr.ptr, (1,))})
    sums = (L.ScalarSum * 2)()
    name = C.c_int()
    for i in range(2):
        L.check(L.lib.cnh_kernel_scalar(k, i, C.byref(name)))
        if name.value == 5:
            sums[i].ptr, sums[i].count, sums[i].folded = s5.ptr, 37, folded.ptr
        else:
            sums[i].ptr, sums[i].count, sums[i].folded = s6.ptr, 1, None
    ia, oa = (L.Memref * 4)(*ins), (L.Memref * 4)(*outs)
    L.check(L.lib.cnh_launch_group_sums(k, 1, 4, ia, 2, sums, 4, oa, None))
    S = folded.get()[0]
    chk = dev.array(np.array([np.nan]))
    L.check(L.lib.cnh_fold_sums(s5.ptr, 37, chk.ptr, None))
    assert S.tobytes() == chk.get()[0].tobytes()
    a = S / 1.75
    got_alpha = alpha_out.get()
    assert got_alpha[0] == a and got_alpha[1] == 7.0 and got_alpha[2] == 7.0
    want_r = hr - a * hq
    assert np.array_equal(x2.get(), hx + a * hp) and np.array_equal(r2.get(), want_r)
    assert abs(rr.get()[0] - np.sum(want_r * want_r)) <= 1e-12 * np.sum(want_r * want_r)
    # the plain launch (scalars by pointer) stores the same alpha
    s5v = dev.array(np.array([S]))
    alpha_out.put(np.array([np.nan, 7.0, 7.0]))
    names = []
    for i in range(2):
        L.check(L.lib.cnh_kernel_scalar(k, i, C.byref(name)))
        names.append(name.value)
    ptrs = L.vparr([s5v.ptr if nm == 5 else s6.ptr for nm in names])
    L.check(L.lib.cnh_launch_group(k, 1, 4, ia, 2, ptrs, 1, 4, oa, None))
    assert alpha_out.get()[0] == a and np.array_equal(r2.get(), want_r)
    # a value with an index cannot be a scalar output, and strided launches refuse such a group
    bad = AstBuilder(L.F64, 1)
    v = bad.binary(L.OP_MUL, 10, bad.leaf(0), bad.broadcast(5), is_temp=False)
    bad.unary(L.OP_SCALAR_OF, 20, v, is_temp=False)
    with pytest.raises(L.CnhError):
        H.compile_group(bad.finish(), L.F64, 1)
    dev.free_all()
