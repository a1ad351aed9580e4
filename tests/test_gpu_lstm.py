"""GPU parity: the LSTM forward step (gate matmatmul + fused gate groups) vs a NumPy/host-libm
restatement of examples/lstm_forward.py:29-49 upstream."""
import math

import numpy as np
import pytest

import bench
from charmnumeric_amd import _lib as L
from tests import helpers as H

pytestmark = pytest.mark.gpu

_exp = np.vectorize(math.exp, otypes=[np.float64])    # host libm, as the reference JIT resolves it
_tanh = np.vectorize(math.tanh, otypes=[np.float64])


def _reference(steps, batch, nin, d, seed=5, extended=True):
    X = H.np_uniform(steps * batch * nin, seed, 0, -1.0, 1.0).reshape(steps, batch, nin)
    Wih = H.np_uniform(4 * d * nin, seed, 1, -1 / 32, 1 / 32).reshape(4 * d, nin)
    Whh = H.np_uniform(4 * d * d, seed, 2, -1 / 32, 1 / 32).reshape(4 * d, d)
    W = np.concatenate([Wih.T, Whh.T], axis=0)
    Hout = np.zeros((steps, batch, d))
    Cc = np.zeros((steps, batch, d))
    IFOG = np.zeros((steps, batch, 4 * d))
    for t in range(steps):
        prev = Hout[t - 1] if t > 0 else np.zeros((batch, d))
        hin = np.concatenate([X[t], prev], axis=1)
        if extended:
            IFOG[t] = (hin.astype(np.longdouble) @ W.astype(np.longdouble)).astype(np.float64)
        else:
            IFOG[t] = hin @ W          # BLAS, fp64: at the full shape extended precision takes minutes
        f3 = 1.0 / (1.0 + _exp(IFOG[t][:, :3 * d] * -1))
        g = _tanh(IFOG[t][:, 3 * d:])
        Cc[t] = f3[:, :d] * g
        if t > 0:
            Cc[t] = Cc[t] + f3[:, d:2 * d] * Cc[t - 1]
        Hout[t] = f3[:, 2 * d:3 * d] * _tanh(Cc[t])
    return Hout, Cc, IFOG, np.abs(X).max()


def test_lstm_forward_full_shape_four_steps(dev):
    """Batch 256, input 1024, hidden 1024 (the benchmark's shape), 4 steps: gate pre-activations
    within 1e-12 * sum_k |a_ik| |w_kj|, cell and hidden states at rtol 1e-12."""
    steps, batch, nin, d = 4, 256, 1024, 1024
    got = bench.run_lstm(L, steps=steps, batch=batch, nin=nin, d=d, timed=False, keep=True)
    Hout, Cc, IFOG, _ = _reference(steps, batch, nin, d, extended=False)
    Wih = H.np_uniform(4 * d * nin, 5, 1, -1 / 32, 1 / 32).reshape(4 * d, nin)
    Whh = H.np_uniform(4 * d * d, 5, 2, -1 / 32, 1 / 32).reshape(4 * d, d)
    Wabs = np.abs(np.concatenate([Wih.T, Whh.T], axis=0))
    X = H.np_uniform(steps * batch * nin, 5, 0, -1.0, 1.0).reshape(steps, batch, nin)
    for t in range(steps):
        prev = Hout[t - 1] if t > 0 else np.zeros((batch, d))
        bound = np.abs(np.concatenate([X[t], prev], axis=1)) @ Wabs
        # the device's own h feeds the next step's product: its deviation (<= 1e-12 relative) adds
        # at most 1e-12 * sum |w| <= 1e-12 * d / 32 on top
        assert np.all(np.abs(got["IFOG"][t] - IFOG[t]) <= 1e-12 * (bound + d / 32.0)), t
    assert np.allclose(got["C"], Cc, rtol=1e-12, atol=1e-13)
    assert np.allclose(got["Hout"], Hout, rtol=1e-12, atol=1e-13)
    assert np.all(np.abs(got["Hout"]) <= 1.0)


@pytest.mark.parametrize("fused", [True, False], ids=["one-gate-launch", "six-gate-launches"])
@pytest.mark.parametrize("steps,batch,nin,d", [(3, 8, 16, 16), (4, 64, 64, 32), (2, 70, 24, 40)])
def test_lstm_forward_small(dev, steps, batch, nin, d, fused):
    got = bench.run_lstm(L, steps=steps, batch=batch, nin=nin, d=d, timed=False, keep=True, fused=fused)
    Hout, Cc, IFOG, _ = _reference(steps, batch, nin, d)
    # gate pre-activations: 1e-12 relative to sum |a||b| (here <= (nin + d) / 32)
    assert np.max(np.abs(got["IFOG"] - IFOG)) <= 1e-12 * (nin + d) / 32
    # step 0 has h0 = c0 = 0, so C[0] = i * g exactly in terms of the device's own gates
    assert np.allclose(got["C"], Cc, rtol=1e-12, atol=1e-13)
    assert np.allclose(got["Hout"], Hout, rtol=1e-12, atol=1e-13)
    assert np.all(np.abs(got["Hout"]) <= 1.0)


def test_gemm_full_lstm_shape_properties(dev):
    """M=256, K=2048, N=4096 (the C5 gate shape): ones closed form and linearity in A."""
    M, K, N = 256, 2048, 4096
    A = dev.array(np.ones((M, K)))
    B = dev.array(np.ones((K, N)))
    Cz = dev.array(np.zeros((M, N)))
    L.check(L.lib.cnh_gemm_acc(L.F64, M, N, K, A.ptr, K, B.ptr, N, Cz.ptr, N, None))
    assert np.all(Cz.get() == float(K))
    rng = np.random.default_rng(0)
    a1 = rng.integers(-4, 5, (M, K)).astype(np.float64)   # small integers: products and sums exact
    b1 = rng.integers(-4, 5, (K, N)).astype(np.float64)
    A.put(a1)
    B.put(b1)
    Cz.put(np.zeros((M, N)))
    L.check(L.lib.cnh_gemm_acc(L.F64, M, N, K, A.ptr, K, B.ptr, N, Cz.ptr, N, None))
    assert np.array_equal(Cz.get(), a1 @ b1)               # exact in fp64, any summation order
    dev.free_all()


@pytest.mark.parametrize("steps,batch,nin,d", [(3, 256, 1024, 1024), (4, 128, 512, 512), (3, 64, 256, 256),
                                               (2, 192, 64, 64),
                                               # more tiles than CUs: one set of eight wavefronts per workgroup
                                               (2, 512, 1024, 1024), (2, 576, 256, 256),
                                               # 1024 tiles and more: four wavefronts of 32 x 32
                                               (2, 1024, 1024, 1024)])
def test_gate_statements_in_the_products_epilogue_change_no_bit(dev, steps, batch, nin, d):
    """One launch per step (the gate statements evaluated on the product's tile of sums before its
    workgroup ends, a workgroup's 64 columns being 16 of each gate) against the product and the gate
    launch one after the other: every array of the program, bit for bit."""
    one = bench.run_lstm(L, steps=steps, batch=batch, nin=nin, d=d, timed=False, keep=True, epilogue=True)
    two = bench.run_lstm(L, steps=steps, batch=batch, nin=nin, d=d, timed=False, keep=True, epilogue=False)
    assert one["launches_per_step"] == 1 and two["launches_per_step"] == 2
    for name in ("IFOG", "IFOGf", "C", "Ct", "Hout", "Hin"):
        assert np.array_equal(one[name], two[name]), name
    assert np.any(one["Hout"][-1] != 0.0)


def test_shapes_the_fused_product_does_not_take_fall_back_to_two_launches(dev):
    """70 rows are no multiple of the 64-row tile: cnh_launch_product_group answers -17 and launches nothing."""
    got = bench.run_lstm(L, steps=2, batch=70, nin=24, d=24, timed=False, keep=True, epilogue=True)
    assert got["launches_per_step"] == 2
    Hout, Cc, IFOG, _ = _reference(2, 70, 24, 24)
    assert np.allclose(got["Hout"], Hout, rtol=1e-12, atol=1e-13)


# ---- cnh_launch_product_group called directly ----

def _affine_group(blocks):
    """out_b = C_b * 2 + E for every column block b of the product (leaves 1..blocks are the blocks,
    leaf 9 is E), and one more root that adds all blocks up."""
    from charmnumeric_amd.astbuild import AstBuilder
    b = AstBuilder(L.F64, 2)
    outs, total = [], None
    for q in range(blocks):
        t = b.binary(L.OP_MUL, 100 + q, b.leaf(1 + q), b.scalar(2.0))
        outs.append(b.binary(L.OP_ADD, 20 + q, t, b.leaf(9), is_temp=False))
        total = b.leaf(1 + q) if total is None else b.binary(L.OP_ADD, 110 + q, total, b.leaf(1 + q))
    b.binary(L.OP_SUB, 30, total, b.leaf(9), is_temp=False)
    return b.finish()


def _bind(k, ins, outs):
    import ctypes as C
    n_in, n_sc, n_out = C.c_int(), C.c_int(), C.c_int()
    L.check(L.lib.cnh_kernel_signature(k, C.byref(n_in), C.byref(n_sc), C.byref(n_out)))
    name, has, tgt, sr = C.c_int(), C.c_int(), C.c_int(), C.c_int()
    reg = L.Region()
    ia, oa = (L.Memref * max(1, n_in.value))(), (L.Memref * max(1, n_out.value))()
    blocks = (C.c_int32 * max(1, n_in.value))()
    for i in range(n_in.value):
        L.check(L.lib.cnh_kernel_input(k, i, C.byref(name), C.byref(has), C.byref(reg)))
        ia[i] = ins[name.value]
        blocks[i] = name.value - 1 if name.value < 9 else -1
    for i in range(n_out.value):
        L.check(L.lib.cnh_kernel_output(k, i, C.byref(name), C.byref(tgt), C.byref(sr), C.byref(reg)))
        oa[i] = outs[name.value]
    return n_in.value, ia, blocks, n_out.value, oa


@pytest.mark.parametrize("blocks", [1, 2, 4])
@pytest.mark.parametrize("M,N,K", [(128, 256, 96), (128, 256, 48), (1280, 1024, 64), (1024, 4096, 32)])
def test_product_with_a_group_by_direct_calls(dev, blocks, M, N, K):
    """C = A @ B and a group on C's column blocks in one launch, all three forms of the kernel (by
    tile count and K), C inside a wider array (ldc > N), E read with a row stride: against NumPy to
    1e-12 of sum |a||b|, and against the product and the group as two launches bit for bit."""
    rng = np.random.default_rng(7 * blocks + M)
    n = N // blocks
    hA, hB, hE = rng.uniform(-1, 1, (M, K)), rng.uniform(-1, 1, (K, N)), rng.uniform(-1, 1, (M, n + 6))
    ldc = N + 64
    A, B, E = dev.array(hA), dev.array(hB), dev.array(hE)
    results = []
    k = H.compile_group(_affine_group(blocks), L.F64, 2)
    for fused in (True, False):
        Cw = dev.array(np.zeros((M, ldc)))
        outs = [dev.array(np.zeros((M, n))) for _ in range(blocks + 1)]
        job = (L.GemmJob * 1)()
        job[0].M, job[0].N, job[0].K = M, N, K
        job[0].A, job[0].lda, job[0].B, job[0].ldb = A.ptr, K, B.ptr, N
        job[0].C, job[0].ldc = Cw.ptr + 32 * 8, ldc
        ins = {1 + q: L.Memref.strided(Cw.ptr + (32 + q * n) * 8, (M, n), (ldc, 1)) for q in range(blocks)}
        ins[9] = L.Memref.strided(E.ptr + 3 * 8, (M, n), (n + 6, 1))
        om = {20 + q: outs[q].memref() for q in range(blocks)}
        om[30] = outs[blocks].memref()
        n_in, ia, blk, n_out, oa = _bind(k, ins, om)
        if fused:
            L.check(L.lib.cnh_launch_product_group(k, job, blocks, 2, n_in, ia, blk, 0, None, 1, n_out, oa, None))
        else:
            L.check(L.lib.cnh_gemm_batch(L.F64, 1, job, 1, None))
            L.check(L.lib.cnh_launch_group(k, 2, n_in, ia, 0, None, 1, n_out, oa, None))
        dev.sync()
        results.append([Cw.get()] + [o.get() for o in outs])
    for a, b_ in zip(*results):
        assert np.array_equal(a, b_)
    Cw, outs = results[0][0], results[0][1:]
    want = hA @ hB
    bound = 1e-12 * (np.abs(hA) @ np.abs(hB))
    got = Cw[:, 32:32 + N]
    assert np.all(np.abs(got - want) <= bound)
    assert np.all(Cw[:, :32] == 0) and np.all(Cw[:, 32 + N:] == 0)
    Eh = hE[:, 3:3 + n]
    for q in range(blocks):
        assert np.array_equal(outs[q], got[:, q * n:(q + 1) * n] * 2.0 + Eh)
    total = got[:, :n].copy()
    for q in range(1, blocks):
        total = total + got[:, q * n:(q + 1) * n]
    assert np.array_equal(outs[blocks], total - Eh)
    dev.free_all()


def test_product_with_a_group_refuses_what_it_cannot_run(dev):
    """-17 (nothing launched, the caller issues two launches) for shapes the fused kernel is not built
    for; -4 / -2 for arguments that are wrong whatever the shape."""
    M, N, K, blocks = 128, 256, 64, 4
    n = N // blocks
    A, B, Cw, E = (dev.array(np.zeros(s)) for s in ((M, K), (K, N), (M, N), (M, n)))
    outs = [dev.array(np.full((M, n), 7.0)) for _ in range(blocks + 1)]
    k = H.compile_group(_affine_group(blocks), L.F64, 2)
    ins = {1 + q: L.Memref.strided(Cw.ptr + q * n * 8, (M, n), (N, 1)) for q in range(blocks)}
    ins[9] = E.memref()
    om = {20 + q: outs[q].memref() for q in range(blocks)}
    om[30] = outs[blocks].memref()
    n_in, ia, blk, n_out, oa = _bind(k, ins, om)

    def call(m=M, nn=N, kk=K, nb=blocks, a_off=0, blocks_arg=None, n_in_arg=None):
        job = (L.GemmJob * 1)()
        job[0].M, job[0].N, job[0].K = m, nn, kk
        job[0].A, job[0].lda, job[0].B, job[0].ldb = A.ptr + a_off, K, B.ptr, N
        job[0].C, job[0].ldc = Cw.ptr, N
        return L.lib.cnh_launch_product_group(k, job, nb, 2, n_in if n_in_arg is None else n_in_arg, ia,
                                              blk if blocks_arg is None else blocks_arg, 0, None, 1, n_out, oa, None)

    assert call(m=M - 8) == -17                    # rows no multiple of 64
    assert call(kk=K - 8) == -17                   # K no multiple of 16
    assert call(a_off=8) == -17                    # A not 16-byte aligned
    assert call(nb=3) == -17 and call(nb=8) == -17
    assert call(nb=2) == -17                       # the group's memrefs are a quarter of the columns wide
    import ctypes as C
    bad = (C.c_int32 * n_in)(*[9 if b >= 0 else -1 for b in blk])
    assert call(blocks_arg=bad) == -4              # a column block that does not exist
    assert call(n_in_arg=n_in - 1) == -4
    L.check(L.lib.cnh_set_option(b"product_statements", 0))
    try:
        assert call() == -17
    finally:
        L.check(L.lib.cnh_set_option(b"product_statements", 1))
    dev.sync()
    for o in outs:                                  # none of the refused calls stored anything
        assert np.all(o.get() == 7.0)
    L.check(call())
    dev.sync()
    assert np.all(outs[0].get() == 0.0)
    dev.free_all()
