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
