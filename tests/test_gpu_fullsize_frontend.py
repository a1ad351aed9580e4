"""The elementwise, CG and LSTM configurations at their full sizes THROUGH THE FRONTEND: statements
written with the NumPy-like operators, shipped as a statement log, planned, merged and routed by the
host executor. At these sizes the executor picks what small shapes never reach: the two-level fold
of 32 768 partials, the matvec that stages its vector in LDS, the product whose workgroups split
the K steps over two sets of wavefronts, buffer loads."""
import math
import os

import numpy as np
import pytest

import bench
import charmnumeric_amd as cnp
from tests import helpers as H
from tests.test_gpu_lstm import _reference as lstm_reference

pytestmark = pytest.mark.gpu

THREADS = min(os.cpu_count() or 1, 16)


def _connect(odf=4, fusion=True, flat_rank3=True, pipeline=False):
    cnp.reset()
    it = cnp.CharmNumericInterface(device=0)
    it.set_layout(flat_rank3)
    it.connect(odf=odf)
    it.set_fusion(fusion)
    if pipeline:
        it.set_pipeline(True)
    return it


@pytest.mark.parametrize("fusion", [True, False], ids=["fused", "node-by-node"])
def test_c1_2p24_in_four_partitions(fusion):
    """examples/simple.py upstream at 2^24 elements: z bit for bit, sum(z), z @ ones and z @ z within
    1e-12 * sum|terms| of the exactly rounded sums."""
    n = 1 << 24
    itf = _connect(4, fusion)
    try:
        x = cnp.random.uniform((n,), seed=0, stream=0, low=-1.0, high=1.0)
        y = cnp.random.uniform((n,), seed=0, stream=1, low=-1.0, high=1.0)
        ones = cnp.ones((n,))
        z = 2.5 * x - 0.5 * y + x * y
        s_dot = z @ ones
        zz = z @ z
        cnp.execute(itf)
        s_sum = cnp.sum(z)                      # on the array that exists by now: a pass of its own
        assert itf.array_info(z.name)["tile"] == n // 4
        hx, hy = H.np_uniform(n, 0, 0, -1.0, 1.0), H.np_uniform(n, 0, 1, -1.0, 1.0)
        hz = ((2.5 * hx) - (0.5 * hy)) + (hx * hy)
        got = z.get(itf)
        bad = np.count_nonzero(got != hz)
        assert bad == 0, f"{bad} elements of z differ"
        exact_sum = math.fsum(hz)
        abs_sum = float(np.sum(np.abs(hz)))
        for name, handle in (("z @ ones", s_dot), ("sum(z)", s_sum)):
            v = handle.get(itf).item()
            assert abs(v - exact_sum) <= 1e-12 * abs_sum, (name, v, exact_sum)
        sq = hz * hz
        v = zz.get(itf).item()
        assert abs(v - math.fsum(sq)) <= 1e-12 * float(np.sum(sq)), (v,)
        if fusion:
            # the reductions rode on the statement: one launch with two reducing roots
            assert itf.stats()["group_launches"] >= 1
        del x, y, ones, z, s_dot, s_sum, zz
    finally:
        cnp.reset()
        itf.close()


@pytest.mark.parametrize("fusion", [True, False], ids=["fused", "node-by-node"])
def test_cg_n16384_ten_iterations_as_the_example_writes_them(cpu_cg_system, fusion):
    """examples/cg.py:40-52 upstream with cnp operators on the benchmark's system: alpha, beta and
    r.r of every iteration and x at the end against the oracle's kernels running the same
    iterations (same bounds as the direct-call test of this configuration)."""
    n, iters = 16384, 10
    itf = _connect(4, fusion)
    try:
        A = cnp.random.cg_matrix(n, 2)
        b = cnp.random.uniform((n,), seed=2, stream=1, low=-1.0, high=1.0)
        x = cnp.zeros((n,))
        r = b.copy()
        p = b.copy()
        rtr = r @ r
        handles = []
        for _ in range(iters):
            Ap = A @ p
            pAp = p @ Ap
            alpha = rtr / pAp
            x = x + alpha * p
            r = r - alpha * Ap
            rtr_new = r @ r
            beta = rtr_new / rtr
            p = r + beta * p
            rtr = rtr_new
            handles.append((alpha, beta, rtr))
        cnp.execute(itf)
        assert itf.array_info(A.name)["tile"] == 8192
        trace = {"alpha": [a.get(itf).item() for a, _, _ in handles],
                 "beta": [b_.get(itf).item() for _, b_, _ in handles],
                 "rtr": [r_.get(itf).item() for _, _, r_ in handles],
                 "x": x.get(itf)}
        _, _, _, cpu_trace = bench.cpu_cg(cpu_cg_system, n, iters, THREADS, keep_x_at=iters)
        par = bench.cg_parity(trace, cpu_trace, cpu_trace["rtr0"])
        assert par["x_max_rel_diff"] <= 1e-10, par
        assert par["scalar_iterations"] >= 4, par
        assert par["alpha_max_rel_dev"] <= 1e-10, par
        assert par["beta_max_rel_dev"] <= 1e-10, par
        assert par["rtr_max_rel_dev"] <= 1e-10, par
        rr = trace["rtr"]
        assert all(rr[i + 1] < rr[i] for i in range(par["scalar_iterations"])), rr
        del A, b, x, r, p, rtr, Ap, pAp, alpha, beta, rtr_new, handles
    finally:
        cnp.reset()
        itf.close()


@pytest.mark.parametrize("flat_rank3", [True, False], ids=["one-block", "buffer-per-partition"])
def test_lstm_forward_full_shape_through_the_frontend(flat_rank3):
    """examples/lstm_forward.py:29-49 upstream, batch 256, input 1024, hidden 1024, three steps:
    gate pre-activations within 1e-12 * sum_k |a_ik| |w_kj|, cell and hidden states at rtol 1e-12."""
    steps, b, word, d = 3, 256, 1024, 1024
    itf = _connect(4, True, flat_rank3)
    try:
        hX = H.np_uniform(steps * b * word, 5, 0, -1.0, 1.0).reshape(steps, b, word)
        Wih = H.np_uniform(4 * d * word, 5, 1, -1 / 32, 1 / 32).reshape(4 * d, word)
        Whh = H.np_uniform(4 * d * d, 5, 2, -1 / 32, 1 / 32).reshape(4 * d, d)
        hW = np.concatenate([Wih.T, Whh.T], axis=0)
        X, W = cnp.array(hX), cnp.array(hW)
        h0 = cnp.zeros((1, d))
        Hin = cnp.zeros((steps, b, word + d))
        Hout = cnp.zeros((steps, b, d))
        IFOG = cnp.zeros((steps, b, 4 * d))
        IFOGf = cnp.zeros((steps, b, 4 * d))
        Cs = cnp.zeros((steps, b, d))
        Ct = cnp.zeros((steps, b, d))
        for t in range(steps):
            prev = cnp.tile(h0, (b, 1)) if t == 0 else Hout[t - 1]
            Hin[t, :, :word] = X[t]
            Hin[t, :, word:] = prev
            IFOG[t] = Hin[t].dot(W)
            IFOGf[t, :, : 3 * d] = 1.0 / (1.0 + cnp.exp(-IFOG[t, :, : 3 * d]))
            IFOGf[t, :, 3 * d:] = cnp.tanh(IFOG[t, :, 3 * d:])
            Cs[t] = IFOGf[t, :, :d] * IFOGf[t, :, 3 * d:]
            if t > 0:
                Cs[t] += IFOGf[t, :, d: 2 * d] * Cs[t - 1]
            Ct[t] = cnp.tanh(Cs[t])
            Hout[t] = IFOGf[t, :, 2 * d: 3 * d] * Ct[t]
        gI, gC, gH = IFOG.get(itf), Cs.get(itf), Hout.get(itf)
        wH, wC, wI, _ = lstm_reference(steps, b, word, d, extended=False)
        Wabs = np.abs(hW)
        for t in range(steps):
            prev = wH[t - 1] if t > 0 else np.zeros((b, d))
            bound = np.abs(np.concatenate([hX[t], prev], axis=1)) @ Wabs
            assert np.all(np.abs(gI[t] - wI[t]) <= 1e-12 * (bound + d / 32.0)), t
        assert np.allclose(gC, wC, rtol=1e-12, atol=1e-13)
        assert np.allclose(gH, wH, rtol=1e-12, atol=1e-13)
        del X, W, h0, Hin, Hout, IFOG, IFOGf, Cs, Ct, prev
    finally:
        cnp.reset()
        itf.close()


def _lstm_arrays(itf, steps, b, word, d):
    """The program of examples/lstm_forward.py upstream; returns every array it leaves, on the host."""
    hX = H.np_uniform(steps * b * word, 5, 0, -1.0, 1.0).reshape(steps, b, word)
    hW = H.np_uniform((word + d) * 4 * d, 5, 1, -1 / 32, 1 / 32).reshape(word + d, 4 * d)
    X, W = cnp.array(hX), cnp.array(hW)
    h0 = cnp.zeros((1, d))
    Hin = cnp.zeros((steps, b, word + d))
    Hout = cnp.zeros((steps, b, d))
    IFOG = cnp.zeros((steps, b, 4 * d))
    IFOGf = cnp.zeros((steps, b, 4 * d))
    Cs = cnp.zeros((steps, b, d))
    Ct = cnp.zeros((steps, b, d))
    for t in range(steps):
        prev = cnp.tile(h0, (b, 1)) if t == 0 else Hout[t - 1]
        Hin[t, :, :word] = X[t]
        Hin[t, :, word:] = prev
        IFOG[t] = Hin[t].dot(W)
        IFOGf[t, :, : 3 * d] = 1.0 / (1.0 + cnp.exp(-IFOG[t, :, : 3 * d]))
        IFOGf[t, :, 3 * d:] = cnp.tanh(IFOG[t, :, 3 * d:])
        Cs[t] = IFOGf[t, :, :d] * IFOGf[t, :, 3 * d:]
        if t > 0:
            Cs[t] += IFOGf[t, :, d: 2 * d] * Cs[t - 1]
        Ct[t] = cnp.tanh(Cs[t])
        Hout[t] = IFOGf[t, :, 2 * d: 3 * d] * Ct[t]
    got = {name: a.get(itf) for name, a in (("Hin", Hin), ("IFOG", IFOG), ("IFOGf", IFOGf), ("C", Cs),
                                            ("Ct", Ct), ("Hout", Hout))}
    del X, W, h0, Hin, Hout, IFOG, IFOGf, Cs, Ct, prev
    return got


@pytest.mark.parametrize("steps,b,word,d", [(4, 256, 1024, 1024), (3, 128, 256, 256), (3, 64, 192, 64)])
def test_an_lstm_step_is_one_launch_and_the_same_bits_as_two(steps, b, word, d):
    """The gate statements of a step ride on the step's product (the product's launch evaluates them
    on its tiles of sums); with that switched off the product and the merged statements are two
    launches. Every array of the program agrees bit for bit."""
    from charmnumeric_amd import _lib as L
    runs = {}
    for on in (1, 0):
        itf = _connect(4, True, True)
        try:
            L.check(L.lib.cnh_set_option(b"product_statements", on))
            itf.set_trace()
            runs[on] = _lstm_arrays(itf, steps, b, word, d)
            trace = itf.trace()
            if os.environ.get("CHARMNUMERIC_SOLVER", "0") in ("", "0"):
                assert sum(" with_statements" in ln for ln in trace) == (steps if on else 0)
                assert sum(" in_product" in ln for ln in trace) == (steps if on else 0)
        finally:
            L.check(L.lib.cnh_set_option(b"product_statements", 1))
            cnp.reset()
            itf.close()
    for name in runs[1]:
        assert np.array_equal(runs[1][name], runs[0][name]), name
    assert np.any(runs[1]["Hout"][-1] != 0.0)


@pytest.mark.parametrize("flush_at", [3, 5, 7, 11, 16])
def test_where_the_frontend_cuts_its_messages_does_not_change_what_is_merged(flush_at):
    """Automatic flushes every few statements cut the recording anywhere — right behind a product,
    in the middle of the gate statements: the product waits for the statements that read it, so
    every step is still one launch, and the arrays are the same bits as with one message."""
    from charmnumeric_amd import _lib as L
    steps, b, word, d = 3, 128, 256, 256
    runs = {}
    for cut in (flush_at, 100000):
        itf = _connect(4, True, True)
        try:
            cnp.set_auto_flush(itf, cut)
            itf.set_trace()
            runs[cut] = _lstm_arrays(itf, steps, b, word, d)
            if os.environ.get("CHARMNUMERIC_SOLVER", "0") in ("", "0"):
                assert sum(" with_statements" in ln for ln in itf.trace()) == steps
        finally:
            cnp.reset()
            itf.close()
    for name in runs[flush_at]:
        assert np.array_equal(runs[flush_at][name], runs[100000][name]), name
