"""The native planner of the statement log (csrc/stmtlog.cpp behind cnx_receive_log) against an
independent Python model of the same rules (tests/planner_model.py): every DAG message it plans,
byte for byte, over the example programs and over random programs, with and without automatic
flushes. Runs on the executor's dry mode: no GPU."""
import random
import struct

import numpy as np
import pytest

import charmnumeric_amd as cnp
from charmnumeric_amd import _lib as L
from charmnumeric_amd import lazy

from tests import planner_model


class Recorded:
    """An interface in dry mode whose log traffic is mirrored into the model."""

    def __init__(self, auto_flush=None):
        cnp.reset()
        self.itf = cnp.CharmNumericInterface(device=-1)
        self.itf.connect(odf=4)
        self.itf.set_capture()
        self.model = planner_model.Planner()
        self.expected = []
        inner = self.itf.send_log

        def send_log(log, window=-1):
            msg = self.model.feed(log, window)
            if msg is not None:
                self.expected.append(msg)
            inner(log, window)

        self.itf.send_log = send_log
        if auto_flush:
            cnp.set_auto_flush(self.itf, auto_flush)

    def check(self):
        cnp.execute(self.itf)
        got = self.itf.captured()
        assert len(got) == len(self.expected)
        for i, (g, e) in enumerate(zip(got, self.expected)):
            assert g == e, f"message {i} differs"
        n = len(got)
        self.expected.clear()
        return n

    def close(self):
        cnp.reset()
        self.itf.close()


@pytest.fixture(params=[None, 5, 12, 48], ids=lambda v: f"autoflush={v}")
def rec(request):
    r = Recorded(request.param)
    yield r
    r.close()


def test_jacobi_loops_with_named_updates(rec):
    u = cnp.zeros((40, 40))
    f = cnp.zeros((40, 40))
    for _ in range(12):
        upd = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
        u[1:-1, 1:-1] = upd + f[1:-1, 1:-1]
    v = cnp.zeros((12, 12, 12))
    for _ in range(5):
        v[1:-1, 1:-1, 1:-1] = (v[:-2, 1:-1, 1:-1] + v[2:, 1:-1, 1:-1] + v[1:-1, :-2, 1:-1]
                               + v[1:-1, 2:, 1:-1] + v[1:-1, 1:-1, :-2] + v[1:-1, 1:-1, 2:]) * (1.0 / 6.0)
    assert rec.check() >= 1


def test_cg_iterations(rec):
    n = 64
    A = cnp.random.cg_matrix(n, 3)
    b = cnp.random.uniform((n,), seed=1)
    x = cnp.zeros((n,))
    r = b - A @ x
    p = r.copy()
    rtr = r.dot(r)
    for _ in range(6):
        Ap = A @ p
        alpha = rtr / p.dot(Ap)
        x = x + alpha * p
        r = r - alpha * Ap
        rtr_new = r.dot(r)
        beta = rtr_new / rtr
        p = r + beta * p
        rtr = rtr_new
    rec.check()


def test_lstm_steps(rec):
    n, b, word, d = 6, 4, 8, 8
    X = cnp.zeros((n, b, word))
    W = cnp.zeros((word + d, 4 * d))
    h0 = cnp.zeros((1, d))
    Hin, Hout = cnp.zeros((n, b, word + d)), cnp.zeros((n, b, d))
    IFOG, IFOGf = cnp.zeros((n, b, 4 * d)), cnp.zeros((n, b, 4 * d))
    Cs, Ct = cnp.zeros((n, b, d)), cnp.zeros((n, b, d))
    for t in range(n):
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
    rec.check()


def test_results_kept_dropped_and_reused(rec):
    a = cnp.array(np.arange(24.0).reshape(4, 6))       # an upload in the middle of the log
    b = cnp.full((4, 6), 2.0)
    c = a + b                   # kept: becomes an array
    d = (a * b) - c             # its product is a temporary
    del c
    e = d * 2.0
    f = e + d                   # d read twice, by two operations of one group
    g = cnp.sum(f)
    s = a[1:3, ::2] * 3.0       # strided slice
    a[0:2, 0:3] = s + 1.0
    h = a * g                   # a one-element array as a run-time scalar
    unused = h + 1.0            # never read, handle dropped: dead code
    del unused
    a[...] = 7.0
    col = cnp.zeros((4, 1))
    vec = cnp.zeros((4,))
    vec[:] = col
    rec.check()
    del d, e, f, h, s
    rec.check()


@pytest.mark.parametrize("seed", range(12))
def test_random_programs(seed):
    rng = random.Random(seed)
    r = Recorded(rng.choice([None, 3, 7, 16, 40]))
    try:
        shapes = [(8,), (6, 4), (3, 4, 5)]
        live = {sh: [cnp.zeros(sh) for _ in range(2)] for sh in shapes}

        def operand(sh):
            kind = rng.random()
            if kind < 0.2:
                return rng.choice([0.5, 2, -1.25])
            x = rng.choice(live[sh])
            if kind < 0.45:
                return x[tuple(slice(None) for _ in sh)]
            return x

        def window(sh):
            return tuple(slice(rng.randrange(0, 2), s - rng.randrange(0, 2)) for s in sh)

        for _ in range(rng.randrange(40, 160)):
            sh = rng.choice(shapes)
            act = rng.random()
            if act < 0.45:
                a, b = operand(sh), operand(sh)
                if isinstance(a, (int, float)) and isinstance(b, (int, float)):
                    a = rng.choice(live[sh])
                op = rng.choice(["+", "-", "*", "/"])
                res = {"+": lambda: a + b, "-": lambda: a - b, "*": lambda: a * b, "/": lambda: a / b}[op]()
                if rng.random() < 0.6:
                    live[sh].append(res)
            elif act < 0.55:
                live[sh].append(cnp.tanh(rng.choice(live[sh])))
            elif act < 0.75:
                w = window(sh)
                target, src = rng.choice(live[sh]), rng.choice(live[sh])
                target[w] = src[w] * 0.5 + (rng.choice(live[sh])[w] if rng.random() < 0.5 else 1.0)
            elif act < 0.8:
                rng.choice(live[sh])[window(sh)] = rng.choice([0.0, 3.5])
            elif act < 0.88 and len(live[sh]) > 2:
                live[sh].pop(rng.randrange(len(live[sh])))
            elif act < 0.94:
                live[(8,)].append(rng.choice(live[(8,)]) * cnp.sum(rng.choice(live[sh])))
            elif act < 0.97:
                x = rng.choice(live[(8,)])
                y = rng.choice(live[(8,)])
                live[(8,)].append(x + x.dot(y))
            else:
                r.check()
        r.check()
        live.clear()
        r.check()
    finally:
        r.close()


def test_malformed_logs_are_refused():
    cnp.reset()
    itf = cnp.CharmNumericInterface(device=-1)
    itf.connect(odf=4)
    try:
        with pytest.raises(RuntimeError, match="statement log"):
            itf.send_log(struct.pack("<2i", 9, 1))                       # unknown record kind
        with pytest.raises(RuntimeError, match="truncated"):
            itf.send_log(struct.pack("<6i", 1, 1, 0, L.F64, 0, 0))       # a creation without its shape
        with pytest.raises(RuntimeError, match="statement log"):
            itf.send_log(struct.pack("<6i4i", 2, 1, L.OP_ADD, L.F64, 3, 0, 1, 8, 0, 0))   # three operands
        itf.send_log(b"")                                                # nothing recorded: fine
    finally:
        cnp.reset()
        itf.close()
