"""Seeded random programs against NumPy: a few arrays of one rank, then a sequence of statements
drawn from what the frontend offers (element-wise expressions over shifted and strided slices,
assignments into slices from expressions, literals and other slices, copies, named temporaries,
sums, dots and products on windows). NumPy runs the same statements in the same order. Element-wise
results must agree bit for bit; reductions and products to 1e-12 of the sum of absolute terms
(1e-5 in the fp32 programs). Integer programs (wrap-around arithmetic) are element-wise only.
Every program runs twice: with the tile rule alone and with the decomposition solver laying the
arrays out (tiles that do not start at element 0)."""
import numpy as np
import pytest

import charmnumeric_amd as cnp

pytestmark = pytest.mark.gpu

MIN_TILE = {1: 64, 2: 16, 3: 8}


def random_slice(rng, n, min_len=2):
    """A slice of extent n with at least min_len elements, unit or small positive step."""
    step = int(rng.choice([1, 1, 1, 2, 3]))
    count = int(rng.integers(min_len, max(min_len + 1, (n - 1) // step + 1)))
    span = (count - 1) * step + 1
    start = int(rng.integers(0, n - span + 1))
    return slice(start, start + span, step), count


def same_count_slice(rng, n, count):
    """Another slice of extent n with exactly `count` elements (None if it cannot fit)."""
    steps = [s for s in (1, 1, 2, 3) if (count - 1) * s + 1 <= n]
    if not steps:
        return None
    step = int(rng.choice(steps))
    span = (count - 1) * step + 1
    start = int(rng.integers(0, n - span + 1))
    return slice(start, start + span, step)


class Program:
    def __init__(self, seed, rank, dtype=np.float64):
        self.rng = np.random.default_rng(seed)
        self.rank = rank
        self.rel = 1e-12 if dtype == np.float64 else 1e-5
        edge = {1: (150, 400), 2: (20, 70), 3: (9, 26)}[rank]
        self.shape = tuple(int(self.rng.integers(*edge)) for _ in range(rank))
        self.integer = np.issubdtype(dtype, np.integer)
        if self.integer:        # values near the top of the range: sums and products wrap around
            info = np.iinfo(dtype)
            self.host = [self.rng.integers(info.min // 2, info.max // 2, self.shape, dtype=dtype)
                         for _ in range(3)]
        else:
            self.host = [self.rng.standard_normal(self.shape).astype(dtype) for _ in range(3)]
        self.dev = [cnp.array(h) for h in self.host]
        self.checks = []     # (device value, host value, kind)

    def key_pair(self):
        """A key on one array and a key of the same shape on another (or the same) array."""
        key, other = [], []
        for n in self.shape:
            s, count = random_slice(self.rng, n)
            o = same_count_slice(self.rng, n, count)
            key.append(s)
            other.append(o if o is not None else s)
        return tuple(key), tuple(other)

    def expression(self, keys):
        """A small expression over slices of equal shape; returns (device value, host value)."""
        rng = self.rng
        terms = []
        for _ in range(int(rng.integers(2, 5))):
            i = int(rng.integers(0, 3))
            k = keys[int(rng.integers(0, len(keys)))]
            terms.append((self.dev[i][k], self.host[i][k]))
        d, h = terms[0]
        for td, th in terms[1:]:
            op = int(rng.integers(0, 3 if self.integer else 4))
            c = int(rng.choice([2, -3, 5])) if self.integer else float(rng.choice([0.5, 2.0, -1.25, 3.0]))
            if op == 0:
                d, h = d + td, h + th
            elif op == 1:
                d, h = d - c * td, h - c * th
            elif op == 2:
                d, h = d * td, h * th
            else:
                d, h = (d + c) / (td * td + 1.5), (h + c) / (th * th + 1.5)
        return d, h

    def statement(self):
        rng = self.rng
        kind = int(rng.integers(0, 8))
        key, other = self.key_pair()
        t = int(rng.integers(0, 3))
        if self.integer and kind in (1, 3, 6, 7):       # integer programs: element-wise work only
            kind = 0
        if kind == 0:                                   # slice = expression of slices
            d, h = self.expression([key, other])
            self.dev[t][key] = d
            self.host[t][key] = h
        elif kind == 1:                                 # slice = literal
            v = float(rng.choice([0.0, 1.0, -2.5]))
            self.dev[t][key] = v
            self.host[t][key] = v
        elif kind == 2:                                 # slice = another slice (maybe of itself)
            s = int(rng.integers(0, 3))
            src_h = self.host[s][other].copy()
            self.dev[t][key] = self.dev[s][other]
            self.host[t][key] = src_h
        elif kind == 3:                                 # named temporary used twice
            d, h = self.expression([key])
            d2, h2 = d * 0.5 + d, h * 0.5 + h
            self.dev[t][key] = d2
            self.host[t][key] = h2
            self.checks.append((d, h, "exact"))
        elif kind == 4:                                 # copy of a slice, kept
            self.checks.append((self.dev[t][key].copy(), self.host[t][key].copy(), "exact"))
        elif kind == 5:                                 # whole-array expression into a new array
            d, h = self.expression([tuple(slice(None) for _ in self.shape)])
            self.checks.append((d, h, "exact"))
        elif kind == 6 and self.rank == 1:              # dot of two windows
            n = self.shape[0]
            s, count = random_slice(rng, n, 8)
            s = slice(s.start, s.start + count)          # unit step
            o = same_count_slice(rng, n, count)
            o = slice(o.start, o.start + count)
            a, b = int(rng.integers(0, 3)), int(rng.integers(0, 3))
            want = float(self.host[a][s] @ self.host[b][o])
            bound = float(np.abs(self.host[a][s]) @ np.abs(self.host[b][o]))
            self.checks.append((self.dev[a][s] @ self.dev[b][o], (want, bound), "sum"))
        elif kind == 6 and self.rank == 2:              # product of two windows
            r, c = self.shape
            k = int(rng.integers(2, min(r, c)))
            r0, c0 = int(rng.integers(0, r - k + 1)), int(rng.integers(0, c - k + 1))
            a, b = int(rng.integers(0, 3)), int(rng.integers(0, 3))
            wa, wb = (slice(None), slice(c0, c0 + k)), (slice(r0, r0 + k), slice(None))
            ha, hb = self.host[a][wa], self.host[b][wb]
            self.checks.append((self.dev[a][wa] @ self.dev[b][wb],
                                (ha @ hb, np.abs(ha) @ np.abs(hb)), "product"))
        elif kind == 6:                                 # plane of a rank-3 array times a plane
            p, q = int(rng.integers(0, self.shape[0])), int(rng.integers(0, self.shape[1]))
            ha, hb = self.host[0][p], self.host[1][:, q, :]          # (s1, s2) and (s0, s2)
            m = min(ha.shape[1], hb.shape[0])                       # cut to a common inner extent
            ha, hb = ha[:, :m], hb[:m, :]
            da, db = self.dev[0][p, :, :m], self.dev[1][:m, q, :]
            self.checks.append((da @ db, (ha @ hb, np.abs(ha) @ np.abs(hb)), "product"))
        else:                                           # sum of an array
            if self.host[t].dtype != np.float64:        # whole-array sums are checked in fp64 programs
                return
            self.checks.append((cnp.sum(self.dev[t]), (float(self.host[t].sum()),
                                                       float(np.abs(self.host[t]).sum())), "sum"))

    def verify(self, itf):
        for d, h in zip(self.dev, self.host):
            got = d.get(itf)
            assert np.array_equal(got, h), "array contents differ"
        for d, h, kind in self.checks:
            got = d.get(itf)
            if kind == "exact":
                assert got.shape == h.shape and np.array_equal(got, h)
            elif kind == "sum":
                want, bound = h
                assert abs(float(got.reshape(-1)[0]) - want) <= self.rel * bound + 1e-300
            else:
                want, bound = h
                assert got.shape == want.shape and np.all(np.abs(got - want) <= self.rel * bound)


@pytest.mark.parametrize("solver", [False, True])
@pytest.mark.parametrize("rank", [1, 2, 3])
@pytest.mark.parametrize("seed", range(10))
def test_random_program(seed, rank, solver):
    cnp.reset()
    itf = cnp.CharmNumericInterface(device=0)
    itf.connect(odf=4)
    for nd, t in MIN_TILE.items():
        itf.set_min_tile(nd, t)
    itf.set_solver(solver)
    itf.set_pipeline(seed % 2 == 1)       # odd seeds: messages queue for the executor's own thread
    cnp.set_auto_flush(itf, int(np.random.default_rng(seed).choice([4, 16, 1000])))
    try:
        dtype = {4: np.float32, 3: np.int64, 8: np.int32}.get(seed % 10, np.float64)
        prog = Program(1000 * rank + seed, rank, dtype)
        for _ in range(18):
            prog.statement()
        prog.verify(itf)
    finally:
        cnp.reset()
        itf.close()


class MixedProgram:
    """Four arrays of one shape, one per element type; statements meet arrays of two types.
    Results must have np.result_type's element type and NumPy's bits (the operand of the other
    type is converted first, exactly); assignments convert to the target's type (truncation into
    integers; values stay far inside every integer range, beyond which C leaves the result open)."""
    TYPES = (np.float64, np.float32, np.int32, np.int64)

    def __init__(self, seed, rank):
        self.rng = np.random.default_rng(seed)
        self.rank = rank
        edge = {1: (150, 400), 2: (20, 70), 3: (9, 26)}[rank]
        self.shape = tuple(int(self.rng.integers(*edge)) for _ in range(rank))
        self.host = []
        for dt in self.TYPES:
            if np.issubdtype(dt, np.integer):
                self.host.append(self.rng.integers(-1000, 1000, self.shape).astype(dt))
            else:
                self.host.append((self.rng.standard_normal(self.shape) * 10).astype(dt))
        self.dev = [cnp.array(h) for h in self.host]
        self.checks = []

    def keys(self):
        key, other = [], []
        for n in self.shape:
            s, count = random_slice(self.rng, n)
            o = same_count_slice(self.rng, n, count)
            key.append(s)
            other.append(o if o is not None else s)
        return tuple(key), tuple(other)

    def statement(self):
        rng = self.rng
        kind = int(rng.integers(0, 5))
        key, other = self.keys()
        i, j, t = (int(v) for v in rng.integers(0, 4, 3))
        if kind == 0:                                   # expression of two types, kept
            op = int(rng.integers(0, 3))
            d, h = self.dev[i][key], self.host[i][key]
            e, g = self.dev[j][other], self.host[j][other]
            with np.errstate(over="ignore"):
                d, h = ((d + e, h + g), (d - e, h - g), (d * e, h * g))[op]
            self.checks.append((d, h.copy(), "exact"))
        elif kind == 1:                                 # slice of one type = sum of slices of others
            h = self.host[i][other] + self.host[j][other]
            self.dev[t][key] = self.dev[i][other] + self.dev[j][other]
            self.host[t][key] = h
        elif kind == 2:                                 # slice = slice of another type
            h = self.host[i][other].copy()
            self.dev[t][key] = self.dev[i][other]
            self.host[t][key] = h
        elif kind == 3:                                 # astype of a whole array and of a slice
            dt = self.TYPES[int(rng.integers(0, 4))]
            self.checks.append((self.dev[i].astype(dt), self.host[i].astype(dt), "exact"))
            self.checks.append((self.dev[j][key].astype(dt), self.host[j][key].astype(dt), "exact"))
        elif self.rank == 1:                            # dot of windows of two types
            n = self.shape[0]
            s, count = random_slice(rng, n, 8)
            s = slice(s.start, s.start + count)
            o = same_count_slice(rng, n, count)
            o = slice(o.start, o.start + count)
            ha, hb = self.host[i][s], self.host[j][o]
            rt = np.result_type(ha.dtype, hb.dtype)
            with np.errstate(over="ignore"):
                want = ha.astype(rt) @ hb.astype(rt)
            bound = float(np.abs(ha.astype(np.float64)) @ np.abs(hb.astype(np.float64)))
            self.checks.append((self.dev[i][s] @ self.dev[j][o], (want, bound, rt), "dot"))
        else:                                           # matrix of one type times a vector of another
            if self.rank != 2:
                return
            v = cnp.array(self.host[j][0].copy())
            hv = self.host[j][0]
            rt = np.result_type(self.host[i].dtype, hv.dtype)
            want = self.host[i].astype(rt) @ hv.astype(rt)
            bound = np.abs(self.host[i].astype(np.float64)) @ np.abs(hv.astype(np.float64))
            self.checks.append((self.dev[i] @ v, (want, bound, rt), "matvec"))

    def verify(self, itf):
        for d, h in zip(self.dev, self.host):
            got = d.get(itf)
            assert got.dtype == h.dtype and np.array_equal(got, h), "array contents differ"
        for d, h, kind in self.checks:
            got = d.get(itf)
            if kind == "exact":
                assert got.dtype == h.dtype and got.shape == h.shape and got.tobytes() == h.tobytes()
            else:
                want, bound, rt = h
                assert got.dtype == rt
                if np.issubdtype(rt, np.integer):
                    assert np.array_equal(got.reshape(np.shape(want) or (1,)), np.reshape(want, np.shape(want) or (1,)))
                else:
                    rel = 1e-12 if rt == np.float64 else 1e-5
                    assert np.all(np.abs(got.reshape(np.shape(want) or (1,)).astype(np.float64)
                                         - np.asarray(want, np.float64).reshape(np.shape(want) or (1,)))
                                  <= rel * np.asarray(bound).reshape(np.shape(want) or (1,)) + 1e-300)


@pytest.mark.parametrize("rank", [1, 2, 3])
@pytest.mark.parametrize("seed", range(8))
def test_random_program_of_mixed_element_types(seed, rank):
    cnp.reset()
    itf = cnp.CharmNumericInterface(device=0)
    itf.connect(odf=4)
    for nd, t in MIN_TILE.items():
        itf.set_min_tile(nd, t)
    itf.set_solver(seed % 4 == 3)
    itf.set_pipeline(seed % 2 == 1)
    cnp.set_auto_flush(itf, int(np.random.default_rng(seed).choice([4, 16, 1000])))
    try:
        prog = MixedProgram(5000 * rank + seed, rank)
        for _ in range(14):
            prog.statement()
        prog.verify(itf)
    finally:
        cnp.reset()
        itf.close()
