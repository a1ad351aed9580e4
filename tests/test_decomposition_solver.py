"""Decomposition solver (cnx_solve_decompositions) against upstream's own known answers
(tests/test_compute_decompositions.cpp upstream, built there with minimum tile 64 for every rank,
odf 4, one PE) and against what the definition of an aligned offset fixes.

An offset o of an array with tile T means: element i lives in tile (i + o) // T. Two arrays are
aligned along a read `out[i] = src[start + i*step]` when, for every i, the tile index of out's
element equals the tile index of the source element scaled by the step, i.e.
(o_out + i) // T_out == (o_src + start + i*step) // (T_out * step) whenever T_src == T_out*step.
"""
import ctypes as C
import struct

import numpy as np
import pytest

from charmnumeric_amd import _lib as L
from charmnumeric_amd import lazy

MIN64 = (64, 64, 64)


class Ref:
    def __init__(self, name, ndims, broadcast=False):
        self.name, self.base_ndims, self.broadcast, self.dtype = name, ndims, broadcast, L.F64


def reg(start, stop, step=None):
    start, stop = tuple(start), tuple(stop)
    return (start, stop, tuple(step) if step else tuple(1 for _ in start))


def message(*nodes):
    return struct.pack("<iii", lazy.DAG_MAGIC, 1, len(nodes)) + b"".join(
        w.to_bytes(i, True) for i, w in enumerate(nodes))


def solve(arrays, msg, odf=4, pes=1, min_tile=MIN64):
    """arrays: {name: (shape, offset, tile, final)} -> {name: (tile, offset tuple)}"""
    names = sorted(arrays)
    buf = (L.Decomp * len(names))()
    for d, name in zip(buf, names):
        shape, offset, tile, final = arrays[name]
        d.name, d.ndims, d.tile, d.final = name, len(shape), tile, int(final)
        for k in range(len(shape)):
            d.shape[k] = shape[k]
            d.offset[k] = offset[k]
    mt = (C.c_int32 * 3)(*min_tile)
    L.check(L.lib.cnx_solve_decompositions(odf, pes, mt, len(names), buf, len(msg), msg))
    assert all(d.final == 1 for d in buf)
    return {d.name: (d.tile, tuple(d.offset[: d.ndims])) for d in buf}


def copy_node(out, src, region, nd=1):
    w = lazy._NodeWriter()
    w.op(out, L.OP_COPY, False, nd, L.F64, [w.leaf(Ref(src, nd))], [region])
    return w


# ---- upstream known answers (tests/test_compute_decompositions.cpp:141-397) ----

def test_shifted_copy_takes_the_absolute_offset_of_its_source():
    # :141-166  B = A[150:350], A placed at 0 with tile 64
    out = solve({1: ((512,), (0,), 64, True), 2: ((200,), (0,), 0, False)},
                message(copy_node(2, 1, reg([150], [350]))))
    assert out[2] == (64, (150,))
    assert out[2][1][0] % 64 == 22
    assert out[1] == (64, (0,))


def test_shifted_copy_from_a_source_that_sits_at_an_offset():
    # :168-192  A placed at 132; B = A[70:170]
    out = solve({1: ((512,), (132,), 64, True), 2: ((100,), (0,), 0, False)},
                message(copy_node(2, 1, reg([70], [170]))))
    assert out[2] == (64, (202,))
    assert out[2][1][0] % 64 == 10


def jacobi_like(nd, n, with_source):
    """tmp_stencil = sum of the 2*nd shifted reads of U (+ F's interior); tmp_weighted =
    U interior + tmp_stencil; U[interior] = tmp_weighted -- the roots of upstream's
    test_jacobi{1,2,3}d_temp_offset (:226-387), with nested binary ADDs for their n-ary ones."""
    U, F, TS, TW, SET = 1, 2, 10, 11, 12
    w = lazy._NodeWriter()
    u = w.leaf(Ref(U, nd))
    reads = []
    for d in range(nd):
        for lo in (0, 2):
            start = [1] * nd
            start[d] = lo
            reads.append((u, reg(start, [s + n - 2 for s in start])))
    inner = reg([1] * nd, [n - 1] * nd)
    if with_source:
        reads.append((w.leaf(Ref(F, nd)), inner))
    acc, acc_reg = reads[0]
    for k, (node, region) in enumerate(reads[1:]):
        last = k == len(reads) - 2
        acc = w.op(TS if last else 100 + k, L.OP_ADD, True, nd, L.F64, [acc, node], [acc_reg, region],
                   root=last)
        acc_reg = None
    w.op(TW, L.OP_ADD, True, nd, L.F64, [u, w.leaf(Ref(TS, nd))], [inner, None])
    w.op(SET, L.OP_SET_REGION, False, nd, L.F64, [u, w.leaf(Ref(TW, nd))], [None, None], region=inner)
    arrays = {U: ((n,) * nd, (0,) * nd, 64, True),
              TS: ((n - 2,) * nd, (0,) * nd, 64, False),
              TW: ((n - 2,) * nd, (0,) * nd, 64, False)}
    if with_source:
        arrays[F] = ((n,) * nd, (0,) * nd, 64, True)
    return arrays, message(w), (TS, TW)


@pytest.mark.parametrize("nd,n,with_source", [(1, 129, True), (2, 129, True), (3, 65, False)])
def test_jacobi_temporaries_sit_one_element_in(nd, n, with_source):
    # :226-387: both temporaries get tile 64 and offset (1,..,1): their tiles line up with U's
    arrays, msg, (ts, tw) = jacobi_like(nd, n, with_source)
    out = solve(arrays, msg)
    assert out[ts] == (64, (1,) * nd)
    assert out[tw] == (64, (1,) * nd)
    assert out[1] == (64, (0,) * nd)


def test_expression_temporary_takes_one_absolute_representative():
    # :194-224  TMP = A[100:300] + A[150:350]; A[200:400] = TMP
    A, TMP, SET = 1, 10, 11
    w = lazy._NodeWriter()
    a = w.leaf(Ref(A, 1))
    w.op(TMP, L.OP_ADD, True, 1, L.F64, [a, a], [reg([100], [300]), reg([150], [350])])
    w.op(SET, L.OP_SET_REGION, False, 1, L.F64, [a, w.leaf(Ref(TMP, 1))], [None, None],
         region=reg([200], [400]))
    out = solve({A: ((512,), (0,), 64, True), TMP: ((200,), (0,), 0, False)}, message(w))
    assert out[TMP] == (64, (150,))
    assert out[TMP][1][0] % 64 == 22
    assert out[A] == (64, (0,))


def test_strided_copy_halves_the_tile_and_sets_the_offset():
    # :389-413  B = A[2:202:2], A with tile 128
    out = solve({1: ((512,), (0,), 128, True), 2: ((100,), (0,), 128, False)},
                message(copy_node(2, 1, reg([2], [202], [2]))))
    assert out[2] == (64, (1,))


# ---- the tile rule alone (src/decomposition_solver.hpp:100-122) ----

@pytest.mark.parametrize("shape,min_tile,odf,pes,want", [
    ((16384, 16384), (262144, 512, 64), 4, 1, 8192),
    ((8192, 8192), (262144, 512, 64), 16, 1, 2048),
    ((512, 512, 512), (262144, 512, 64), 64, 1, 128),
    ((1 << 24,), (262144, 512, 64), 4, 1, 1 << 22),
    ((200,), MIN64, 4, 1, 64),
    ((100,), MIN64, 4, 1, 64),
])
def test_tile_rule_without_a_dag(shape, min_tile, odf, pes, want):
    out = solve({7: (shape, (0,) * len(shape), 0, False)}, b"", odf=odf, pes=pes, min_tile=min_tile)
    assert out[7] == (want, (0,) * len(shape))


# ---- what alignment means, checked by brute force ----

def tiles_line_up(o_out, t_out, o_src, t_src, start, step, count):
    """Every element of the result sits in the tile that holds its source element."""
    i = np.arange(count)
    scale = t_src // t_out
    if scale == step:
        return np.array_equal((o_out + i) // t_out, (o_src + start + i * step) // t_src)
    return np.array_equal((o_out + i) // t_out, (o_src + start + i * step) // t_out)


@pytest.mark.parametrize("src_off,start,step,count", [
    (0, 150, 1, 200), (132, 70, 1, 100), (0, 1, 1, 127), (64, 0, 1, 300), (5, 59, 1, 64),
    (0, 2, 2, 100), (0, 0, 2, 256), (0, 64, 2, 200), (0, 4, 4, 100),
])
def test_single_read_is_aligned_exactly(src_off, start, step, count):
    tile = 64 * step
    out = solve({1: ((1024,), (src_off,), tile, True), 2: ((count,), (0,), tile, False)},
                message(copy_node(2, 1, reg([start], [start + count * step], [step]))), odf=64)
    t_out, (o_out,) = out[2]
    assert t_out == 64
    assert tiles_line_up(o_out, t_out, src_off, tile, start, step, count)


def test_whole_array_statement_shares_one_decomposition():
    # c = a + b over whole, freshly produced arrays: one class, offset 0, same tile
    a, b, c, d = 1, 2, 3, 4
    w0 = copy_node(a, 9, reg([10], [210]))
    w1 = lazy._NodeWriter()
    w1.op(b, L.OP_MUL, False, 1, L.F64, [w1.leaf(Ref(a, 1)), w1.scalar(2.0, 1, L.F64)], [None, None])
    w2 = lazy._NodeWriter()
    w2.op(c, L.OP_ADD, False, 1, L.F64, [w2.leaf(Ref(a, 1)), w2.leaf(Ref(b, 1))], [None, None])
    w3 = copy_node(d, c, reg([0], [100]))
    out = solve({9: ((512,), (0,), 64, True), a: ((200,), (0,), 0, False), b: ((200,), (0,), 0, False),
                 c: ((200,), (0,), 0, False), d: ((100,), (0,), 0, False)}, message(w0, w1, w2, w3))
    assert out[a] == out[b] == out[c] == (64, (10,))
    assert out[d] == (64, (10,))


def test_product_operands_and_results_stay_at_offset_zero():
    # src/decomposition_solver.hpp:590-595,1705-1709
    A, x, y, xs = 1, 2, 3, 4
    w0 = copy_node(xs, x, reg([7], [135]))
    w1 = lazy._NodeWriter()
    w1.op(y, L.OP_MATMUL, False, 1, L.F64, [w1.leaf(Ref(A, 2)), w1.leaf(Ref(xs, 1))], [None, None])
    out = solve({A: ((128, 128), (0, 0), 64, True), x: ((256,), (0,), 64, True),
                 xs: ((128,), (0,), 0, False), y: ((128,), (0,), 0, False)}, message(w0, w1))
    assert out[xs] == (64, (0,))
    assert out[y] == (64, (0,))


def test_two_sources_pull_with_their_volumes():
    # r = big[3:203] + small[40:240]: the larger source decides the phase (weights are source
    # volumes, src/decomposition_solver.hpp:651-655); the absolute offset is then the value of
    # that phase nearest to what the tree parent asks for (:1309-1324,1450-1478)
    big, small, r = 1, 2, 3
    for shapes, want in ((((4096,), (512,)), 3), (((512,), (4096,)), 40)):
        w = lazy._NodeWriter()
        w.op(r, L.OP_ADD, False, 1, L.F64, [w.leaf(Ref(big, 1)), w.leaf(Ref(small, 1))],
             [reg([3], [203]), reg([40], [240])])
        out = solve({big: (shapes[0], (0,), 64, True), small: (shapes[1], (0,), 64, True),
                     r: ((200,), (0,), 0, False)}, message(w), odf=64)
        assert out[r][0] == 64 and out[r][1][0] % 64 == want, (shapes, out[r])
        assert abs(out[r][1][0] - 40) <= 32


def test_cycle_falls_back_to_per_array_wishes():
    # t = a[8:108] + b[8:108] with a, b both placed makes the triangle a - t - b plus the
    # assignment b[8:108] = t a cycle through t; all wishes agree on 8
    a, b, t = 1, 2, 3
    w = lazy._NodeWriter()
    w.op(t, L.OP_ADD, False, 1, L.F64, [w.leaf(Ref(a, 1)), w.leaf(Ref(b, 1))],
         [reg([8], [108]), reg([8], [108])])
    w2 = lazy._NodeWriter()
    w2.op(20, L.OP_SET_REGION, False, 1, L.F64, [w2.leaf(Ref(b, 1)), w2.leaf(Ref(t, 1))], [None, None],
          region=reg([8], [108]))
    out = solve({a: ((256,), (0,), 64, True), b: ((256,), (0,), 64, True), t: ((100,), (0,), 0, False)},
                message(w, w2))
    assert out[t] == (64, (8,))


def test_bad_arguments_are_refused():
    buf = (L.Decomp * 1)()
    buf[0].name, buf[0].ndims = 1, 4
    mt = (C.c_int32 * 3)(*MIN64)
    assert L.lib.cnx_solve_decompositions(4, 1, mt, 1, buf, 0, b"") < 0
    buf[0].ndims = 1
    buf[0].shape[0] = 0
    assert L.lib.cnx_solve_decompositions(4, 1, mt, 1, buf, 0, b"") < 0
    buf[0].shape[0] = 10
    assert L.lib.cnx_solve_decompositions(4, 1, mt, 1, buf, 5, b"12345") < 0
    assert L.lib.cnx_solve_decompositions(4, 1, mt, 1, buf, 0, b"") == 0


def test_tree_phases_minimise_the_weighted_misalignment():
    """Brute force over every phase of the three free arrays of a tree with two placed arrays:
    the solver's phases reach the minimum of sum(weight * circular distance between the phase an
    edge asks for and the phase taken), which is what its dynamic programme is for
    (src/decomposition_solver.hpp:1070-1166)."""
    A, E, B, Cc, D = 1, 2, 3, 4, 5
    T = 64
    nodes = [copy_node(B, A, reg([5], [205])), copy_node(Cc, B, reg([9], [109]))]
    w = lazy._NodeWriter()
    w.op(D, L.OP_ADD, False, 1, L.F64, [w.leaf(Ref(B, 1)), w.leaf(Ref(E, 1))],
         [reg([30], [130]), reg([3], [103])])
    nodes.append(w)
    shapes = {A: 1000, E: 700, B: 200, Cc: 100, D: 100}
    fixed = {A: 17, E: 40}
    arrays = {n: ((shapes[n],), (fixed.get(n, 0),), T, n in fixed) for n in shapes}
    out = solve(arrays, message(*nodes), odf=64)
    # (from, to, shift, weight = volume of the array read)
    edges = [(A, B, 5, shapes[A]), (B, Cc, 9, shapes[B]), (B, D, 30, shapes[B]), (E, D, 3, shapes[E])]
    ph = np.arange(T)
    grid = dict(zip((B, Cc, D), np.meshgrid(ph, ph, ph, indexing="ij")))
    for n, o in fixed.items():
        grid[n] = np.full((T, T, T), o % T)
    total = np.zeros((T, T, T), dtype=np.int64)
    for src, dst, shift, weight in edges:
        d = (grid[src] + shift - grid[dst]) % T
        total += weight * np.minimum(d, T - d)
    got = total[out[B][1][0] % T, out[Cc][1][0] % T, out[D][1][0] % T]
    assert got == total.min(), (out, int(got), int(total.min()))
    assert all(out[n] == (T, (fixed[n],)) for n in fixed)


# ---- the executor under the solver (dry mode: decisions only) ----

@pytest.fixture
def planned_itf():
    import charmnumeric_amd as cnp
    cnp.reset()
    it = cnp.CharmNumericInterface(device=-1)
    it.connect(odf=4)
    for nd in (1, 2, 3):
        it.set_min_tile(nd, 64)
    it.set_solver(True)
    it.set_trace()
    yield it
    cnp.reset()
    it.close()


def test_executor_lays_results_out_as_planned(planned_itf):
    import charmnumeric_amd as cnp
    it = planned_itf
    a = cnp.zeros(512)
    b = a[150:350] + 1.0
    c = b + b
    d = a[2:202:2] * 2.0
    lazy.execute(it)
    log = it.trace()
    assert it.array_info(a.name)["offset"] == (0,)
    assert it.array_info(b.name) == {"ndims": 1, "dtype": L.F64, "tile": 64, "shape": (200,),
                                     "offset": (150,)}
    assert it.array_info(c.name)["offset"] == (150,)
    assert it.array_info(d.name)["tile"] == 64 and it.array_info(d.name)["offset"] == (1,)
    assert any(ln.startswith(f"plan {b.name} tile=64 offset=(150)") for ln in log)
    # b and c are cut alike: per-tile launch; b against a needs the gather
    kinds = {ln.split("out=")[1].split()[0]: ln for ln in log if ln.startswith("group")}
    assert "path=dense" in kinds[str(c.name)]
    assert "path=tiles" in kinds[str(b.name)]


def test_executor_without_the_solver_keeps_offset_zero(planned_itf):
    import charmnumeric_amd as cnp
    it = planned_itf
    it.set_solver(False)
    a = cnp.zeros(512)
    b = a[150:350] + 1.0
    lazy.execute(it)
    assert it.array_info(b.name)["offset"] == (0,)
    assert not any(ln.startswith("plan") for ln in it.trace())


def test_products_of_offset_operands_are_copied_first(planned_itf):
    import charmnumeric_amd as cnp
    it = planned_itf
    A = cnp.zeros((200, 180))
    v = cnp.zeros(400)
    B = A[3:163, 5:165] * 1.0
    x = v[11:171] * 1.0
    lazy.execute(it)                       # B and x are placed before any product names them
    assert it.array_info(B.name)["offset"] == (3, 5)
    assert it.array_info(x.name)["offset"] == (11,)
    it.trace()
    y = B @ x
    C2 = B @ B
    lazy.execute(it)
    log = it.trace()
    assert sum(ln.startswith("relayout") for ln in log) == 3
    assert it.array_info(y.name)["offset"] == (0,) and it.array_info(C2.name)["offset"] == (0, 0)
    # the copies are gone again
    assert it.stats()["live_arrays"] == 6
    # within one message the solver keeps product operands at 0 itself (no copy needed)
    B2 = A[3:163, 5:165] * 2.0
    y2 = B2 @ x
    lazy.execute(it)
    assert it.array_info(B2.name)["offset"] == (0, 0)
    assert sum(ln.startswith("relayout") for ln in it.trace()) == 0


# ---- assignments across ranks (src/decomposition_solver.hpp:333-353,728-786) ----

def test_plane_assigned_into_a_slab_lines_up_with_it():
    """X[3, 10:110, 20:120] = Y with Y a fresh 2-D array: Y's rows meet X's dimension 1 and its
    columns dimension 2, so Y wants offset (10, 20); the lower-rank array also takes the tile of
    the higher-rank one."""
    X, Y, SET = 1, 2, 9
    w = lazy._NodeWriter()
    w.op(SET, L.OP_SET_REGION, False, 3, L.F64, [w.leaf(Ref(X, 3)), w.leaf(Ref(Y, 2))], [None, None],
         region=reg([3, 10, 20], [4, 110, 120]))
    out = solve({X: ((8, 200, 200), (0, 0, 0), 64, True), Y: ((100, 100), (0, 0), 128, False)},
                message(w), odf=64)
    assert out[Y] == (64, (10, 20))
    assert out[X] == (64, (0, 0, 0))


def test_slab_read_into_a_plane_lines_up_with_it():
    """The other way round: P[5:105, 7:107] = Z with Z a fresh (1, 100, 100) array read whole:
    Z's dimensions 1 and 2 meet P's 0 and 1; dimension 0 (extent 1) meets nothing and stays 0."""
    P, Z, SET = 1, 2, 9
    w = lazy._NodeWriter()
    w.op(SET, L.OP_SET_REGION, False, 2, L.F64, [w.leaf(Ref(P, 2)), w.leaf(Ref(Z, 3))], [None, None],
         region=reg([5, 7], [105, 107]))
    out = solve({P: ((300, 300), (0, 0), 64, True), Z: ((1, 100, 100), (0, 0, 0), 0, False)},
                message(w), odf=64)
    assert out[Z][0] == 64
    assert out[Z][1] == (0, 5, 7)


def test_cycle_with_conflicting_wishes_follows_the_heavier_one():
    """t reads a[8:108] and b[40:140]; b[8:108] = t closes a cycle through t, so t is settled from
    the wishes of its producers and its consumer one by one, weighted by volume: phase 8 is asked
    for by a (256 elements) and by the assignment (t's own 100), phase 40 by b (256 or 4096)."""
    a, b, t = 1, 2, 3
    for nb, want in ((256, 8), (4096, 40)):
        w = lazy._NodeWriter()
        w.op(t, L.OP_ADD, False, 1, L.F64, [w.leaf(Ref(a, 1)), w.leaf(Ref(b, 1))],
             [reg([8], [108]), reg([40], [140])])
        w2 = lazy._NodeWriter()
        w2.op(20, L.OP_SET_REGION, False, 1, L.F64, [w2.leaf(Ref(b, 1)), w2.leaf(Ref(t, 1))], [None, None],
              region=reg([8], [108]))
        out = solve({a: ((256,), (0,), 64, True), b: ((nb,), (0,), 64, True), t: ((100,), (0,), 0, False)},
                    message(w, w2), odf=64)
        assert out[t][0] == 64 and out[t][1][0] % 64 == want, (nb, out[t])


# ---- robustness: random DAGs never crash the solver and always give usable tiles ----

def test_random_dags_give_power_of_two_tiles_and_finite_offsets():
    rng = np.random.default_rng(2024)
    for case in range(300):
        nd = int(rng.integers(1, 4))
        names = list(range(1, 7))
        arrays = {}
        for name in names:
            shape = tuple(int(rng.integers(1, 300)) for _ in range(nd))
            final = bool(rng.integers(0, 2))
            tile = int(rng.choice([0, 16, 64, 128])) if not final else int(rng.choice([16, 64, 128]))
            offset = tuple(int(rng.integers(0, 200)) if final else 0 for _ in range(nd))
            arrays[name] = (shape, offset, tile, final)
        # one lower- or higher-rank array for assignments across ranks
        other_nd = nd - 1 if nd > 1 else nd + 1
        arrays[9] = (tuple(int(rng.integers(1, 100)) for _ in range(other_nd)), (0,) * other_nd, 0, False)

        def region(shape):
            start, stop, step = [], [], []
            for n in shape:
                st = int(rng.choice([1, 1, 2, 3]))
                a = int(rng.integers(0, n))
                b = int(rng.integers(a + 1, n + 1))
                start.append(a), stop.append(b), step.append(st)
            return reg(start, stop, step)

        nodes = []
        for _ in range(int(rng.integers(1, 6))):
            w = lazy._NodeWriter()
            kind = int(rng.integers(0, 4))
            a, b, out = (int(x) for x in rng.choice(names, 3))
            la, lb = w.leaf(Ref(a, nd)), w.leaf(Ref(b, nd))
            ra = region(arrays[a][0]) if rng.integers(0, 2) else None
            rb = region(arrays[b][0]) if rng.integers(0, 2) else None
            if kind == 0:
                w.op(out, L.OP_ADD, False, nd, L.F64, [la, lb], [ra, rb])
            elif kind == 1:
                t = w.op(100 + len(nodes), L.OP_MUL, True, nd, L.F64, [la, lb], [ra, rb])
                w.op(200 + len(nodes), L.OP_SET_REGION, False, nd, L.F64, [w.leaf(Ref(out, nd)), t],
                     [None, None], region=region(arrays[out][0]))
            elif kind == 2:
                w.op(300 + len(nodes), L.OP_SET_REGION, False, nd, L.F64,
                     [w.leaf(Ref(out, nd)), w.leaf(Ref(9, other_nd))], [None, None],
                     region=region(arrays[out][0]))
            else:
                w.op(out, L.OP_MATMATMUL if nd == 2 else L.OP_COPY, False, nd, L.F64,
                     [la, lb] if nd == 2 else [la], [ra, rb] if nd == 2 else [ra])
            nodes.append(w)
        got = solve(arrays, message(*nodes), odf=int(rng.choice([1, 4, 64])), min_tile=(16, 16, 16))
        for name, (tile, offset) in got.items():
            shape, off0, tile0, final = arrays[name]
            assert tile >= 16 and tile & (tile - 1) == 0, (case, name, tile)
            assert all(abs(o) < (1 << 24) for o in offset), (case, name, offset)
            if final:
                assert (tile, offset) == (tile0, off0), (case, name)


def test_the_seven_known_answers_of_the_golden_file():
    """The same seven cases, with inputs and expectations taken from the committed fixture."""
    from tests import helpers as H
    cases = {c["name"]: c for c in H.golden()["decomposition_offsets"]["cases"]}
    assert len(cases) == 7

    def as_tuple(v):
        return tuple(v) if isinstance(v, list) else (v,)

    for name in ("shifted_copy_uses_absolute_offset", "shifted_copy_from_nonzero_source_offset",
                 "strided_copy_reduces_tile_and_sets_offset"):
        c = cases[name]
        src, (lo, hi, step) = c["source_array"], c["copy_region"]
        count = (hi - lo + step - 1) // step
        out = solve({1: ((src["size"],), (src["offset"],), src["tile"], True),
                     2: ((count,), (0,), src["tile"] if step > 1 else 0, False)},
                    message(copy_node(2, 1, reg([lo], [hi], [step]))))
        assert out[2] == (c["expect"]["tile"], as_tuple(c["expect"]["offset"])), name
        assert out[2][1][0] % out[2][0] == c["expect"]["phase"], name
    c = cases["shifted_expression_temp_uses_absolute_representative"]
    w = lazy._NodeWriter()
    a = w.leaf(Ref(1, 1))
    w.op(10, L.OP_ADD, True, 1, L.F64, [a, a], [reg([r[0]], [r[1]], [r[2]]) for r in c["operand_regions"]])
    s0, s1, s2 = c["set_region"]
    w.op(11, L.OP_SET_REGION, False, 1, L.F64, [a, w.leaf(Ref(10, 1))], [None, None], region=reg([s0], [s1], [s2]))
    out = solve({1: ((512,), (0,), 64, True), 10: ((s1 - s0,), (0,), 0, False)}, message(w))
    assert out[10] == (c["expect"]["tile"], (c["expect"]["offset"],))
    assert out[1][1] == (c["expect"]["target_offset"],)
    for nd, name in ((1, "jacobi1d_temp_offset"), (2, "jacobi2d_temp_offset"), (3, "jacobi3d_temp_offset")):
        c = cases[name]
        n = c["shape"][0]
        arrays, msg, (ts, tw) = jacobi_like(nd, n, with_source=nd < 3)
        out = solve(arrays, msg)
        assert out[ts] == out[tw] == (c["expect"]["tile"], as_tuple(c["expect"]["offset"])), name
