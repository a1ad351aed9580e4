"""Host logic of the frontend and the executor, exercised without a GPU: the executor's dry mode
takes every decision (shapes, tiles, kernel compilation and cache, launch path) and logs it."""
import struct
import sys

import numpy as np
import pytest

import charmnumeric_amd as cnp
from charmnumeric_amd import _lib as L
from charmnumeric_amd import lazy
from charmnumeric_amd.array import parse_key, compose, region_shape


@pytest.fixture
def itf():
    cnp.reset()
    it = cnp.CharmNumericInterface(device=-1)
    it.connect(odf=4)
    it.set_trace()
    yield it
    cnp.reset()
    it.close()


def lines(itf, prefix):
    """Log lines starting with `prefix`; reading the log clears it."""
    return [ln for ln in itf.trace() if ln.startswith(prefix)]


# ---- slicing rules (charmnumeric.py:272-343 upstream) ----

def test_parse_key_follows_numpy_for_slices_and_keeps_integer_dims():
    shape = (10, 7, 5)
    assert parse_key((slice(1, -1), 3), shape) == ((1, 3, 0), (9, 4, 5), (1, 1, 1))
    assert parse_key(Ellipsis, shape) == ((0, 0, 0), (10, 7, 5), (1, 1, 1))
    assert parse_key((Ellipsis, -1), shape) == ((0, 0, 4), (10, 7, 5), (1, 1, 1))
    assert parse_key((slice(2, -2, 2),), (17,)) == ((2,), (15,), (2,))
    assert region_shape(((2,), (15,), (2,))) == (7,)
    with pytest.raises(NotImplementedError):
        parse_key(slice(None, None, -1), (4,))
    with pytest.raises(ValueError):
        parse_key(slice(None, None, 0), (4,))
    with pytest.raises(IndexError):
        parse_key(10, (4,))
    with pytest.raises(IndexError):
        parse_key((0, 0), (4,))
    with pytest.raises(NotImplementedError):
        parse_key((None, 0), (4,))
    with pytest.raises(TypeError):
        parse_key("a", (4,))


def test_view_of_view_composes_like_numpy():
    base = np.arange(200)
    outer = parse_key(slice(10, 190, 3), base.shape)
    inner = parse_key(slice(2, 50, 4), region_shape(outer))
    r = compose(outer, inner)
    want = base[10:190:3][2:50:4]
    got = base[r[0][0]:r[1][0]:r[2][0]]
    assert np.array_equal(got, want)


def test_region_through_a_strided_view_stays_inside_the_base_array(itf):
    # extent 10 is not a multiple of the step: the composed stop must not pass the array's end
    outer = parse_key(slice(None, None, 4), (10,))
    assert compose(outer, parse_key(slice(None), region_shape(outer))) == ((0,), (9,), (4,))
    assert compose(outer, parse_key(slice(0, 3), region_shape(outer))) == ((0,), (9,), (4,))
    assert compose(outer, parse_key(slice(1, 1), region_shape(outer))) == ((4,), (4,), (4,))
    for n, so, si in ((10, 4, 1), (17, 3, 2), (200, 7, 5), (11, 2, 3)):
        base = np.arange(n)
        o = parse_key(slice(1, None, so), base.shape)
        i = parse_key(slice(None, None, si), region_shape(o))
        r = compose(o, i)
        assert r[1][0] <= n
        assert np.array_equal(base[r[0][0]:r[1][0]:r[2][0]], base[1::so][::si])
    # the executor accepts the assignments (dry mode: decisions only)
    a = cnp.zeros(10)
    a[::4][:] = 1.0
    u = cnp.zeros(11)
    u[::3].fill(2.0)
    b = cnp.ones(3)
    a[::4][0:3] = b + b
    cnp.execute(itf)
    assert not [ln for ln in itf.trace() if "error" in ln.lower()]


def test_dtype_and_shape_rules(itf):
    a = cnp.zeros((8,), dtype=cnp.float32)
    assert (a + 1.5).dtype == np.float32          # scalars never promote (charmnumeric.py:369-373)
    assert (2 * a).shape == (8,)
    i = cnp.zeros((8,), dtype=cnp.int32)
    assert (i / 2).dtype == np.int32
    # arrays of two element types meet in np.result_type (charmnumeric.py:369-373 upstream); the
    # operand of the other type is converted by an ASTYPE node first
    assert (a + i).dtype == np.float64 and (i * a).dtype == np.float64
    assert (i + cnp.zeros((8,), dtype=cnp.int64)).dtype == np.int64
    assert (a - cnp.zeros((8,))).dtype == np.float64
    assert (a @ cnp.zeros((8,))).dtype == np.float64
    assert (cnp.zeros((4, 8), dtype=cnp.int32) @ a).dtype == np.float64
    assert (cnp.zeros((4, 8), dtype=cnp.float32) @ cnp.zeros((8, 2))).dtype == np.float64
    assert i.astype(np.float32).dtype == np.float32 and i.astype(np.int32, copy=False) is i
    cnp.execute(itf)
    conv = lines(itf, "astype")
    assert len(conv) == 11 and all("launches=1" in ln for ln in conv)
    with pytest.raises(ValueError):
        a + cnp.zeros((9,), dtype=cnp.float32)
    with pytest.raises(TypeError):
        cnp.zeros((4,), dtype=np.float16)
    with pytest.raises(ValueError):
        bool(a)
    with pytest.raises(TypeError):
        np.asarray(a)
    with pytest.raises(ValueError):
        a @ cnp.zeros((9,), dtype=cnp.float32)
    with pytest.raises(ValueError):
        cnp.zeros((4, 5)) @ cnp.zeros((4,))
    with pytest.raises(ValueError):
        cnp.zeros((4, 5)) @ cnp.zeros((4, 5))
    assert a.size == 8 and a.size() == 8 and a.nbytes == 32 and len(a) == 8 and a.ndim == 1
    assert a[2:6].shape == (4,) and cnp.zeros((4, 6))[1].shape == (1, 6)


def test_dot_with_an_array_of_ones_is_recorded_as_a_sum(itf):
    z = cnp.zeros((4096,)) + 2.0
    one = cnp.ones((4096,))
    s1 = z @ one
    s2 = one @ z
    cnp.execute(itf)
    log = itf.trace()
    assert not [ln for ln in log if ln.startswith("reduce ")], log
    # any assignment into the array ends it, also through a view; a dot with it is a dot again
    one[5:9] = 3.0
    s3 = z @ one
    w = cnp.full((4096,), 1.0)
    v = w[:]
    v[0] = 2.0
    s4 = z @ w
    s5 = z[8:24] @ cnp.ones((16,))          # a slice is not summed whole: stays a dot
    cnp.execute(itf)
    log = itf.trace()
    assert len([ln for ln in log if ln.startswith("reduce ")]) == 3, log
    del s1, s2, s3, s4, s5


# ---- grouping ----

def test_statement_with_dead_temporaries_is_one_group(itf):
    a = cnp.zeros((128,), dtype=cnp.float32)
    b = cnp.zeros((128,), dtype=cnp.float32)
    x = 2 * (a + b + 3)
    cnp.execute(itf)
    g = lines(itf, "group")
    assert len(g) == 1 and "path=dense" in g[0] and "inputs=2" in g[0]
    assert itf.stats()["live_arrays"] == 3       # a, b, x: the two temporaries never became arrays
    assert itf.array_info(x.name)["shape"] == (128,)


def test_live_intermediate_is_materialised_and_splits_the_group(itf):
    a = cnp.zeros((64,))
    t = a + 1.0
    u = t * 2.0
    cnp.execute(itf)
    g = lines(itf, "group")
    # two DAG nodes (t is an array of its own); the executor runs them as one launch that stores both
    assert len(g) == 1 and "path=run statements=2" in g[0]
    assert itf.array_info(t.name)["shape"] == (64,) and itf.array_info(u.name)["shape"] == (64,)
    itf.set_fusion(False)
    v = a + 3.0
    w = v * 2.0
    cnp.execute(itf)
    assert len(lines(itf, "group")) == 2


def test_unused_results_are_dropped(itf):
    a = cnp.zeros((64,))
    a + 1.0                                      # result dropped immediately
    cnp.execute(itf)
    assert lines(itf, "group") == []


def test_stencil_statement_fuses_into_set_region_with_pingpong(itf):
    u = cnp.zeros((64, 64))
    u[0, :] = 1.0
    u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
    cnp.execute(itf)
    tr = itf.trace()
    assert sum(ln.startswith("fill") for ln in tr) == 1
    g = [ln for ln in tr if ln.startswith("group")]
    assert len(g) == 1 and "path=tiles" in g[0] and "pingpong" in g[0] and "inputs=4" in g[0]


def test_assignment_from_a_live_array_is_a_copy_group(itf):
    a = cnp.zeros((17, 17))
    c = cnp.zeros((9, 9))
    c[1:-1, 1:-1] = a[2:-2:2, 2:-2:2]
    cnp.execute(itf)
    g = lines(itf, "group")
    assert len(g) == 1 and "path=tiles" in g[0] and "inplace" in g[0]


def test_pending_reader_runs_before_a_later_assignment(itf):
    """t = u + 1 recorded before u[...] = 5 must see the old u: the assignment closes t's group."""
    u = cnp.zeros((32,))
    t = u + 1.0
    u[...] = 5.0
    cnp.execute(itf)
    tr = itf.trace()
    assert [ln.split()[0] for ln in tr if ln.split()[0] in ("group", "fill")] == ["group", "fill"]
    assert t.shape == (32,)


def test_cg_iteration_compiles_once_and_reuses_buffers(itf):
    n = 256
    A = cnp.zeros((n, n))
    b = cnp.ones((n,))
    x = cnp.zeros((n,))
    r = b.copy()
    p = b.copy()
    rtr = r @ r
    cnp.execute(itf)
    compiled = []
    for k in range(4):
        Ap = A @ p
        pAp = p @ Ap
        alpha = rtr / pAp
        x = x + alpha * p
        r = r - alpha * Ap
        rtr_new = r @ r
        beta = rtr_new / rtr
        p = r + beta * p
        rtr = rtr_new
        cnp.execute(itf)
        compiled.append(itf.stats()["compiled"])
    assert compiled[1] == compiled[0] == compiled[-1]         # every later iteration hits the cache
    st = itf.stats()
    assert st["reuses"] > 0 and st["live_arrays"] <= 12
    tr = itf.trace()
    assert sum(ln.startswith("matmul") for ln in tr) == 4
    # p.Ap follows a product and runs on its own (the matrix is too small for the fused matvec)
    assert sum(ln.startswith("reduce") for ln in tr) == 4
    # alpha, x, r and r.r are one launch, beta and p another (and the two copies of b with the
    # first r.r ahead of the loop a third kind)
    runs = [ln for ln in tr if "path=run" in ln]
    assert len(runs) == 1 + 2 * 4 and "statements=2 scalars_formed=0 reductions=1" in runs[0]
    assert sum("statements=3 scalars_formed=1 reductions=1" in ln for ln in runs) == 4
    assert sum("statements=2 scalars_formed=1 reductions=0" in ln for ln in runs) == 4


def test_a_cg_iteration_on_a_large_system_is_two_launches(itf):
    """examples/cg.py:40-52 upstream at n = 16384: the matvec takes the p update before it and the
    dot behind it along, the x and r updates form alpha in registers from the dot's partial sums and
    leave those of r.r. Partial sums are folded by the launch that reads them; a value somebody
    else asks for gets a fold of its own."""
    n = 16384
    A = cnp.zeros((n, n))
    b = cnp.ones((n,))
    x = cnp.zeros((n,))
    r = b.copy()
    p = b.copy()
    rtr = r @ r
    cnp.execute(itf)
    itf.trace()
    for k in range(3):
        Ap = A @ p
        pAp = p @ Ap
        alpha = rtr / pAp
        x = x + alpha * p
        r = r - alpha * Ap
        rtr_new = r @ r
        beta = rtr_new / rtr
        p = r + beta * p
        rtr = rtr_new
    cnp.execute(itf)
    tr = [ln for ln in itf.trace() if not ln.startswith(("create", "delete"))]
    assert len(tr) == 2 * 3 + 1, tr
    assert tr[0].startswith("matmul") and "fused dot=" in tr[0] and "vector=" not in tr[0]
    for k in (1, 2):
        assert tr[2 * k].startswith("matmul") and "fused vector=" in tr[2 * k] and "dot=" in tr[2 * k]
    for k in range(3):
        assert "path=run statements=3 scalars_formed=1 reductions=1" in tr[2 * k + 1] and "sums_taken=1" in tr[2 * k + 1]
    # the program ends: beta and p of the last iteration are a launch of their own
    assert "path=run statements=2 scalars_formed=1 reductions=0" in tr[6] and "sums_taken=1" in tr[6]
    assert not any(ln.startswith("fold") for ln in tr)
    st = itf.stats()
    assert st["live_arrays"] <= 12
    # a value that is read back while it stands as partial sums is folded first
    Ap = A @ p
    pAp = p @ Ap
    cnp.execute(itf)
    info = itf.array_info(pAp.name)
    assert info["shape"] == (1,)
    tr = [ln for ln in itf.trace() if not ln.startswith(("create", "delete"))]
    assert len(tr) == 2 and tr[0].startswith("matmul") and tr[1].startswith("fold") and "partials=256" in tr[1]
    # switched off: node by node
    itf.set_fusion(False)
    Ap = A @ p
    pAp = p @ Ap
    alpha = rtr / pAp
    x = x + alpha * p
    cnp.execute(itf)
    tr = [ln for ln in itf.trace() if not ln.startswith(("create", "delete"))]
    assert [ln.split()[0] for ln in tr] == ["matmul", "reduce", "group", "group"] and "fused" not in tr[0]


def test_tile_rule_and_minimum_tile_override(itf):
    """Tile = minimum tile of the rank doubled until the array has at most odf*PEs tiles
    (src/decomposition_solver.hpp:100-122 upstream); the upstream tests build with minimum 64."""
    a = cnp.zeros((1 << 24,))
    m = cnp.zeros((16384, 16384))
    u2 = cnp.zeros((8192, 8192))
    cnp.execute(itf)
    assert itf.array_info(a.name)["tile"] == 4194304
    assert itf.array_info(m.name)["tile"] == 8192
    assert itf.array_info(u2.name)["tile"] == 4096           # odf 4, one PE: 2x2 tiles
    itf.set_min_tile(1, 64)
    v = cnp.zeros((200,))
    w = cnp.zeros((100,))
    cnp.execute(itf)
    assert itf.array_info(v.name)["tile"] == 64 and itf.array_info(w.name)["tile"] == 64
    it16 = cnp.CharmNumericInterface(device=-1)
    it16.connect(odf=16)
    u3 = cnp.zeros((8192, 8192))
    u4 = cnp.zeros((512, 512, 512))
    cnp.execute(it16)
    assert it16.array_info(u3.name)["tile"] == 2048
    assert it16.array_info(u4.name)["tile"] == 256           # 16 tiles allowed: 128 would need 64
    del u3, u4
    it16.close()


def test_matmatmul_panel_products_follow_the_tile_grids(itf):
    itf.set_min_tile(2, 64)
    A = cnp.zeros((128, 192))
    B = cnp.zeros((192, 64))
    Cm = A @ B
    cnp.execute(itf)
    # A: tile 128 (2 tiles allowed after doubling), B, C per the same rule; every product is logged
    ln = lines(itf, "matmatmul")
    assert len(ln) == 1 and "panel_products=" in ln[0]
    assert itf.array_info(Cm.name)["shape"] == (128, 64)


def test_diag_copies_once_per_tile_the_diagonal_crosses(itf):
    itf.set_min_tile(1, 64)
    itf.set_min_tile(2, 16)
    v = cnp.ones((100,))
    D = cnp.diag(v, 1)                  # 101 x 101 in 64-tiles: the super-diagonal meets 3 of 4
    d = cnp.diag(D, -40)                # rows 40..100, columns 0..60: tiles (0,0) and (1,0)
    e = cnp.diag(cnp.ones((64, 128)))
    cnp.execute(itf)
    log = [ln for ln in itf.trace() if ln.startswith("diag")]
    assert log[0].endswith("k=1 copies=3") and log[1].endswith("k=-40 copies=2")
    assert D.shape == (101, 101) and d.shape == (61,) and e.shape == (64,)


def test_matvec_of_a_plane_keeps_the_tile_grid_of_the_rank3_array(itf):
    itf.set_min_tile(3, 8)
    A3 = cnp.ones((2, 40, 24))
    y = A3[1, :, :].matvec(cnp.ones((24,)))
    z = cnp.ones((40, 1, 24)).matvec(cnp.ones((24,)))
    cnp.execute(itf)
    assert y.shape == (40,) and z.shape == (40,)
    assert sum(ln.startswith("matmul") for ln in itf.trace()) == 2


def test_pipelined_interface_does_the_same_work_and_defers_errors(itf):
    def program():
        a = cnp.ones((300,))
        b = cnp.arange(300, dtype=np.float64)
        for _ in range(5):
            b[1:-1] = 0.5 * (b[:-2] + b[2:]) + a[1:-1]
            cnp.execute(itf)
        s = b.dot(a)
        cnp.execute(itf)
        return s

    kinds = lambda log: [ln.split()[0] for ln in log]
    program()
    cnp.execute(itf)
    plain = kinds(itf.trace())
    itf.set_pipeline(True)
    program()
    cnp.execute(itf)
    assert kinds(itf.trace()) == plain          # reading the log waits for the queue
    # an executor error surfaces at the next call that reads state back, and the queue keeps working
    itf.send_dag(7, b"not a dag message")
    with pytest.raises(RuntimeError):
        itf.sync()
    itf.sync()
    itf.set_pipeline(False)
    with pytest.raises(RuntimeError):
        itf.send_dag(8, b"not a dag message")


def test_in_place_when_read_and_written_lattices_miss_each_other(itf):
    """An operand that reads the target array forces ping-pong buffers only if its index lattice can
    meet the assigned one; red-black colours, other slabs and interleaved strides run in place."""
    itf.set_min_tile(1, 64)
    itf.set_min_tile(2, 16)
    b = cnp.arange(200, dtype=np.float64)
    phi = cnp.zeros((40, 40))
    cnp.execute(itf)
    itf.trace()

    def how(stmt):
        stmt()
        cnp.execute(itf)
        (line,) = lines(itf, "group")
        # a statement whose boxes are single blocks and do not meet goes out through the memref
        # launch (in place by construction)
        return "inplace" if "path=statements" in line else line.split()[-1]

    def assign(dst, src):
        def stmt():
            b[dst] = b[src] * 2.0
        return stmt

    assert how(assign(slice(1, -1), slice(0, -2))) == "pingpong"             # shifted overlap
    assert how(assign(slice(1, -1, 2), slice(0, -2, 2))) == "inplace"        # odd <- even
    assert how(assign(slice(0, 10, 3), slice(1, 11, 3))) == "inplace"        # {0,3,6,9} <- {1,4,7,10}
    assert how(assign(slice(0, 10, 2), slice(4, 14, 2))) == "pingpong"       # share 4, 6, 8
    assert how(assign(slice(0, 9, 2), slice(3, 18, 3))) == "pingpong"        # share 6
    assert how(assign(slice(0, 5, 2), slice(3, 12, 3))) == "inplace"         # {0,2,4} vs {3,6,9}
    assert how(assign(slice(100, 150), slice(0, 50))) == "inplace"           # apart

    def red():
        phi[1:-1:2, 1:-1:2] = 0.25 * (phi[0:-2:2, 1:-1:2] + phi[2::2, 1:-1:2] + phi[1:-1:2, 0:-2:2]
                                      + phi[1:-1:2, 2::2])
    assert how(red) == "inplace"

    def jacobi():
        phi[1:-1, 1:-1] = 0.25 * (phi[:-2, 1:-1] + phi[2:, 1:-1] + phi[1:-1, :-2] + phi[1:-1, 2:])
    assert how(jacobi) == "pingpong"


def test_the_two_lattices_of_a_colour_are_one_sweep(itf):
    """examples/gauss_seidel.py upstream: four statements a sweep, two launches; the arrays become
    one block the first time."""
    n = 8192
    phi, f = cnp.zeros((n, n)), cnp.zeros((n, n))
    cnp.execute(itf)
    assert itf.array_info(phi.name)["tile"] == 4096
    itf.trace()
    for _ in range(2):
        for r0, c0 in ((1, 1), (2, 2), (1, 2), (2, 1)):
            rows, cols = slice(r0, -1, 2), slice(c0, -1, 2)
            up, down = slice(r0 - 1, -2, 2), slice(r0 + 1, None, 2)
            left, right = slice(c0 - 1, -2, 2), slice(c0 + 1, None, 2)
            phi[rows, cols] = 0.25 * (phi[up, cols] + phi[down, cols] + phi[rows, left] + phi[rows, right]
                                      - 0.5 * f[rows, cols])
    cnp.execute(itf)
    tr = [ln for ln in itf.trace() if ln.startswith(("group", "block"))]
    assert [ln.split()[0] for ln in tr] == ["block", "block", "group", "group", "group", "group"]
    assert all("path=lattices roots=2" in ln and "inplace" in ln for ln in tr[2:])
    assert itf.stats()["compiled"] <= 3
    # a statement that reads what the one before it assigns stays on its own
    phi[1:-1:2, 1:-1:2] = phi[0:-2:2, 1:-1:2] * 2.0
    phi[2:-1:2, 1:-1:2] = phi[1:-2:2, 1:-1:2] * 2.0
    cnp.execute(itf)
    assert not any("path=lattices" in ln for ln in itf.trace())


def test_malformed_messages_are_refused(itf):
    with pytest.raises(RuntimeError, match="bad magic"):
        itf.send_dag(0, struct.pack("<iii", 1, 1, 0))
    good = struct.pack("<iii", lazy.DAG_MAGIC, 1, 1)
    with pytest.raises(RuntimeError, match="truncated|AST nodes"):
        itf.send_dag(0, good + struct.pack("<ii", 0, 0))
    with pytest.raises(RuntimeError, match="version"):
        itf.send_dag(0, struct.pack("<iii", lazy.DAG_MAGIC, 7, 0))
    # a group that reads an array the executor has never seen
    a = cnp.Array((8,), np.float64)
    b = a + 1.0
    with pytest.raises(RuntimeError, match="does not exist"):
        cnp.execute(itf)
    del b


def test_get_checks_rank_size_and_dtype(itf):
    a = cnp.zeros((8, 4))
    cnp.execute(itf)
    with pytest.raises(RuntimeError, match="asked for"):
        itf.get(1, a.name, 32, dtype=np.float64)
    with pytest.raises(RuntimeError, match="asked for"):
        itf.get(2, a.name, 32, dtype=np.float32)
    assert itf.get(2, a.name, 32, dtype=np.float64).shape == (32,)


def test_auto_flush_happens_between_statements(itf):
    itf.set_fusion(False)      # one launch per statement, so that the flushes can be counted
    cnp.set_auto_flush(itf, 5)
    a = cnp.zeros((16,))
    for _ in range(6):
        a[...] = (a + 1.0) * 2.0
    assert lazy.pending_count() < 5 + 4                      # threshold + one statement
    tr = itf.trace()
    groups = [ln for ln in tr if ln.startswith("group")]
    assert len(groups) >= 3
    # a flush in the middle of an expression would have turned its temporaries into arrays
    assert all("path=" in ln for ln in groups) and itf.stats()["live_arrays"] == 1


def test_auto_flush_never_splits_a_stencil_statement(itf):
    cnp.set_auto_flush(itf, 3)
    u = cnp.zeros((64, 64))
    u[0, :] = 1.0
    for _ in range(10):
        u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
    cnp.execute(itf)
    groups = [ln for ln in itf.trace() if ln.startswith("group")]
    assert len(groups) == 10 and all("pingpong" in g and "inputs=4" in g for g in groups)
    st = itf.stats()
    assert st["live_arrays"] == 1 and st["compiled"] == 1 and st["cache_hits"] == 9


def test_auto_flush_keeps_a_named_intermediate_fused(itf):
    """upd = f(u); u[...] = g(u, upd) in a loop: `upd` is alive at every statement boundary (its
    handle goes when the name is bound again). An automatic flush holds the newest statements back
    instead of turning `upd` into an array; only the explicit flush at the end has to."""
    n = 96
    u, f = cnp.zeros((n, n)), cnp.ones((n, n))
    cnp.execute(itf)
    itf.trace()
    cnp.set_auto_flush(itf, 24)
    for _ in range(20):
        upd = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:] + 0.1 * f[1:-1, 1:-1])
        u[1:-1, 1:-1] = (1.0 / 3.0) * u[1:-1, 1:-1] + (2.0 / 3.0) * upd
    cnp.execute(itf)
    log = itf.trace()
    groups = [ln for ln in log if ln.startswith("group")]
    assert len(groups) == 21 and sum("inputs=6" in ln for ln in groups) == 19
    assert sum(ln.startswith("create") for ln in log) == 1      # the last upd only
    assert not any(ln.startswith("delete") for ln in log)
    del upd
    cnp.execute(itf)
    assert sum(ln.startswith("delete") for ln in itf.trace()) == 1


def test_state_queries_complete_what_a_hold_back_flush_left(itf):
    """A flush with a hold-back window may leave its newest statements unplanned. Every call that
    reads or writes array state (sync, get, array_info, put) and every DAG message that follows
    sees them done, in order."""
    n = 32
    u, f = cnp.zeros((n, n)), cnp.ones((n, n))
    cnp.execute(itf)
    itf.trace()

    def held_back_step():
        f[0, :] = 2.0          # a flush that would hold everything back holds nothing back
        upd = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:] + 0.1 * f[1:-1, 1:-1])
        u[1:-1, 1:-1] = (1.0 / 3.0) * u[1:-1, 1:-1] + (2.0 / 3.0) * upd
        log = b"".join(lazy._state.pending)
        lazy._state.pending = []
        itf.send_log(log, 16)
        assert not any(ln.startswith("group") for ln in itf.trace())      # still unplanned
        return upd

    upd = held_back_step()
    itf.sync()
    assert sum(ln.startswith("group") for ln in itf.trace()) == 2
    assert itf.array_info(upd.name)["shape"][:2] == (n - 2, n - 2)
    del upd
    cnp.execute(itf)
    itf.trace()
    # a DAG message behind a held-back log runs behind its statements
    upd = held_back_step()
    itf.send_dag(0, _message([_create(900, (8,), L.F64)]))
    kinds = [ln.split()[0] for ln in itf.trace()]
    assert kinds.index("create") < len(kinds) and kinds[-1] == "create" and kinds.count("group") == 2
    del upd
    # get
    upd = held_back_step()
    got = u.get(itf)
    assert got.shape == (n, n) and sum(ln.startswith("group") for ln in itf.trace()) == 2


def _message(nodes_bytes):
    return struct.pack("<iii", lazy.DAG_MAGIC, 1, len(nodes_bytes)) + b"".join(nodes_bytes)


def _create(name, shape, dtype, node_id=0):
    w = lazy._NodeWriter()
    w.op(name, L.OP_CREATE, False, len(shape), dtype, [], [], lazy._full_region(shape))
    return w.to_bytes(node_id, False)


def test_runs_of_same_extent_assignments_become_one_launch(itf):
    """Assignments of one extent whose boxes are single blocks of memory merge; a box that overlaps
    an earlier one of the same array without being identical ends the run; a matrix product
    assigned to a slab is written there directly."""
    n, b, d = 6, 8, 16
    A = cnp.zeros((n, b, 2 * d))
    C = cnp.zeros((n, b, d))
    H = cnp.zeros((n, b, d))
    W = cnp.zeros((d, 2 * d))
    cnp.execute(itf)
    itf.trace()
    t = 2
    A[t] = H[t - 1].dot(W)
    C[t] = A[t, :, :d] * A[t, :, d:]
    C[t] += A[t, :, :d] * C[t - 1]
    H[t] = cnp.tanh(C[t])
    cnp.execute(itf)
    log = itf.trace()
    assert any("matmatmul" in ln and "into_region" in ln for ln in log)
    assert not any(ln.startswith("create") for ln in log)          # no temporary for the product
    runs = [ln for ln in log if "path=statements" in ln]
    # three statements, two of them assigning C[t]: the first store is dropped
    assert len(runs) == 1 and "count=3" in runs[0] and "outputs=2" in runs[0]
    # overlapping, not identical: u[1:5] is read, then u[2:6] assigned -> two launches
    u, v = cnp.zeros(8), cnp.zeros(8)
    cnp.execute(itf)
    itf.trace()
    v[0:4] = u[1:5] * 2.0
    u[2:6] = v[2:6] + 1.0
    cnp.execute(itf)
    runs = [ln for ln in itf.trace() if "path=statements" in ln]
    assert len(runs) == 2 and all("count=1" in ln for ln in runs)
    # switched off: node by node
    itf.set_fusion(False)
    H[3] = C[3] * 2.0
    C[4] = H[3] + 1.0
    cnp.execute(itf)
    assert not any("path=statements" in ln for ln in itf.trace())


@pytest.mark.parametrize("shape,box", [((4,), (slice(0, 3),)), ((1, 4), (slice(0, 1), slice(0, 4))),
                                       ((1, 1), (slice(0, 1), slice(0, 1)))])
def test_a_run_never_assigns_an_array_it_reads_as_a_kernel_scalar(itf, shape, box):
    """A one-element array used as a scalar is fetched once when the launch starts: the statement
    that assigns it and the statement that reads it as a scalar stay separate launches, in either
    order."""
    c, a = cnp.zeros((1,)), cnp.zeros((1,))
    x, y = cnp.zeros(shape), cnp.zeros(shape)
    cnp.execute(itf)
    itf.trace()
    c[0:1] = a[0:1] + 1.0
    y[box] = x[box] * c
    cnp.execute(itf)
    runs = [ln for ln in itf.trace() if "path=statements" in ln]
    assert len(runs) == 2 and all("count=1" in ln for ln in runs)
    # read as a scalar first, assigned afterwards
    y[box] = x[box] * c
    c[0:1] = a[0:1] + 2.0
    cnp.execute(itf)
    runs = [ln for ln in itf.trace() if "path=statements" in ln]
    assert len(runs) == 2 and all("count=1" in ln for ln in runs)
    # a scalar nobody assigns in the run does not keep statements apart
    y[box] = x[box] * c
    x[box] = y[box] + c
    cnp.execute(itf)
    runs = [ln for ln in itf.trace() if "path=statements" in ln]
    assert len(runs) == 1 and "count=2" in runs[0]


def test_reductions_ride_on_the_group_that_produces_their_operand(itf):
    """A new array and the reductions of it that follow go out as one launch with reducing roots;
    slices, other layouts and results that are not fresh keep every node on its own."""
    n = 4096
    x, y, ones = cnp.zeros((n,)), cnp.zeros((n,)), cnp.ones((n,))
    cnp.execute(itf)
    itf.trace()
    z = 2.5 * x - 0.5 * y + x * y
    s1 = z @ ones
    s2 = z @ z
    s3 = cnp.sumsq_diff(z, x)
    s4 = cnp.maxabs_diff(y, z)
    s5 = cnp.sum(z)                 # the fifth: a launch carries four at most
    cnp.execute(itf)
    log = itf.trace()
    fused = [ln for ln in log if "path=dense+reduce" in ln]
    assert len(fused) == 1 and "reductions=4" in fused[0]
    assert sum(ln.startswith("reduce") for ln in log) == 1
    assert sum(ln.startswith("create") for ln in log) == 6       # z and five one-element results
    # a 3-D field and its norms
    u, f = cnp.zeros((12, 10, 8)), cnp.zeros((12, 10, 8))
    cnp.execute(itf)
    itf.trace()
    r = f - 6.0 * u
    nrm = cnp.sumsq_diff(r, f)
    top = cnp.maxabs_diff(r, u)
    cnp.execute(itf)
    fused = [ln for ln in itf.trace() if "path=dense+reduce" in ln]
    assert len(fused) == 1 and "reductions=2" in fused[0]
    # not a fresh array (an assignment into a slice), or a reduction over a window: node by node
    y[0:n // 2] = x[0:n // 2] * 2.0
    w1 = y @ ones
    t = x + y
    w2 = t[0:n // 2] @ ones[0:n // 2]
    cnp.execute(itf)
    log = itf.trace()
    assert not any("path=dense+reduce" in ln for ln in log)
    assert sum(ln.startswith("reduce") for ln in log) == 2
    # switched off
    itf.set_fusion(False)
    t2 = x * 3.0
    w3 = t2 @ t2
    cnp.execute(itf)
    assert not any("path=dense+reduce" in ln for ln in itf.trace())


def test_kernel_cache_is_bounded_over_a_long_slab_loop(itf):
    """Each step assigns another slab: another group (same code, other regions). The executor keeps
    a bounded number of them and lets the oldest go."""
    n = 4500
    itf.set_fusion(False)              # one group per statement: that is what fills the cache
    a = cnp.zeros((n, 8))
    for t in range(1, n):
        a[t] = a[t - 1] * 0.5
    cnp.execute(itf)
    st = itf.stats()
    assert st["compiled"] == n - 1 and st["group_launches"] == n - 1
    # the first slabs were evicted: assigning them again compiles again instead of hitting the cache
    a[1] = a[0] * 0.5
    cnp.execute(itf)
    assert itf.stats()["compiled"] == n


# ---- error behaviour of the executor (messages built by hand where the frontend would refuse) ----

def test_executor_refuses_what_it_cannot_do(itf):
    itf.send_dag(0, _message([_create(1, (8, 8), L.F64), _create(2, (8,), L.F64), _create(3, (8,), L.F32),
                              _create(4, (9,), L.F64)]))
    ref = lambda name, nd, dt=L.F64: lazy.ArrayRef(name, None, (8,) * nd, nd, dt)

    def nonfusible(opcode, operands, shape, dtype=L.F64, name=50):
        w = lazy._NodeWriter()
        w.op(name, opcode, False, len(shape), dtype, [w.leaf(o) for o in operands], [None] * len(operands),
             lazy._full_region(shape))
        return _message([w.to_bytes(9, False)])

    with pytest.raises(RuntimeError, match="not supported"):
        itf.send_dag(1, nonfusible(55, [ref(2, 1)], (8, 8)))
    itf.send_dag(0, _message([_create(5, (2, 2, 2), L.F64)]))
    with pytest.raises(RuntimeError, match="1-D or 2-D"):
        itf.send_dag(1, nonfusible(L.OP_DIAG, [lazy.ArrayRef(5, None, (2, 2, 2), 3, L.F64)], (2,)))
    with pytest.raises(RuntimeError, match="1-D operands"):
        itf.send_dag(1, nonfusible(L.OP_REDUCE, [ref(1, 2), ref(1, 2)], (1,)))
    with pytest.raises(RuntimeError, match="dtypes"):
        itf.send_dag(1, nonfusible(L.OP_REDUCE, [ref(2, 1), ref(3, 1, L.F32)], (1,)))
    with pytest.raises(RuntimeError, match="lengths"):
        itf.send_dag(1, nonfusible(L.OP_REDUCE, [ref(2, 1), ref(4, 1)], (1,)))
    with pytest.raises(RuntimeError, match="columns"):
        itf.send_dag(1, nonfusible(L.OP_MATMUL, [ref(1, 2), ref(4, 1)], (8,)))
    with pytest.raises(RuntimeError, match="does not exist"):
        itf.send_dag(1, nonfusible(L.OP_REDUCE, [ref(77, 1), ref(2, 1)], (1,)))
    with pytest.raises(RuntimeError, match="already exists"):
        itf.send_dag(1, _message([_create(2, (8,), L.F64)]))
    # a fill whose region leaves the array
    w = lazy._NodeWriter()
    t = w.leaf(ref(2, 1))
    v = w.scalar(1.0, 1, L.F64)
    w.op(60, L.OP_SET_REGION, False, 1, L.F64, [t, v], [None, None], ((0,), (12,), (1,)))
    with pytest.raises(RuntimeError, match="leaves extent"):
        itf.send_dag(1, _message([w.to_bytes(3, False)]))
    # a group over arrays of another dtype than it computes in
    w = lazy._NodeWriter()
    a32 = w.leaf(ref(3, 1, L.F32))
    w.op(61, L.OP_ADD, False, 1, L.F64, [a32, w.scalar(1.0, 1, L.F64)], [None, None], lazy._full_region((8,)))
    with pytest.raises(RuntimeError, match="dtype"):
        itf.send_dag(1, _message([w.to_bytes(4, True)]))
    # nothing of the above left a half-made result behind that blocks later work
    a = cnp.Array((8,), np.float64, name=2)
    a._gen = -1                                   # a borrowed name: never deleted by this handle
    assert itf.get(1, 2, 8).shape == (8,)


def test_frontend_refuses_like_upstream():
    cnp.reset()
    a = cnp.zeros((4, 5))
    with pytest.raises(ValueError):
        cnp.diag(a, 5)                                # diagonal out of range
    with pytest.raises(ValueError):
        cnp.diag(cnp.zeros((2, 2, 2)))
    with pytest.raises(ValueError):
        cnp.zeros((2, 3, 4)).matvec(cnp.zeros((4,)))  # no extent of 1 to drop
    with pytest.raises(NotImplementedError):
        a[::-1]
    with pytest.raises(TypeError):
        a.astype(np.float16)
    with pytest.raises(ValueError):
        a[0:2, 0:2] = cnp.zeros((3, 3))
    with pytest.raises(ValueError):
        cnp.zeros((2, 3, 4)) @ cnp.zeros((4, 2))      # no extent of 1 to drop
    with pytest.raises(ValueError):
        cnp.matmul(2.0, a)
    with pytest.raises(NotImplementedError):
        cnp.zeros((0, 3))
    with pytest.raises(NotImplementedError):
        cnp.zeros((2, 2, 2, 2))
    assert cnp.add(2, 3) == 5 and cnp.dot(2.0, 4.0) == 8.0
    assert cnp.tanh(0.0) == 0.0 and cnp.exp(0) == 1.0
    assert cnp.full((3,), 7).dtype == np.int64 and cnp.ones((2, 2)).dtype == np.float64
    assert cnp.arange(5).shape == (5,) and cnp.eye(3).shape == (3, 3)
    assert cnp.zeros_like(a).shape == (4, 5) and cnp.empty_like(a, dtype=np.int32).dtype == np.int32
    cnp.reset()


def test_get_region_is_the_slice_of_the_same_bounds(itf):
    a = cnp.zeros((40, 30))
    v = a.get_region(((2, 5), (38, 29), (3, 2)))
    w = a[2:38:3, 5:29:2]
    assert v.shape == w.shape == (12, 12) and v.region == w.region
    inner = v.get_region(((1, 0), (5, 12), (2, 1)))             # a view of a view composes
    assert inner.region == w[1:5:2, :].region

    class R:
        start, stop, step = (0, 0), (40, 30), (1, 1)
    assert a.get_region(R()).shape == (40, 30)
    for bad in (((0,), (40,), (1,)), ((0, 0), (41, 30), (1, 1)), ((0, 0), (40, 30), (0, 1)),
                ((5, 0), (5, 30), (1, 1))):
        with pytest.raises(IndexError):
            a.get_region(bad)


def test_randn_is_upstreams_placeholder(itf):
    r = cnp.random.randn(3, 5)
    assert r.shape == (3, 5) and r.dtype == np.float32


def test_an_lstm_step_is_a_product_and_one_merged_launch(itf):
    """examples/lstm_forward.py upstream, steps after the first two: the sigmoid over three gates'
    columns is cut into three pieces that join the run of the statements on one gate's columns (and
    the copies that prepare the next step's operand), so a step is the product plus one launch."""
    n, b, word, d = 6, 32, 16, 16
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
    cnp.execute(itf)
    work = [ln for ln in itf.trace() if ln.startswith("group") or ln.startswith("matmatmul")]
    # from the second product on: product, merged launch, product, merged launch, ...
    at = [i for i, ln in enumerate(work) if ln.startswith("matmatmul")]
    assert len(at) == n
    for a, b_ in zip(at[1:], at[2:] + [len(work)]):
        assert b_ - a == 2 and "path=statements" in work[a + 1]
    # three pieces + tanh + C + C += + Ct + Hout + the two copies for the next step
    assert sum("count=10" in ln for ln in work) == n - 2


def test_a_one_block_matrix_is_assigned_into_a_slab_of_a_rank3_array():
    """IFOG[t] = M and Hin[t, :, w:] = prev with M, prev rank-2 arrays stored as one block (their
    tile grid is ragged): presented to the rank-3 group with an extent-1 dimension in front."""
    cnp.reset()
    it = cnp.CharmNumericInterface(device=-1)
    it.connect(odf=4)
    it.set_trace()
    it.set_solver(True)
    it.set_layout(True)
    it.set_min_tile(2, 16)
    it.set_min_tile(3, 8)
    try:
        n, b, d, word = 2, 48, 40, 24
        h0 = cnp.zeros((1, d))
        Hin = cnp.zeros((n, b, word + d))
        prev = cnp.tile(h0, (b, 1))
        Hin[0, :, word:] = prev
        Hin[1, :, word:] = prev * 2.0
        cnp.execute(it)
        tr = it.trace()
        made = [ln for ln in tr if ln.startswith("create") and "shape=(48,40)" in ln]
        assert made and all("tile=32" in ln for ln in made)        # 40 columns in tiles of 32: ragged
        assert len([ln for ln in tr if ln.startswith("group") and "path=tiles" in ln]) == 2
    finally:
        cnp.reset()
        it.close()


# ---- the recording fast paths in C against the Python methods they stand in for ----

def _recorded(program, fast):
    """The statement log `program` leaves (records as bytes; direct calls by name and opcode)."""
    A = sys.modules["charmnumeric_amd.array"]
    cnp.reset()
    before = A.set_fast_recording(fast)
    try:
        program()
        out = [item if type(item) is bytes else ("call", item.name, item.opcode) for item in lazy._state.pending]
    finally:
        A.set_fast_recording(before)
        cnp.reset()
    return out


def _program_stencils():
    u, f = cnp.zeros((33, 65)), cnp.ones((33, 65))
    for _ in range(2):
        upd = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:] + 0.001 * f[1:-1, 1:-1])
        u[1:-1, 1:-1] = (1.0 - 2.0 / 3.0) * u[1:-1, 1:-1] + (2.0 / 3.0) * upd
    u[0, :] = 1.0
    u[-1] = 2
    u[3:9:2, ::4] = f[3:9:2, ::4] * 3 - 1
    u[5, 2:7] = u[6][:, 3:8] / 2.0
    v = u[::2][1:5]                       # a view of a view, strided outside, unit inside
    w = v[:, ::3][1:, 2:]
    u[20:23, 0:7] = -w[0:3, 0:7] + 1
    del upd, v, w


def _program_ranks_and_types():
    a, b = cnp.zeros(100), cnp.ones(100)
    c = 2 * a - b / 4 + (a - 1) * (3 - b)
    a[10:20] = c[30:40]
    a[::7] = -b[::7]
    a[5] = 1.5
    s = a @ b                             # one-element results as run-time scalars: Python's route
    a[:] = a * s + b
    i = cnp.zeros((8, 9), dtype=cnp.int32)
    i[1:3] = i[2:4] + 7
    j = i / 2 + i * 3
    x = cnp.zeros((4, 5, 6))
    x[1] = x[2] + x[3, :, :] * 0.5
    x[:, 1:4, ::2] = x[:, 0:3, 1::2] - 2
    x[..., 0] = 1.0                       # an ellipsis: Python's route
    y = cnp.zeros((4, 5, 6), dtype=cnp.float32)
    z = x + y                             # two element types: converted first, Python's route
    k = cnp.zeros((5, 6))
    x[2] = k                              # a matrix into a slab: Python's route
    del c, s, j, z


@pytest.mark.parametrize("program", [_program_stencils, _program_ranks_and_types])
def test_recording_in_c_leaves_the_same_log_as_the_python_methods(program):
    A = sys.modules["charmnumeric_amd.array"]
    if A._cnrec is None:
        pytest.skip("recording in Python only (CHARMNUMERIC_PYREC)")
    fast, slow = _recorded(program, True), _recorded(program, False)
    assert len(fast) == len(slow) and len(fast) > 20
    for n, (x, y) in enumerate(zip(fast, slow)):
        assert x == y, f"record {n} differs"


def test_errors_raised_through_the_c_paths_are_the_python_ones():
    cnp.reset()
    a, b = cnp.zeros((4, 6)), cnp.zeros((4, 7))
    with pytest.raises(IndexError):
        a[4]
    with pytest.raises(IndexError):
        a[0, 0, 0]
    with pytest.raises(NotImplementedError):
        a[::-1]
    with pytest.raises(NotImplementedError):
        a[2:2]
    with pytest.raises(ValueError):
        a + b
    with pytest.raises(ValueError):
        a[0:2] = b[0:2]
    with pytest.raises(TypeError):
        a["x"]
    with pytest.raises((TypeError, AttributeError)):
        del a[0]
    with pytest.raises(ValueError):
        a + "x"
    assert (1 - a).shape == (4, 6) and (-a).shape == (4, 6) and (np.float64(2.0) * a).shape == (4, 6)
    assert (a[1:3] / 2).shape == (2, 6) and a[1:3, 2].shape == (2, 1) and a[-1].shape == (1, 6)
    v = a[1:4][1:, ::2]
    assert v.region == ((2, 0), (4, 5), (1, 2)) and v.base is a and v.shape == (2, 3) and v.name == a.name
    cnp.reset()


def test_a_dying_array_leaves_one_deletion_record_and_an_old_generation_none():
    cnp.reset()
    a = cnp.zeros(10)
    t = a + 1
    name = t.name
    n = len(lazy._state.pending)
    del t
    assert lazy._state.pending[n:] == [struct.pack("<2i", 5, name)]
    old = a * 2
    cnp.reset()                                   # names restart: the handle names nothing any more
    del old, a
    assert lazy._state.pending == []


@pytest.mark.parametrize("rank", [1, 2, 3])
@pytest.mark.parametrize("seed", range(6))
def test_random_programs_record_the_same_log_through_c_and_python(seed, rank):
    """The random programs of the GPU suite (expressions over shifted and strided slices,
    assignments, copies, named temporaries, sums, dots and products on windows, two element types
    meeting), recorded twice: the two logs must be the same bytes, uploads included."""
    A = sys.modules["charmnumeric_amd.array"]
    if A._cnrec is None:
        pytest.skip("recording in Python only (CHARMNUMERIC_PYREC)")
    from tests.test_gpu_random_programs import MixedProgram, Program

    def record(fast):
        cnp.reset()
        before = A.set_fast_recording(fast)
        try:
            dtype = {4: np.float32, 3: np.int64, 5: np.int32}.get(seed, np.float64)
            prog = Program(1000 * rank + seed, rank, dtype)
            for _ in range(18):
                prog.statement()
            mixed = MixedProgram(77 * rank + seed, rank)
            for _ in range(8):
                mixed.statement()
            del prog, mixed
            return [item if type(item) is bytes else ("call", item.name, item.opcode, item.dtype,
                                                      item.payload.tobytes())
                    for item in lazy._state.pending]
        finally:
            A.set_fast_recording(before)
            cnp.reset()

    fast, slow = record(True), record(False)
    assert len(fast) == len(slow) and len(fast) > 50
    assert fast == slow
