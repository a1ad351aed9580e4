#!/usr/bin/env python3
"""Benchmark of the per-partition array execution path on one MI355X.

Headline (one JSON line on stdout): dense conjugate gradient at n = 16384 in fp64, iterations per
second, with the roofline of its dominant kernel (the tiled matvec, HBM-bound) and a CPU baseline
(the oracle's restatement of the reference CPU path) timed on the host cores of the same box.
A "step" is one CG iteration: one matvec over the 2x2 tile grid, two dots, two scalar ops and three
fused vector updates. Inputs are generated on the device before the timed region starts.

The other workloads (fused elementwise 2^24, Jacobi 2-D 8192^2, Jacobi 3-D 512^3, LSTM step) are
measured the same way and reported under "also" in the same line.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
FP64_MFMA_PEAK_TFLOPS = 78.6
# HBM bytes per launch of the tiled matvec at n = 16384, from rocprofv3 FETCH_SIZE (x 2.0, the
# factor a plain streaming kernel of known size gives on gfx950) + WRITE_SIZE (x 1.0):
# (2 099 620 + 259.9) KiB for the fused form, (2 098 440 + 128.1) KiB for the plain one,
# see profiles/bench_hbm_traffic_pmc.txt.
GEMV_N16384_TRAFFIC_BYTES = 2150277018
GEMV_N16384_TRAFFIC_BYTES_PLAIN = 2148933734


def _dev():
    from charmnumeric_amd import _lib as L

    L.check(L.lib.cnh_init(0))
    return L


class Buf:
    def __init__(self, L, nbytes, zero=False):
        p = C.c_void_p()
        L.check(L.lib.cnh_alloc(int(nbytes), 1 if zero else 0, C.byref(p)))
        self.ptr = p.value
        self.L = L
        self.nbytes = int(nbytes)

    def get(self, dtype=np.float64, count=None):
        n = self.nbytes // np.dtype(dtype).itemsize if count is None else count
        out = np.empty(n, dtype=dtype)
        self.L.check(self.L.lib.cnh_d2h(out.ctypes.data, self.ptr, out.nbytes, None))
        return out

    def free(self):
        if self.ptr:
            self.L.lib.cnh_free(self.ptr)
            self.ptr = None


class Events:
    """Pairs of HIP events on one stream; elapsed times read after a sync."""

    def __init__(self, L, n):
        self.L = L
        self.a = [C.c_void_p() for _ in range(n)]
        self.b = [C.c_void_p() for _ in range(n)]
        for e in self.a + self.b:
            L.check(L.lib.cnh_event_create(C.byref(e)))

    def times_ms(self, used):
        out = []
        ms = C.c_float()
        for i in range(used):
            self.L.check(self.L.lib.cnh_event_elapsed_ms(self.a[i], self.b[i], C.byref(ms)))
            out.append(ms.value)
        return out

    def free(self):
        for e in self.a + self.b:
            self.L.lib.cnh_event_destroy(e)


def _compile(L, ast, dtype, nd):
    k = C.c_void_p()
    L.check(L.lib.cnh_compile_group(C.byref(ast), dtype, nd, 0, C.byref(k)))
    return k


def _launch1(L, k, nd, ins, scalars, outs, stream=None):
    """One partition, broadcast scalars resident on the device."""
    n_in, n_out = len(ins), len(outs)
    ia = (L.Memref * max(1, n_in))(*ins)
    oa = (L.Memref * max(1, n_out))(*outs)
    sp = (C.c_void_p * max(1, len(scalars)))(*[C.c_void_p(s) for s in scalars])
    L.check(L.lib.cnh_launch_group(k, nd, n_in, ia, len(scalars), sp, 1, n_out, oa, stream))


# -------------------------------------------------------------------------------------------------
# C2: dense CG, n = 16384
# -------------------------------------------------------------------------------------------------
def cg_asts(L):
    """The element-wise part of one CG iteration as two groups. The scalar statements
    (alpha = r.r / p.Ap, beta = r.r_new / r.r) are formed in registers by the group that uses them,
    and r.r_new is taken by the launch that produces r_new: it leaves one partial sum per workgroup,
    which the p update sums (every workgroup in the same order) and stores for the next iteration.
    An iteration is four launches (matvec, dot, x and r, p) instead of eight; with the fused matvec
    (cnh_gemv_tiles_fused), which also forms p and leaves the partial sums of p.Ap, two.
    Group 1 (leaves 1 = p, 2 = x, 3 = Ap, 4 = r; scalars 5 = r.r, 6 = p.Ap):
        7 = x + alpha p, 8 = r - alpha Ap, 9 = sum of (8)^2 as partial sums.
    Group 2 (leaves 1 = p, 2 = r_new; scalars 5 = r.r_new given as those partial sums, 6 = r.r):
        7 = r_new + beta p."""
    from charmnumeric_amd.astbuild import AstBuilder

    def update_x_r():
        b = AstBuilder(L.F64, 1)
        alpha = b.binary(L.OP_DIV, 100, b.broadcast(5), b.broadcast(6))
        t1 = b.binary(L.OP_MUL, 101, alpha, b.leaf(1))
        b.binary(L.OP_ADD, 7, b.leaf(2), t1, is_temp=False)
        t2 = b.binary(L.OP_MUL, 102, alpha, b.leaf(3))
        r_new = b.binary(L.OP_SUB, 8, b.leaf(4), t2, is_temp=False)
        b.unary(L.OP_SUM_OF, 9, b.binary(L.OP_MUL, 103, r_new, r_new), is_temp=False)
        return b.finish()

    def update_p():
        b = AstBuilder(L.F64, 1)
        beta = b.binary(L.OP_DIV, 100, b.broadcast(5), b.broadcast(6))
        t = b.binary(L.OP_MUL, 101, beta, b.leaf(1))
        b.binary(L.OP_ADD, 7, b.leaf(2), t, is_temp=False)
        return b.finish()

    return update_x_r(), update_p()


def prepare_launch(L, k, nd, ins, scalars, outs, stream=None):
    """A launch of group kernel `k` over one partition, put together once: memrefs by leaf name,
    run-time scalars by name (a device address, or (address, count, where the sum goes) for one that
    is given as partial sums), memrefs by output name. Returns what fires it."""
    n_in, n_sc, n_out = C.c_int(), C.c_int(), C.c_int()
    L.check(L.lib.cnh_kernel_signature(k, C.byref(n_in), C.byref(n_sc), C.byref(n_out)))
    name, has, tgt, sr = C.c_int(), C.c_int(), C.c_int(), C.c_int()
    reg = L.Region()
    ia = (L.Memref * max(1, n_in.value))()
    oa = (L.Memref * max(1, n_out.value))()
    sp = (L.ScalarSum * max(1, n_sc.value))()
    for i in range(n_in.value):
        L.check(L.lib.cnh_kernel_input(k, i, C.byref(name), C.byref(has), C.byref(reg)))
        ia[i] = ins[name.value]
    for i in range(n_sc.value):
        L.check(L.lib.cnh_kernel_scalar(k, i, C.byref(name)))
        what = scalars[name.value]
        sp[i].ptr, sp[i].count, sp[i].folded = what if isinstance(what, tuple) else (what, 1, None)
    for i in range(n_out.value):
        L.check(L.lib.cnh_kernel_output(k, i, C.byref(name), C.byref(tgt), C.byref(sr), C.byref(reg)))
        oa[i] = outs[name.value]
    n_i, n_s, n_o = n_in.value, n_sc.value, n_out.value
    return lambda: L.check(L.lib.cnh_launch_group_sums(k, nd, n_i, ia, n_s, sp, n_o, oa, stream))


def run_cg(L, n, steps, warmup, tile_rule_tile=None, seed=2, check=True, trace_iters=0, fuse=True):
    """`steps` timed CG iterations. With trace_iters > 0 an untimed pass over the same system runs
    first and reads alpha, beta and r.r back after each of its iterations (and x at its end):
    what the parity check against the CPU leg compares."""
    tile = tile_rule_tile or cg_tile(n)
    g = (n + tile - 1) // tile
    t0 = time.time()
    tiles = []
    for i in range(g):
        for j in range(g):
            nr, nc = min(tile, n - i * tile), min(tile, n - j * tile)
            b = Buf(L, nr * nc * 8)
            L.check(L.lib.cnh_fill_cg_matrix(b.ptr, n, i * tile, nr, j * tile, nc, nc, seed, None))
            tiles.append(b)
    tptr = L.vparr([t.ptr for t in tiles])
    vec = lambda: Buf(L, n * 8, zero=True)
    bvec, x, r, p, Ap = vec(), vec(), vec(), vec(), vec()
    x2, r2, p2 = vec(), vec(), vec()
    L.check(L.lib.cnh_fill_uniform(bvec.ptr, n, seed, 1, 0, -1.0, 1.0, None))
    sc = Buf(L, 8 * 8, zero=True)  # slot 0 / 3: r.r of the current / next iterate (swapping), 1: p.Ap
    # partial sums of r_new . r_new, one per workgroup (512 elements) of the launch that updates r
    n_partials = (n + 511) // 512
    partials = Buf(L, n_partials * 8, zero=True)
    S = lambda i: sc.ptr + 8 * i
    k_xr, k_p = (_compile(L, a, L.F64, 1) for a in cg_asts(L))
    mr = lambda b_, cnt=n: L.Memref.dense(b_.ptr, (cnt,))

    # Vectors ping-pong between two buffers and r.r between two slots: an iteration's launches exist
    # in two prepared forms, for even and odd iterations.
    bufs = [{"x": x, "r": r, "p": p, "rtr": 0}, {"x": x2, "r": r2, "p": p2, "rtr": 3}]
    forms = []
    for cur, nxt in ((bufs[0], bufs[1]), (bufs[1], bufs[0])):
        forms.append({
            "p": cur["p"], "x_new": nxt["x"], "rtr": cur["rtr"], "rtr_new": nxt["rtr"], "r_new": nxt["r"],
            "update_x_r": prepare_launch(L, k_xr, 1, {1: mr(cur["p"]), 2: mr(cur["x"]), 3: mr(Ap), 4: mr(cur["r"])},
                                         {5: S(cur["rtr"]), 6: S(1)},
                                         {7: mr(nxt["x"]), 8: mr(nxt["r"]),
                                          9: L.Memref.dense(partials.ptr, (n_partials,))}),
            "update_p": prepare_launch(L, k_p, 1, {1: mr(cur["p"]), 2: mr(nxt["r"])},
                                       {5: (partials.ptr, n_partials, S(nxt["rtr"])), 6: S(cur["rtr"])},
                                       {7: mr(nxt["p"])}),
        })
    state = {"parity": 0, "first": True}

    # Two launches per iteration where the fused matvec applies (16384 rows or more): the matvec
    # forms p = r + beta p on the way (beta from the partial sums of r.r the previous launch left,
    # which it also folds and stores) and leaves the partial sums of p.Ap, one per workgroup; the
    # x and r update forms alpha from those. The p of the LAST iteration is formed by one closing
    # launch of the p update, so that the timed iterations leave the full CG state behind.
    n_pap = (n + 63) // 64
    pap = Buf(L, n_pap * 8, zero=True)
    fused = fuse and n >= 16384 and tile * 8 <= 65536 and tile % 2 == 0 and n % 2 == 0
    fforms = []
    if fused:
        for cur, nxt in ((bufs[0], bufs[1]), (bufs[1], bufs[0])):
            # iteration k of parity e: p_k -> cur["p"], formed from r_k = cur["r"] and p_{k-1} = nxt["p"];
            # r.r_k -> slot cur["rtr"], r.r_{k-1} in slot nxt["rtr"]
            fforms.append({
                "form_p": L.GemvFusion(cur["r"].ptr, nxt["p"].ptr, partials.ptr, n_partials, S(nxt["rtr"]),
                                       S(cur["rtr"]), cur["p"].ptr, pap.ptr, n_pap),
                "plain": L.GemvFusion(None, None, None, 0, None, None, cur["p"].ptr, pap.ptr, n_pap),
                "p": cur["p"],
                "update_x_r": prepare_launch(L, k_xr, 1, {1: mr(cur["p"]), 2: mr(cur["x"]), 3: mr(Ap), 4: mr(cur["r"])},
                                             {5: S(cur["rtr"]), 6: (pap.ptr, n_pap, S(1))},
                                             {7: mr(nxt["x"]), 8: mr(nxt["r"]),
                                              9: L.Memref.dense(partials.ptr, (n_partials,))}),
                # closes a run of iterations: p_{k+1} = r_{k+1} + beta p_k, r.r_{k+1} folded and stored
                "close": prepare_launch(L, k_p, 1, {1: mr(cur["p"]), 2: mr(nxt["r"])},
                                        {5: (partials.ptr, n_partials, S(nxt["rtr"])), 6: S(cur["rtr"])},
                                        {7: mr(nxt["p"])}),
            })

    def reset():
        # x = 0, r = p = b, r.r; the ping-pong roles go back to their starting assignment too
        state["parity"] = 0
        state["first"] = True
        L.check(L.lib.cnh_memset0(x.ptr, n * 8, None))
        L.check(L.lib.cnh_d2d(r.ptr, bvec.ptr, n * 8, None))
        L.check(L.lib.cnh_d2d(p.ptr, bvec.ptr, n * 8, None))
        L.check(L.lib.cnh_dot_partial(L.F64, n, r.ptr, r.ptr, S(0), None))

    def iteration(ev=None, i=0):
        if fused:
            f = fforms[state["parity"]]
            if ev is not None:
                L.check(L.lib.cnh_event_record(ev.a[i], None))
            # the first iteration after a reset (or after a closing launch) finds p ready
            fu = f["plain"] if state["first"] else f["form_p"]
            L.check(L.lib.cnh_gemv_tiles_fused(n, n, tile, tptr, f["p"].ptr, Ap.ptr, C.byref(fu), None, None))
            if ev is not None:
                L.check(L.lib.cnh_event_record(ev.b[i], None))
            f["update_x_r"]()                  # alpha from the partial sums of p.Ap; x, r, partial sums of r.r
            state["first"] = False
            state["parity"] ^= 1
            return
        f = forms[state["parity"]]
        if ev is not None:
            L.check(L.lib.cnh_event_record(ev.a[i], None))
        L.check(L.lib.cnh_gemv_tiles(L.F64, n, n, tile, tptr, f["p"].ptr, Ap.ptr, None))
        if ev is not None:
            L.check(L.lib.cnh_event_record(ev.b[i], None))
        L.check(L.lib.cnh_dot_partial(L.F64, n, f["p"].ptr, Ap.ptr, S(1), None))
        f["update_x_r"]()                      # x + alpha p, r - alpha Ap, partial sums of r_new . r_new
        f["update_p"]()                        # r.r_new summed and stored, r_new + beta p
        state["parity"] ^= 1

    def close():
        """After a run of fused iterations: forms the p (and stores the r.r) the last one left open."""
        if fused and not state["first"]:
            fforms[state["parity"] ^ 1]["close"]()
            state["first"] = True

    def current():
        return bufs[state["parity"]]

    reset()
    for _ in range(warmup):
        iteration()
    close()
    L.check(L.lib.cnh_device_sync())
    setup_s = time.time() - t0

    trace = None
    if trace_iters > 0:
        reset()
        trace = {"alpha": [], "beta": [], "rtr": []}
        for _ in range(trace_iters):
            before = current()["rtr"]
            iteration()
            close()                          # r.r of the new iterate is folded by the p update
            v = sc.get(np.float64)           # waits for the iteration
            after = current()["rtr"]
            # alpha and beta exist in registers only; the same two divisions on the host, from the
            # reduction results the device used (IEEE division: the same bits)
            trace["alpha"].append(float(v[before] / v[1]))
            trace["beta"].append(float(v[after] / v[before]))
            trace["rtr"].append(float(v[after]))
        trace["x"] = current()["x"].get()

    reset()
    ev = Events(L, steps)
    e0, e1 = C.c_void_p(), C.c_void_p()
    L.check(L.lib.cnh_event_create(C.byref(e0)))
    L.check(L.lib.cnh_event_create(C.byref(e1)))
    L.check(L.lib.cnh_device_sync())
    w0 = time.perf_counter()
    L.check(L.lib.cnh_event_record(e0, None))
    for i in range(steps):
        iteration(ev, i)
    close()                                  # inside the timed region: the last iteration's p and r.r
    L.check(L.lib.cnh_event_record(e1, None))
    L.check(L.lib.cnh_device_sync())
    wall = time.perf_counter() - w0
    ms = C.c_float()
    L.check(L.lib.cnh_event_elapsed_ms(e0, e1, C.byref(ms)))
    gemv_ms = ev.times_ms(steps)
    res = {
        "n": n, "tile": tile, "steps": steps, "wall_s": wall, "gpu_ms": ms.value,
        "ms_per_step": wall * 1e3 / steps, "iters_per_s": steps / wall,
        "gemv_avg_us": 1e3 * float(np.mean(gemv_ms)), "gemv_min_us": 1e3 * float(np.min(gemv_ms)),
        "setup_s": setup_s, "launches_per_iteration": 2 if fused else 4,
        "rtr_final": float(sc.get(np.float64)[current()["rtr"]]),
        "x": current()["x"].get() if check else None,
        "trace": trace,
    }
    ev.free()
    for b_ in tiles + [bvec, x, r, p, Ap, x2, r2, p2, sc, partials, pap]:
        b_.free()
    return res


def cg_tile(n, odf=4, pes=1, min_tile=512):
    """Tile edge of a 2-D array under the reference rule (decomposition_solver.hpp:100-122)."""
    tile = min_tile
    while ((n + tile - 1) // tile) ** 2 > odf * pes:
        tile *= 2
    return tile


def cpu_cg_setup(n, seed=2):
    from oracle import cn_oracle as O

    orc = O.Oracle()
    tile = cg_tile(n)
    g = (n + tile - 1) // tile
    tiles = [[orc.cg_matrix(n, i * tile, min(tile, n - i * tile), j * tile, min(tile, n - j * tile),
                            seed) for j in range(g)] for i in range(g)]
    b = orc.uniform(n, seed, 1, -1.0, 1.0)
    return orc, tile, g, tiles, b


def cpu_cg(setup, n, iters, threads, keep_x_at=None):
    """CG with the oracle's kernels in the reference's order of operations; returns
    (it/s, x, rtr, trace) where trace holds alpha, beta and r.r of every iteration and, with
    keep_x_at = k, a copy of x after k iterations."""
    from oracle import cn_oracle as O

    orc, tile, g, tiles, b = setup
    lib = orc.lib
    x = np.zeros(n)
    r = b.copy()
    p = b.copy()
    rtr = orc.dot(r, r)
    Ap = np.zeros(n)
    part = np.zeros(tile)
    trace = {"alpha": [], "beta": [], "rtr": [], "x": None, "rtr0": rtr}
    t0 = time.perf_counter()
    for it in range(iters):
        # tile GEMV + partial accumulate on the 1-D owner, column tiles in order
        for i in range(g):
            rows = tiles[i][0].shape[0]
            seg = Ap[i * tile:i * tile + rows]
            for j in range(g):
                t = tiles[i][j]
                xs = p[j * tile:j * tile + t.shape[1]]
                lib.orc_gemv_sub_mt(O.F64, O.ptr(t), t.shape[1], 0, 0, t.shape[0], t.shape[1],
                                    O.ptr(xs), O.ptr(part), threads)
                if j == 0:
                    seg[:] = part[:rows]
                else:
                    lib.orc_axpy1(O.F64, rows, O.ptr(part), O.ptr(seg))
        pAp = orc.dot(p, Ap)
        alpha = rtr / pAp
        x = x + alpha * p
        r = r - alpha * Ap
        rtr_new = orc.dot(r, r)
        beta = rtr_new / rtr
        p = r + beta * p
        rtr = rtr_new
        trace["alpha"].append(alpha)
        trace["beta"].append(beta)
        trace["rtr"].append(rtr)
        if keep_x_at == it + 1:
            trace["x"] = x.copy()
    dt = time.perf_counter() - t0
    return iters / dt, x, rtr, trace


def cg_parity(gpu_trace, cpu_trace, rtr0, floor=1e-24):
    """Agreement of the device's CG with the CPU leg on the same system: the solutions after the
    same number of iterations, and alpha, beta, r.r of every iteration whose r.r is still above
    `floor` times the initial one. Below that the recursion works on rounding noise (on this system
    from the sixth iteration on) and two correct implementations differ by factors."""
    n = min(len(gpu_trace["alpha"]), len(cpu_trace["alpha"]))
    k = 0
    while k < n and cpu_trace["rtr"][k] >= floor * rtr0:
        k += 1
    out = {"iterations_compared": n, "scalar_iterations": k}
    for key in ("alpha", "beta", "rtr"):
        g = np.array(gpu_trace[key][:k])
        c = np.array(cpu_trace[key][:k])
        out[f"{key}_max_rel_dev"] = float(np.max(np.abs(g - c) / np.abs(c))) if k else None
    xc = cpu_trace["x"]
    out["x_max_rel_diff"] = float(np.max(np.abs(gpu_trace["x"] - xc)) / np.max(np.abs(xc)))
    return out


# -------------------------------------------------------------------------------------------------
# C1: fused elementwise 2^24 + sum + dot
# -------------------------------------------------------------------------------------------------
def c1_ast(L, reduced=False):
    """z = 2.5 x - 0.5 y + x y (name 10). With `reduced`, sum(z) (20) and z.z (21) as reducing
    roots of the same group: the launch that stores z also sums it."""
    from charmnumeric_amd.astbuild import AstBuilder

    b = AstBuilder(L.F64, 1)
    x, y = b.leaf(0), b.leaf(1)
    t1 = b.binary(L.OP_MUL, 100, b.scalar(2.5), x)
    t2 = b.binary(L.OP_MUL, 101, b.scalar(0.5), y)
    t3 = b.binary(L.OP_SUB, 102, t1, t2)
    t4 = b.binary(L.OP_MUL, 103, x, y)
    z = b.binary(L.OP_ADD, 10, t3, t4, is_temp=False)
    if reduced:
        b.unary(L.OP_SUM_OF, 20, z, is_temp=False)
        zz = b.binary(L.OP_MUL, 104, z, z)
        b.unary(L.OP_SUM_OF, 21, zz, is_temp=False)
    return b.finish()


def run_c1(L, n=1 << 24, parts=4, reps=20):
    per = n // parts
    xs, ys, zs = [], [], []
    for q in range(parts):
        xb, yb, zb = Buf(L, per * 8), Buf(L, per * 8), Buf(L, per * 8)
        L.check(L.lib.cnh_fill_uniform(xb.ptr, per, 0, 0, q * per, -1.0, 1.0, None))
        L.check(L.lib.cnh_fill_uniform(yb.ptr, per, 0, 1, q * per, -1.0, 1.0, None))
        xs.append(xb); ys.append(yb); zs.append(zb)
    k = _compile(L, c1_ast(L), L.F64, 1)
    ins = (L.Memref * (4 * parts))()
    outs = (L.Memref * parts)()
    for q in range(parts):
        mx, my = L.Memref.dense(xs[q].ptr, (per,)), L.Memref.dense(ys[q].ptr, (per,))
        ins[4 * q], ins[4 * q + 1], ins[4 * q + 2], ins[4 * q + 3] = mx, my, mx, my
        outs[q] = L.Memref.dense(zs[q].ptr, (per,))
    ones = Buf(L, 8)
    res = Buf(L, 16, zero=True)
    zp = L.vparr([z.ptr for z in zs])
    lens = L.i64arr([per] * parts)

    def ew():
        L.check(L.lib.cnh_launch_group_batched(k, 1, parts, 4, ins, 0, None, 0, 1, outs, None))

    def sm():
        L.check(L.lib.cnh_sum_tiles(L.F64, parts, zp, lens, res.ptr, None))

    def dt():
        L.check(L.lib.cnh_dot_tiles(L.F64, parts, zp, zp, lens, res.ptr + 8, None))

    # the three as one group with reducing roots: one pass over x and y, z stored once and never
    # read back (the results go to a second pair of slots, compared with the first below)
    kr = _compile(L, c1_ast(L, reduced=True), L.F64, 1)
    res2 = Buf(L, 16, zero=True)
    outs_r = (L.Memref * (3 * parts))()
    for q in range(parts):
        outs_r[3 * q] = outs[q]
        outs_r[3 * q + 1] = L.Memref.dense(res2.ptr, (1,))
        outs_r[3 * q + 2] = L.Memref.dense(res2.ptr + 8, (1,))

    def fused():
        L.check(L.lib.cnh_launch_group_batched(kr, 1, parts, 4, ins, 0, None, 0, 3, outs_r, None))

    out = {}
    for name, fn, nbytes in (("elementwise", ew, 24 * n), ("sum", sm, 8 * n), ("dot_zz", dt, 8 * n),
                             ("elementwise_sum_dot_one_pass", fused, 24 * n)):
        for _ in range(3):
            fn()
        ev = Events(L, reps)
        L.check(L.lib.cnh_device_sync())
        for i in range(reps):
            L.check(L.lib.cnh_event_record(ev.a[i], None))
            fn()
            L.check(L.lib.cnh_event_record(ev.b[i], None))
        L.check(L.lib.cnh_device_sync())
        t = ev.times_ms(reps)
        # the same call issued `reps` times back to back between ONE pair of events: what it costs
        # inside a stream of launches, without an event record before and after every call
        L.check(L.lib.cnh_event_record(ev.a[0], None))
        for i in range(reps):
            fn()
        L.check(L.lib.cnh_event_record(ev.b[0], None))
        L.check(L.lib.cnh_device_sync())
        stream_us = 1e3 * ev.times_ms(1)[0] / reps
        ev.free()
        us = 1e3 * float(np.median(t))
        out[name] = {"us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1),
                     "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                     "us_back_to_back": round(stream_us, 2),
                     "hbm_frac_back_to_back": round(nbytes / stream_us / 1e3 / HBM_PEAK_GBS, 4)}
    separate, one_pass = res.get(np.float64), res2.get(np.float64)
    out["one_pass_vs_separate_rel_diff"] = float(np.max(np.abs(separate - one_pass) / np.abs(separate)))
    out["separate_passes_us"] = round(out["elementwise"]["us"] + out["sum"]["us"] + out["dot_zz"]["us"], 2)
    for b_ in xs + ys + zs + [ones, res, res2]:
        b_.free()
    return out


# -------------------------------------------------------------------------------------------------
# C3 / C4: Jacobi sweeps over tiles resident on the device
# -------------------------------------------------------------------------------------------------
def jacobi_ast(L, nd, n):
    from charmnumeric_amd.astbuild import AstBuilder

    b = AstBuilder(L.F64, nd)
    u = b.leaf(0)

    def reg(shift):
        return (tuple(shift), tuple(s + n - 2 for s in shift), (1,) * nd)

    shifts = []
    for d in range(nd):
        lo, hi = [1] * nd, [1] * nd
        lo[d], hi[d] = 0, 2
        shifts += [reg(lo), reg(hi)]
    t = b.binary(L.OP_ADD, 100, u, u, shifts[0], shifts[1])
    for i, r in enumerate(shifts[2:]):
        t = b.binary(L.OP_ADD, 101 + i, t, u, None, r)
    coef = 0.25 if nd == 2 else 0.16666666666666666
    t = b.binary(L.OP_MUL, 120, b.scalar(coef), t)
    b.set_region(121, u, t, reg([1] * nd))
    return b.finish()


class SubBuf:
    """A piece of a larger device allocation."""

    def __init__(self, L, ptr, nbytes):
        self.L, self.ptr, self.nbytes = L, ptr, int(nbytes)

    def free(self):
        pass


class TiledDev:
    """n^nd fp64 array in tiles of edge `tile`, laid out the way the host executor lays arrays out:
    rank 2 — every tile a row-major buffer of its own extents, carved back to back from one
    allocation; rank 3 — one row-major block over the whole array with the tiles as views into it
    (common row and plane pitches). CNH_BENCH_TILE_MAJOR=1 gives rank 3 separate tile buffers too,
    `skew` extra bytes apart (equally sized power-of-two tiles back to back start at addresses
    that differ by a multiple of their size: 462 us per 512^3 sweep against 424 us with 2 MiB +
    256 B between them)."""

    def __init__(self, L, nd, n, tile, skew=None):
        self.L, self.nd, self.n, self.tile = L, nd, n, tile
        self.g = (n + tile - 1) // tile
        self.flat = (nd == 3 or bool(os.environ.get("CNH_BENCH_FLAT2"))) and not os.environ.get("CNH_BENCH_TILE_MAJOR")
        if skew is None:
            skew = (2 << 20) + 256 if nd == 3 else 0
            if os.environ.get("CNH_BENCH_SKEW"):
                skew = int(os.environ["CNH_BENCH_SKEW"])
        idxs = list(np.ndindex(*([self.g] * nd)))
        exts = [[min(tile, n - i * tile) for i in idx] for idx in idxs]
        offs, off = [], 0
        if self.flat:
            offs = [sum(i * tile * n ** (nd - 1 - d) for d, i in enumerate(idx)) * 8 for idx in idxs]
            off = n ** nd * 8
        else:
            for ext in exts:
                offs.append(off)
                off += (int(np.prod(ext)) * 8 + 255) // 256 * 256 + skew
        self.slab = Buf(L, off, zero=True)
        self.bufs = [(idx, ext, SubBuf(L, self.slab.ptr + o, int(np.prod(ext)) * 8))
                     for idx, ext, o in zip(idxs, exts, offs)]
        self.ptrs = (C.c_void_p * len(self.bufs))(*[C.c_void_p(b.ptr) for _, _, b in self.bufs])
        d = L.Tiled()
        d.ndims, d.tile = nd, tile
        for i in range(nd):
            d.offset[i], d.shape[i], d.grid_lo[i], d.grid[i] = 0, n, 0, self.g
            if self.flat:
                d.pitch[i] = n ** (nd - 1 - i)
        d.tiles = C.cast(self.ptrs, C.POINTER(C.c_void_p))
        self.desc = d

    def strides(self, ext):
        """Elements between consecutive indices of each dimension inside a tile of extents ext."""
        if self.flat:
            return [self.n ** (self.nd - 1 - d) for d in range(self.nd)]
        return [int(np.prod(ext[d + 1:])) for d in range(self.nd)]

    def free(self):
        self.slab.free()


def run_jacobi(L, nd, n, tile, sweeps, reduce_every=10, reps_note=""):
    a, b = TiledDev(L, nd, n, tile), TiledDev(L, nd, n, tile)
    # initial state: 2-D hot top row; 3-D uniform[0,1) interior with zero faces
    for (idx, ext, buf), (_, _, buf2) in zip(a.bufs, b.bufs):
        if nd == 2:
            if idx[0] == 0:
                one = np.array([1.0]).view(np.uint8)
                L.check(L.lib.cnh_fill_region(2, 8, buf.ptr, L.i64arr(a.strides(ext)), L.i64arr([0, 0]),
                                              L.i64arr([1, 1]), L.i64arr([1, ext[1]]),
                                              one.ctypes.data, None))
    if nd == 3:
        _fill_3d(L, a, n)
    k = _compile(L, jacobi_ast(L, nd, n), L.F64, nd)
    nleaf = 2 * nd
    res = Buf(L, 8, zero=True)
    ntile = len(a.bufs)
    lens = L.i64arr([int(np.prod(e)) for _, e, _ in a.bufs])
    if a.flat:      # one block: the reductions read it as a single chunk
        ntile, lens = 1, L.i64arr([n ** nd])

    def sweep(src, dst):
        descs = (L.Tiled * nleaf)(*([src.desc] * nleaf))
        L.check(L.lib.cnh_launch_group_tiles(k, nleaf, descs, 0, None, 0, C.byref(src.desc),
                                             C.byref(dst.desc), None))

    def sweep_with_residual(src, dst):
        # the sweep accumulates sum (new - old)^2 (2-D) or max |new - old| (3-D) on the way
        descs = (L.Tiled * nleaf)(*([src.desc] * nleaf))
        L.check(L.lib.cnh_launch_group_tiles_residual(k, nleaf, descs, 0, None, 0, C.byref(src.desc),
                                                      C.byref(dst.desc), 0 if nd == 2 else 1, res.ptr, None))

    def residual(src, dst):
        fn = L.lib.cnh_sumsq_diff_tiles if nd == 2 else L.lib.cnh_maxabs_diff_tiles
        if a.flat:
            L.check(fn(1, L.vparr([dst.slab.ptr]), L.vparr([src.slab.ptr]), lens, res.ptr, None))
        else:
            L.check(fn(ntile, dst.ptrs, src.ptrs, lens, res.ptr, None))

    for _ in range(3):
        sweep(a, b)
        sweep_with_residual(b, a)
    L.check(L.lib.cnh_device_sync())
    ev = Events(L, sweeps)
    e0, e1 = C.c_void_p(), C.c_void_p()
    L.check(L.lib.cnh_event_create(C.byref(e0)))
    L.check(L.lib.cnh_event_create(C.byref(e1)))
    L.check(L.lib.cnh_event_record(e0, None))
    cur, nxt = a, b
    reducing = []
    for i in range(sweeps):
        L.check(L.lib.cnh_event_record(ev.a[i], None))
        if (i + 1) % reduce_every == 0:
            sweep_with_residual(cur, nxt)
            reducing.append(i)
        else:
            sweep(cur, nxt)
        L.check(L.lib.cnh_event_record(ev.b[i], None))
        cur, nxt = nxt, cur
    L.check(L.lib.cnh_event_record(e1, None))
    L.check(L.lib.cnh_device_sync())
    ms = C.c_float()
    L.check(L.lib.cnh_event_elapsed_ms(e0, e1, C.byref(ms)))
    t = ev.times_ms(sweeps)
    last_fused = float(res.get(np.float64)[0])
    # the same residual by a second pass over both buffers (what every tenth sweep cost before the
    # sweep accumulated it on the way), for comparison and as a check
    evr = Events(L, 5)
    for i in range(5):
        L.check(L.lib.cnh_event_record(evr.a[i], None))
        residual(nxt, cur)              # cur holds the newest contents, nxt the ones before
        L.check(L.lib.cnh_event_record(evr.b[i], None))
    L.check(L.lib.cnh_device_sync())
    tr = evr.times_ms(5)
    last_separate = float(res.get(np.float64)[0])
    # The whole run again between two events only (an event pair around every sweep costs a few
    # microseconds per sweep itself): once with the residual every reduce_every sweeps, once without.
    totals = {}
    for label, with_res in (("with", True), ("without", False)):
        L.check(L.lib.cnh_device_sync())
        L.check(L.lib.cnh_event_record(e0, None))
        cur, nxt = a, b
        for i in range(sweeps):
            if with_res and (i + 1) % reduce_every == 0:
                sweep_with_residual(cur, nxt)
            else:
                sweep(cur, nxt)
            cur, nxt = nxt, cur
        L.check(L.lib.cnh_event_record(e1, None))
        L.check(L.lib.cnh_device_sync())
        L.check(L.lib.cnh_event_elapsed_ms(e0, e1, C.byref(ms)))
        totals[label] = ms.value
    plain = [t[i] for i in range(sweeps) if i not in reducing]
    us_pair = 1e3 * float(np.median(plain))          # one sweep between its own pair of events
    # a sweep's cost in the loop: all sweeps between ONE pair of events (what the kernel trace shows
    # too; the event pair around every single sweep adds 2-4 us of its own)
    us = 1e3 * totals["without"] / sweeps
    us_red = 1e3 * float(np.median([t[i] for i in reducing])) if reducing else None
    interior = (n - 2) ** nd
    nbytes = 8.0 * ((n ** nd - (4 if nd == 2 else 0)) + interior) if nd == 2 else 8.0 * (n ** 3 + interior)
    out = {"sweeps": sweeps, "us_per_sweep": round(us, 2), "GBps": round(nbytes / us / 1e3, 1),
           "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
           "bytes_per_sweep": nbytes, "total_ms_with_reductions": round(totals["with"], 3),
           "total_ms_without_reductions": round(totals["without"], 3),
           "reductions_add_pct": round(100.0 * (totals["with"] / totals["without"] - 1.0), 2),
           "us_per_sweep_between_its_own_events": round(us_pair, 2),
           "hbm_frac_between_its_own_events": round(nbytes / us_pair / 1e3 / HBM_PEAK_GBS, 4),
           "us_per_reducing_sweep": round(us_red, 2) if us_red else None,
           "separate_reduction_pass_us": round(1e3 * float(np.median(tr)), 2),
           "last_reduction": last_fused, "last_reduction_by_separate_pass": last_separate,
           "partitions": len(a.bufs), "tile": tile,
           "layout": "one block, partitions as views" if a.flat else "one buffer per partition"}
    ev.free()
    evr.free()
    a.free()
    b.free()
    res.free()
    return out


def _fill_3d(L, arr, n):
    """Interior uniform[0,1) (seed 1, element index = row-major flat index), faces 0."""
    t = arr.tile
    if arr.flat:
        L.check(L.lib.cnh_fill_uniform(arr.slab.ptr, n ** 3, 1, 0, 0, 0.0, 1.0, None))
    else:
        for idx, ext, buf in arr.bufs:
            L.check(L.lib.cnh_fill_uniform_tile(buf.ptr, 3, L.i64arr(ext), L.i64arr([i * t for i in idx]),
                                                L.i64arr([n, n, n]), 1, 0, 0.0, 1.0, None))
    # zero the six faces
    zero = np.zeros(1).view(np.uint8)
    for idx, ext, buf in arr.bufs:
        st = L.i64arr(arr.strides(ext))
        for d in range(3):
            for side in (0, 1):
                if (side == 0 and idx[d] != 0) or (side == 1 and idx[d] != arr.g - 1):
                    continue
                start = [0, 0, 0]
                cnt = list(ext)
                start[d] = 0 if side == 0 else ext[d] - 1
                cnt[d] = 1
                L.check(L.lib.cnh_fill_region(3, 8, buf.ptr, st, L.i64arr(start), L.i64arr([1, 1, 1]),
                                              L.i64arr(cnt), zero.ctypes.data, None))


# -------------------------------------------------------------------------------------------------
# C5: LSTM forward (gate matmatmul on the fp64 matrix cores + fused gate groups)
# -------------------------------------------------------------------------------------------------
def lstm_asts(L, d):
    """The per-step statements of examples/lstm_forward.py:40-49 as SET_REGION groups on 2-D views
    (batch x columns) of the step's slice."""
    from charmnumeric_amd.astbuild import AstBuilder

    def sigmoid():        # IFOGf[:, :3d] = 1.0 / (1.0 + exp(IFOG[:, :3d] * -1))
        b = AstBuilder(L.F64, 2)
        x = b.leaf(1)
        t0 = b.binary(L.OP_MUL, 100, x, b.scalar(-1))
        t1 = b.unary(L.OP_EXP, 101, t0)
        t2 = b.binary(L.OP_ADD, 102, b.scalar(1.0), t1)
        b.binary(L.OP_DIV, 2, b.scalar(1.0), t2, is_temp=False)
        return b.finish()

    def tanh():           # out = tanh(in)
        b = AstBuilder(L.F64, 2)
        b.unary(L.OP_TANH, 2, b.leaf(1), is_temp=False)
        return b.finish()

    def mul():            # out = a * b
        b = AstBuilder(L.F64, 2)
        b.binary(L.OP_MUL, 3, b.leaf(1), b.leaf(2), is_temp=False)
        return b.finish()

    def muladd():         # out = c + f * cprev   (C[t] += f * C[t-1])
        b = AstBuilder(L.F64, 2)
        t = b.binary(L.OP_MUL, 100, b.leaf(2), b.leaf(3))
        b.binary(L.OP_ADD, 4, b.leaf(1), t, is_temp=False)
        return b.finish()

    return sigmoid(), tanh(), mul(), muladd()


def lstm_fused_ast(L, first, with_x=False):
    """All gate statements of one step (examples/lstm_forward.py:40-49 upstream) as one group with
    several output roots, each statement over its (batch x d) column window; later roots read
    earlier ones from registers. Leaves: 1..4 = the i, f, o, g windows of IFOG[t], 5 = C[t-1].
    Outputs: 11..14 = the windows of IFOGf[t], 15 = C[t], 16 = tanh(C[t]), 17 = Hout[t],
    18 = the same values again, for the right half of Hin[t+1]. with_x: leaf 6 = X[t+1] and output 19 =
    its copy for the left half of Hin[t+1] (`Hin[t+1, :, :word] = X[t+1]`, same extents when the input
    is as wide as the state)."""
    from charmnumeric_amd.astbuild import AstBuilder

    b = AstBuilder(L.F64, 2)

    def sigmoid(src, name, tmp):
        t0 = b.binary(L.OP_MUL, tmp, b.leaf(src), b.scalar(-1))
        t1 = b.unary(L.OP_EXP, tmp + 1, t0)
        t2 = b.binary(L.OP_ADD, tmp + 2, b.scalar(1.0), t1)
        return b.binary(L.OP_DIV, name, b.scalar(1.0), t2, is_temp=False)

    gi = sigmoid(1, 11, 100)
    gf = sigmoid(2, 12, 110)
    go = sigmoid(3, 13, 120)
    gg = b.unary(L.OP_TANH, 14, b.leaf(4), is_temp=False)
    if first:
        c = b.binary(L.OP_MUL, 15, gi, gg, is_temp=False)
    else:
        c0 = b.binary(L.OP_MUL, 130, gi, gg)
        fc = b.binary(L.OP_MUL, 131, gf, b.leaf(5))
        c = b.binary(L.OP_ADD, 15, c0, fc, is_temp=False)
    ct = b.unary(L.OP_TANH, 16, c, is_temp=False)
    h = b.binary(L.OP_MUL, 17, go, ct, is_temp=False)
    idx = b._new(18, L.OP_COPY, is_temp=False)
    node = b._nodes[idx]
    node.n_operands = 1
    b._attach(node, 0, h, None)
    b._roots.append(idx)
    if with_x:
        idx = b._new(19, L.OP_COPY, is_temp=False)
        node = b._nodes[idx]
        node.n_operands = 1
        b._attach(node, 0, b.leaf(6), None)
        b._roots.append(idx)
    return b.finish()


def run_lstm(L, steps=64, batch=256, nin=1024, d=1024, seed=5, timed=True, keep=False, fused=True, warm_passes=5,
             merge_x=True, epilogue=True):
    """epilogue: the gate launch of a step rides on the step's product (cnh_launch_product_group) where
    the shape is one the product kernel takes that way; the events "around the product" then cover
    the whole step's launch."""
    k_in = nin + d
    merge_x = merge_x and fused and nin == d     # the copy of x_{t+1} rides on step t's gate launch
    X = Buf(L, steps * batch * nin * 8)
    W = Buf(L, k_in * 4 * d * 8)
    L.check(L.lib.cnh_fill_uniform(X.ptr, steps * batch * nin, seed, 0, 0, -1.0, 1.0, None))
    # W = [W_ih^T ; W_hh^T] (k_in x 4d): streams 1 and 2 hold W_ih, W_hh as (4d x nin), (4d x d);
    # the transpose is laid out directly by generating row r of W from column r of the stream.
    bound = 1.0 / 32.0
    Wih = Buf(L, 4 * d * nin * 8)
    Whh = Buf(L, 4 * d * d * 8)
    L.check(L.lib.cnh_fill_uniform(Wih.ptr, 4 * d * nin, seed, 1, 0, -bound, bound, None))
    L.check(L.lib.cnh_fill_uniform(Whh.ptr, 4 * d * d, seed, 2, 0, -bound, bound, None))
    i64 = L.i64arr
    one = i64([1, 1])
    zero2 = i64([0, 0])
    # W[r, c] = Wih[c, r] for r < nin: a strided copy with swapped strides
    L.check(L.lib.cnh_copy_region(2, 8, W.ptr, i64([4 * d, 1]), zero2, one, Wih.ptr, i64([1, nin]),
                                  zero2, one, i64([nin, 4 * d]), None))
    L.check(L.lib.cnh_copy_region(2, 8, W.ptr + nin * 4 * d * 8, i64([4 * d, 1]), zero2, one, Whh.ptr,
                                  i64([1, d]), zero2, one, i64([d, 4 * d]), None))
    Wih.free()
    Whh.free()
    Hin = Buf(L, steps * batch * k_in * 8, zero=True)
    IFOG = Buf(L, steps * batch * 4 * d * 8, zero=True)
    IFOGf = Buf(L, steps * batch * 4 * d * 8, zero=True)
    Cc = Buf(L, steps * batch * d * 8, zero=True)
    Ct = Buf(L, steps * batch * d * 8, zero=True)
    Hout = Buf(L, steps * batch * d * 8, zero=True)
    a_sig, a_tanh, a_mul, a_muladd = lstm_asts(L, d)
    k_sig, k_tanh, k_mul, k_muladd = (_compile(L, a, L.F64, 2) for a in (a_sig, a_tanh, a_mul, a_muladd))
    k_first, k_later = (_compile(L, lstm_fused_ast(L, f, merge_x), L.F64, 2) for f in (True, False))
    k_last = _compile(L, lstm_fused_ast(L, steps == 1), L.F64, 2) if merge_x else k_later
    spare = Buf(L, batch * d * 8)      # where the last step's copy of h goes (no Hin[steps])

    def view(buf, t, row_len, c0, ncols):
        base = buf.ptr + (t * batch * row_len + c0) * 8
        return L.Memref.strided(base, (batch, ncols), (row_len, 1))

    ev = Events(L, steps)
    stream = C.c_void_p()
    L.check(L.lib.cnh_stream_create(C.byref(stream)))

    # Everything a step launches is put together before the clock starts (descriptor tables,
    # memrefs by leaf name): the timed loop only fires prepared launches, as a compiled caller would.
    def prepared_group(k, nd, ins, outs):
        n_in, n_sc, n_out = C.c_int(), C.c_int(), C.c_int()
        L.check(L.lib.cnh_kernel_signature(k, C.byref(n_in), C.byref(n_sc), C.byref(n_out)))
        name, has, tgt, sr = C.c_int(), C.c_int(), C.c_int(), C.c_int()
        reg = L.Region()
        ia = (L.Memref * max(1, n_in.value))()
        oa = (L.Memref * max(1, n_out.value))()
        for i in range(n_in.value):
            L.check(L.lib.cnh_kernel_input(k, i, C.byref(name), C.byref(has), C.byref(reg)))
            ia[i] = ins[name.value]
        for i in range(n_out.value):
            L.check(L.lib.cnh_kernel_output(k, i, C.byref(name), C.byref(tgt), C.byref(sr), C.byref(reg)))
            oa[i] = outs[name.value]
        return lambda: L.check(L.lib.cnh_launch_group(k, nd, n_in.value, ia, 0, None, 1, n_out.value, oa, stream))

    def prepared1(k, nd, ins, outs):
        ia = (L.Memref * max(1, len(ins)))(*ins)
        oa = (L.Memref * max(1, len(outs)))(*outs)
        return lambda: L.check(L.lib.cnh_launch_group(k, nd, len(ins), ia, 0, None, 1, len(outs), oa, stream))

    def prepared_copy(dst, dst_strides, src, src_strides, extent):
        args = (2, 8, dst, i64(dst_strides), zero2, one, src, i64(src_strides), zero2, one, i64(extent), stream)
        return lambda: L.check(L.lib.cnh_copy_region(*args))

    def product_job(t):
        # IFOG[t] = Hin[t] @ W, written without reading what IFOG[t] held
        jobs = (L.GemmJob * 1)()
        jobs[0].M, jobs[0].N, jobs[0].K = batch, 4 * d, k_in
        jobs[0].A, jobs[0].lda = Hin.ptr + t * batch * k_in * 8, k_in
        jobs[0].B, jobs[0].ldb = W.ptr, 4 * d
        jobs[0].C, jobs[0].ldc = IFOG.ptr + t * batch * 4 * d * 8, 4 * d
        return jobs

    def prepared_product(t):
        jobs = product_job(t)
        return lambda: L.check(L.lib.cnh_gemm_batch(L.F64, 1, jobs, 1, stream))

    one_launch = []      # per step: did the product take the gate statements along?

    def prepared_product_group(t, k, ins, outs):
        """The product of step t and the gate group in one launch, the group's leaves 1..4 being the
        product's four column blocks; falls back to two launches where the kernel does not take the shape."""
        jobs = product_job(t)
        n_in, n_sc, n_out = C.c_int(), C.c_int(), C.c_int()
        L.check(L.lib.cnh_kernel_signature(k, C.byref(n_in), C.byref(n_sc), C.byref(n_out)))
        name, has, tgt, sr = C.c_int(), C.c_int(), C.c_int(), C.c_int()
        reg = L.Region()
        ia = (L.Memref * max(1, n_in.value))()
        oa = (L.Memref * max(1, n_out.value))()
        blocks = (C.c_int32 * max(1, n_in.value))()
        for i in range(n_in.value):
            L.check(L.lib.cnh_kernel_input(k, i, C.byref(name), C.byref(has), C.byref(reg)))
            ia[i] = ins[name.value]
            blocks[i] = name.value - 1 if 1 <= name.value <= 4 else -1
        for i in range(n_out.value):
            L.check(L.lib.cnh_kernel_output(k, i, C.byref(name), C.byref(tgt), C.byref(sr), C.byref(reg)))
            oa[i] = outs[name.value]
        two = [lambda: L.check(L.lib.cnh_gemm_batch(L.F64, 1, jobs, 1, stream)),
               lambda: L.check(L.lib.cnh_launch_group(k, 2, n_in.value, ia, 0, None, 1, n_out.value, oa, stream))]
        state = {"fused": None}

        def fire():
            if state["fused"] is not False:
                rc = L.lib.cnh_launch_product_group(k, jobs, 4, 2, n_in.value, ia, blocks, 0, None, 1, n_out.value,
                                                    oa, stream)
                if rc == -17 and state["fused"] is None:
                    state["fused"] = False
                else:
                    L.check(rc)
                    state["fused"] = True
                    return
            for f in two:
                f()
        one_launch.append(state)
        return fire

    def prepare(t):
        """(what runs before the product, the product, what runs after it) of step t."""
        # Hin[t, :, :nin] = X[t]; Hin[t, :, nin:] = Hout[t-1] (h0 = 0 at t = 0)
        before = []
        if t == 0 or not merge_x:
            before.append(prepared_copy(Hin.ptr + t * batch * k_in * 8, [k_in, 1], X.ptr + t * batch * nin * 8,
                                        [nin, 1], [batch, nin]))
        if t > 0 and not fused:
            before.append(prepared_copy(Hin.ptr + (t * batch * k_in + nin) * 8, [k_in, 1],
                                        Hout.ptr + (t - 1) * batch * d * 8, [d, 1], [batch, d]))
        after = []
        if fused:
            # every gate statement of the step in one launch; h goes to Hout[t] and, for the next
            # step's product, to the right half of Hin[t+1]
            ins = {1: view(IFOG, t, 4 * d, 0, d), 2: view(IFOG, t, 4 * d, d, d),
                   3: view(IFOG, t, 4 * d, 2 * d, d), 4: view(IFOG, t, 4 * d, 3 * d, d)}
            if t > 0:
                ins[5] = view(Cc, t - 1, d, 0, d)
            nxt = (view(Hin, t + 1, k_in, nin, d) if t + 1 < steps
                   else L.Memref.strided(spare.ptr, (batch, d), (d, 1)))
            outs = {11: view(IFOGf, t, 4 * d, 0, d), 12: view(IFOGf, t, 4 * d, d, d),
                    13: view(IFOGf, t, 4 * d, 2 * d, d), 14: view(IFOGf, t, 4 * d, 3 * d, d),
                    15: view(Cc, t, d, 0, d), 16: view(Ct, t, d, 0, d), 17: view(Hout, t, d, 0, d), 18: nxt}
            kern = k_first if t == 0 else k_later
            if merge_x and t + 1 < steps:
                ins[6] = view(X, t + 1, nin, 0, nin)
                outs[19] = view(Hin, t + 1, k_in, 0, nin)
            elif merge_x:
                kern = k_last
            if epilogue:
                return before, prepared_product_group(t, kern, ins, outs), []
            after.append(prepared_group(kern, 2, ins, outs))
        else:
            after.append(prepared1(k_sig, 2, [view(IFOG, t, 4 * d, 0, 3 * d)], [view(IFOGf, t, 4 * d, 0, 3 * d)]))
            after.append(prepared1(k_tanh, 2, [view(IFOG, t, 4 * d, 3 * d, d)], [view(IFOGf, t, 4 * d, 3 * d, d)]))
            after.append(prepared1(k_mul, 2, [view(IFOGf, t, 4 * d, 0, d), view(IFOGf, t, 4 * d, 3 * d, d)],
                                   [view(Cc, t, d, 0, d)]))
            if t > 0:
                # leaf uses are collected root by root: (f, C[t-1]) of the product, then C[t]
                after.append(prepared1(k_muladd, 2, [view(IFOGf, t, 4 * d, d, d), view(Cc, t - 1, d, 0, d),
                                                     view(Cc, t, d, 0, d)], [view(Cc, t, d, 0, d)]))
            after.append(prepared1(k_tanh, 2, [view(Cc, t, d, 0, d)], [view(Ct, t, d, 0, d)]))
            after.append(prepared1(k_mul, 2, [view(IFOGf, t, 4 * d, 2 * d, d), view(Ct, t, d, 0, d)],
                                   [view(Hout, t, d, 0, d)]))
        return before, prepared_product(t), after

    plan = [prepare(t) for t in range(steps)]
    L.check(L.lib.cnh_device_sync())         # the fills above ran on the default stream

    def run_steps(count, product_events):
        for t in range(count):
            before, product, after = plan[t]
            for fire in before:
                fire()
            if product_events:
                L.check(L.lib.cnh_event_record(ev.a[t], stream))
            product()
            if product_events:
                L.check(L.lib.cnh_event_record(ev.b[t], stream))
            for fire in after:
                fire()

    out = {}
    e0, e1 = C.c_void_p(), C.c_void_p()
    L.check(L.lib.cnh_event_create(C.byref(e0)))
    L.check(L.lib.cnh_event_create(C.byref(e1)))
    flop = 2.0 * batch * k_in * 4 * d
    if timed:
        run_steps(min(steps, 3), False)      # builds the kernels
        L.check(L.lib.cnh_stream_sync(stream))

    def measure(warm):
        """(median product time, whole-pass time per step), each after `warm` untimed passes queued
        right ahead of it: no pause, the device never idles between them and the measured pass."""
        total_ms = C.c_float(0.0)
        for _ in range(warm):
            run_steps(steps, False)
        run_steps(steps, True)               # an event pair around every product
        L.check(L.lib.cnh_stream_sync(stream))
        g = ev.times_ms(steps)
        if timed:
            for _ in range(warm):
                run_steps(steps, False)
            L.check(L.lib.cnh_event_record(e0, stream))
            run_steps(steps, False)          # one event pair around all steps, nothing between the launches
            L.check(L.lib.cnh_event_record(e1, stream))
            L.check(L.lib.cnh_stream_sync(stream))
            L.check(L.lib.cnh_event_elapsed_ms(e0, e1, C.byref(total_ms)))
        return 1e3 * float(np.median(g)), 1e3 * total_ms.value / steps

    # The matrix pipe's clock rises under sustained load: right after an idle device the product
    # takes 81-87 us, after about 30 ms of uninterrupted steps 72-73 us (measured on MI355X; the
    # HBM-bound workloads do not change). Both are measured.
    gus_idle, step_idle = measure(0)
    gus, step_us = measure(warm_passes) if (timed and warm_passes > 0) else (gus_idle, step_idle)
    ceiling = C.c_double()
    L.check(L.lib.cnh_probe_mfma_f64(8192, C.byref(ceiling)))   # ~1 ms of back-to-back matrix instructions
    # Primary figures: one forward pass of the configuration (64 steps, about 6 ms) started on an
    # idle device, which is what the configuration as stated runs at. The same pass queued behind
    # untimed ones (a long sequence, a training loop) is reported beside it as `sustained`.
    out = {"steps": steps, "gemm_us": round(gus_idle, 2), "gemm_tflops": round(flop / gus_idle / 1e6, 2),
           "mfma_frac": round(flop / gus_idle / 1e6 / FP64_MFMA_PEAK_TFLOPS, 4),
           "step_us": round(step_idle, 2),
           "step_frac_of_mfma_roofline": round(flop / FP64_MFMA_PEAK_TFLOPS / 1e6 / step_idle, 4)
           if step_idle else None,
           "measured_from": "an idle device (one pass of 64 steps)",
           "mfma_measured_ceiling_tflops": round(ceiling.value, 1),
           "sustained": {"gemm_us": round(gus, 2), "gemm_tflops": round(flop / gus / 1e6, 2),
                         "mfma_frac": round(flop / gus / 1e6 / FP64_MFMA_PEAK_TFLOPS, 4),
                         "mfma_frac_of_measured_ceiling": round(flop / gus / 1e6 / ceiling.value, 4)
                         if ceiling.value else None,
                         "step_us": round(step_us, 2),
                         "step_frac_of_mfma_roofline":
                             round(flop / FP64_MFMA_PEAK_TFLOPS / 1e6 / step_us, 4) if step_us else None,
                         "untimed_passes_queued_ahead": warm_passes if timed else 0},
           "flop_per_step": flop}
    if keep:
        out["Hout"] = Hout.get().reshape(steps, batch, d)
        out["C"] = Cc.get().reshape(steps, batch, d)
        out["IFOG"] = IFOG.get().reshape(steps, batch, 4 * d)
        out["IFOGf"] = IFOGf.get().reshape(steps, batch, 4 * d)
        out["Ct"] = Ct.get().reshape(steps, batch, d)
        out["Hin"] = Hin.get().reshape(steps, batch, k_in)
    ev.free()
    for e in (e0, e1):
        L.lib.cnh_event_destroy(e)
    L.check(L.lib.cnh_stream_destroy(stream))
    out["gate_launches_per_step"] = 1 if fused else 6
    # the product, the gate launch (which also lays x_{t+1} into the next step's operand when the
    # input is as wide as the state) and otherwise the copy of x_t
    out["launches_per_step"] = (2 if merge_x else 3) if fused else 9
    if one_launch and all(st["fused"] for st in one_launch):
        # the gate statements ran in the product's epilogue: the events "around the product" covered the
        # step's whole launch (product, gate statements, the copies for the next step)
        out["launches_per_step"] -= 1
        out["gate_launches_per_step"] = 0
        for part in (out, out["sustained"]):
            part["launch_us"] = part.pop("gemm_us")
            for key in ("gemm_tflops", "mfma_frac", "mfma_frac_of_measured_ceiling"):
                part.pop(key, None)
    for b_ in (X, W, Hin, IFOG, IFOGf, Cc, Ct, Hout, spare):
        b_.free()
    return out


def cpu_jacobi(nd, n, tile, sweeps, threads):
    """The same sweep on the host through the oracle's chare-by-chare restatement of the reference
    path (halo pack + delivery, aligned cells, one interpreted kernel per cell, SET_REGION copy),
    `threads` chares side by side. A bounded sample: `sweeps` sweeps of the full-size array."""
    from charmnumeric_amd import _lib as L
    from oracle import cn_oracle as O

    orc = O.Oracle()
    ast = jacobi_ast(L, nd, n)
    g = (n + tile - 1) // tile
    tiles = []
    for idx in np.ndindex(*([g] * nd)):
        ext = [min(tile, n - i * tile) for i in idx]
        t = np.zeros(ext)
        if idx[0] == 0:
            t[0] = 1.0
        tiles.append(t)
    t0 = time.perf_counter()
    for _ in range(sweeps):
        rc, st = orc.world_group(ast, L.F64, (n,) * nd, tile, tiles, threads)
        if rc:
            raise RuntimeError(f"oracle world sweep failed: {rc}")
    dt = time.perf_counter() - t0
    return {"us_per_sweep": round(dt / sweeps * 1e6, 1), "threads": threads, "sweeps": sweeps,
            "messages_per_sweep": st["messages"], "halo_bytes_per_sweep": st["bytes"],
            "kernel_calls_per_sweep": st["kernels"],
            "what": "oracle restatement of the reference's fragment path, one thread per chare"}


def _physical_cores():
    """(logical CPUs the process may use, physical cores of the box as /proc/cpuinfo lists them)."""
    logical = os.cpu_count() or 1
    try:
        logical = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        pass
    cores = set()
    try:
        phys = core = None
        with open("/proc/cpuinfo") as f:
            for ln in f:
                if ln.startswith("physical id"):
                    phys = ln.split(":")[1].strip()
                elif ln.startswith("core id"):
                    core = ln.split(":")[1].strip()
                elif not ln.strip():
                    if core is not None:
                        cores.add((phys, core))
                    phys = core = None
    except OSError:
        pass
    return logical, (len(cores) or None)


def cpu_c1(threads, n=1 << 24, parts=4, passes=3):
    """Configuration 1 on the host as the reference's fast path runs it
    (src/execute_node.cpp:1263-1336 upstream): the fused statement chare by chare over the 4 tiles
    (one interpreted kernel per chare, `threads` chares side by side, at most one thread per chare),
    then z . ones and z . z tile by tile with the partials added in tile order
    (src/executor_reduce.cpp:62-94 upstream). A bounded sample: `passes` passes at full size."""
    from concurrent.futures import ThreadPoolExecutor

    from charmnumeric_amd import _lib as L
    from oracle import cn_oracle as O

    orc = O.Oracle()
    per = n // parts
    ast = c1_ast(L)
    xs = [orc.uniform(per, 0, 0, -1.0, 1.0, first=q * per) for q in range(parts)]
    ys = [orc.uniform(per, 0, 1, -1.0, 1.0, first=q * per) for q in range(parts)]
    zs = [np.empty(per) for _ in range(parts)]
    ones = np.ones(per)
    workers = max(1, min(threads, parts))

    def chare(q):
        if orc.eval_group(ast, L.F64, 1, [xs[q], ys[q], xs[q], ys[q]], [], [zs[q]]):
            raise RuntimeError("oracle group evaluation failed")

    def dots(q):
        return orc.dot(zs[q], ones), orc.dot(zs[q], zs[q])

    t_elem = t_red = 0.0
    s = nrm2 = 0.0
    with ThreadPoolExecutor(workers) as pool:
        list(pool.map(chare, range(parts)))       # untimed: the result tiles' pages are touched here
        for _ in range(passes):
            t0 = time.perf_counter()
            list(pool.map(chare, range(parts)))
            t1 = time.perf_counter()
            partials = list(pool.map(dots, range(parts)))
            s = nrm2 = 0.0
            for a, b in partials:                 # tile order, as the reducer adds them
                s += a
                nrm2 += b
            t2 = time.perf_counter()
            t_elem += t1 - t0
            t_red += t2 - t1
    elem_us = t_elem / passes * 1e6
    return {"elementwise_us": round(elem_us, 1), "elementwise_GBs": round(24.0 * n / (elem_us * 1e-6) / 1e9, 2),
            "two_reductions_us": round(t_red / passes * 1e6, 1), "threads": workers, "passes": passes,
            "sum": float(s), "norm": float(np.sqrt(nrm2)),
            "what": "oracle restatement of the reference's fast path: one fused loop per chare over 4 chares, "
                    "then tile dots added in tile order"}


def cpu_lstm(threads, steps=2, batch=256, nin=1024, d=1024, seed=5):
    """Configuration 5 on the host: per step the gate product as the reference's panel accumulate
    (C zeroed, C += A.B, src/executor_incremental.cpp:120-132 upstream; rows split over `threads`)
    and the gate statements of examples/lstm_forward.py:40-49 upstream as one interpreted group
    each. A bounded sample: `steps` steps at the full shape."""
    from charmnumeric_amd import _lib as L
    from oracle import cn_oracle as O

    orc = O.Oracle()
    k_in = nin + d
    X = orc.uniform(steps * batch * nin, seed, 0, -1.0, 1.0).reshape(steps, batch, nin)
    Wih = orc.uniform(4 * d * nin, seed, 1, -1.0 / 32, 1.0 / 32).reshape(4 * d, nin)
    Whh = orc.uniform(4 * d * d, seed, 2, -1.0 / 32, 1.0 / 32).reshape(4 * d, d)
    W = np.ascontiguousarray(np.concatenate([Wih.T, Whh.T], axis=0))
    Hin = np.zeros((steps, batch, k_in))
    IFOG = np.zeros((steps, batch, 4 * d))
    IFOGf = np.zeros((steps, batch, 4 * d))
    Cc = np.zeros((steps, batch, d))
    Ct = np.zeros((steps, batch, d))
    Hout = np.zeros((steps, batch, d))
    a_sig, a_tanh, a_mul, a_muladd = lstm_asts(L, d)

    def group(ast, ins, outs):
        if orc.eval_group(ast, L.F64, 2, ins, [], outs):
            raise RuntimeError("oracle group evaluation failed")

    t_gemm = t_gate = 0.0
    for t in range(steps):
        Hin[t, :, :nin] = X[t]
        if t > 0:
            Hin[t, :, nin:] = Hout[t - 1]
        t0 = time.perf_counter()
        IFOG[t] = 0.0
        orc.gemm_acc(Hin[t], W, IFOG[t], threads=threads)
        t1 = time.perf_counter()
        group(a_sig, [IFOG[t, :, :3 * d]], [IFOGf[t, :, :3 * d]])
        group(a_tanh, [IFOG[t, :, 3 * d:]], [IFOGf[t, :, 3 * d:]])
        group(a_mul, [IFOGf[t, :, :d], IFOGf[t, :, 3 * d:]], [Cc[t]])
        if t > 0:
            group(a_muladd, [IFOGf[t, :, d:2 * d], Cc[t - 1], Cc[t]], [Cc[t]])
        group(a_tanh, [Cc[t]], [Ct[t]])
        group(a_mul, [IFOGf[t, :, 2 * d:3 * d], Ct[t]], [Hout[t]])
        t2 = time.perf_counter()
        t_gemm += t1 - t0
        t_gate += t2 - t1
    flop = 2.0 * batch * k_in * 4 * d
    return {"gemm_us": round(t_gemm / steps * 1e6, 1), "gemm_GFLOPs": round(flop * steps / t_gemm / 1e9, 2),
            "gates_us": round(t_gate / steps * 1e6, 1), "step_us": round((t_gemm + t_gate) / steps * 1e6, 1),
            "threads": threads, "steps": steps, "h_last_abs_mean": float(np.mean(np.abs(Hout[steps - 1]))),
            "what": "oracle restatement: panel accumulate C += A.B with rows over threads, then the six gate "
                    "statements as interpreted groups on one thread"}


def run_frontend_cg(n, steps, warmup, trace_iters=0):
    """The headline: the CG iteration of examples/cg.py:40-52 upstream written with the frontend's
    operators and run by the host executor (statement log -> planner -> DAG nodes -> kernels), the
    route a user of the drop-in takes. One step = one CG iteration; the timed region is `steps`
    iterations between two syncs, recording and flushing included. The matvec launches of the
    timed stretch are bracketed by events on the executor's own stream. With trace_iters > 0 an
    untimed pass over the same system first keeps alpha, beta and r.r of every iteration and x at
    its end for the parity check against the CPU leg."""
    import charmnumeric_amd as cnp
    out = {}
    cnp.reset()
    itf = cnp.CharmNumericInterface(device=0)
    itf.connect(odf=4)
    itf.set_pipeline(True)               # the executor works on its own thread while Python records
    try:
        cnp.set_auto_flush(itf, 48)      # keep the device busy while later statements are recorded
        A = cnp.random.cg_matrix(n, 2)
        b = cnp.random.uniform((n,), seed=2, stream=1, low=-1.0, high=1.0)
        cnp.execute(itf)
        out["tile"] = itf.array_info(A.name)["tile"]
        state = {}

        def start():
            state["x"] = cnp.zeros((n,))
            state["r"] = b.copy()
            state["p"] = b.copy()
            state["rtr"] = state["r"] @ state["r"]

        def iterate(k, keep=None):
            x, r, p, rtr = state["x"], state["r"], state["p"], state["rtr"]
            for _ in range(k):
                Ap = A @ p
                pAp = p @ Ap
                alpha = rtr / pAp
                x = x + alpha * p
                r = r - alpha * Ap
                rtr_new = r @ r
                beta = rtr_new / rtr
                p = r + beta * p
                rtr = rtr_new
                if keep is not None:
                    keep.append((alpha, beta, rtr))
            state.update(x=x, r=r, p=p, rtr=rtr)
            cnp.execute(itf)
            itf.sync()

        start()
        iterate(warmup)
        if trace_iters > 0:
            start()
            kept = []
            iterate(trace_iters, kept)
            out["trace"] = {"alpha": [a.get(itf).item() for a, _, _ in kept],
                            "beta": [b_.get(itf).item() for _, b_, _ in kept],
                            "rtr": [r_.get(itf).item() for _, _, r_ in kept],
                            "x": state["x"].get(itf)}
            del kept
        # the timed iterations start again from x = 0
        start()
        cnp.execute(itf)
        itf.sync()
        itf.time_matvecs(True)
        t0 = time.perf_counter()
        iterate(steps)
        dt = time.perf_counter() - t0
        gemv_ms = itf.matvec_times_ms()
        itf.time_matvecs(False)
        out.update({"iters_per_s": steps / dt, "ms_per_step": dt * 1e3 / steps, "wall_s": dt,
                    "gemv_avg_us": 1e3 * float(np.mean(gemv_ms)), "gemv_min_us": 1e3 * float(np.min(gemv_ms)),
                    "gemv_launches_timed": len(gemv_ms),
                    "rtr_final": state["rtr"].get(itf).item()})
        st = itf.stats()
        out["executor"] = {"group_launches": st["group_launches"], "compiled": st["compiled"],
                           "live_arrays": st["live_arrays"]}
        state.clear()
        del A, b
    finally:
        cnp.reset()
        itf.close()
    return out


def run_strided(reps=10, only=None):
    """Programs whose statements do not fit the aligned, unit-step, even-width mould of the five
    configurations: the sweeps and grid transfers of examples/multigrid2d.py and
    examples/gauss_seidel.py upstream (odd 2^k + 1 grids, step-2 lattices). Through the frontend,
    wall clock between two syncs. Bytes are the elements each statement has to touch, 8 bytes each
    (no allowance for the halves of cache lines a stride of two leaves unused)."""
    import charmnumeric_amd as cnp
    out = {}
    cnp.reset()
    itf = cnp.CharmNumericInterface(device=0)
    itf.connect(odf=4)
    itf.set_pipeline(True)
    try:
        cnp.set_auto_flush(itf, 48)

        def timed(fn, n, warm=2, batches=3):
            """Median over `batches` batches of n operations each, every batch between two syncs
            (steady-state rate: a batch is several milliseconds, so the one flush and wait that end
            it weigh little, and the median keeps one late wake-up of a host thread out)."""
            for _ in range(warm):
                fn()
            cnp.execute(itf)
            itf.sync()
            per = []
            for _ in range(batches):
                t0 = time.perf_counter()
                for _ in range(n):
                    fn()
                cnp.execute(itf)
                itf.sync()
                per.append((time.perf_counter() - t0) / n * 1e6)
            return float(np.median(per))

        def want(name):
            return only is None or only == name

        def entry(us, nbytes, **more):
            d = {"us": round(us, 1), "algorithmic_bytes": int(nbytes), "GBs": round(nbytes / (us * 1e-6) / 1e9, 1),
                 "frac_of_hbm_peak": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 3)}
            d.update(more)
            return d

        # weighted Jacobi with a source term on a 2^12 + 1 grid (examples/multigrid2d.py smoother)
        n = 4097
        u = cnp.random.uniform((n, n), seed=7, stream=0, low=0.0, high=1.0)
        f = cnp.random.uniform((n, n), seed=7, stream=1, low=-1.0, high=1.0)
        h2, omega = (1.0 / (n - 1)) ** 2, 2.0 / 3.0

        def smooth():
            upd = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:] + h2 * f[1:-1, 1:-1])
            u[1:-1, 1:-1] = (1.0 - omega) * u[1:-1, 1:-1] + omega * upd

        if want("weighted_jacobi_4097"):
            out["weighted_jacobi_4097"] = entry(timed(smooth, 10 * reps), 3 * 8.0 * n * n)

        # residual into a third array, restriction to 2049^2 and prolongation back
        r = cnp.zeros((n, n))

        def residual():
            r[1:-1, 1:-1] = f[1:-1, 1:-1] - (1.0 / h2) * (4.0 * u[1:-1, 1:-1] - u[:-2, 1:-1] - u[2:, 1:-1]
                                                           - u[1:-1, :-2] - u[1:-1, 2:])

        if want("residual_4097"):
            out["residual_4097"] = entry(timed(residual, 10 * reps), 3 * 8.0 * n * n)
        nc = (n - 1) // 2 + 1
        coarse = cnp.zeros((nc, nc))
        c_, lo, hi = slice(2, -2, 2), slice(1, -3, 2), slice(3, -1, 2)

        def restrict():
            coarse[1:-1, 1:-1] = (0.25 * r[c_, c_]
                                  + 0.125 * (r[lo, c_] + r[hi, c_] + r[c_, lo] + r[c_, hi])
                                  + 0.0625 * (r[lo, lo] + r[lo, hi] + r[hi, lo] + r[hi, hi]))

        if want("restriction_4097_to_2049"):
            out["restriction_4097_to_2049"] = entry(timed(restrict, 10 * reps), 8.0 * n * n + 8.0 * nc * nc)
        e = cnp.zeros((n, n))

        def prolong():
            e[2:-2:2, 2:-2:2] = coarse[1:-1, 1:-1]
            e[1:-1:2, 2:-2:2] = 0.5 * (coarse[:-1, 1:-1] + coarse[1:, 1:-1])
            e[2:-2:2, 1:-1:2] = 0.5 * (coarse[1:-1, :-1] + coarse[1:-1, 1:])
            e[1:-1:2, 1:-1:2] = 0.25 * (coarse[:-1, :-1] + coarse[1:, :-1] + coarse[:-1, 1:] + coarse[1:, 1:])

        if want("prolongation_2049_to_4097"):
            out["prolongation_2049_to_4097"] = entry(timed(prolong, 10 * reps), 8.0 * n * n + 4 * 8.0 * nc * nc,
                                                     statements=4)
            # the four statements run as one launch that reads the coarse array once: the same time
            # against the bytes of that single pass
            once = 8.0 * n * n + 8.0 * nc * nc
            us = out["prolongation_2049_to_4097"]["us"]
            out["prolongation_2049_to_4097"].update(
                bytes_read_once=int(once), frac_of_hbm_peak_read_once=round(once / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 3))
        del u, f, r, coarse, e
        cnp.execute(itf)

        # red-black Gauss-Seidel on 8192^2 (examples/gauss_seidel.py): four statements a sweep
        n = 8192
        phi = cnp.zeros((n, n))
        g = cnp.random.uniform((n, n), seed=8, stream=0, low=-1.0, high=1.0)
        h2 = (1.0 / (n - 1)) ** 2

        def red_black():
            for r0, c0 in ((1, 1), (2, 2), (1, 2), (2, 1)):
                rows, cols = slice(r0, -1, 2), slice(c0, -1, 2)
                up, down = slice(r0 - 1, -2, 2), slice(r0 + 1, None, 2)
                left, right = slice(c0 - 1, -2, 2), slice(c0 + 1, None, 2)
                phi[rows, cols] = 0.25 * (phi[up, cols] + phi[down, cols] + phi[rows, left] + phi[rows, right]
                                          - h2 * g[rows, cols])

        if want("red_black_8192"):
            out["red_black_8192"] = entry(timed(red_black, 2 * reps), 4 * 8.0 * n * n, statements=4)
        del phi, g
        cnp.execute(itf)

        # 7-point Poisson sweep with a source term on 257^3
        n = 257
        itf.close()
        itf = cnp.CharmNumericInterface(device=0)
        itf.connect(odf=64)
        itf.set_pipeline(True)
        cnp.set_auto_flush(itf, 48)
        v = cnp.random.uniform((n, n, n), seed=9, stream=0, low=0.0, high=1.0)
        q = cnp.random.uniform((n, n, n), seed=9, stream=1, low=-1.0, high=1.0)
        c6, h2 = 0.16666666666666666, (1.0 / (n - 1)) ** 2

        def poisson():
            v[1:-1, 1:-1, 1:-1] = c6 * (v[:-2, 1:-1, 1:-1] + v[2:, 1:-1, 1:-1] + v[1:-1, :-2, 1:-1]
                                        + v[1:-1, 2:, 1:-1] + v[1:-1, 1:-1, :-2] + v[1:-1, 1:-1, 2:]
                                        + h2 * q[1:-1, 1:-1, 1:-1])

        if want("poisson_257_cubed"):
            out["poisson_257_cubed"] = entry(timed(poisson, 10 * reps), 3 * 8.0 * n ** 3)
        del v, q
        cnp.execute(itf)

        # a whole V-cycle of examples/multigrid2d.py upstream on 4097^2 down to 5^2: two smoothing
        # sweeps before and after, residual, full-weighting restriction, bilinear prolongation and
        # correction, temporaries created and dropped at every level (about a hundred launches, most
        # of them on the small grids, where the host sets the pace)
        if want("multigrid_v_cycle_4097"):
            itf.close()
            itf = cnp.CharmNumericInterface(device=0)
            itf.connect(odf=4)
            itf.set_pipeline(True)
            cnp.set_auto_flush(itf, 48)
            omega = 2.0 / 3.0

            def smooth_on(ug, fg, hh2, sweeps):
                for _ in range(sweeps):
                    upd = 0.25 * (ug[:-2, 1:-1] + ug[2:, 1:-1] + ug[1:-1, :-2] + ug[1:-1, 2:] + hh2 * fg[1:-1, 1:-1])
                    ug[1:-1, 1:-1] = (1.0 - omega) * ug[1:-1, 1:-1] + omega * upd

            def v_cycle(ug, fg, h):
                m, hh2 = ug.shape[0], h * h
                if m <= 5:
                    smooth_on(ug, fg, hh2, 40)
                    return
                smooth_on(ug, fg, hh2, 2)
                rg = cnp.zeros((m, m))
                rg[1:-1, 1:-1] = fg[1:-1, 1:-1] - (1.0 / hh2) * (4.0 * ug[1:-1, 1:-1] - ug[:-2, 1:-1] - ug[2:, 1:-1]
                                                                  - ug[1:-1, :-2] - ug[1:-1, 2:])
                mc = (m - 1) // 2 + 1
                rc, ec = cnp.zeros((mc, mc)), cnp.zeros((mc, mc))
                cc, lo_, hi_ = slice(2, -2, 2), slice(1, -3, 2), slice(3, -1, 2)
                rc[1:-1, 1:-1] = (0.25 * rg[cc, cc] + 0.125 * (rg[lo_, cc] + rg[hi_, cc] + rg[cc, lo_] + rg[cc, hi_])
                                  + 0.0625 * (rg[lo_, lo_] + rg[lo_, hi_] + rg[hi_, lo_] + rg[hi_, hi_]))
                v_cycle(ec, rc, 2.0 * h)
                eg = cnp.zeros((m, m))
                eg[2:-2:2, 2:-2:2] = ec[1:-1, 1:-1]
                eg[1:-1:2, 2:-2:2] = 0.5 * (ec[:-1, 1:-1] + ec[1:, 1:-1])
                eg[2:-2:2, 1:-1:2] = 0.5 * (ec[1:-1, :-1] + ec[1:-1, 1:])
                eg[1:-1:2, 1:-1:2] = 0.25 * (ec[:-1, :-1] + ec[1:, :-1] + ec[:-1, 1:] + ec[1:, 1:])
                ug[1:-1, 1:-1] = ug[1:-1, 1:-1] + eg[1:-1, 1:-1]
                smooth_on(ug, fg, hh2, 2)

            n = 4097
            xs_ = np.linspace(0.0, 1.0, n)
            fv = cnp.array(2.0 * np.pi ** 2 * np.outer(np.sin(np.pi * xs_), np.sin(np.pi * xs_)))
            uv = cnp.zeros((n, n))
            us = timed(lambda: v_cycle(uv, fv, 1.0 / (n - 1)), reps, warm=2)
            exact = np.outer(np.sin(np.pi * xs_), np.sin(np.pi * xs_))
            out["multigrid_v_cycle_4097"] = {"us": round(us, 1), "levels": 11,
                                             "max_error_after_the_cycles": float(np.max(np.abs(uv.get(itf) - exact)))}
            del uv, fv
            cnp.execute(itf)
    finally:
        cnp.reset()
        itf.close()
    return out


def run_frontend():
    """The other configurations written against the NumPy-like frontend: statements -> statement log
    -> host executor -> the same kernels. Shows what the whole stack costs on top of the direct
    C ABI calls timed above (wall clock, flush + sync included)."""
    import charmnumeric_amd as cnp
    out = {}
    cnp.reset()
    itf = cnp.CharmNumericInterface(device=0)
    itf.connect(odf=4)
    itf.set_pipeline(True)               # the executor works on its own thread while Python records
    out["pipelined"] = True
    try:
        cnp.set_auto_flush(itf, 48)      # keep the device busy while later statements are recorded
        # configuration 1 as examples/simple.py upstream writes it: one fused statement, sum, norm
        m = 1 << 24
        xs = cnp.random.uniform((m,), seed=0, stream=0, low=-1.0, high=1.0)
        ys = cnp.random.uniform((m,), seed=0, stream=1, low=-1.0, high=1.0)
        ones = cnp.ones((m,))

        def c1(k):
            for _ in range(k):
                z = 2.5 * xs - 0.5 * ys + xs * ys
                s_ = z @ ones
                nrm2 = z @ z
            cnp.execute(itf)
            itf.sync()
            return s_, nrm2

        c1(3)
        t0 = time.perf_counter()
        s_, nrm2 = c1(100)
        dt = time.perf_counter() - t0
        out["c1_us_per_pass"] = round(dt / 100 * 1e6, 1)         # elementwise + two reductions
        out["c1_sum"] = s_.get(itf).item()
        out["c1_norm"] = float(np.sqrt(nrm2.get(itf).item()))
        del xs, ys, ones, s_, nrm2

        for key, shape, sweeps in (("jacobi2d_8192", (8192, 8192), 100), ("jacobi3d_512", (512, 512, 512), 50)):
            it16 = cnp.CharmNumericInterface(device=0)
            it16.connect(odf=16 if len(shape) == 2 else 64)
            it16.set_pipeline(True)
            cnp.set_auto_flush(it16, 48)
            u = cnp.zeros(shape)
            if len(shape) == 2:
                u[0, :] = 1.0
            else:
                u[0, :, :] = 1.0

            def sweep(k):
                for _ in range(k):
                    if len(shape) == 2:
                        u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
                    else:
                        u[1:-1, 1:-1, 1:-1] = 0.16666666666666666 * (
                            u[:-2, 1:-1, 1:-1] + u[2:, 1:-1, 1:-1] + u[1:-1, :-2, 1:-1]
                            + u[1:-1, 2:, 1:-1] + u[1:-1, 1:-1, :-2] + u[1:-1, 1:-1, 2:])
                cnp.execute(it16)
                it16.sync()

            sweep(5)
            t0 = time.perf_counter()
            sweep(sweeps)
            dt = time.perf_counter() - t0
            out[key + "_us_per_sweep"] = round(dt / sweeps * 1e6, 1)
            out[key + "_tile"] = it16.array_info(u.name)["tile"]
            del u
            cnp.execute(it16)
            it16.close()
        # configuration 5 written as upstream's example writes it (examples/lstm_forward.py upstream)
        n, b, word, d = 64, 256, 1024, 1024
        itl = cnp.CharmNumericInterface(device=0)
        itl.connect(odf=4)
        itl.set_pipeline(True)
        cnp.set_auto_flush(itl, 48)
        X = cnp.random.uniform((n, b, word), seed=5, stream=0, low=-1.0, high=1.0)
        W = cnp.random.uniform((word + d, 4 * d), seed=5, stream=1, low=-1.0 / 32, high=1.0 / 32)
        h0 = cnp.zeros((1, d))
        Hin = cnp.zeros((n, b, word + d))
        Hout = cnp.zeros((n, b, d))
        IFOG = cnp.zeros((n, b, 4 * d))
        IFOGf = cnp.zeros((n, b, 4 * d))
        Cs = cnp.zeros((n, b, d))
        Ct = cnp.zeros((n, b, d))

        def lstm_steps(t0, t1, wait=True):
            for t in range(t0, t1):
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
            cnp.execute(itl)
            if wait:
                itl.sync()

        # the whole sequence twice: the first pass also compiles every kernel the program needs
        # (the merged statement runs of steps 0, 1 and of the later ones), the second is what a
        # longer sequence costs per step
        t0 = time.perf_counter()
        lstm_steps(0, n)
        out["lstm_first_pass_us_per_step"] = round((time.perf_counter() - t0) / n * 1e6, 1)
        # six passes without a pause between them (the executor's thread and the device run on while
        # the next pass is recorded): what a long sequence costs per step. Timed twice: starting
        # from an idle device (clock rise included), then again right behind those passes, as the
        # direct calls are measured behind untimed passes.
        passes = 6
        for label in ("lstm_us_per_step_from_idle", "lstm_us_per_step"):
            t0 = time.perf_counter()
            for q in range(passes):
                lstm_steps(0, n, wait=q == passes - 1)
            dt = time.perf_counter() - t0
            out[label] = round(dt / (passes * n) * 1e6, 1)
        out["lstm_passes_timed"] = passes
        out["lstm_h_last_abs_mean"] = float(np.mean(np.abs(Hout[n - 1].get(itl))))
        del X, W, h0, Hin, Hout, IFOG, IFOGf, Cs, Ct
        cnp.execute(itl)
        itl.close()
    finally:
        cnp.reset()
        itf.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--n", type=int, default=16384, help="order of the CG system")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-also", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--cpu-iters", type=int, default=50)
    ap.add_argument("--strided", action="store_true",
                    help="only the strided and odd-sized programs (multigrid transfers, red-black sweeps); "
                         "prints their figures as one JSON line of their own")
    ap.add_argument("--only", default=None, help="with --strided: the one program to run (by its key in the output)")
    ap.add_argument("--config", default=None, choices=["c1", "c3", "c4", "c5"],
                    help="only that configuration by direct C ABI calls (for profiling one kernel family); "
                         "prints its figures as one JSON line of their own")
    ap.add_argument("--cg-separate", action="store_true",
                    help="CG iteration as four launches (matvec, dot, x and r, p) instead of the fused two")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every partition of the path lives on a single MI355X; "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    L = _dev()
    if args.strided:
        print(json.dumps({"metric": "strided_programs_through_the_frontend", "unit": "us per operation",
                          "n_gpus": 1, "data": "synthetic", "programs": run_strided(only=args.only)}))
        return
    if args.config:
        one = {"c1": lambda: run_c1(L), "c3": lambda: run_jacobi(L, 2, 8192, 2048, 200),
               "c4": lambda: run_jacobi(L, 3, 512, 128, 100), "c5": lambda: run_lstm(L)}[args.config]()
        print(json.dumps({"metric": "configuration_" + args.config, "n_gpus": 1, "data": "synthetic", "figures": one}))
        return
    if os.environ.get("CNH_BENCH_MARCH2D"):
        L.check(L.lib.cnh_set_option(b"slide2d_march", 1))
    name = C.create_string_buffer(256)
    L.check(L.lib.cnh_device_name(name, 256))
    n = args.n
    parity_iters = 0 if args.no_cpu else min(args.steps, args.cpu_iters)
    # The headline is the route a user of the drop-in takes: the frontend's operators through the
    # host executor. The same iteration by direct C ABI calls is timed beside it.
    cgf = run_frontend_cg(n, args.steps, args.warmup, trace_iters=parity_iters)
    cg = run_cg(L, n, args.steps, args.warmup, trace_iters=parity_iters, fuse=not args.cg_separate)
    gemv_bytes = 8.0 * n * n + 2 * 8.0 * n
    achieved = gemv_bytes / (cgf["gemv_avg_us"] * 1e-6) / 1e9
    two = cgf["gemv_launches_timed"] == args.steps and n >= 16384
    line = {
        "metric": "cg_iterations_per_second_n16384_fp64",
        "value": round(cgf["iters_per_s"], 2),
        "unit": "iterations/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(cgf["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64",
        "data": "synthetic",
        "config": {"workload": f"dense CG, n={n}, A in {cgf['tile']}^2 row-major tiles, one CG iteration per step "
                               "(matvec, 2 dots, 2 scalar statements, 3 vector updates) written with the frontend's "
                               "operators as examples/cg.py:40-52 upstream and run by the host executor, which "
                               "launches it as "
                               + ("two kernels: the matvec, which forms p = r + beta p on the way (beta from the "
                                  "partial sums of r.r) and leaves the partial sums of p.Ap; x and r with alpha "
                                  "formed in registers and the partial sums of r.r taken on the way" if two else
                                  "a matvec, a dot and two merged launches of the vector and scalar statements"),
                   "route": "charmnumeric_amd frontend -> statement log -> host executor -> HIP kernels",
                   "device": name.value.decode()},
        "roofline": {"bound": "hbm",
                     "kernel": "gemv_rows_xlds<double,8,8,4,true>" if two else "gemv_rows_xlds<double,8,8,4>",
                     "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": (GEMV_N16384_TRAFFIC_BYTES if two else GEMV_N16384_TRAFFIC_BYTES_PLAIN)
                     if n == 16384 else None,
                     "traffic_source": "rocprofv3 --pmc counters of an earlier run of this kernel "
                                       "(profiles/bench_hbm_traffic_pmc.txt), not measured in this run",
                     "avg_us": round(cgf["gemv_avg_us"], 2),
                     "timed_by": "HIP events around every matvec launch on the executor's stream, inside the timed "
                                 "iterations",
                     "bytes_per_launch": gemv_bytes},
        "gemv_roofline_iters_per_s": round(HBM_PEAK_GBS * 1e9 / gemv_bytes, 1),
        "rtr_final": cgf["rtr_final"],
        "executor": cgf["executor"],
        "direct_c_abi": {"what": "the same iterations as direct calls of the C ABI with prepared launches "
                                 "(cnh_gemv_tiles_fused + cnh_launch_group_sums), no frontend and no executor",
                         "iterations_per_s": round(cg["iters_per_s"], 2), "ms_per_step": round(cg["ms_per_step"], 4),
                         "gemv_avg_us": round(cg["gemv_avg_us"], 2),
                         "launches_per_iteration": cg["launches_per_iteration"], "rtr_final": cg["rtr_final"]},
    }
    if not args.no_also:
        also = {}
        try:
            also["c1_fused_elementwise_2p24"] = run_c1(L)
        except Exception as exc:  # report, do not hide
            also["c1_error"] = str(exc)
        try:
            also["c3_jacobi2d_8192"] = run_jacobi(L, 2, 8192, 2048, 200)
        except Exception as exc:
            also["c3_error"] = str(exc)
        try:
            also["c4_jacobi3d_512"] = run_jacobi(L, 3, 512, 128, 100)
        except Exception as exc:
            also["c4_error"] = str(exc)
        try:
            also["c5_lstm_forward"] = run_lstm(L)
            # the same pass as two launches per step: the product timed alone (its fraction of the
            # matrix peak), and what the one launch is compared with
            two = run_lstm(L, epilogue=False)
            also["c5_lstm_forward"]["as_two_launches_per_step"] = {
                k: two[k] for k in ("gemm_us", "gemm_tflops", "mfma_frac", "step_us", "sustained", "launches_per_step")}
        except Exception as exc:
            also["c5_error"] = str(exc)
        try:
            also["strided_programs"] = run_strided()
        except Exception as exc:
            also["strided_error"] = str(exc)
        try:
            also["through_frontend"] = run_frontend()
        except Exception as exc:
            also["frontend_error"] = str(exc)
        line["also"] = also
    if not args.no_cpu:
        logical, physical = _physical_cores()
        threads = min(logical, 16)
        setup = cpu_cg_setup(n)
        ips1, _, _, _ = cpu_cg(setup, n, args.cpu_iters, 1)
        ipsN, _, _, cpu_trace = cpu_cg(setup, n, args.cpu_iters, threads, keep_x_at=parity_iters)
        line["cpu_baseline"] = {
            "value": round(ipsN, 3), "unit": "iterations/s", "cores": threads, "kind": "port",
            "threads_used": threads, "host_logical_cpus": logical, "host_physical_cores": physical,
            "sample": f"same system (n={n}, {cgf['tile']}^2 tiles), {args.cpu_iters} CG iterations, "
                      f"oracle kernels, tile matvec split over {threads} threads",
            "one_core": round(ips1, 3),
        }
        if not args.no_also and "also" in line:
            try:
                line["also"]["c3_jacobi2d_8192"]["cpu_port"] = cpu_jacobi(2, 8192, 2048, 3, threads)
                line["also"]["c4_jacobi3d_512"]["cpu_port"] = cpu_jacobi(3, 512, 128, 2, threads)
                line["also"]["c1_fused_elementwise_2p24"]["cpu_port"] = {
                    "one_core": cpu_c1(1), "threads": cpu_c1(threads)}
                line["also"]["c5_lstm_forward"]["cpu_port"] = {
                    "one_core": cpu_lstm(1, steps=1), "threads": cpu_lstm(threads, steps=2)}
                # the frontend's C1 results against the host's, relative to the sum of |terms|
                # (sum: about 2^24 * 0.55; norm: relative to itself)
                fe, cp = line["also"].get("through_frontend", {}), line["also"]["c1_fused_elementwise_2p24"]["cpu_port"]
                if "c1_sum" in fe:
                    fe["c1_sum_vs_cpu_rel_to_abs_terms"] = abs(fe["c1_sum"] - cp["threads"]["sum"]) / (0.55 * (1 << 24))
                    fe["c1_norm_vs_cpu_rel"] = abs(fe["c1_norm"] - cp["threads"]["norm"]) / cp["threads"]["norm"]
            except Exception as exc:
                line["also"]["cpu_port_error"] = str(exc)
        # same system, same number of iterations (an untimed pass of the device path before the
        # timed one): the two solutions and the per-iteration scalars must agree
        par = cg_parity(cgf["trace"], cpu_trace, cpu_trace["rtr0"])
        line["cg_parity_max_rel_diff"] = par["x_max_rel_diff"]
        line["cg_parity"] = par
        line["direct_c_abi"]["cg_parity"] = cg_parity(cg["trace"], cpu_trace, cpu_trace["rtr0"])
    print(json.dumps(line))


if __name__ == "__main__":
    main()
