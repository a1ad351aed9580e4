"""Shared test helpers: device buffers over the C ABI, ulp distance, NumPy generator, ASTs."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from charmnumeric_amd import _lib as L
from charmnumeric_amd.astbuild import AstBuilder

NP = {L.F32: np.float32, L.F64: np.float64, L.I32: np.int32, L.I64: np.int64}
DT = {np.dtype(v): k for k, v in NP.items()}

MASK = (1 << 64) - 1


# ---- NumPy restatement of the counter-based SplitMix64 generator -------------------------------
def np_splitmix(seed, stream, idx):
    idx = np.asarray(idx, dtype=np.uint64)
    with np.errstate(over="ignore"):
        s = (np.uint64((seed * 0x9E3779B97F4A7C15) & MASK)
             + np.uint64((stream * 0xD1B54A32D192ED03) & MASK) + idx)
        z = s + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def np_u01(seed, stream, idx):
    return (np_splitmix(seed, stream, idx) >> np.uint64(11)).astype(np.float64) * 2.0 ** -53


def np_uniform(n, seed, stream, lo, hi, first=0):
    u = np_u01(seed, stream, np.arange(first, first + n, dtype=np.uint64))
    return lo + (hi - lo) * u


def ulp_distance(a, b):
    """Max distance in units in the last place between two float arrays (same dtype)."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    assert a.dtype == b.dtype and a.shape == b.shape
    it = np.int64 if a.dtype == np.float64 else np.int32
    ia = a.view(it).astype(np.int64)
    ib = b.view(it).astype(np.int64)
    # map the sign-magnitude float order onto a monotone integer line
    top = np.int64(1) << (63 if a.dtype == np.float64 else 31)
    ia = np.where(ia < 0, -(ia + top), ia)
    ib = np.where(ib < 0, -(ib + top), ib)
    both_nan = np.isnan(a) & np.isnan(b)
    d = np.abs(ia - ib)
    d = np.where(both_nan, 0, d)
    return int(d.max()) if d.size else 0


# ---- device side -------------------------------------------------------------------------------
class DevBuf:
    def __init__(self, dev, nbytes, dtype, shape):
        self.dev = dev
        self.nbytes = int(nbytes)
        self.dtype = np.dtype(dtype)
        self.shape = tuple(shape)
        p = C.c_void_p()
        L.check(L.lib.cnh_alloc(max(self.nbytes, 16), 1, C.byref(p)))
        self.ptr = p.value

    def get(self):
        out = np.empty(self.shape, dtype=self.dtype)
        L.check(L.lib.cnh_d2h(out.ctypes.data, self.ptr, self.nbytes, None))
        return out

    def put(self, a):
        a = np.ascontiguousarray(a, dtype=self.dtype)
        assert a.nbytes == self.nbytes
        L.check(L.lib.cnh_h2d(self.ptr, a.ctypes.data, self.nbytes, None))

    def free(self):
        if self.ptr:
            L.check(L.lib.cnh_free(self.ptr))
            self.ptr = None

    def memref(self, shape=None):
        return L.Memref.dense(self.ptr, shape or self.shape)


class Device:
    def __init__(self):
        L.check(L.lib.cnh_init(0))
        self._bufs = []

    def name(self):
        buf = C.create_string_buffer(256)
        L.check(L.lib.cnh_device_name(buf, 256))
        return buf.value.decode()

    def empty(self, shape, dtype):
        shape = tuple(int(s) for s in np.atleast_1d(shape))
        b = DevBuf(self, int(np.prod(shape)) * np.dtype(dtype).itemsize, dtype, shape)
        self._bufs.append(b)
        return b

    def array(self, a):
        a = np.ascontiguousarray(a)
        b = self.empty(a.shape, a.dtype)
        if a.nbytes:
            b.put(a)
        return b

    def sync(self):
        L.check(L.lib.cnh_device_sync())

    def free_all(self):
        for b in self._bufs:
            b.free()
        self._bufs = []


def compile_group(ast, dtype, ndims, key=0):
    k = C.c_void_p()
    L.check(L.lib.cnh_compile_group(C.byref(ast), dtype, ndims, key, C.byref(k)))
    return k


def kernel_source(k, variant):
    n = L.lib.cnh_kernel_source(k, variant.encode(), None, 0)
    L.check(n)
    buf = C.create_string_buffer(int(n))
    L.check(L.lib.cnh_kernel_source(k, variant.encode(), buf, int(n)))
    return buf.value.decode()


def launch_batched(k, ndims, parts_in, scalars, parts_out, scalars_on_device=False):
    """parts_in / parts_out: list over partitions of lists of Memref."""
    n_parts = len(parts_out)
    n_in = len(parts_in[0]) if parts_in and parts_in[0] else 0
    n_out = len(parts_out[0])
    ins = (L.Memref * max(1, n_parts * n_in))()
    outs = (L.Memref * max(1, n_parts * n_out))()
    for p in range(n_parts):
        for i in range(n_in):
            ins[p * n_in + i] = parts_in[p][i]
        for o in range(n_out):
            outs[p * n_out + o] = parts_out[p][o]
    sp = (C.c_void_p * max(1, len(scalars)))(*[C.c_void_p(s) for s in scalars])
    L.check(L.lib.cnh_launch_group_batched(k, ndims, n_parts, n_in, ins, len(scalars), sp,
                                           1 if scalars_on_device else 0, n_out, outs, None))


# ---- ASTs of the workloads ---------------------------------------------------------------------
def ast_c1(dtype=L.F64):
    """z = ((2.5*x) - (0.5*y)) + (x*y); names x=0, y=1, z=10 (leaf uses x, y, x, y)."""
    b = AstBuilder(dtype, 1)
    x, y = b.leaf(0), b.leaf(1)
    t1 = b.binary(L.OP_MUL, 100, b.scalar(2.5), x)
    t2 = b.binary(L.OP_MUL, 101, b.scalar(0.5), y)
    t3 = b.binary(L.OP_SUB, 102, t1, t2)
    t4 = b.binary(L.OP_MUL, 103, x, y)
    b.binary(L.OP_ADD, 10, t3, t4, is_temp=False)
    return b.finish()


def ast_jacobi2d(n, dtype=L.F64, name=0, coef=0.25):
    """u[1:-1,1:-1] = coef*(((u[:-2,1:-1]+u[2:,1:-1])+u[1:-1,:-2])+u[1:-1,2:])."""
    b = AstBuilder(dtype, 2)
    u = b.leaf(name)
    r_up = ((0, 1), (n - 2, n - 1), (1, 1))
    r_dn = ((2, 1), (n, n - 1), (1, 1))
    r_lf = ((1, 0), (n - 1, n - 2), (1, 1))
    r_rt = ((1, 2), (n - 1, n), (1, 1))
    t1 = b.binary(L.OP_ADD, 100, u, u, r_up, r_dn)
    t2 = b.binary(L.OP_ADD, 101, t1, u, None, r_lf)
    t3 = b.binary(L.OP_ADD, 102, t2, u, None, r_rt)
    t4 = b.binary(L.OP_MUL, 103, b.scalar(coef), t3)
    b.set_region(104, u, t4, ((1, 1), (n - 1, n - 1), (1, 1)))
    return b.finish()


def ast_jacobi3d(n, dtype=L.F64, name=0, coef=0.16666666666666666):
    """7-point form of examples/jacobi3d.py:14 upstream (six neighbours, left-assoc adds)."""
    b = AstBuilder(dtype, 3)
    u = b.leaf(name)

    def reg(s0, s1, s2):
        return ((s0, s1, s2), (s0 + n - 2, s1 + n - 2, s2 + n - 2), (1, 1, 1))

    shifts = [reg(0, 1, 1), reg(2, 1, 1), reg(1, 0, 1), reg(1, 2, 1), reg(1, 1, 0), reg(1, 1, 2)]
    t = b.binary(L.OP_ADD, 100, u, u, shifts[0], shifts[1])
    for i, r in enumerate(shifts[2:]):
        t = b.binary(L.OP_ADD, 101 + i, t, u, None, r)
    t = b.binary(L.OP_MUL, 110, b.scalar(coef), t)
    b.set_region(111, u, t, reg(1, 1, 1))
    return b.finish()


def ast_poisson2d(n, dtype=L.F64, u_name=0, f_name=1, coef=0.25):
    """u[1:-1,1:-1] = coef*((((up+down)+left)+right)+f[1:-1,1:-1]): a Jacobi sweep with a source
    term held in a second array."""
    b = AstBuilder(dtype, 2)
    u, f = b.leaf(u_name), b.leaf(f_name)
    mid = ((1, 1), (n - 1, n - 1), (1, 1))
    t1 = b.binary(L.OP_ADD, 100, u, u, ((0, 1), (n - 2, n - 1), (1, 1)), ((2, 1), (n, n - 1), (1, 1)))
    t2 = b.binary(L.OP_ADD, 101, t1, u, None, ((1, 0), (n - 1, n - 2), (1, 1)))
    t3 = b.binary(L.OP_ADD, 102, t2, u, None, ((1, 2), (n - 1, n), (1, 1)))
    t4 = b.binary(L.OP_ADD, 103, t3, f, None, mid)
    t5 = b.binary(L.OP_MUL, 104, b.scalar(coef), t4)
    b.set_region(105, u, t5, mid)
    return b.finish()


def ast_poisson3d(n, dtype=L.F64, u_name=0, f_name=1, coef=0.16666666666666666):
    """The 7-point sweep with a source term: u[1:-1,..] = coef*((sum of six neighbours)+f[1:-1,..])."""
    b = AstBuilder(dtype, 3)
    u, f = b.leaf(u_name), b.leaf(f_name)

    def reg(s0, s1, s2):
        return ((s0, s1, s2), (s0 + n - 2, s1 + n - 2, s2 + n - 2), (1, 1, 1))

    shifts = [reg(0, 1, 1), reg(2, 1, 1), reg(1, 0, 1), reg(1, 2, 1), reg(1, 1, 0), reg(1, 1, 2)]
    t = b.binary(L.OP_ADD, 100, u, u, shifts[0], shifts[1])
    for i, r in enumerate(shifts[2:]):
        t = b.binary(L.OP_ADD, 101 + i, t, u, None, r)
    t = b.binary(L.OP_ADD, 109, t, f, None, reg(1, 1, 1))
    t = b.binary(L.OP_MUL, 110, b.scalar(coef), t)
    b.set_region(111, u, t, reg(1, 1, 1))
    return b.finish()


def np_poisson(u, f, coef):
    v = u.copy()
    if u.ndim == 2:
        v[1:-1, 1:-1] = coef * ((((u[:-2, 1:-1] + u[2:, 1:-1]) + u[1:-1, :-2]) + u[1:-1, 2:]) + f[1:-1, 1:-1])
    else:
        v[1:-1, 1:-1, 1:-1] = coef * (((((((u[:-2, 1:-1, 1:-1] + u[2:, 1:-1, 1:-1]) + u[1:-1, :-2, 1:-1])
                                          + u[1:-1, 2:, 1:-1]) + u[1:-1, 1:-1, :-2]) + u[1:-1, 1:-1, 2:]))
                                      + f[1:-1, 1:-1, 1:-1])
    return v


def np_jacobi2d(u, coef=0.25):
    v = u.copy()
    v[1:-1, 1:-1] = coef * (((u[:-2, 1:-1] + u[2:, 1:-1]) + u[1:-1, :-2]) + u[1:-1, 2:])
    return v


def np_jacobi3d(u, coef=0.16666666666666666):
    v = u.copy()
    v[1:-1, 1:-1, 1:-1] = coef * (
        ((((u[:-2, 1:-1, 1:-1] + u[2:, 1:-1, 1:-1]) + u[1:-1, :-2, 1:-1]) + u[1:-1, 2:, 1:-1])
         + u[1:-1, 1:-1, :-2]) + u[1:-1, 1:-1, 2:])
    return v


# ---- tiled arrays on the device ----------------------------------------------------------------
class TiledArray:
    """A global array cut into row-major tiles of edge `tile`, each tile its own device buffer."""

    def __init__(self, dev, host, tile, offset=None):
        self.dev = dev
        self.shape = host.shape
        self.nd = host.ndim
        self.tile = tile
        self.offset = tuple(offset) if offset is not None else (0,) * self.nd
        self.dtype = host.dtype
        self.grid_lo = tuple(o // tile for o in self.offset)
        self.grid = tuple((o + s + tile - 1) // tile - o // tile
                          for o, s in zip(self.offset, self.shape))
        self.bufs = []
        for ti in np.ndindex(*self.grid):
            sl = self._slice(ti)
            self.bufs.append(dev.array(host[sl]))
        self._ptrs = (C.c_void_p * len(self.bufs))(*[C.c_void_p(b.ptr) for b in self.bufs])

    def _slice(self, ti):
        sl = []
        for d in range(self.nd):
            g = self.grid_lo[d] + ti[d]
            lo = max(g * self.tile, self.offset[d]) - self.offset[d]
            hi = min((g + 1) * self.tile, self.offset[d] + self.shape[d]) - self.offset[d]
            sl.append(slice(lo, hi))
        return tuple(sl)

    def desc(self):
        t = L.Tiled()
        t.ndims = self.nd
        t.tile = self.tile
        for d in range(self.nd):
            t.offset[d] = self.offset[d]
            t.shape[d] = self.shape[d]
            t.grid_lo[d] = self.grid_lo[d]
            t.grid[d] = self.grid[d]
        t.tiles = C.cast(self._ptrs, C.POINTER(C.c_void_p))
        return t

    def gather(self):
        out = np.empty(self.shape, dtype=self.dtype)
        for b, ti in zip(self.bufs, np.ndindex(*self.grid)):
            out[self._slice(ti)] = b.get()
        return out


def launch_tiles(k, inputs, scalars, cur, dst, scalars_on_device=False):
    descs = (L.Tiled * max(1, len(inputs)))(*[a.desc() for a in inputs])
    sp = (C.c_void_p * max(1, len(scalars)))(*[C.c_void_p(s) for s in scalars])
    cd = cur.desc() if cur is not None else None
    dd = dst.desc()
    L.check(L.lib.cnh_launch_group_tiles(k, len(inputs), descs, len(scalars), sp,
                                         1 if scalars_on_device else 0,
                                         C.byref(cd) if cd is not None else None, C.byref(dd), None))


def golden():
    """The known-answer vectors of upstream's tests, kept as data under tests/golden."""
    import json
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "upstream_known_answers.json")) as f:
        return json.load(f)


def host_libm_is_the_restated_one():
    """True where the host's exp/tanh are the algorithms the device code restates: x86-64 glibc
    2.28..2.38 (table-driven exp with its FMA build selected at load time, fdlibm tanh/expm1)."""
    import platform
    if platform.machine() != "x86_64":
        return False
    lib, ver = platform.libc_ver()
    if lib != "glibc":
        return False
    try:
        major, minor = (int(t) for t in ver.split(".")[:2])
    except ValueError:
        return False
    if (major, minor) < (2, 28) or (major, minor) > (2, 38):
        return False
    try:
        with open("/proc/cpuinfo") as f:
            flags = next((ln for ln in f if ln.startswith("flags")), "")
    except OSError:
        return False
    return " fma " in flags + " " and " avx2 " in flags + " "
