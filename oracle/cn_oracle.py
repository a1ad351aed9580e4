"""ctypes binding of the CPU oracle (oracle/libcn_oracle.so).

TEST INFRASTRUCTURE: imported only by tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg. The product package never imports this module.

Struct layouts are identical to the ones in include/cnhip.h, so struct pointers are declared as
void pointers here and the same ctypes objects can be handed to both libraries.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libcn_oracle.so")

F32, F64, I32, I64 = 0, 1, 2, 3
NP_DTYPES = {F32: np.float32, F64: np.float64, I32: np.int32, I64: np.int64}
DTYPE_OF = {np.dtype(v): k for k, v in NP_DTYPES.items()}


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libcn_oracle.so"])
    return _SO


def load():
    build()
    lib = C.CDLL(_SO)
    vp, i32, i64, dbl = C.c_void_p, C.c_int, C.c_int64, C.c_double
    u64 = C.c_uint64
    protos = {
        "orc_first_aligned_point": (i32, [i32] * 6 + [vp, vp]),
        "orc_region_size_dim": (i32, [vp, i32]),
        "orc_region_size": (i32, [vp]),
        "orc_region_overlaps": (i32, [vp, vp]),
        "orc_region_covers": (i32, [vp, vp]),
        "orc_region_intersect": (i32, [vp, vp, vp]),
        "orc_region_subtract": (i32, [vp, vp, vp]),
        "orc_region_map": (None, [vp, vp, vp, vp]),
        "orc_decomp_num_chares": (i32, [vp, i32]),
        "orc_decomp_chare_region_global": (None, [vp, vp, vp]),
        "orc_decompose": (i32, [vp, vp, i32, vp, vp]),
        "orc_local_inputs": (i32, [vp, i32, vp, vp, vp, vp, vp, vp]),
        "orc_send_remote_inputs": (i32, [vp, i32, vp, vp, vp, vp, i32, vp, vp, vp]),
        "orc_align_fragments": (i32, [i32, i32, vp, vp, vp, i32, vp, vp, vp, vp, vp]),
        "orc_next_pow2": (i32, [i32]),
        "orc_tile_rule": (i32, [i32, vp, i32, i32, i32]),
        "orc_group_signature": (i32, [vp, i32, vp, vp, vp, vp, vp, vp, vp, vp]),
        "orc_group_dtype": (i32, [vp]),
        "orc_eval_group": (i32, [vp, i32, i32, i32, vp, i32, vp, i32, vp]),
        "orc_world_group": (i32, [vp, i32, i32, vp, i32, vp, i32, vp]),
        "orc_fill_region": (i32, [i32, i32, vp, vp, vp, vp, vp, vp]),
        "orc_copy_region": (i32, [i32, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp]),
        "orc_scalar_to_dtype": (i32, [i32, dbl, vp]),
        "orc_dot": (i32, [i32, i64, vp, vp, vp]),
        "orc_reduce_partials": (i32, [i32, i32, vp, vp]),
        "orc_gemv_sub": (i32, [i32, vp, i64, i64, i64, i64, i64, vp, vp]),
        "orc_gemv_sub_mt": (i32, [i32, vp, i64, i64, i64, i64, i64, vp, vp, i32]),
        "orc_axpy1": (i32, [i32, i64, vp, vp]),
        "orc_gemm_acc": (i32, [i32, i64, i64, i64, vp, i64, vp, i64, vp, i64]),
        "orc_gemm_acc_mt": (i32, [i32, i64, i64, i64, vp, i64, vp, i64, vp, i64, i32]),
        "orc_sum": (i32, [i32, i64, vp, vp]),
        "orc_sumsq_diff": (i32, [i64, vp, vp, vp]),
        "orc_maxabs_diff": (i32, [i64, vp, vp, vp]),
        "orc_splitmix": (u64, [u64, u64, u64]),
        "orc_u01": (dbl, [u64, u64, u64]),
        "orc_fill_uniform": (None, [vp, i64, u64, u64, u64, dbl, dbl]),
        "orc_fill_cg_matrix": (None, [vp, i64, i64, i64, i64, i64, i64, u64]),
    }
    for name, (res, args) in protos.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


class Memref(C.Structure):
    """orc_memref: sizes, strides and offset in elements."""

    _fields_ = [
        ("allocated", C.c_void_p),
        ("aligned", C.c_void_p),
        ("offset", C.c_int64),
        ("sizes", C.c_int64 * 3),
        ("strides", C.c_int64 * 3),
    ]


def ptr(a):
    """Address of a numpy array's first element."""
    return a.ctypes.data


# ---- numpy-friendly wrappers -----------------------------------------------------------------

class Oracle:
    def __init__(self):
        self.lib = load()

    # synthetic inputs
    def uniform(self, n, seed, stream, lo, hi, first=0):
        out = np.empty(int(n), dtype=np.float64)
        self.lib.orc_fill_uniform(ptr(out), int(n), seed, stream, first, lo, hi)
        return out

    def cg_matrix(self, n, row0, nrows, col0, ncols, seed):
        out = np.empty((nrows, ncols), dtype=np.float64)
        self.lib.orc_fill_cg_matrix(ptr(out), n, row0, nrows, col0, ncols, ncols, seed)
        return out

    # fused group on numpy operands. `ins`/`outs` are lists of numpy arrays (views allowed:
    # strides are translated to element strides), scalars a list of python numbers.
    def eval_group(self, ast, dtype, ndims, ins, scalars, outs):
        def mr(a):
            m = Memref()
            m.allocated = a.ctypes.data
            m.aligned = a.ctypes.data
            m.offset = 0
            for d in range(a.ndim):
                m.sizes[d] = a.shape[d]
                m.strides[d] = a.strides[d] // a.itemsize
            return m

        npdt = NP_DTYPES[dtype]
        in_arr = (Memref * max(1, len(ins)))(*[mr(a) for a in ins])
        out_arr = (Memref * max(1, len(outs)))(*[mr(a) for a in outs])
        svals = [np.array([s], dtype=npdt) for s in scalars]
        sptr = (C.c_void_p * max(1, len(svals)))(*[C.c_void_p(ptr(s)) for s in svals])
        rc = self.lib.orc_eval_group(C.addressof(ast), dtype, ndims, len(ins),
                                     C.addressof(in_arr), len(svals), C.addressof(sptr),
                                     len(outs), C.addressof(out_arr))
        return rc

    # One SET_REGION group over a tiled array, chare by chare as the reference's fragment path
    # runs it. `tiles` are the row-major tiles (row-major grid order), updated in place.
    def world_group(self, ast, dtype, shape, tile, tiles, threads=1):
        nd = len(shape)
        shp = (C.c_int32 * 3)(*list(shape) + [1] * (3 - nd))
        tp = (C.c_void_p * len(tiles))(*[C.c_void_p(ptr(t)) for t in tiles])
        stats = (C.c_int64 * 4)()
        rc = self.lib.orc_world_group(C.addressof(ast), dtype, nd, shp, int(tile), tp, int(threads), stats)
        return rc, {"messages": stats[0], "bytes": stats[1], "kernels": stats[2], "max_cells": stats[3]}

    @staticmethod
    def split_tiles(arr, tile):
        """Row-major tiles of a global array in row-major grid order (copies)."""
        grid = [(n + tile - 1) // tile for n in arr.shape]
        out = []
        for idx in np.ndindex(*grid):
            sl = tuple(slice(i * tile, min((i + 1) * tile, n)) for i, n in zip(idx, arr.shape))
            out.append(np.array(arr[sl], order="C", copy=True))
        return out

    @staticmethod
    def join_tiles(tiles, shape, tile):
        grid = [(n + tile - 1) // tile for n in shape]
        out = np.empty(shape, dtype=tiles[0].dtype)
        for t, idx in zip(tiles, np.ndindex(*grid)):
            sl = tuple(slice(i * tile, min((i + 1) * tile, n)) for i, n in zip(idx, shape))
            out[sl] = t
        return out

    def dot(self, a, b):
        dt = DTYPE_OF[a.dtype]
        out = np.zeros(1, dtype=a.dtype)
        self.lib.orc_dot(dt, a.size, ptr(a), ptr(b), ptr(out))
        return out[0]

    def gemv(self, A, x):
        dt = DTYPE_OF[A.dtype]
        y = np.zeros(A.shape[0], dtype=A.dtype)
        self.lib.orc_gemv_sub(dt, ptr(A), A.shape[1], 0, 0, A.shape[0], A.shape[1], ptr(x), ptr(y))
        return y

    def gemm_acc(self, A, B, Cm, threads=1):
        dt = DTYPE_OF[A.dtype]
        self.lib.orc_gemm_acc_mt(dt, A.shape[0], B.shape[1], A.shape[1], ptr(A), A.shape[1], ptr(B),
                                 B.shape[1], ptr(Cm), Cm.shape[1], threads)
        return Cm
