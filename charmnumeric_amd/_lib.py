"""ctypes binding of libcnhip.so (the C ABI declared in include/cnhip.h).

The library is the only execution path: importing this module fails loudly when the shared
object has not been built, and every call raises CnhError when the library reports an error
(for example when no HIP device is present). There is no CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import os

MAX_ND = 3

F32, F64, I32, I64 = 0, 1, 2, 3

OP_COPY, OP_SET_REGION, OP_GET_REGION, OP_CREATE, OP_NOOP = -5, -4, -3, -2, -1
OP_ADD, OP_SUB, OP_MUL, OP_DIV, OP_MATMUL, OP_TANH, OP_EXP = 0, 1, 2, 3, 4, 5, 6
OP_TILE, OP_REDUCE, OP_MATMATMUL, OP_DIAG = 7, 8, 9, 10
OP_SUM_OF, OP_MAXABS_OF = 20, 21          # reducing roots of a fused group (extension)
OP_SCALAR_OF = 22                         # an output formed from scalars alone, stored once (extension)


class CnhError(RuntimeError):
    pass


class Region(C.Structure):
    _fields_ = [
        ("is_global", C.c_int32),
        ("ndims", C.c_int32),
        ("start", C.c_int32 * MAX_ND),
        ("stop", C.c_int32 * MAX_ND),
        ("step", C.c_int32 * MAX_ND),
    ]

    @classmethod
    def make(cls, start=None, stop=None, step=None):
        r = cls()
        if start is None:
            r.is_global = 1
            return r
        r.is_global = 0
        r.ndims = len(start)
        for d in range(len(start)):
            r.start[d] = int(start[d])
            r.stop[d] = int(stop[d])
            r.step[d] = int(step[d]) if step is not None else 1
        return r

    def as_tuple(self):
        n = self.ndims
        return (tuple(self.start[:n]), tuple(self.stop[:n]), tuple(self.step[:n]))


class AstNode(C.Structure):
    _fields_ = [
        ("result_name", C.c_int32),
        ("opcode", C.c_int32),
        ("is_temp", C.c_int32),
        ("is_scalar", C.c_int32),
        ("is_broadcast", C.c_int32),
        ("ndims", C.c_int32),
        ("dtype", C.c_int32),
        ("n_operands", C.c_int32),
        ("operands", C.c_int32 * 2),
        ("has_operand_region", C.c_int32 * 2),
        ("scalar", C.c_double),
        ("operand_regions", Region * 2),
        ("region", Region),
    ]


class Ast(C.Structure):
    _fields_ = [
        ("n_nodes", C.c_int32),
        ("n_roots", C.c_int32),
        ("nodes", C.POINTER(AstNode)),
        ("roots", C.POINTER(C.c_int32)),
    ]


class GemmJob(C.Structure):
    """cnh_gemm_job: one C += A * B panel product of a batch."""
    _fields_ = [("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64), ("A", C.c_void_p), ("lda", C.c_int64),
                ("B", C.c_void_p), ("ldb", C.c_int64), ("C", C.c_void_p), ("ldc", C.c_int64)]


class GemvFusion(C.Structure):
    """cnh_gemv_fusion: the vector work a fused matvec takes along."""
    _fields_ = [("xa", C.c_void_p), ("xb", C.c_void_p), ("num", C.c_void_p), ("num_count", C.c_int64),
                ("den", C.c_void_p), ("num_folded", C.c_void_p), ("w", C.c_void_p),
                ("dot_partials", C.c_void_p), ("dot_capacity", C.c_int64), ("quotient_out", C.c_void_p)]


class ScalarSum(C.Structure):
    """cnh_scalar_sum: a run-time scalar given as `count` partial sums at `ptr`."""

    _fields_ = [("ptr", C.c_void_p), ("count", C.c_int64), ("folded", C.c_void_p)]


class Memref(C.Structure):
    _fields_ = [
        ("allocated", C.c_void_p),
        ("aligned", C.c_void_p),
        ("offset", C.c_int64),
        ("sizes", C.c_int64 * MAX_ND),
        ("strides", C.c_int64 * MAX_ND),
    ]

    @classmethod
    def dense(cls, ptr, shape, offset=0):
        m = cls()
        m.allocated = ptr
        m.aligned = ptr
        m.offset = offset
        stride = 1
        for d in range(len(shape) - 1, -1, -1):
            m.sizes[d] = shape[d]
            m.strides[d] = stride
            stride *= shape[d]
        return m

    @classmethod
    def strided(cls, ptr, sizes, strides, offset=0):
        m = cls()
        m.allocated = ptr
        m.aligned = ptr
        m.offset = offset
        for d in range(len(sizes)):
            m.sizes[d] = sizes[d]
            m.strides[d] = strides[d]
        return m


class GemvPanel(C.Structure):
    _fields_ = [("base", C.c_void_p), ("ld", C.c_int64), ("ncols", C.c_int64), ("xoff", C.c_int64)]


class Decomp(C.Structure):
    """cnx_decomp: ArrayMetadata as the decomposition solver reads and writes it."""
    _fields_ = [
        ("name", C.c_int32),
        ("ndims", C.c_int32),
        ("shape", C.c_int32 * 3),
        ("offset", C.c_int32 * 3),
        ("tile", C.c_int32),
        ("final", C.c_int32),
    ]


class Tiled(C.Structure):
    _fields_ = [
        ("ndims", C.c_int32),
        ("tile", C.c_int32),
        ("offset", C.c_int32 * MAX_ND),
        ("shape", C.c_int32 * MAX_ND),
        ("grid_lo", C.c_int32 * MAX_ND),
        ("grid", C.c_int32 * MAX_ND),
        ("tiles", C.POINTER(C.c_void_p)),
        ("pitch", C.c_int64 * MAX_ND),
    ]


def _lib_path():
    here = os.path.dirname(os.path.abspath(__file__))
    return os.path.join(here, "libcnhip.so")


def _load():
    path = _lib_path()
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `make -C charmnumeric_amd/csrc` "
            "(or python -c 'import __graft_entry__ as g; g.build()'). "
            "charmnumeric_amd has no CPU fallback."
        )
    return C.CDLL(path, mode=C.RTLD_GLOBAL)


lib = _load()

_i64p = C.POINTER(C.c_int64)
_vpp = C.POINTER(C.c_void_p)

# name -> (restype, argtypes); mirrors include/cnhip.h declaration by declaration.
_PROTOS = {
    "cnh_init": (C.c_int, [C.c_int]),
    "cnh_last_error": (C.c_char_p, []),
    "cnh_device_name": (C.c_int, [C.c_char_p, C.c_size_t]),
    "cnh_version": (C.c_int, []),
    "cnh_set_option": (C.c_int, [C.c_char_p, C.c_int]),
    "cnh_code_objects": (C.c_int64, []),
    "cnh_code_objects_from_disk": (C.c_int64, []),
    "cnh_alloc": (C.c_int, [C.c_size_t, C.c_int, _vpp]),
    "cnh_free": (C.c_int, [C.c_void_p]),
    "cnh_memset0": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p]),
    "cnh_h2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "cnh_d2h": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "cnh_d2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "cnh_d2h_region": (C.c_int, [C.c_int, C.c_int, C.c_void_p, _i64p, _i64p, C.c_void_p, _i64p,
                                 _i64p, _i64p, C.c_void_p]),
    "cnh_stream_create": (C.c_int, [_vpp]),
    "cnh_stream_destroy": (C.c_int, [C.c_void_p]),
    "cnh_stream_sync": (C.c_int, [C.c_void_p]),
    "cnh_stream_callback": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "cnh_device_sync": (C.c_int, []),
    "cnh_event_create": (C.c_int, [_vpp]),
    "cnh_event_destroy": (C.c_int, [C.c_void_p]),
    "cnh_event_record": (C.c_int, [C.c_void_p, C.c_void_p]),
    "cnh_event_sync": (C.c_int, [C.c_void_p]),
    "cnh_event_elapsed_ms": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "cnh_fill_region": (C.c_int, [C.c_int, C.c_int, C.c_void_p, _i64p, _i64p, _i64p, _i64p,
                                  C.c_void_p, C.c_void_p]),
    "cnh_copy_region": (C.c_int, [C.c_int, C.c_int, C.c_void_p, _i64p, _i64p, _i64p, C.c_void_p,
                                  _i64p, _i64p, _i64p, _i64p, C.c_void_p]),
    "cnh_convert_region": (C.c_int, [C.c_int, C.c_int, C.c_void_p, _i64p, _i64p, _i64p, C.c_int, C.c_void_p,
                                     _i64p, _i64p, _i64p, _i64p, C.c_void_p]),
    "cnh_scalar_to_dtype": (C.c_int, [C.c_int, C.c_double, C.c_void_p]),
    "cnh_compile_group": (C.c_int, [C.POINTER(Ast), C.c_int, C.c_int, C.c_uint64, _vpp]),
    "cnh_kernel_release": (C.c_int, [C.c_void_p]),
    "cnh_launch_group_sums": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int,
                                        C.c_void_p, C.c_void_p]),
    "cnh_fold_sums": (C.c_int, [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]),
    "cnh_alloc_on": (C.c_int, [C.c_size_t, C.c_int, C.c_void_p, _vpp]),
    "cnh_allocation_count": (C.c_int64, []),
    "cnh_kernel_lattice": (C.c_int, [C.c_void_p]),
    "cnh_kernel_matches": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_int]),
    "cnh_kernel_signature": (C.c_int, [C.c_void_p, C.POINTER(C.c_int), C.POINTER(C.c_int),
                                       C.POINTER(C.c_int)]),
    "cnh_kernel_input": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int),
                                   C.POINTER(Region)]),
    "cnh_kernel_scalar": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_int)]),
    "cnh_kernel_output": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int),
                                    C.POINTER(C.c_int), C.POINTER(Region)]),
    "cnh_kernel_source": (C.c_int64, [C.c_void_p, C.c_char_p, C.c_char_p, C.c_size_t]),
    "cnh_kernel_build": (C.c_int, [C.c_void_p, C.c_char_p]),
    "cnh_kernel_variants_loaded": (C.c_int, [C.c_void_p, C.c_char_p]),
    "cnh_launch_group": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.POINTER(Memref), C.c_int, _vpp,
                                   C.c_int, C.c_int, C.POINTER(Memref), C.c_void_p]),
    "cnh_launch_group_batched": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int,
                                           C.POINTER(Memref), C.c_int, _vpp, C.c_int, C.c_int,
                                           C.POINTER(Memref), C.c_void_p]),
    "cnh_launch_group_tiles": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(Tiled), C.c_int, _vpp,
                                         C.c_int, C.POINTER(Tiled), C.POINTER(Tiled), C.c_void_p]),
    "cnh_launch_group_tiles_residual": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(Tiled), C.c_int, _vpp,
                                                  C.c_int, C.POINTER(Tiled), C.POINTER(Tiled), C.c_int,
                                                  C.c_void_p, C.c_void_p]),
    "cnh_dot_partial": (C.c_int, [C.c_int, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p,
                                  C.c_void_p]),
    "cnh_dot_partial_noalloc": (C.c_int, [C.c_int, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p,
                                          C.c_void_p]),
    "cnh_reduce_final": (C.c_int, [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "cnh_dot_tiles": (C.c_int, [C.c_int, C.c_int, _vpp, _vpp, _i64p, C.c_void_p, C.c_void_p]),
    "cnh_sum_tiles": (C.c_int, [C.c_int, C.c_int, _vpp, _i64p, C.c_void_p, C.c_void_p]),
    "cnh_sumsq_diff_tiles": (C.c_int, [C.c_int, _vpp, _vpp, _i64p, C.c_void_p, C.c_void_p]),
    "cnh_maxabs_diff_tiles": (C.c_int, [C.c_int, _vpp, _vpp, _i64p, C.c_void_p, C.c_void_p]),
    "cnh_gemv": (C.c_int, [C.c_int, C.c_int64, C.c_int64, C.c_void_p, C.c_int64, C.c_void_p,
                           C.c_void_p, C.c_int, C.c_void_p]),
    "cnh_axpy1": (C.c_int, [C.c_int, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p]),
    "cnh_gemv_tiles": (C.c_int, [C.c_int, C.c_int64, C.c_int64, C.c_int32, _vpp, C.c_void_p,
                                 C.c_void_p, C.c_void_p]),
    "cnh_gemv_tiles_fused": (C.c_int, [C.c_int64, C.c_int64, C.c_int32, _vpp, C.c_void_p, C.c_void_p,
                                       C.c_void_p, C.POINTER(C.c_int64), C.c_void_p]),
    "cnh_gemm_acc": (C.c_int, [C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_int64,
                               C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_void_p]),
    "cnh_gemm_acc_batch": (C.c_int, [C.c_int, C.c_int, C.POINTER(GemmJob), C.c_void_p]),
    "cnh_gemv_panels": (C.c_int, [C.c_int, C.c_int64, C.c_int32, C.c_int64, C.c_int64, C.c_int64,
                                  C.POINTER(GemvPanel), C.c_void_p, C.c_void_p, C.c_void_p]),
    "cnh_gemm_batch": (C.c_int, [C.c_int, C.c_int, C.POINTER(GemmJob), C.c_int, C.c_void_p]),
    "cnh_launch_product_group": (C.c_int, [C.c_void_p, C.POINTER(GemmJob), C.c_int, C.c_int, C.c_int,
                                           C.POINTER(Memref), C.POINTER(C.c_int32), C.c_int, _vpp, C.c_int,
                                           C.c_int, C.POINTER(Memref), C.c_void_p]),
    "cnh_probe_mfma_f64": (C.c_int, [C.c_int, C.POINTER(C.c_double)]),
    "cnh_fill_uniform": (C.c_int, [C.c_void_p, C.c_int64, C.c_uint64, C.c_uint64, C.c_uint64,
                                   C.c_double, C.c_double, C.c_void_p]),
    "cnh_fill_uniform_tile": (C.c_int, [C.c_void_p, C.c_int, _i64p, _i64p, _i64p, C.c_uint64,
                                        C.c_uint64, C.c_double, C.c_double, C.c_void_p]),
    "cnh_fill_cg_matrix": (C.c_int, [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int64,
                                     C.c_int64, C.c_int64, C.c_uint64, C.c_void_p]),
}

# Host executor (include/cnexec.h).
_i32p = C.POINTER(C.c_int32)
_PROTOS.update({
    "cnx_create": (C.c_int, [C.c_int, C.c_int, C.c_int, _vpp]),
    "cnx_destroy": (C.c_int, [C.c_void_p]),
    "cnx_set_min_tile": (C.c_int, [C.c_void_p, C.c_int, C.c_int]),
    "cnx_receive_dag": (C.c_int, [C.c_void_p, C.c_int, C.c_int64, C.c_char_p]),
    "cnx_receive_log": (C.c_int, [C.c_void_p, C.c_int64, C.c_char_p, C.c_int]),
    "cnx_discard_log": (C.c_int, [C.c_void_p]),
    "cnx_set_capture": (C.c_int, [C.c_void_p, C.c_int]),
    "cnx_captured": (C.c_int64, [C.c_void_p, C.c_char_p, C.c_size_t]),
    "cnx_set_async": (C.c_int, [C.c_void_p, C.c_int]),
    "cnx_get": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int, C.c_void_p]),
    "cnx_put": (C.c_int, [C.c_void_p, C.c_int, C.c_int64, C.c_int, C.c_void_p]),
    "cnx_fill_uniform": (C.c_int, [C.c_void_p, C.c_int, C.c_uint64, C.c_uint64, C.c_double, C.c_double]),
    "cnx_fill_cg_matrix": (C.c_int, [C.c_void_p, C.c_int, C.c_uint64]),
    "cnx_sync": (C.c_int, [C.c_void_p]),
    "cnx_array_info": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int),
                                 C.POINTER(C.c_int), _i32p, _i32p]),
    "cnx_stats": (C.c_int, [C.c_void_p, _i64p]),
    "cnx_set_matvec_timing": (C.c_int, [C.c_void_p, C.c_int]),
    "cnx_matvec_times": (C.c_int64, [C.c_void_p, C.POINTER(C.c_float), C.c_int64]),
    "cnx_solve_decompositions": (C.c_int, [C.c_int, C.c_int, _i32p, C.c_int, C.POINTER(Decomp),
                                           C.c_int64, C.c_char_p]),
    "cnx_set_trace": (C.c_int, [C.c_void_p, C.c_int]),
    "cnx_set_solver": (C.c_int, [C.c_void_p, C.c_int]),
    "cnx_set_layout": (C.c_int, [C.c_void_p, C.c_int]),
    "cnx_set_fusion": (C.c_int, [C.c_void_p, C.c_int]),
    "cnx_trace": (C.c_int64, [C.c_void_p, C.c_char_p, C.c_size_t]),
})

EXPORTS = tuple(_PROTOS)

for _name, (_res, _args) in _PROTOS.items():
    _fn = getattr(lib, _name)  # AttributeError here = the library lacks a declared symbol
    _fn.restype = _res
    _fn.argtypes = _args


def check(rc):
    """Raise CnhError for a negative return code."""
    if rc is not None and rc < 0:
        msg = lib.cnh_last_error()
        raise CnhError(f"libcnhip error {rc}: {msg.decode(errors='replace') if msg else ''}")
    return rc


def i64arr(values):
    return (C.c_int64 * len(values))(*[int(v) for v in values])


def vparr(values):
    return (C.c_void_p * len(values))(*[C.c_void_p(v) for v in values])
