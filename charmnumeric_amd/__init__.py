"""MI355X-native back end for charmnumeric's per-partition array execution path, with the lazy
NumPy-like frontend that feeds it (API of upstream's `charmnumeric` package)."""
import numpy as _np

from . import _lib  # noqa: F401  (fails loudly when libcnhip.so has not been built)
from . import random  # noqa: F401
from .array import (Array, ArrayView, DType, arange, array, asarray, copy, copyto, create_array, empty,
                    empty_like, eye, full, full_like, identity, ones, ones_like, zeros, zeros_like)
from .interface import CharmNumericInterface, LocalCluster
from .lazy import execute, reset, set_auto_flush
from .operations import (add, diag, divide, dot, exp, matmul, maxabs_diff, multiply, norm2, subtract, sum,
                         sumsq_diff, tanh, tile)

ndarray = Array
float32, float64, int32, int64 = _np.float32, _np.float64, _np.int32, _np.int64
dtype = _np.dtype
newaxis = None
pi, e = _np.pi, _np.e

__all__ = [
    "Array", "ArrayView", "CharmNumericInterface", "DType", "LocalCluster", "add", "arange", "array",
    "asarray", "copy", "copyto", "create_array", "diag", "divide", "dot", "dtype", "e", "empty",
    "empty_like", "exp", "eye", "execute", "float32", "float64", "full", "full_like", "identity", "int32",
    "int64", "matmul", "maxabs_diff", "multiply", "ndarray", "newaxis", "norm2", "ones", "ones_like", "pi",
    "random", "reset", "set_auto_flush", "subtract", "sum", "sumsq_diff", "tanh", "tile", "zeros",
    "zeros_like",
]
