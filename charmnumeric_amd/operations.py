"""Function forms of the array operations (charmnumeric/operations.py upstream), plus reductions
upstream lacks (sum, squared-difference sum, max-abs difference; upstream's only reduction is the
1-D dot, src/executor_reduce.cpp:9-12 upstream)."""
from __future__ import annotations

import numpy as np

from . import _lib as L
from . import lazy
from .array import (_ArrayLike, _as_operand, _coerce_scalar, _is_scalar_like, asarray, nonfusible, unary)
from .array import tile as _tile_array


def tanh(x):
    if isinstance(x, _ArrayLike):
        return unary(L.OP_TANH, x)
    if _is_scalar_like(x):
        return np.tanh(_coerce_scalar(x))
    return unary(L.OP_TANH, x)


def exp(x):
    if isinstance(x, _ArrayLike):
        return unary(L.OP_EXP, x)
    if _is_scalar_like(x):
        return np.exp(_coerce_scalar(x))
    return unary(L.OP_EXP, x)


def _both_scalars(a, b):
    return _is_scalar_like(a) and _is_scalar_like(b)


def add(x1, x2):
    if _both_scalars(x1, x2):
        return _coerce_scalar(x1) + _coerce_scalar(x2)
    return _as_operand(x1) + _as_operand(x2)


def subtract(x1, x2):
    if _both_scalars(x1, x2):
        return _coerce_scalar(x1) - _coerce_scalar(x2)
    return _as_operand(x1) - _as_operand(x2)


def multiply(x1, x2):
    if _both_scalars(x1, x2):
        return _coerce_scalar(x1) * _coerce_scalar(x2)
    return _as_operand(x1) * _as_operand(x2)


def divide(x1, x2):
    if _both_scalars(x1, x2):
        return _coerce_scalar(x1) / _coerce_scalar(x2)
    return _as_operand(x1) / _as_operand(x2)


def matmul(x1, x2):
    if _is_scalar_like(x1) or _is_scalar_like(x2):
        raise ValueError("matmul does not support scalar operands")
    return asarray(x1) @ asarray(x2)


def dot(x1, x2):
    if _both_scalars(x1, x2):
        return _coerce_scalar(x1) * _coerce_scalar(x2)
    lhs, rhs = _as_operand(x1), _as_operand(x2)
    if not isinstance(lhs, _ArrayLike) or not isinstance(rhs, _ArrayLike):
        return lhs * rhs
    return lhs.dot(rhs)


def norm2(x):
    """Squared L2 norm of a 1-D array."""
    x = asarray(x)
    if x.ndims != 1:
        raise ValueError(f"norm2 requires a 1D array, got {x.ndims}D")
    return x.dot(x)


def tile(x, reps):
    if _is_scalar_like(x):
        return asarray(np.tile(_coerce_scalar(x), reps))
    return _tile_array(x, reps)


def diag(v, k=0):
    """numpy.diag: a 1-D array becomes the k-th diagonal of a square matrix of zeros, a 2-D array
    gives its k-th diagonal (charmnumeric/operations.py:125-148 upstream)."""
    v = asarray(v)
    k = int(k)
    if v.ndims == 1:
        n = v.shape[0] + abs(k)
        return nonfusible(L.OP_DIAG, [v, k], (n, n), v.dtype)
    if v.ndims == 2:
        rows, cols = v.shape
        length = max(0, min(rows, cols - k)) if k >= 0 else max(0, min(rows + k, cols))
        if length == 0:
            raise ValueError(f"k={k} is out of range for shape ({rows}, {cols})")
        return nonfusible(L.OP_DIAG, [v, k], (length,), v.dtype)
    raise ValueError(f"diag requires a 1D or 2D array, got {v.ndims}D")


# ---- reductions without upstream counterpart: results are size-1 fp64 arrays on the device ----


def sum(x):
    """Sum of all elements of an array of any rank."""
    x = asarray(x)
    return nonfusible(lazy.OP_SUM, [x], (1,), x.dtype)


def sumsq_diff(a, b):
    """sum((a - b)**2) over whole fp64 arrays of one shape."""
    a, b = asarray(a), asarray(b)
    if tuple(a.shape) != tuple(b.shape):
        raise ValueError(f"shapes {a.shape} and {b.shape} differ")
    return nonfusible(lazy.OP_SUMSQ_DIFF, [a, b], (1,), a.dtype)


def maxabs_diff(a, b):
    """max(|a - b|) over whole fp64 arrays of one shape."""
    a, b = asarray(a), asarray(b)
    if tuple(a.shape) != tuple(b.shape):
        raise ValueError(f"shapes {a.shape} and {b.shape} differ")
    return nonfusible(lazy.OP_MAXABS_DIFF, [a, b], (1,), a.dtype)
