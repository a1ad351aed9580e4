"""Array and ArrayView: the NumPy-like lazy frontend objects.

API contract of upstream's frontend (charmnumeric/charmnumeric.py upstream): operators and their
reflected forms (:394-482), slicing rules (:272-343: integers keep their dimension as extent 1,
negative steps and newaxis are refused), dtype rules (:369-373: scalars never promote), matmul routing
(:485-533), creation routines (:860-1062) and `.get(interface)` (:683-688). Everything is recorded
through `lazy` and runs when something calls `execute` or `.get`.
"""
from __future__ import annotations

import numbers

import numpy as np

from . import _lib as L
from . import lazy

# The recording hot path in C (csrc/recorder.c): the base type of the classes below, which then
# take indexing, the binary operators, slice assignment and deletion records from it and keep the
# methods here (`_py_*`, `_binary`) as the route for every form the C code does not handle.
# CHARMNUMERIC_PYREC=1 runs on the Python methods alone.
import os as _os

if _os.environ.get("CHARMNUMERIC_PYREC", "0") not in ("", "0"):
    _cnrec = None
else:
    try:
        from . import _cnrec
    except ImportError as exc:  # pragma: no cover
        raise ImportError("charmnumeric_amd/_cnrec has not been built: run "
                          "python -c 'import __graft_entry__ as g; g.build()' "
                          "(or set CHARMNUMERIC_PYREC=1 to record in Python)") from exc
_HandleBase = object if _cnrec is None else _cnrec.Handle

_DEFAULT_DTYPE = np.dtype("float64")
_SUPPORTED = (np.dtype("float32"), np.dtype("float64"), np.dtype("int32"), np.dtype("int64"))


class DType:
    """Element type numbers shared with the executor (charmnumeric.py:34-40 upstream)."""

    FLOAT32, FLOAT64, INT32, INT64 = 0, 1, 2, 3

    @staticmethod
    def from_numpy(np_dtype):
        return lazy.wire_dtype(_normalize_dtype(np_dtype))

    @staticmethod
    def to_numpy(wire):
        try:
            return _SUPPORTED[(0, 1, 2, 3).index(wire)]
        except ValueError:
            raise TypeError(f"Unsupported wire dtype {wire!r}") from None

    @staticmethod
    def promote(a, b):
        return DType.from_numpy(np.result_type(DType.to_numpy(a), DType.to_numpy(b)))


_PLAIN_NUMBERS = (int, float)


class _CallableInt(int):
    """`a.size` that may also be called as `a.size()` (both spellings occur upstream)."""

    def __call__(self):
        return int(self)


def _normalize_dtype(dtype, allow_none=False):
    if dtype is None:
        return None if allow_none else _DEFAULT_DTYPE
    dt = np.dtype(dtype)
    if dt not in _SUPPORTED:
        raise TypeError(f"charmnumeric only supports float32, float64, int32, and int64; got {dt}")
    return dt


def _normalize_shape(shape):
    out = (int(shape),) if isinstance(shape, numbers.Integral) else tuple(int(s) for s in shape)
    if any(s < 0 for s in out):
        raise ValueError(f"negative dimensions are not allowed: {out}")
    if not 1 <= len(out) <= 3:
        raise NotImplementedError(f"arrays of rank {len(out)} are not supported (1 to 3)")
    if any(s == 0 for s in out):
        raise NotImplementedError("zero-sized arrays are not supported")
    return out


def _is_scalar_like(v):
    if type(v) in _PLAIN_NUMBERS:          # the common case, without the abstract-class checks
        return True
    if isinstance(v, np.ndarray):
        return v.ndim == 0
    return isinstance(v, (bool, numbers.Real, np.generic))


def _coerce_scalar(v):
    if type(v) in _PLAIN_NUMBERS:
        return v
    if isinstance(v, (np.ndarray, np.generic)):
        v = v.item()
    if isinstance(v, bool):
        return int(v)
    if isinstance(v, numbers.Integral):
        return int(v)
    return float(v)


def _size(shape):
    n = 1
    for s in shape:
        n *= int(s)
    return n


# ---------------------------------------------------------------------------------------------
# regions


def _expand_key(key, ndims):
    if not isinstance(key, tuple):
        key = (key,)
    if sum(1 for k in key if k is Ellipsis) > 1:
        raise IndexError("an index can only have a single ellipsis")
    if any(k is None for k in key):
        raise NotImplementedError("np.newaxis is not supported yet")
    explicit = sum(1 for k in key if k is not Ellipsis)
    if explicit > ndims:
        raise IndexError(f"too many indices for array: array is {ndims}-dimensional, "
                         f"but {explicit} were indexed")
    out = []
    for k in key:
        if k is Ellipsis:
            out.extend([slice(None)] * (ndims - explicit))
        else:
            out.append(k)
    out.extend([slice(None)] * (ndims - len(out)))
    return out


def parse_key(key, shape):
    """Index expression -> (start, stop, step) per dimension, relative to an object of `shape`."""
    ndims = len(shape)
    if type(key) is not tuple:
        key = (key,)
    if len(key) <= ndims:
        # the common form, plain slices and integers only (dimensions not named are taken whole):
        # nothing to expand
        start, stop, step = [0] * ndims, list(shape), [1] * ndims
        d = 0
        for item in key:
            kind = type(item)
            if kind is int:
                extent = shape[d]
                if item < 0:
                    item += extent
                if not 0 <= item < extent:
                    break
                start[d] = item
                stop[d] = item + 1
            elif kind is slice:
                st = item.step
                if st is not None and not (type(st) is int and st > 0):
                    break
                start[d], stop[d], step[d] = item.indices(shape[d])
            else:
                break
            d += 1
        else:
            return tuple(start), tuple(stop), tuple(step)
    start, stop, step = [0] * ndims, [0] * ndims, [1] * ndims
    for d, item in enumerate(_expand_key(key, ndims)):
        if isinstance(item, slice):
            st = 1 if item.step is None else int(item.step)
            if st == 0:
                raise ValueError("slice step cannot be zero")
            if st < 0:
                raise NotImplementedError("negative slicing is not supported yet")
            start[d], stop[d], step[d] = item.indices(shape[d])
        elif isinstance(item, numbers.Integral):
            i = int(item)
            if i < 0:
                i += shape[d]
            if not 0 <= i < shape[d]:
                raise IndexError(f"index {item} is out of bounds for axis {d} with size {shape[d]}")
            start[d], stop[d], step[d] = i, i + 1, 1
        else:
            raise TypeError("only integers, slices, and ellipsis are valid charmnumeric indices")
    return tuple(start), tuple(stop), tuple(step)


def region_shape(region):
    start, stop, step = region
    if step in _UNIT:
        if len(start) == 3:
            return (max(0, stop[0] - start[0]), max(0, stop[1] - start[1]), max(0, stop[2] - start[2]))
        return tuple(max(0, stop[d] - start[d]) for d in range(len(start)))
    return tuple(max(0, (stop[d] - start[d] + step[d] - 1) // step[d]) for d in range(len(start)))


_UNIT = {(1,), (1, 1), (1, 1, 1)}


def _unit_steps(step):
    return step in _UNIT


def compose(outer, inner):
    """Region `inner` (relative to the view `outer`) expressed relative to outer's base array.
    The stop is one past the last selected element, so a region taken through a strided view never
    reaches beyond the view's own last element (`a[::4][:]` on 10 elements is [0:9:4], not
    [0:12:4]); upstream keeps the outer region as it is when the inner one is the whole view
    (charmnumeric.py:215-220 upstream), with the same effect."""
    if outer is None:
        return inner
    if inner[2] == outer[2] and _unit_steps(inner[2]):
        # unit steps on both sides: plain offsets
        ostart = outer[0]
        n = len(ostart)
        if n == 3:
            return ((ostart[0] + inner[0][0], ostart[1] + inner[0][1], ostart[2] + inner[0][2]),
                    (ostart[0] + inner[1][0], ostart[1] + inner[1][1], ostart[2] + inner[1][2]), inner[2])
        return (tuple(ostart[d] + inner[0][d] for d in range(n)),
                tuple(ostart[d] + inner[1][d] for d in range(n)), inner[2])
    ostart, _, ostep = outer
    istart, istop, istep = inner
    nd = len(istart)
    start, stop, step = [], [], []
    for d in range(nd):
        count = max(0, (istop[d] - istart[d] + istep[d] - 1) // istep[d])
        first = ostart[d] + istart[d] * ostep[d]
        start.append(first)
        step.append(ostep[d] * istep[d])
        stop.append(first + (count - 1) * step[-1] + 1 if count else first)
    return tuple(start), tuple(stop), tuple(step)


def _is_whole(region, shape):
    return region is None or all(region[0][d] == 0 and region[1][d] == shape[d] and region[2][d] == 1
                                 for d in range(len(shape)))


# ---------------------------------------------------------------------------------------------
# the objects


class _ArrayLike(_HandleBase):
    __array_priority__ = 1000

    # -- basic properties --
    @property
    def ndim(self):
        return self.ndims

    @property
    def size(self):
        return _CallableInt(self._n)

    @property
    def itemsize(self):
        return self.dtype.itemsize

    @property
    def nbytes(self):
        return int(self.size) * self.itemsize

    def wire_dtype(self):
        return self._wire

    def __len__(self):
        return self.shape[0]

    def __bool__(self):
        raise ValueError("The truth value of a charmnumeric array is ambiguous. "
                         "Use .get(interface) to materialize it first.")

    def __array__(self, dtype=None, copy=None):
        raise TypeError("charmnumeric arrays are lazy frontend objects. "
                        "Call .get(interface) before converting to numpy.")

    # -- operand form: the bytes that name this object in a record of the statement log --
    def _refb(self, broadcast=False):
        raise NotImplementedError

    def _base(self):
        raise NotImplementedError

    # -- slicing --
    def _py_getitem(self, key):
        inner = parse_key(key, self.shape)
        return ArrayView(self._base(), compose(self._region(), inner))

    def get_region(self, region, **kwargs):
        """The view of `region` = (start, stop, step) per dimension, in this object's own
        coordinates, or any object with those three attributes (upstream's ArrayRegion,
        charmnumeric.py:690-695,789-794 upstream; its keyword arguments are derived here)."""
        if not isinstance(region, tuple):
            region = (region.start, region.stop, region.step)
        start, stop, step = (tuple(int(v) for v in part) for part in region)
        if not len(start) == len(stop) == len(step) == self.ndims:
            raise IndexError(f"region of rank {len(start)} on an array of rank {self.ndims}")
        for d in range(self.ndims):
            if step[d] < 1 or start[d] < 0 or stop[d] > self.shape[d] or stop[d] <= start[d]:
                raise IndexError(f"region [{start[d]}:{stop[d]}:{step[d]}] does not fit extent "
                                 f"{self.shape[d]} in dimension {d}")
        return ArrayView(self._base(), compose(self._region(), (start, stop, step)))

    def _py_setitem(self, key, rhs):
        inner = parse_key(key, self.shape)
        region = compose(self._region(), inner)
        shape = region_shape(inner)
        base = self._base()
        base._all_ones = False
        if isinstance(rhs, _ArrayLike):
            value = rhs
        else:
            value = _coerce_assignment_operand(rhs, shape, self.dtype)
        if isinstance(value, _ArrayLike):
            if value._wire != base._wire:
                value = _converted(value, base.dtype)      # NumPy's rule: the target's type wins
            if value.shape != shape:
                # a lower-rank value fits a region whose extra dimensions have extent 1
                # (IFOG[t] = M with M 2-D), and a whole higher-rank one whose extra dimensions
                # have extent 1 fits a lower-rank target (vec[:] = column)
                squeeze = lambda sh: tuple(x for x in sh if x != 1)
                if not (value.ndims != len(shape) and squeeze(value.shape) == squeeze(shape)):
                    raise ValueError(
                        f"could not broadcast input from shape {value.shape} into shape {shape}")
                if not _is_whole(value._region(), value._base().shape):
                    value = value.copy()        # a slice of another rank: copied out first
            operand = value._refb()
        else:
            operand = lazy.scalar_bytes(value)
        lazy.record_set(base.name, base._wire, base.ndims, shape, region, operand)

    # -- arithmetic, indexing, assignment: from the C base type when it is there --
    if _cnrec is None:
        __getitem__ = _py_getitem
        __setitem__ = _py_setitem

        def __add__(self, o):
            return _binary(L.OP_ADD, self, o)

        def __radd__(self, o):
            return _binary(L.OP_ADD, o, self)

        def __sub__(self, o):
            return _binary(L.OP_SUB, self, o)

        def __rsub__(self, o):
            return _binary(L.OP_SUB, o, self)

        def __mul__(self, o):
            return _binary(L.OP_MUL, self, o)

        def __rmul__(self, o):
            return _binary(L.OP_MUL, o, self)

        def __truediv__(self, o):
            return _binary(L.OP_DIV, self, o)

        def __rtruediv__(self, o):
            return _binary(L.OP_DIV, o, self)

        def __neg__(self):
            # upstream spells negation as multiplication by -1 (charmnumeric.py:427-434)
            return _binary(L.OP_MUL, self, -1)

    def __matmul__(self, o):
        return _matmul(self, o)

    def dot(self, o):
        return _matmul(self, o)

    def matvec(self, vec):
        return _matvec(self, vec)

    def copy(self):
        """A new array holding these values: one COPY node (upstream's opcode -5), which fuses like
        any element-wise operation, instead of a zero-filled array assigned afterwards."""
        out = Array(self.shape, self.dtype)
        lazy.record_op(out.name, L.OP_COPY, out._wire, out.shape, self._refb())
        return out

    def fill(self, value):
        self[...] = value

    def astype(self, dtype, copy=True):
        """Upstream refuses a change of element type (charmnumeric.py:738-744, 842-848); here it is
        one converting copy on the device (C conversion rules, as numpy.ndarray.astype)."""
        want = _normalize_dtype(dtype)
        if want != self.dtype:
            return _converted(self, want)
        return self.copy() if copy else self


class Array(_ArrayLike):
    """A whole distributed array, existing or about to be computed."""

    # True while every element is known to be exactly 1 (set by ones()/full(.., 1), dropped by any
    # assignment into the array): a dot with such an array is recorded as a sum, which reads one
    # array instead of two and gives the same bits (a * 1 is a, the order of additions is the same).
    if _cnrec is None:
        _all_ones = False

    def __init__(self, shape, dtype, name=None):
        self.shape = tuple(shape)
        self.ndims = len(self.shape)
        self.dtype = np.dtype(dtype)
        self._wire = lazy.wire_dtype(self.dtype)
        self._n = _size(self.shape)
        self.name = lazy.new_name() if name is None else name
        self._gen = lazy.generation()
        self._rb = None

    @classmethod
    def _result_of(cls, like, shape):
        """A new array of `shape` with the element type of the array-like `like` (shape already a
        tuple of ints): the result of an operation, without re-deriving what the operand knows."""
        out = cls.__new__(cls)
        out.shape = shape
        out.ndims = len(shape)
        out.dtype = like.dtype
        out._wire = like._wire
        out._n = like._n if shape is like.shape else _size(shape)
        out.name = lazy.new_name()
        out._gen = lazy.generation()
        out._rb = None
        return out

    if _cnrec is None:
        def __del__(self):
            lazy.record_delete(self.name, self._gen)

    def __repr__(self):
        return f"Array(shape={self.shape}, dtype={self.dtype.name}, name={self.name})"

    def _base(self):
        return self

    def _region(self):
        return None

    def _refb(self, broadcast=False):
        if broadcast:
            return lazy.ref_bytes(self.name, self.ndims, self._wire, None, True)
        rb = self._rb
        if rb is None:
            rb = self._rb = lazy.ref_bytes(self.name, self.ndims, self._wire, None)
        return rb

    def get(self, interface):
        lazy.execute(interface)
        data = interface.get(self.ndims, self.name, int(self.size), dtype=self.dtype)
        return data.reshape(self.shape) if self.ndims > 1 else data


class ArrayView(_ArrayLike):
    """A rectangular, possibly strided, slice of an Array. Keeps its base alive."""

    def __init__(self, base, region):
        self.base = base
        self.region = region
        self.shape = shape = region_shape(region)
        self.ndims = base.ndims
        self.dtype = base.dtype
        self._wire = base._wire
        n = 1
        for extent in shape:
            n *= extent
        self._n = n
        self._rb = None
        if n == 0:
            raise NotImplementedError("zero-sized slices are not supported")

    @property
    def name(self):
        return self.base.name

    def __repr__(self):
        return f"ArrayView(shape={self.shape}, dtype={self.dtype.name}, name={self.name})"

    def _base(self):
        return self.base

    def _region(self):
        return self.region

    def _refb(self, broadcast=False):
        rb = self._rb
        if rb is None or broadcast:
            base = self.base
            region = None if self._n == base._n and _is_whole(self.region, base.shape) else self.region
            rb = lazy.ref_bytes(base.name, base.ndims, self._wire, region, broadcast)
            if not broadcast:
                self._rb = rb
        return rb

    def get(self, interface):
        out = empty(self.shape, dtype=self.dtype)
        out[...] = self
        return out.get(interface)


# ---------------------------------------------------------------------------------------------
# operations


def _as_operand(v):
    if isinstance(v, _ArrayLike):
        return v
    if _is_scalar_like(v):
        return _coerce_scalar(v)
    host = np.asarray(v)
    if host.ndim == 0:
        return _coerce_scalar(host.item())
    return asarray(host)


def _binary(opcode, lhs, rhs):
    la, ra = isinstance(lhs, _ArrayLike), isinstance(rhs, _ArrayLike)
    if not la:
        lhs = _as_operand(lhs)
        la = isinstance(lhs, _ArrayLike)
    if not ra:
        rhs = _as_operand(rhs)
        ra = isinstance(rhs, _ArrayLike)
    if la and ra:
        if lhs.dtype != rhs.dtype:
            lhs, rhs = _promoted(lhs, rhs)
        # the result takes the shape of the operand with more than one element; a one-element
        # whole array beside it is a run-time scalar
        if lhs._n > 1 and rhs._n > 1:
            if lhs.shape != rhs.shape:
                raise ValueError(f"operands could not be broadcast together with shapes "
                                 f"{lhs.shape} and {rhs.shape}")
            like, lb, rb = lhs, False, False
        elif lhs._n > 1:
            like, lb, rb = lhs, False, True
        elif rhs._n > 1:
            like, lb, rb = rhs, True, False
        else:
            like, lb, rb = lhs, False, False
        for x, bc in ((lhs, lb), (rhs, rb)):
            if bc and not _is_whole(x._region(), x._base().shape):
                raise NotImplementedError("a one-element slice cannot be used as a scalar operand")
        a, b = lhs._refb(lb), rhs._refb(rb)
    elif la:
        like = lhs
        a, b = lhs._refb(), lazy.scalar_bytes(rhs)
    else:
        like = rhs
        a, b = lazy.scalar_bytes(lhs), rhs._refb()
    out = Array._result_of(like, like.shape)
    lazy.record_op(out.name, opcode, out._wire, out.shape, a, b)
    return out


def unary(opcode, x):
    if not isinstance(x, _ArrayLike):
        x = asarray(x)
    if x._wire > L.F64:                    # the two integer types follow the floating-point ones
        raise TypeError("tanh/exp need a floating-point array")
    out = Array._result_of(x, x.shape)
    lazy.record_op(out.name, opcode, out._wire, out.shape, x._refb())
    return out


def _whole(x):
    """An operand of a non-fusible operation must be a whole array: slices are copied out first."""
    if isinstance(x, ArrayView) and not _is_whole(x.region, x.base.shape):
        return x.copy()
    return x


def _window_ok(x):
    """Products and dots read unit-step slices in place (upstream sends the view's region with the
    node, charmnumeric.py:595-616 upstream); anything else is copied out first. A 3-D operand
    gives up its first extent-1 dimension, and the rows of what remains must be contiguous."""
    if not isinstance(x, ArrayView) or _is_whole(x.region, x.base.shape):
        return True
    if any(st != 1 for st in x.region[2]):
        return False
    if x.ndims == 3:
        ones = [d for d in range(3) if x.shape[d] == 1]
        return bool(ones) and (ones[0] != 2 or x.base.shape[2] == 1)
    return True


_WINDOWED = (L.OP_REDUCE, L.OP_MATMUL, L.OP_MATMATMUL)


def nonfusible(opcode, operands, shape, dtype):
    operands = [_whole(o) if isinstance(o, _ArrayLike) and not (opcode in _WINDOWED and _window_ok(o))
                else o for o in operands]
    out = Array(shape, dtype)
    lazy.record_nonfusible(out.name, opcode, out._wire, out.shape,
                           [o._refb() if isinstance(o, _ArrayLike) else lazy.scalar_bytes(o) for o in operands])
    return out


def tile(x, reps):
    """numpy.tile for arrays (charmnumeric/operations.py:52-72 upstream): the operand's shape is
    left-padded with ones to the rank of `reps` and repeated."""
    x = asarray(x)
    reps = (int(reps),) if isinstance(reps, numbers.Integral) else tuple(int(r) for r in reps)
    rank = max(x.ndims, len(reps))
    if rank > 3:
        raise NotImplementedError("arrays of rank above 3 are not supported")
    shape = (1,) * (rank - x.ndims) + tuple(x.shape)
    reps = (1,) * (rank - len(reps)) + reps
    if any(r < 1 for r in reps):
        raise NotImplementedError("zero-sized arrays are not supported")
    return nonfusible(L.OP_TILE, [x], tuple(s * r for s, r in zip(shape, reps)), x.dtype)


def _converted(x, dtype):
    """x as a new array of element type `dtype`: one ASTYPE node (slices are copied out first)."""
    dtype = np.dtype(dtype)
    src = _whole(x)
    out = Array(src.shape, dtype)
    lazy.record_nonfusible(out.name, lazy.OP_ASTYPE, out._wire, out.shape, [src._refb()])
    return out


def _promoted(a, b):
    """Both operands in np.result_type of their element types, the type upstream gives the result
    (charmnumeric.py:369-373 upstream). Upstream's kernels then read every operand in that one type
    whatever it holds (src/jit.cpp:47-69); here the operand of the other type is converted first."""
    want = _normalize_dtype(np.result_type(a.dtype, b.dtype))
    return (a if a.dtype == want else _converted(a, want),
            b if b.dtype == want else _converted(b, want))


def _matmul(lhs, rhs):
    rhs = _as_operand(rhs)
    if not isinstance(rhs, _ArrayLike):
        raise ValueError("matmul does not support scalar operands")
    if lhs.ndims == 1 and rhs.ndims == 1:
        if lhs.shape[0] != rhs.shape[0]:
            raise ValueError(f"Shape mismatch for dot product: ({lhs.shape[0]},) @ ({rhs.shape[0]},)")
        if lhs.dtype != rhs.dtype:
            lhs, rhs = _promoted(lhs, rhs)
        for a, b in ((lhs, rhs), (rhs, lhs)):
            if isinstance(b, Array) and b._all_ones and (isinstance(a, Array) or _is_whole(a.region, a.base.shape)):
                return nonfusible(lazy.OP_SUM, [a], (1,), a.dtype)
        return nonfusible(L.OP_REDUCE, [lhs, rhs], (1,), lhs.dtype)
    if lhs.ndims not in (2, 3):
        raise ValueError(f"matmul requires a 2D matrix, got {lhs.ndims}D")
    if rhs.ndims == 1:
        return _matvec(lhs, rhs)
    if rhs.ndims == 2 and rhs.shape[1] == 1:
        return _matvec(lhs, _column_as_vector(rhs))
    lr, lc = _matrix_shape(lhs)
    rr, rc = _matrix_shape(rhs)
    if lc != rr:
        raise ValueError(f"Shape mismatch: ({lr},{lc}) @ ({rr},{rc})")
    if lhs.dtype != rhs.dtype:
        lhs, rhs = _promoted(lhs, rhs)
    return nonfusible(L.OP_MATMATMUL, [lhs, rhs], (lr, rc), lhs.dtype)


def _column_as_vector(col):
    """An (N, 1) operand of a matvec becomes a 1-D temporary, and the result is 1-D
    (charmnumeric.py:528-531,542-545 upstream)."""
    temp = create_array((col.shape[0],), dtype=col.dtype)
    temp[:] = _whole(col)
    return temp


def _matrix_shape(x):
    """(rows, cols) of a matmul operand: a 2-D array, or a 3-D one with exactly one extent of 1,
    which is dropped (charmnumeric.py:579-592 upstream)."""
    if x.ndims == 2:
        return x.shape[0], x.shape[1]
    if x.ndims == 3:
        ones = [d for d in range(3) if x.shape[d] == 1]
        if len(ones) != 1:
            raise ValueError(f"3D matmatmul requires exactly one singleton dim, got shape {x.shape}")
        rest = [d for d in range(3) if d != ones[0]]
        return x.shape[rest[0]], x.shape[rest[1]]
    raise ValueError(f"matmatmul requires 2D or 3D operand, got {x.ndims}D")


def _matvec(mat, vec):
    if not isinstance(vec, _ArrayLike):
        raise ValueError("matvec requires an Array vector")
    if vec.ndims == 2 and vec.shape[1] == 1:
        vec = _column_as_vector(vec)
    if vec.ndims != 1:
        raise ValueError("matvec requires a 1D vector (N,) or 2D column vector (N, 1)")
    if mat.ndims == 2:
        rows, cols = mat.shape
    elif mat.ndims == 3:
        ones = [d for d in range(3) if mat.shape[d] == 1]
        if len(ones) != 1:
            raise ValueError(f"3D matvec requires exactly one singleton dimension, got shape {mat.shape}")
        rows, cols = (mat.shape[d] for d in range(3) if d != ones[0])
    else:
        raise ValueError(f"matvec requires a 2D or 3D matrix, got {mat.ndims}D")
    if cols != vec.shape[0]:
        raise ValueError(f"Shape mismatch: matrix cols {cols} != vector size {vec.shape[0]}")
    if mat.dtype != vec.dtype:
        mat, vec = _promoted(mat, vec)
    return nonfusible(L.OP_MATMUL, [mat, vec], (rows,), mat.dtype)


# ---------------------------------------------------------------------------------------------
# creation
#
# Every constructor ends in one of two recorded forms: CREATE alone (the executor zero-fills new
# arrays), CREATE followed by either one fill (constant contents) or one bulk upload. Host values
# pass through _HostValues, which settles rank, dtype and broadcasting once for all constructors.


class _HostValues:
    """Host-side contents for a device array: a NumPy array of a wire dtype, rank >= 1."""

    __slots__ = ("data",)

    def __init__(self, values, dtype=None, copy=False, ndmin=0, broadcast=None, what="input"):
        want = _normalize_dtype(dtype, allow_none=True)
        data = np.array(values, dtype=want, copy=True) if copy else np.asarray(values, dtype=want)
        if data.ndim < ndmin:
            data = data.reshape((1,) * (ndmin - data.ndim) + data.shape)
        if broadcast is not None and data.ndim > 0:
            try:
                data = np.broadcast_to(data, broadcast)
            except ValueError as exc:
                label = "fill_value" if what == "fill_value" else "input"
                raise ValueError(f"could not broadcast {label} from shape {data.shape} into shape "
                                 f"{tuple(broadcast)}") from exc
        self.data = data

    @property
    def is_scalar(self):
        return self.data.ndim == 0

    def constant(self):
        """The single value all elements share, or None."""
        flat = self.data.reshape(-1)
        if flat.size and (flat.size == 1 or bool(np.all(flat == flat[0]))):
            return flat[0]
        return None

    def upload(self):
        """A new device array holding these values."""
        if self.is_scalar:
            raise NotImplementedError("0D charmnumeric arrays are not supported yet")
        out = create_array(self.data.shape, dtype=_normalize_dtype(self.data.dtype))
        return _assign_host_data(out, self.data)


def create_array(shape, dtype=_DEFAULT_DTYPE):
    out = Array(_normalize_shape(shape), _normalize_dtype(dtype))
    lazy.record_create(out.name, out._wire, out.shape)
    return out


def _assign_host_data(target, values):
    """Whole-array load from host data: one fill when all elements are equal, else one bulk upload
    (upstream assigns element by element here, charmnumeric.py:863-878)."""
    src = _HostValues(values, dtype=target.dtype)
    if src.data.shape != tuple(target.shape):
        raise ValueError(f"cannot assign data with shape {src.data.shape} into shape {target.shape}")
    if src.data.size == 0:
        return target
    same = src.constant()
    if same is not None:
        target[...] = _coerce_scalar(same)
    else:
        lazy.record_call(lazy.Call(target.name, "put", target.wire_dtype(),
                                   np.ascontiguousarray(src.data).copy()))
    return target


def _coerce_assignment_operand(rhs, shape, dtype):
    """Right-hand side of an assignment: device objects and scalars pass, host data is uploaded."""
    if isinstance(rhs, _ArrayLike):
        return rhs
    if _is_scalar_like(rhs):
        return _coerce_scalar(rhs)
    src = _HostValues(rhs, dtype=dtype, broadcast=shape)
    return _coerce_scalar(src.data.item()) if src.is_scalar else src.upload()


def empty(shape, dtype=_DEFAULT_DTYPE):
    return create_array(shape, dtype)


zeros = empty          # new arrays are zero-filled by the executor


def full(shape, fill_value, dtype=None):
    shape = _normalize_shape(shape)
    src = None if _is_scalar_like(fill_value) else _HostValues(fill_value, dtype=dtype, broadcast=shape,
                                                                what="fill_value")
    if src is not None and not src.is_scalar:
        return src.upload()
    value = fill_value if src is None else src.data.item()
    dt = _normalize_dtype(dtype, allow_none=True) or _normalize_dtype(np.asarray(value).dtype)
    out = create_array(shape, dt)
    out[...] = _coerce_scalar(value)
    out._all_ones = value == 1
    return out


def ones(shape, dtype=_DEFAULT_DTYPE):
    return full(shape, 1, dtype=dtype)


def _like_constructor(make, doc):
    """X_like(a, ..., dtype=None, shape=None): shape and dtype of `a` unless overridden."""
    def ctor(a, *args, dtype=None, shape=None):
        if isinstance(a, _ArrayLike):
            s, d = a.shape, a.dtype
        else:
            host = np.asarray(a)
            if host.ndim == 0:
                raise NotImplementedError("0D charmnumeric arrays are not supported yet")
            s, d = host.shape, _normalize_dtype(host.dtype)
        return make(s if shape is None else _normalize_shape(shape), *args,
                    dtype=d if dtype is None else _normalize_dtype(dtype))
    ctor.__doc__ = doc
    return ctor


empty_like = _like_constructor(empty, "empty_like(a, dtype=None, shape=None)")
zeros_like = _like_constructor(zeros, "zeros_like(a, dtype=None, shape=None)")
ones_like = _like_constructor(ones, "ones_like(a, dtype=None, shape=None)")
full_like = _like_constructor(full, "full_like(a, fill_value, dtype=None, shape=None)")


def _existing(a, dtype):
    """`a` when it is a device object of the requested dtype (None for host data)."""
    if not isinstance(a, _ArrayLike):
        return None
    want = _normalize_dtype(dtype, allow_none=True)
    if want is not None and want != a.dtype:
        raise NotImplementedError(
            "dtype conversion for existing charmnumeric arrays is not implemented yet")
    return a


def asarray(a, dtype=None):
    have = _existing(a, dtype)
    return have if have is not None else _HostValues(a, dtype=dtype).upload()


def array(a, dtype=None, copy=True, ndmin=0):
    have = _existing(a, dtype)
    if have is None:
        return _HostValues(a, dtype=dtype, copy=copy, ndmin=ndmin).upload()
    if len(have.shape) < ndmin:
        raise NotImplementedError("ndmin on an existing charmnumeric array is not implemented")
    return have.copy() if copy else have


def copy(a, order="K"):
    return array(a, copy=True)


def copyto(dst, src):
    if not isinstance(dst, _ArrayLike):
        raise TypeError("copyto destination must be a charmnumeric Array or ArrayView")
    dst[...] = src
    return dst


def arange(start, stop=None, step=1, dtype=None):
    return _HostValues(np.arange(start, stop, step, dtype=_normalize_dtype(dtype, allow_none=True))).upload()


def eye(N, M=None, k=0, dtype=_DEFAULT_DTYPE):
    rows = int(N)
    cols = rows if M is None else int(M)
    return _HostValues(np.eye(rows, cols, int(k), dtype=_normalize_dtype(dtype))).upload()


def identity(n, dtype=_DEFAULT_DTYPE):
    return eye(n, dtype=dtype)


if _cnrec is not None:
    _cnrec.setup(lazy._state, Array, ArrayView, _ArrayLike._py_getitem, _ArrayLike._py_setitem, _binary,
                 lazy._flush_if_due, (L.OP_ADD, L.OP_SUB, L.OP_MUL, L.OP_DIV))


def set_fast_recording(on=True):
    """Switches the C fast paths of indexing, operators and assignment on or off (off: every call
    takes the Python methods; the statement log is the same bytes either way). Returns the previous
    setting; without the C module it is always off."""
    return bool(_cnrec.set_fast(bool(on))) if _cnrec is not None else False
