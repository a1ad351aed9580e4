"""Lazy recording core of the frontend: every array operation is recorded in program order, as one
small binary record of the statement log (format: include/cnexec.h), and the log is shipped to the
executor when something forces a flush. The executor groups the records into a DAG of fused groups
(csrc/stmtlog.cpp) on its own thread, so recording costs the program one struct.pack per operation.

Upstream delegates this layer to charmtyles (``fusible_op`` / ``nonfusible_op`` / ``create_object``
/ ``execute`` / ``set_auto_flush``, imported at charmnumeric/charmnumeric.py:5-16 and used by
examples/jacobi2d.py:2-6 upstream); charmtyles is not part of the charmnumeric tree, so the grouping
rule and the byte formats here are this package's own. What is kept: the AST node fields and opcode /
dtype numbers the backend consumes, and the observable semantics (program order, lazy execution,
results identical to evaluating statement by statement).

Grouping rule: consecutive elementwise operations of one result shape form a group; a group ends at
the first result that must exist as an array afterwards (its handle is still alive, or something
outside the group reads it), at an assignment ``target[region] = value`` that consumes the group's
last result (which becomes the group's SET_REGION root), and before any other kind of instruction.
Results that die inside their group are temporaries and never touch memory.
"""
from __future__ import annotations

import struct

import numpy as np

from . import _lib as L

# Extension opcodes of include/cnexec.h
OP_DELETE, OP_SUM, OP_SUMSQ_DIFF, OP_MAXABS_DIFF, OP_ASTYPE = 100, 101, 102, 103, 104
DAG_MAGIC = 0x47444E43

_ELEMENTWISE = {L.OP_ADD, L.OP_SUB, L.OP_MUL, L.OP_DIV, L.OP_TANH, L.OP_EXP, L.OP_COPY}


class Call:
    """A call that goes to the executor directly, in program order: a bulk upload or a fill."""

    __slots__ = ("name", "opcode", "dtype", "payload")

    def __init__(self, name, opcode, dtype, payload):
        self.name = name
        self.opcode = opcode          # "put" | "fill_uniform" | "fill_cg_matrix"
        self.dtype = dtype
        self.payload = payload


class _State:
    def __init__(self):
        self.pending = []             # log records (bytes) and Call objects, in program order
        self.next_name = 1
        self.auto_flush = None        # (interface, threshold)
        self.flush_at = 1 << 62       # the threshold while automatic flushes are on
        self.flushing = False
        self.in_expression = False    # the last record that is not a deletion is an elementwise operation
        self.generation = 0           # bumped by reset(): handles of older generations are inert


_state = _State()

# record kinds of the statement log
_CREATE, _OP, _SET, _NONFUSIBLE, _DELETE = 1, 2, 3, 4, 5
_HEAD = struct.Struct("<6i")          # kind, name, opcode, dtype, n_operands, aux
_DELETE_REC = struct.Struct("<2i")
_SHAPE = struct.Struct("<4i")         # ndims, extent[3]
_REGION3 = struct.Struct("<10i")      # ndims, start[3], stop[3], step[3]
_SCALAR = struct.Struct("<iid")       # 0, 0, value
_REF = struct.Struct("<15i")          # 1, name, base_ndims, dtype, broadcast, has_region, start/stop/step[3]
_PAD = ((), (0, 0), (0,), ())         # what fills a rank-n triple up to three entries
_shape_cache = {}


def new_name():
    n = _state.next_name
    _state.next_name += 1
    return n


def shape_bytes(shape):
    out = _shape_cache.get(shape)
    if out is None:
        out = _SHAPE.pack(len(shape), *shape, *_PAD[len(shape)])
        if len(_shape_cache) < 4096:
            _shape_cache[shape] = out
    return out


def ref_bytes(name, base_ndims, dtype, region, broadcast=False):
    """One use of an array (region None) or of a slice of it as an operand."""
    if region is None:
        return _REF.pack(1, name, base_ndims, dtype, 1 if broadcast else 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0)
    start, stop, step = region
    if base_ndims == 3:
        return _REF.pack(1, name, 3, dtype, 1 if broadcast else 0, 1, *start, *stop, *step)
    pad = _PAD[base_ndims]
    return _REF.pack(1, name, base_ndims, dtype, 1 if broadcast else 0, 1, *start, *pad, *stop, *pad, *step, *pad)


def scalar_bytes(value):
    return _SCALAR.pack(0, 0, value)


def _flush_if_due():
    af = _state.auto_flush
    if af is not None and not _state.flushing and len(_state.pending) >= af[1]:
        # never in the middle of an expression (its intermediates are alive only until it is
        # finished, and flushing would turn each into a real array), unless the backlog is large: a
        # program made of elementwise statements only has no other point
        if not _state.in_expression or len(_state.pending) >= 16 * af[1]:
            execute(af[0], hold_back=True)


def record_op(name, opcode, dtype, shape, a, b=None):
    """An elementwise operation over one or two operands (ref_bytes / scalar_bytes)."""
    st = _state
    if len(st.pending) >= st.flush_at:
        _flush_if_due()
    st.in_expression = True
    sb = _shape_cache.get(shape) or shape_bytes(shape)
    if b is None:
        st.pending.append(_HEAD.pack(_OP, name, opcode, dtype, 1, 0) + sb + a)
    else:
        st.pending.append(_HEAD.pack(_OP, name, opcode, dtype, 2, 0) + sb + a + b)


def record_set(name, dtype, base_ndims, shape, region, operand):
    """target[region] = operand; `shape` is the extent of the region."""
    st = _state
    if len(st.pending) >= st.flush_at:
        _flush_if_due()
    st.in_expression = False
    start, stop, step = region
    sb = _shape_cache.get(shape) or shape_bytes(shape)
    if base_ndims == 3:
        rb = _REGION3.pack(3, *start, *stop, *step)
    else:
        pad = _PAD[base_ndims]
        rb = _REGION3.pack(base_ndims, *start, *pad, *stop, *pad, *step, *pad)
    st.pending.append(_HEAD.pack(_SET, name, 0, dtype, 1, base_ndims) + sb + rb + operand)


def record_nonfusible(name, opcode, dtype, shape, operands):
    st = _state
    if len(st.pending) >= st.flush_at:
        _flush_if_due()
    st.in_expression = False
    st.pending.append(_HEAD.pack(_NONFUSIBLE, name, opcode, dtype, len(operands), 0) + shape_bytes(shape)
                      + b"".join(operands))


def record_create(name, dtype, shape):
    st = _state
    if len(st.pending) >= st.flush_at:
        _flush_if_due()
    st.in_expression = False
    st.pending.append(_HEAD.pack(_CREATE, name, 0, dtype, 0, 0) + shape_bytes(shape))


def record_call(call):
    st = _state
    if len(st.pending) >= st.flush_at:
        _flush_if_due()
    st.in_expression = False
    st.pending.append(call)


def generation():
    return _state.generation


def record_delete(name, gen):
    # Called from handle finalisers; never flushes (it may run at any point, even at shutdown).
    # A handle created before the last reset() names nothing any more: names restart there.
    try:
        if gen != _state.generation:
            return
        _state.pending.append(_DELETE_REC.pack(_DELETE, name))
    except Exception:  # interpreter teardown
        pass


def set_auto_flush(interface, threshold):
    """Flush to `interface` whenever `threshold` instructions are pending (examples/jacobi2d.py:6
    upstream)."""
    _state.auto_flush = (interface, int(threshold))
    _state.flush_at = int(threshold)


def reset():
    """Forget everything recorded and restart naming (what upstream's test fixture
    reset_frontend_state does, tests/conftest.py:128-141 upstream)."""
    _state.pending.clear()
    _state.next_name = 1
    af, _state.auto_flush = _state.auto_flush, None
    _state.flush_at = 1 << 62
    _state.in_expression = False
    _state.generation += 1
    if af is not None:
        af[0].discard_log()           # what its automatic flushes held back


def pending_count():
    return len(_state.pending)


def execute(interface, hold_back=False):
    """Ships everything recorded so far to the executor behind `interface`
    (charmtyles.core.execute upstream: examples/jacobi3d.py:2,18). An automatic flush
    (`hold_back`) lets the executor keep the most recent statements unplanned when one of them
    produced a result whose handle is still alive (a loop `upd = f(u[...]); u[...] = g(u[...], upd)`
    frees `upd` only one iteration later; planned now it would become an array of its own)."""
    if _state.flushing:
        return
    _state.flushing = True
    try:
        batch = _state.pending
        _state.pending = []
        window = _state.auto_flush[1] if hold_back and _state.auto_flush is not None else -1
        chunk = []
        for item in batch:
            if type(item) is bytes:
                chunk.append(item)
            else:
                interface.send_log(b"".join(chunk), -1)
                chunk = []
                interface.direct_call(item)
        if chunk or window < 0:
            interface.send_log(b"".join(chunk), window)
    finally:
        _state.flushing = False


# ---------------------------------------------------------------------------------------------
# DAG messages written by hand (include/cnexec.h): for callers of send_dag


class ArrayRef:
    """One use of an array (or of a slice of it) as an operand."""

    __slots__ = ("name", "region", "shape", "base_ndims", "dtype", "broadcast")

    def __init__(self, name, region, shape, base_ndims, dtype, broadcast=False):
        self.name = name
        self.region = region          # (start, stop, step) tuples relative to the base array, or None
        self.shape = shape if type(shape) is tuple else tuple(shape)
        self.base_ndims = base_ndims
        self.dtype = dtype            # wire dtype
        self.broadcast = broadcast


_GLOBAL_REGION = struct.pack("<i", 1)
_region_cache = {}


def _region_bytes(region):
    if region is None:
        return _GLOBAL_REGION
    out = _region_cache.get(region)
    if out is None:
        start, stop, step = region
        flat = [0, len(start)]
        for d in range(len(start)):
            flat += [int(start[d]), int(stop[d]), int(step[d])]
        out = struct.pack("<%di" % len(flat), *flat)
        if len(_region_cache) < 4096:
            _region_cache[region] = out
    return out


def _full_region(shape):
    return (tuple(0 for _ in shape), tuple(int(s) for s in shape), tuple(1 for _ in shape))


_NODE_HEAD = [struct.Struct("<8i%dd" % 1 if k == 0 else "<8i%did" % k) for k in range(3)]
# one DAG node holding a single operand-less AST node (id, fusible, 1 node, 1 root | node | global
# region | root 0)
_LONE_NODE = struct.Struct("<4i8idii")


class _NodeWriter:
    """Collects the AST nodes of one DAG node."""

    def __init__(self):
        self.nodes = []
        self.roots = []
        self._leaf = {}
        self._next_scalar = -1

    def _add(self, name, opcode, is_temp, is_scalar, is_broadcast, ndims, dtype, operands, scalar,
             operand_regions, region):
        self.nodes.append((name, opcode, is_temp, is_scalar, is_broadcast, ndims, dtype, operands, scalar,
                           operand_regions, region))
        return len(self.nodes) - 1

    def leaf(self, ref):
        key = (ref.name, bool(ref.broadcast))
        if key not in self._leaf:
            self._leaf[key] = self._add(ref.name, L.OP_NOOP, 0, 0, 1 if ref.broadcast else 0,
                                        ref.base_ndims, ref.dtype, (), 0.0, (), None)
        return self._leaf[key]

    def scalar(self, value, ndims, dtype):
        idx = self._add(self._next_scalar, L.OP_NOOP, 0, 1, 0, ndims, dtype, (), float(value), (), None)
        self._next_scalar -= 1
        return idx

    def op(self, name, opcode, is_temp, ndims, dtype, operands, operand_regions, region=None, root=True):
        idx = self._add(name, opcode, 1 if is_temp else 0, 0, 0, ndims, dtype, tuple(operands), 0.0,
                        tuple(operand_regions), region)
        if root:
            self.roots.append(idx)
        return idx

    def to_bytes(self, node_id, fusible):
        out = [struct.pack("<iiii", node_id, 1 if fusible else 0, len(self.nodes), len(self.roots))]
        for (name, opcode, is_temp, is_scalar, is_bc, ndims, dtype, operands, scalar, oregs, region) in self.nodes:
            out.append(_NODE_HEAD[len(operands)].pack(name, opcode, is_temp, is_scalar, is_bc, ndims, dtype,
                                                      len(operands), *operands, scalar))
            for r in oregs:
                out.append(_region_bytes(r))
            out.append(_region_bytes(region))
        out.append(struct.pack("<%di" % len(self.roots), *self.roots))
        return b"".join(out)



_WIRE = {np.dtype("float32"): L.F32, np.dtype("float64"): L.F64, np.dtype("int32"): L.I32,
         np.dtype("int64"): L.I64}


def wire_dtype(np_dtype):
    return _WIRE[np.dtype(np_dtype)]
