"""Lazy recording core of the frontend: every array operation is recorded in program order and
shipped to the executor as a DAG of fused groups when something forces a flush.

Upstream delegates this layer to charmtyles (``fusible_op`` / ``nonfusible_op`` / ``create_object``
/ ``execute`` / ``set_auto_flush``, imported at charmnumeric/charmnumeric.py:5-16 and used by
examples/jacobi2d.py:2-6 upstream); charmtyles is not part of the charmnumeric tree, so the grouping
rule and the byte format here are this package's own. What is kept: the AST node fields and opcode /
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
OP_DELETE, OP_SUM, OP_SUMSQ_DIFF, OP_MAXABS_DIFF = 100, 101, 102, 103
DAG_MAGIC = 0x47444E43

_ELEMENTWISE = {L.OP_ADD, L.OP_SUB, L.OP_MUL, L.OP_DIV, L.OP_TANH, L.OP_EXP, L.OP_COPY}


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


class Instr:
    __slots__ = ("kind", "name", "opcode", "operands", "shape", "dtype", "region", "payload")

    def __init__(self, kind, name=None, opcode=None, operands=(), shape=(), dtype=L.F64, region=None,
                 payload=None):
        self.kind = kind              # create | op | set | nonfusible | delete | call
        self.name = name
        self.opcode = opcode
        self.operands = operands if type(operands) is list else list(operands)  # ArrayRef or scalars
        self.shape = shape if type(shape) is tuple else tuple(shape)
        self.dtype = dtype
        self.region = region
        self.payload = payload


class _State:
    def __init__(self):
        self.pending = []
        self.next_name = 1
        self.auto_flush = None        # (interface, threshold)
        self.epoch = 0
        self.flushing = False
        self.generation = 0           # bumped by reset(): handles of older generations are inert


_state = _State()


def new_name():
    n = _state.next_name
    _state.next_name += 1
    return n


def _between_statements():
    """True when what was recorded last is a complete statement: an assignment, a creation or a
    non-elementwise operation, followed only by deletions. While an expression is being built the
    last non-deletion is one of its elementwise operations, whose handle is alive only until the
    expression is finished; flushing then would turn every such intermediate into a real array."""
    p = _state.pending
    i = len(p) - 1
    while i >= 0 and p[i].kind == "delete":
        i -= 1
    return i >= 0 and p[i].kind != "op"


def record(instr):
    af = _state.auto_flush
    if af is not None and not _state.flushing and len(_state.pending) >= af[1]:
        # a program made of elementwise statements only has no such point: flush it anyway once
        # the backlog is large
        if _between_statements() or len(_state.pending) >= 16 * af[1]:
            execute(af[0], hold_back=True)
    _state.pending.append(instr)


def generation():
    return _state.generation


def record_delete(name, gen):
    # Called from handle finalisers; never flushes (it may run at any point, even at shutdown).
    # A handle created before the last reset() names nothing any more: names restart there.
    try:
        if gen != _state.generation:
            return
        _state.pending.append(Instr("delete", name=name))
    except Exception:  # interpreter teardown
        pass


def set_auto_flush(interface, threshold):
    """Flush to `interface` whenever `threshold` instructions are pending (examples/jacobi2d.py:6
    upstream)."""
    _state.auto_flush = (interface, int(threshold))


def reset():
    """Forget everything recorded and restart naming (what upstream's test fixture
    reset_frontend_state does, tests/conftest.py:128-141 upstream)."""
    _state.pending.clear()
    _state.next_name = 1
    _state.auto_flush = None
    _state.epoch = 0
    _state.generation += 1


def pending_count():
    return len(_state.pending)


# ---------------------------------------------------------------------------------------------
# grouping


class _Group:
    __slots__ = ("ops", "set_idx", "shape", "dtype", "names")

    def __init__(self, shape, dtype):
        self.ops = []
        self.set_idx = None
        self.shape = shape
        self.dtype = dtype
        self.names = set()


def _uses_of(batch, dropped=()):
    """name -> indices of the instructions that read it; a negative index -(i+1) marks instruction
    i writing into it (assignment target), which always counts as a use from outside any group."""
    uses = {}
    for i, ins in enumerate(batch):
        if i in dropped:
            continue
        if ins.kind in ("op", "set", "nonfusible", "call"):
            for o in ins.operands:
                if isinstance(o, ArrayRef):
                    uses.setdefault(o.name, []).append(i)
        if ins.kind in ("set", "call") and ins.name is not None:
            uses.setdefault(ins.name, []).append(-(i + 1))
    return uses


def _plan(batch, dead_later=()):
    """Returns the list of work items in execution order:
    ("group", _Group) | ("instr", index) | ("delete", name).
    `dead_later`: results whose handle is known to be dropped, unread, right after this batch."""
    producer = {ins.name: i for i, ins in enumerate(batch) if ins.kind == "op"}
    deleted = {ins.name for ins in batch if ins.kind == "delete"} | set(dead_later)
    dropped = set()                     # dead code: op indices never emitted
    forced = set()                      # op results that must be materialised

    while True:
        uses = _uses_of(batch, dropped)
        items, group_of = [], {}
        cur = None
        deferred = []

        def close():
            nonlocal cur
            if cur is not None and cur.ops:
                items.append(("group", cur))
            cur = None
            for name in deferred:
                items.append(("delete", name))
            deferred.clear()

        for i, ins in enumerate(batch):
            if i in dropped:
                continue
            if ins.kind == "op":
                reads_slice_of_own = cur is not None and any(
                    isinstance(o, ArrayRef) and o.region is not None and o.name in cur.names
                    for o in ins.operands)
                if cur is None or cur.shape != ins.shape or cur.dtype != ins.dtype or reads_slice_of_own:
                    close()
                    cur = _Group(ins.shape, ins.dtype)
                cur.ops.append(i)
                cur.names.add(ins.name)
                group_of[i] = cur
                if ins.name in forced:
                    close()
            elif ins.kind == "delete":
                if ins.name in producer and producer[ins.name] in dropped:
                    continue
                deferred.append(ins.name)
                if cur is None:
                    close()
            elif ins.kind == "set":
                v = ins.operands[0]
                fuse = (cur is not None and isinstance(v, ArrayRef) and v.region is None
                        and batch[cur.ops[-1]].name == v.name and v.name not in forced
                        and not v.broadcast and len(cur.shape) == ins.payload.base_ndims
                        and cur.dtype == ins.dtype)
                if fuse:
                    cur.set_idx = i
                    group_of[i] = cur
                    close()
                else:
                    close()
                    items.append(("instr", i))
            else:
                close()
                items.append(("instr", i))
        close()

        changed = False
        for i, ins in enumerate(batch):
            if ins.kind != "op" or i in dropped:
                continue
            g = group_of[i]
            use_idx = uses.get(ins.name, [])
            dead = ins.name in deleted
            if dead and not use_idx:
                dropped.add(i)          # computed, never read, handle gone
                changed = True
                continue
            inside = all(u >= 0 and group_of.get(u) is g for u in use_idx)
            is_last = g.ops[-1] == i
            temp_ok = dead and inside and (not is_last or g.set_idx is not None)
            if not temp_ok and ins.name not in forced:
                # must exist as an array: its group has to end here
                if not (is_last and g.set_idx is None):
                    forced.add(ins.name)
                    changed = True
        if not changed:
            return items, forced, deleted, producer, dropped


# ---------------------------------------------------------------------------------------------
# serialisation (format: include/cnexec.h)


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


def _emit_group(batch, g, forced, deleted, node_id):
    w = _NodeWriter()
    index_of = {}                      # op result name -> AST node index inside this group
    ndims = len(g.shape)
    last = g.ops[-1]
    for i in g.ops:
        ins = batch[i]
        opnds, oregs = [], []
        for o in ins.operands:
            if isinstance(o, ArrayRef):
                if o.name in index_of and o.region is None:
                    opnds.append(index_of[o.name])
                    oregs.append(None)
                else:
                    opnds.append(w.leaf(o))
                    oregs.append(o.region)
            else:
                opnds.append(w.scalar(o, ndims, ins.dtype))
                oregs.append(None)
        is_root_result = (i == last and g.set_idx is None)
        region = _full_region(ins.shape) if is_root_result else None
        index_of[ins.name] = w.op(ins.name, ins.opcode, not is_root_result, ndims, ins.dtype, opnds, oregs,
                                  region)
    if g.set_idx is not None:
        s = batch[g.set_idx]
        target = w.leaf(s.payload)      # ArrayRef of the whole target
        w.op(new_name(), L.OP_SET_REGION, False, s.payload.base_ndims, s.dtype,
             [target, index_of[batch[last].name]], [None, None], s.region)
    return w.to_bytes(node_id, True)


def _emit_instr(ins, node_id):
    w = _NodeWriter()
    if ins.kind == "create":
        w.op(ins.name, L.OP_CREATE, False, len(ins.shape), ins.dtype, [], [], _full_region(ins.shape))
        return w.to_bytes(node_id, False)
    if ins.kind == "set":
        v = ins.operands[0]
        target = w.leaf(ins.payload)
        if isinstance(v, ArrayRef):
            value, vreg = w.leaf(v), v.region
        else:
            value, vreg = w.scalar(v, ins.payload.base_ndims, ins.dtype), None
        w.op(new_name(), L.OP_SET_REGION, False, ins.payload.base_ndims, ins.dtype, [target, value],
             [None, vreg], ins.region)
        return w.to_bytes(node_id, isinstance(v, ArrayRef))
    if ins.kind == "nonfusible":
        opnds = [w.leaf(o) if isinstance(o, ArrayRef) else w.scalar(o, len(ins.shape), ins.dtype)
                 for o in ins.operands]
        w.op(ins.name, ins.opcode, False, len(ins.shape), ins.dtype, opnds,
             [o.region if isinstance(o, ArrayRef) else None for o in ins.operands], _full_region(ins.shape))
        return w.to_bytes(node_id, False)
    raise AssertionError(ins.kind)


def _emit_delete(name, node_id):
    return _LONE_NODE.pack(node_id, 0, 1, 1, name, OP_DELETE, 0, 0, 0, 1, L.F64, 0, 0.0, 1, 0)


def build_messages(batch, dead_later=(), fused_away=None):
    """Turns a batch of instructions into a list of work for an interface:
    ("dag", bytes) and ("call", Instr) in execution order. Names of `dead_later` that did not
    become arrays are added to `fused_away`."""
    items, forced, deleted, producer, dropped = _plan(batch, dead_later)
    out, nodes = [], []
    node_id = 0

    def flush_nodes():
        if nodes:
            out.append(("dag", struct.pack("<iii", DAG_MAGIC, 1, len(nodes)) + b"".join(nodes)))
            nodes.clear()

    materialised = set()
    for kind, what in items:
        if kind == "group":
            nodes.append(_emit_group(batch, what, forced, deleted, node_id))
            if what.set_idx is None:
                materialised.add(batch[what.ops[-1]].name)
        elif kind == "delete":
            if what in producer and what not in materialised:
                continue                # a temporary: it never became an array
            nodes.append(_emit_delete(what, node_id))
        else:
            ins = batch[what]
            if ins.kind == "call":
                flush_nodes()
                out.append(("call", ins))
                continue
            nodes.append(_emit_instr(ins, node_id))
        node_id += 1
    flush_nodes()
    if fused_away is not None:
        fused_away.update(n for n in dead_later if n in producer and n not in materialised)
    return out


def _hold_back_cut(batch, window):
    """Where an automatic flush stops. A loop of the form

        upd = f(u[...], ...)            # a result with a Python name
        u[...] = g(u[...], upd)         # consumed by the next statement

    leaves `upd` alive at every statement boundary: its handle goes only when the name is bound
    again, one iteration later. Flushing right there would turn it into a real array and split
    the statement in two. So the statements from the one that produced such a recent, still
    undeleted result onwards stay pending; by the next flush their deletions have arrived, and
    what is flushed now is planned knowing which of its results die, unread, in the part held
    back. Returns the number of instructions to send."""
    n = len(batch)
    deleted = {ins.name for ins in batch if ins.kind == "delete"}
    first_live = None
    for i in range(max(0, n - window), n):
        ins = batch[i]
        if ins.kind == "op" and ins.name not in deleted:
            first_live = i
            break
    if first_live is None:
        return n
    # the last statement boundary at or before that producer: a position whose predecessor
    # (deletions aside) is not an elementwise operation
    cut = first_live
    while cut > 0:
        j = cut - 1
        while j >= 0 and batch[j].kind == "delete":
            j -= 1
        if j < 0 or batch[j].kind != "op":
            break
        cut -= 1
    return cut if cut > 0 else n


def execute(interface, hold_back=False):
    """Ships everything recorded so far to the executor behind `interface`
    (charmtyles.core.execute upstream: examples/jacobi3d.py:2,18). An automatic flush
    (`hold_back`) may keep the most recent statements pending, see _hold_back_cut."""
    if _state.flushing or not _state.pending:
        return
    _state.flushing = True
    try:
        batch = _state.pending
        _state.pending = []
        dead_later, fused_away = (), None
        if hold_back and _state.auto_flush is not None:
            cut = _hold_back_cut(batch, _state.auto_flush[1])
            if cut < len(batch):
                tail = batch[cut:]
                batch = batch[:cut]
                read_in_tail = {o.name for ins in tail if ins.kind != "delete"
                                for o in ins.operands if isinstance(o, ArrayRef)}
                read_in_tail |= {ins.name for ins in tail if ins.kind in ("set", "call") and ins.name is not None}
                produced = {ins.name for ins in batch if ins.kind == "op"}
                dead_later = {ins.name for ins in tail if ins.kind == "delete" and ins.name in produced
                              and ins.name not in read_in_tail}
                fused_away = set()
                _state.pending = tail
        for kind, what in build_messages(batch, dead_later, fused_away):
            if kind == "dag":
                interface.send_dag(_state.epoch, what)
                _state.epoch += 1
            else:
                interface.direct_call(what)
        if fused_away:
            # their deletions wait in the part held back and have nothing to delete
            _state.pending = [ins for ins in _state.pending
                              if not (ins.kind == "delete" and ins.name in fused_away)]
    finally:
        _state.flushing = False


_WIRE = {np.dtype("float32"): L.F32, np.dtype("float64"): L.F64, np.dtype("int32"): L.I32,
         np.dtype("int64"): L.I64}


def wire_dtype(np_dtype):
    return _WIRE[np.dtype(np_dtype)]
