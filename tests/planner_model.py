"""A Python model of the statement-log planner of libcnhip (csrc/stmtlog.cpp): the grouping rule,
the hold-back rule of automatic flushes and the DAG message encoding, written out independently so
that the tests can compare the native planner's messages with it byte for byte.

Grouping rule: consecutive elementwise operations of one result shape form a group; a group ends at
the first result that must exist as an array afterwards (its handle is still alive, or something
outside the group reads it), at an assignment ``target[region] = value`` that consumes the group's
last result (which becomes the group's SET_REGION root), and before any other kind of instruction.
Results that die inside their group are temporaries and never touch memory.
"""
import struct

from charmnumeric_amd import _lib as L
from charmnumeric_amd.lazy import (ArrayRef, DAG_MAGIC, OP_DELETE, _LONE_NODE, _NodeWriter, _full_region)

_KINDS = {1: "create", 2: "op", 3: "set", 4: "nonfusible", 5: "delete"}


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



def decode_log(log):
    """The records of a statement log (format: include/cnexec.h) as Instr objects."""
    out, pos = [], 0

    def words(n):
        nonlocal pos
        v = struct.unpack_from("<%di" % n, log, pos)
        pos += 4 * n
        return v

    while pos < len(log):
        kind, name = words(2)
        if kind == 5:
            out.append(Instr("delete", name=name))
            continue
        opcode, dtype, n_operands, aux = words(4)
        nd, *shape = words(4)
        shape = tuple(shape[:nd])
        region = None
        if kind == 3:
            rnd, *v = words(10)
            region = (tuple(v[0:rnd]), tuple(v[3:3 + rnd]), tuple(v[6:6 + rnd]))
        operands = []
        for _ in range(n_operands):
            tag, = words(1)
            if tag == 0:
                words(1)
                operands.append(struct.unpack_from("<d", log, pos)[0])
                pos += 8
                continue
            oname, base_nd, odtype, bc, has = words(5)
            v = words(9)
            oreg = (tuple(v[0:base_nd]), tuple(v[3:3 + base_nd]), tuple(v[6:6 + base_nd])) if has else None
            operands.append(ArrayRef(oname, oreg, (), base_nd, odtype, bool(bc)))
        payload = ArrayRef(name, None, (), aux, dtype) if kind == 3 else None
        out.append(Instr(_KINDS[kind], name, opcode, operands, shape, dtype, region, payload))
    return out


class _Names:
    """Result names of the SET_REGION roots: counted from 2^30, above every array name."""

    def __init__(self):
        self.next = 1 << 30

    def __call__(self):
        self.next += 1
        return self.next - 1


new_name = _Names()


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




class Planner:
    """What the executor does with the stretches of log it receives: keeps what an automatic flush
    holds back, plans the rest. feed() returns the DAG message planned (None when there is nothing)."""

    def __init__(self):
        self.pending = []
        new_name.next = 1 << 30

    def feed(self, log, window):
        self.pending += decode_log(log)
        if not self.pending:
            return None
        batch, self.pending = self.pending, []
        dead_later, fused_away = (), set()
        if window >= 0:
            cut = _hold_back_cut(batch, window)
            if cut < len(batch):
                tail = batch[cut:]
                batch = batch[:cut]
                read_in_tail = {o.name for ins in tail if ins.kind != "delete"
                                for o in ins.operands if isinstance(o, ArrayRef)}
                read_in_tail |= {ins.name for ins in tail if ins.kind == "set"}
                produced = {ins.name for ins in batch if ins.kind == "op"}
                dead_later = {ins.name for ins in tail if ins.kind == "delete" and ins.name in produced
                              and ins.name not in read_in_tail}
                self.pending = tail
        out = build_messages(batch, dead_later, fused_away)
        self.pending = [ins for ins in self.pending if not (ins.kind == "delete" and ins.name in fused_away)]
        assert len(out) <= 1
        return out[0][1] if out else struct.pack("<iii", DAG_MAGIC, 1, 0)
