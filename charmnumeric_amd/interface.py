"""The interface object: where upstream's frontend talks to a Charm++ server over a CCS socket
(charmnumeric/interface.py upstream), this one drives the in-process executor of libcnhip through
its C ABI (include/cnexec.h). `connect` keeps upstream's signature; address and port are ignored."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from . import _lib as L
from . import lazy


class CharmNumericInterface:
    def __init__(self, device=0, max_pes=1):
        """device < 0 selects the executor's dry mode: every decision is taken and logged, nothing
        is allocated or launched (used by tests on machines without a GPU)."""
        self.device = int(device)
        self.max_pes = int(max_pes)
        self.odf = None
        self._ex = None
        self._min_tiles = {}
        self._pipeline = False
        self._solver = os.environ.get("CHARMNUMERIC_SOLVER", "0") not in ("", "0")
        self._flat3 = os.environ.get("CHARMNUMERIC_FLAT3", "1") not in ("", "0")
        self._fusion = os.environ.get("CHARMNUMERIC_FUSE", "1") not in ("", "0")

    # -- decomposition planning ----------------------------------------------------------------
    def set_solver(self, on=True):
        """Plan tile edges and offsets of new arrays per DAG message the way upstream's server
        does (src/decomposition_solver.hpp upstream) instead of the tile rule with offset 0.
        Values never depend on it. Off by default (environment variable CHARMNUMERIC_SOLVER=1
        turns it on for every interface): with all tiles on one device, lined-up tiles save no
        traffic."""
        self._solver = bool(on)
        if self._ex is not None:
            L.check(L.lib.cnx_set_solver(self._ex, 1 if on else 0))

    def set_layout(self, flat_rank3=True):
        """How rank-3 arrays created from now on are stored: one row-major block with the
        partitions as views into it (default; environment variable CHARMNUMERIC_FLAT3=0 turns it
        off for every interface), or one contiguous buffer per partition."""
        self._flat3 = bool(flat_rank3)
        if self._ex is not None:
            L.check(L.lib.cnx_set_layout(self._ex, 1 if flat_rank3 else 0))

    def set_fusion(self, on=True):
        """Whether the executor merges nodes into fewer launches: runs of same-extent assignments,
        products written straight into the slice they are assigned to, dense statements with the
        scalar statements between them and the reductions behind them, a matvec with the vector
        update before it and the dot behind it, the two lattices of a red-black colour (default on;
        environment variable CHARMNUMERIC_FUSE=0 turns it off for every interface). Stored arrays
        of element-wise statements are the same bit for bit either way. Reductions (and what is
        computed from them) agree to the order of summation only: a reduction taken by the launch
        that produces its operand adds other partial sums than one that reads the array again, and
        which form runs can also depend on where a flush falls."""
        self._fusion = bool(on)
        if self._ex is not None:
            L.check(L.lib.cnx_set_fusion(self._ex, 1 if on else 0))

    # -- pipelining --------------------------------------------------------------------------
    def set_pipeline(self, on=True):
        """Upstream's frontend hands DAG messages to a server and goes on recording; with
        pipelining on, the executor does the same with a thread of its own: send_dag returns once
        the message is queued, and the executor works through the queue while Python records the
        next statements. Whatever reads state back (get, sync, array_info, stats, trace, close)
        waits for the queue first. An error of the executor then surfaces at the next call on the
        interface, not at the send that caused it; work queued behind a failed message is
        dropped."""
        self._pipeline = bool(on)
        if self._ex is not None:
            L.check(L.lib.cnx_set_async(self._ex, 1 if on else 0))

    # -- connection --------------------------------------------------------------------------
    def connect(self, server_ip=None, server_port=None, odf=4):
        if self._ex is not None:
            raise RuntimeError("already connected")
        ex = C.c_void_p()
        L.check(L.lib.cnx_create(self.device, self.max_pes, int(odf), C.byref(ex)))
        self._ex = ex
        self.odf = int(odf)
        for nd, t in self._min_tiles.items():
            L.check(L.lib.cnx_set_min_tile(self._ex, nd, t))
        if self._solver:
            L.check(L.lib.cnx_set_solver(self._ex, 1))
        if not self._flat3:
            L.check(L.lib.cnx_set_layout(self._ex, 0))
        if not self._fusion:
            L.check(L.lib.cnx_set_fusion(self._ex, 0))
        if self._pipeline:
            L.check(L.lib.cnx_set_async(self._ex, 1))
        return self

    def set_min_tile(self, ndims, min_tile):
        """Minimum tile edge per rank (CT_MIN_TILE_1D/2D/3D upstream, src/backend.hpp:10-18)."""
        self._min_tiles[int(ndims)] = int(min_tile)
        if self._ex is not None:
            L.check(L.lib.cnx_set_min_tile(self._ex, int(ndims), int(min_tile)))

    def close(self):
        if self._ex is not None:
            # instructions still pending refer to arrays of this executor: drop them
            try:
                lazy.execute(self)
            finally:
                ex, self._ex = self._ex, None
                L.check(L.lib.cnx_destroy(ex))

    def __enter__(self):
        return self

    def __exit__(self, exc_type, exc, tb):
        self.close()

    def _handle(self):
        if self._ex is None:
            raise RuntimeError("interface is not connected")
        return self._ex

    # -- what the lazy core calls ------------------------------------------------------------------
    def send_dag(self, epoch, message):
        L.check(L.lib.cnx_receive_dag(self._handle(), int(epoch), len(message), message))

    def send_log(self, log, hold_back_window=-1):
        """A stretch of the statement log (lazy.py records it; format: include/cnexec.h). The
        executor plans it into DAG nodes and runs them; a window >= 0 marks an automatic flush, which
        may leave the most recent statements unplanned until the next call."""
        L.check(L.lib.cnx_receive_log(self._handle(), len(log), log, int(hold_back_window)))

    def discard_log(self):
        """Drops what automatic flushes left unplanned in the executor (the frontend was reset)."""
        if self._ex is not None:
            L.check(L.lib.cnx_discard_log(self._ex))

    def set_capture(self, on=True):
        """Test hook: keep the DAG messages planned from the log; captured() returns and clears them."""
        L.check(L.lib.cnx_set_capture(self._handle(), 1 if on else 0))

    def captured(self):
        ex = self._handle()
        need = L.lib.cnx_captured(ex, None, 0)
        if need < 0:
            L.check(int(need))
        buf = C.create_string_buffer(max(1, int(need)))
        L.lib.cnx_captured(ex, buf, int(need))
        raw, out, pos = buf.raw[:int(need)], [], 0
        while pos < len(raw):
            size = int.from_bytes(raw[pos:pos + 8], "little")
            out.append(raw[pos + 8:pos + 8 + size])
            pos += 8 + size
        return out

    def direct_call(self, instr):
        ex = self._handle()
        if instr.opcode == "put":
            host = instr.payload
            L.check(L.lib.cnx_put(ex, instr.name, host.size, instr.dtype, host.ctypes.data_as(C.c_void_p)))
        elif instr.opcode == "fill_uniform":
            seed, stream, lo, hi = instr.payload
            L.check(L.lib.cnx_fill_uniform(ex, instr.name, seed, stream, lo, hi))
        elif instr.opcode == "fill_cg_matrix":
            L.check(L.lib.cnx_fill_cg_matrix(ex, instr.name, instr.payload[0]))
        else:
            raise AssertionError(instr.opcode)

    # -- data out ----------------------------------------------------------------------------
    def get(self, ndims, name, size, dtype=np.float64):
        """Array `name` as a flat NumPy array (upstream: interface.get(ndims, name, size, dtype=),
        charmnumeric.py:683-688)."""
        out = np.empty(int(size), dtype=np.dtype(dtype))
        L.check(L.lib.cnx_get(self._handle(), int(ndims), 0, int(name), int(size), lazy.wire_dtype(dtype),
                              out.ctypes.data_as(C.c_void_p)))
        return out

    def sync(self):
        L.check(L.lib.cnx_sync(self._handle()))

    # -- introspection -----------------------------------------------------------------------
    def array_info(self, name):
        nd, dt, tile = C.c_int(), C.c_int(), C.c_int()
        shape, off = (C.c_int32 * 3)(), (C.c_int32 * 3)()
        L.check(L.lib.cnx_array_info(self._handle(), int(name), C.byref(nd), C.byref(dt), C.byref(tile),
                                     shape, off))
        return {"ndims": nd.value, "dtype": dt.value, "tile": tile.value,
                "shape": tuple(shape[:nd.value]), "offset": tuple(off[:nd.value])}

    def time_matvecs(self, on=True):
        """Brackets every matvec launch with events from now on (measurement only)."""
        L.check(L.lib.cnx_set_matvec_timing(self._handle(), 1 if on else 0))

    def matvec_times_ms(self, at_most=4096):
        """Elapsed milliseconds of the matvec launches timed since the last call, oldest first."""
        buf = (C.c_float * at_most)()
        n = L.lib.cnx_matvec_times(self._handle(), buf, at_most)
        if n < 0:
            L.check(int(n))
        return [buf[i] for i in range(n)]

    def stats(self):
        out = (C.c_int64 * 8)()
        L.check(L.lib.cnx_stats(self._handle(), out))
        keys = ("compiled", "cache_hits", "nodes", "allocations", "reuses", "group_launches",
                "live_arrays", "bytes_held")
        return dict(zip(keys, out))

    def set_trace(self, on=True):
        L.check(L.lib.cnx_set_trace(self._handle(), 1 if on else 0))

    def trace(self):
        need = L.lib.cnx_trace(self._handle(), None, 0)
        L.check(need)
        buf = C.create_string_buffer(int(need))
        L.lib.cnx_trace(self._handle(), buf, need)
        return buf.value.decode().splitlines()


class LocalCluster(CharmNumericInterface):
    """Context manager that starts an executor and connects to it; upstream's LocalCluster launches
    `charmrun +p<max_pes> server` and connects with `odf` (charmnumeric/interface.py:25-129
    upstream)."""

    def __init__(self, server_binary=None, *, odf=4, max_pes=1, device=0, **_ignored):
        super().__init__(device=device, max_pes=max_pes)
        self.connect(odf=odf)
