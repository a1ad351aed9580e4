"""Seeded synthetic inputs generated on the device. Upstream has no generator: its `randn`
(charmnumeric/random.py:4-5 upstream) returns a new float32 array of the asked shape, which the
server zero-fills; that function is kept with that behaviour."""
from __future__ import annotations

from . import lazy
from .array import create_array


def randn(*args):
    """As upstream's: a new float32 array of shape `args` (zero-filled, no random numbers)."""
    return create_array(tuple(args), dtype="float32")


def uniform(shape, seed, stream=0, low=0.0, high=1.0):
    """fp64 array with element i (row-major) = low + (high-low)*u01(seed, stream, i), from the
    counter-based SplitMix64 generator the tests restate in NumPy."""
    out = create_array(shape, dtype="float64")
    lazy.record_call(lazy.Call(out.name, "fill_uniform", out.wire_dtype(),
                               (int(seed), int(stream), float(low), float(high))))
    return out


def cg_matrix(n, seed):
    """The dense symmetric test matrix of the CG workload: diagonal 2.0, off-diagonal
    (u01(seed,0,i*n+j) + u01(seed,0,j*n+i)) / (2n)."""
    out = create_array((int(n), int(n)), dtype="float64")
    lazy.record_call(lazy.Call(out.name, "fill_cg_matrix", out.wire_dtype(), (int(seed),)))
    return out
