"""Builds the flat AST structure (cnh_ast) that the executor consumes.

The field set and conventions are those the upstream backend reads from its AST nodes
(src/jit.cpp:223-385, tests/test_jit.cpp:35-46 upstream): leaves are NOOP nodes named after the
array they stand for, scalar leaves carry unique negative names, roots are listed temporaries
first, and a SET_REGION root has operands [target, rhs] plus the assigned region.
"""
from __future__ import annotations

import ctypes as C

from . import _lib as L


class AstBuilder:
    def __init__(self, dtype, ndims):
        self.dtype = int(dtype)
        self.ndims = int(ndims)
        self._nodes = []
        self._roots = []
        self._next_scalar = -1
        self._keep = None

    # -- leaves ---------------------------------------------------------------------------
    def _new(self, name, opcode, is_temp=False, is_scalar=False, scalar=0.0, is_broadcast=False,
             ndims=None):
        n = L.AstNode()
        n.result_name = int(name)
        n.opcode = int(opcode)
        n.is_temp = int(bool(is_temp))
        n.is_scalar = int(bool(is_scalar))
        n.is_broadcast = int(bool(is_broadcast))
        n.ndims = self.ndims if ndims is None else int(ndims)
        n.dtype = self.dtype
        n.n_operands = 0
        n.operands[0] = -1
        n.operands[1] = -1
        n.scalar = float(scalar)
        n.region = L.Region.make()
        n.operand_regions[0] = L.Region.make()
        n.operand_regions[1] = L.Region.make()
        self._nodes.append(n)
        return len(self._nodes) - 1

    def leaf(self, name, ndims=None):
        return self._new(name, L.OP_NOOP, ndims=ndims)

    def broadcast(self, name):
        """A size-1 array used as a run-time scalar (dot results, alpha, beta)."""
        return self._new(name, L.OP_NOOP, is_broadcast=True, ndims=1)

    def scalar(self, value):
        idx = self._new(self._next_scalar, L.OP_NOOP, is_scalar=True, scalar=value)
        self._next_scalar -= 1
        return idx

    # -- roots ----------------------------------------------------------------------------
    def _attach(self, node, slot, operand, region):
        node.operands[slot] = operand
        if region is not None:
            node.has_operand_region[slot] = 1
            node.operand_regions[slot] = region if isinstance(region, L.Region) else L.Region.make(*region)

    def binary(self, opcode, name, lhs, rhs, lhs_region=None, rhs_region=None, is_temp=True):
        idx = self._new(name, opcode, is_temp=is_temp)
        n = self._nodes[idx]
        n.n_operands = 2
        self._attach(n, 0, lhs, lhs_region)
        self._attach(n, 1, rhs, rhs_region)
        self._roots.append(idx)
        return idx

    def unary(self, opcode, name, operand, region=None, is_temp=True):
        idx = self._new(name, opcode, is_temp=is_temp)
        n = self._nodes[idx]
        n.n_operands = 1
        self._attach(n, 0, operand, region)
        self._roots.append(idx)
        return idx

    def set_region(self, name, target, rhs, region, rhs_region=None):
        idx = self._new(name, L.OP_SET_REGION, is_temp=False)
        n = self._nodes[idx]
        n.n_operands = 2
        self._attach(n, 0, target, None)
        self._attach(n, 1, rhs, rhs_region)
        n.region = region if isinstance(region, L.Region) else L.Region.make(*region)
        self._roots.append(idx)
        return idx

    def finish(self):
        nodes = (L.AstNode * len(self._nodes))(*self._nodes)
        roots = (C.c_int32 * len(self._roots))(*self._roots)
        ast = L.Ast()
        ast.n_nodes = len(self._nodes)
        ast.n_roots = len(self._roots)
        ast.nodes = C.cast(nodes, C.POINTER(L.AstNode))
        ast.roots = C.cast(roots, C.POINTER(C.c_int32))
        self._keep = (nodes, roots)
        ast._keep = self._keep  # keep the arrays alive with the struct
        return ast
