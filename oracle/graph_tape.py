"""A whole graph evaluated on the host the reference's way: node by node in
the order of teq::Evaluator (children first, internal/teq/evaluator.hpp:33-45),
every node by the oracle's routine for its opcode, inside one C call
(graph_tape.c) so that no Python runs between the nodes.  TEST INFRASTRUCTURE:
the checker of whole graphs on the CPU and the `cpu_baseline` of the graph
part of the benchmark; nothing under tenncor_amd/ imports it.

The graph is read through the node API any binding of the host layer offers
(`opcode`, `args`, `shape`, `dtype`, `attr`, `data` of a node): attributes are
decoded here the way internal/eigen/packattr.hpp:60-363 packs them.
"""
import ctypes

import numpy as np

from . import oracle as orc

RANK_CAP = 8
_NP = {1: np.float64, 2: np.float32, 3: np.int32, 4: np.int8, 5: np.uint8, 6: np.int16, 7: np.uint16, 8: np.uint32,
       9: np.int64, 10: np.uint64}


class TapeOp(ctypes.Structure):
    _fields_ = [("opcode", ctypes.c_int32), ("dtype", ctypes.c_int32), ("in_dtype", ctypes.c_int32),
                ("nargs", ctypes.c_int32), ("first_arg", ctypes.c_int32), ("out", ctypes.c_int32),
                ("nattr", ctypes.c_int32), ("pad_", ctypes.c_int32), ("n", ctypes.c_uint64),
                ("ashape", ctypes.c_uint64 * 8), ("bshape", ctypes.c_uint64 * 8), ("attr", ctypes.c_uint64 * 32)]


def _mask(ranks):
    m = 0
    for r in ranks:
        if r < RANK_CAP:
            m |= 1 << r
    return m


def _attrs(g, node, op, inshape, outshape):
    """The values graph_tape.c expects in attr[] for this opcode."""
    if op in ("REDUCE_SUM", "REDUCE_PROD", "REDUCE_MIN", "REDUCE_MAX", "REVERSE"):
        return [_mask(g.attr(node, "rank_set"))]
    if op == "ARGMAX":
        return [g.attr(node, "rank")[0]]
    if op == "EXTEND":
        return [outshape[d] // inshape[d] for d in range(RANK_CAP)]
    if op == "PERMUTE":
        order = [r for r in g.attr(node, "ranks")][:RANK_CAP]
        return order + [d for d in range(RANK_CAP) if d not in order]
    if op == "SLICE":
        pairs = g.attr(node, "dimension_pairs")
        offsets, extents = [0] * RANK_CAP, list(inshape)
        for d in range(min(len(pairs) // 2, RANK_CAP)):
            offsets[d] = min(pairs[2 * d], inshape[d] - 1)
            extents[d] = min(pairs[2 * d + 1], inshape[d] - offsets[d])
        return offsets + extents
    if op == "PAD":
        pairs = g.attr(node, "dimension_pairs")
        before, after = [0] * RANK_CAP, [0] * RANK_CAP
        for d in range(min(len(pairs) // 2, RANK_CAP)):
            before[d], after[d] = pairs[2 * d], pairs[2 * d + 1]
        return before + after
    if op in ("STRIDE", "SCATTER"):
        incr = list(g.attr(node, "dimensions"))[:RANK_CAP]
        return incr + [1] * (RANK_CAP - len(incr)) + list(outshape)
    if op == "CONCAT":
        return [g.attr(node, "rank")[0]]
    if op == "CONTRACT":
        return list(g.attr(node, "rank_pairs"))
    if op == "CONV":
        return list(g.attr(node, "ranks"))[:RANK_CAP]
    return []


class Tape:
    """The functors under `targets` as one list of steps over host buffers."""

    def __init__(self, g, targets):
        self.g = g
        order, seen = [], {}

        def visit(node):
            # iterative post-order: unrolled recurrent graphs are thousands of nodes deep
            stack = [(node, iter(g.args(node)))]
            while stack:
                cur, kids = stack[-1]
                if cur.id in seen:
                    stack.pop()
                    continue
                advanced = False
                for kid in kids:
                    if kid.id not in seen:
                        stack.append((kid, iter(g.args(kid))))
                        advanced = True
                        break
                if not advanced:
                    seen[cur.id] = len(order)
                    order.append(cur)
                    stack.pop()

        for t in targets:
            visit(t)
        self.index = seen
        self.nodes = order
        self.buffers, self.leaves = [], []
        ops, arg_ids, arg_shapes = [], [], []
        for node in order:
            shape = orc.shape8(node.shape)
            dtype = g.dtype(node)
            opname = g.opcode(node)
            if opname in (None, "BAD_OP"):
                self.leaves.append(node)
                self.buffers.append(np.array(g.data(node), dtype=_NP[dtype]).reshape(-1).copy())
                continue
            self.buffers.append(np.zeros(orc.n_elems(shape), _NP[dtype]))
            args = g.args(node)
            op = TapeOp()
            op.opcode = orc.OPCODES.index(opname)
            op.dtype = dtype
            op.nargs, op.first_arg, op.out = len(args), len(arg_ids), seen[node.id]
            op.n = orc.n_elems(shape)
            shapes = [orc.shape8(a.shape) for a in args]
            for k, a in enumerate(args):
                arg_ids.append(seen[a.id])
                arg_shapes.extend(shapes[k])
            for d in range(RANK_CAP):
                op.ashape[d] = shapes[0][d]
                op.bshape[d] = shapes[1][d] if len(shapes) > 1 else 1
            if opname == "CAST":
                op.in_dtype = g.dtype(args[0])
            vals = _attrs(g, node, opname, shapes[0], shape)
            assert len(vals) <= 32, opname
            op.nattr = len(vals)
            for i, v in enumerate(vals):
                op.attr[i] = int(v)
            ops.append(op)
        self.ops = (TapeOp * max(len(ops), 1))(*ops)
        self.nops = len(ops)
        self.arg_ids = (ctypes.c_int32 * max(len(arg_ids), 1))(*arg_ids)
        self.arg_shapes = (ctypes.c_uint64 * max(len(arg_shapes), 1))(*arg_shapes)
        self.ptrs = (ctypes.c_void_p * len(self.buffers))(*[b.ctypes.data for b in self.buffers])

    def set(self, node, values):
        """New content for a leaf (the step the benchmark recipe takes before each evaluate)."""
        buf = self.buffers[self.index[node.id]]
        buf[...] = np.asarray(values, buf.dtype).reshape(-1)

    def run(self, reps=1):
        """Evaluates every functor `reps` times; returns the seconds each pass took."""
        lib = orc.lib()
        lib.orc_tape_run.restype = ctypes.c_int
        lib.orc_tape_run.argtypes = [ctypes.POINTER(TapeOp), ctypes.c_int, ctypes.POINTER(ctypes.c_int32),
                                     ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_void_p), ctypes.c_int,
                                     ctypes.POINTER(ctypes.c_double)]
        secs = (ctypes.c_double * reps)()
        rc = lib.orc_tape_run(self.ops, self.nops, self.arg_ids, self.arg_shapes, self.ptrs, reps, secs)
        if rc != 0:
            step = rc - 1000
            raise RuntimeError("step %d of the tape failed (%s)" % (step, orc.OPCODES[self.ops[step].opcode] if step >= 0 else rc))
        return [secs[i] for i in range(reps)]

    def value(self, node):
        return self.buffers[self.index[node.id]]
