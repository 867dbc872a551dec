"""ctypes front end of the CPU oracle (``liboracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``; the shipped package never
imports it.

Tensors are flat numpy arrays plus a tenncor shape: a list of up to 8 dims in
which dim 0 is the fastest-varying one (internal/teq/shape.hpp:56-59), i.e. the
reverse of the numpy shape of the same memory (tenncor/pyutils/convert.hpp:17-27).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

RANK_CAP = 8
DOUBLE, FLOAT, INT32 = 1, 2, 3
# the integer widths the full build adds (cfg/fulltype.yml:11-34)
INT8, UINT8, INT16, UINT16, UINT32, INT64, UINT64 = 4, 5, 6, 7, 8, 9, 10
NP_OF = {DOUBLE: np.float64, FLOAT: np.float32, INT32: np.int32,
         INT8: np.int8, UINT8: np.uint8, INT16: np.int16, UINT16: np.uint16,
         UINT32: np.uint32, INT64: np.int64, UINT64: np.uint64}
_CODE_OF = {np.dtype(t): code for code, t in NP_OF.items()}

# cfg/ops.yml key order (tools/egen/plugins/opcodes.py:16-22)
OPCODES = [
    "BAD_OP", "IDENTITY", "ABS", "NEG", "SIN", "COS", "TAN", "EXP", "LOG", "SQRT", "ROUND",
    "SIGMOID", "TANH", "SQUARE", "CUBE", "RAND_UNIF", "REVERSE", "REDUCE_SUM", "REDUCE_PROD",
    "REDUCE_MIN", "REDUCE_MAX", "ARGMAX", "PERMUTE", "EXTEND", "RESHAPE", "SLICE", "PAD",
    "STRIDE", "SCATTER", "POW", "ADD", "SUB", "MUL", "DIV", "MIN", "MAX", "EQ", "NEQ", "LT",
    "GT", "MATMUL", "CONTRACT", "CONV", "SELECT", "CONCAT", "ASSIGN", "ASSIGN_ADD",
    "ASSIGN_SUB", "ASSIGN_MUL", "ASSIGN_DIV", "CAST",
]
OP = {name: i for i, name in enumerate(OPCODES)}


def build(force=False):
    """Compile liboracle.so with the Makefile next to this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def dtype_code(arr):
    t = np.asarray(arr).dtype
    if t not in _CODE_OF:
        raise TypeError("unsupported dtype %s" % t)
    return _CODE_OF[t]


def shape8(shape, fill=1):
    s = list(shape) + [fill] * (RANK_CAP - len(shape))
    return s[:RANK_CAP]


def n_elems(shape):
    n = 1
    for d in shape8(shape):
        n *= d
    return n


def _u64(vals):
    return (ctypes.c_uint64 * len(vals))(*[int(v) for v in vals])


def _p(arr):
    return arr.ctypes.data_as(ctypes.c_void_p)


def _flat(arr):
    return np.ascontiguousarray(arr).reshape(-1)


def _check(rc, what):
    if rc != 0:
        raise ValueError("oracle rejected %s (rc=%d)" % (what, rc))


def _opcode(op):
    return OP[op] if isinstance(op, str) else int(op)


def unary(op, x):
    x = _flat(x)
    out = np.empty_like(x)
    _check(lib().orc_unary(_opcode(op), dtype_code(x), ctypes.c_uint64(x.size), _p(x), _p(out)), op)
    return out


def binary(op, a, b):
    a, b = _flat(a), _flat(b)
    assert a.dtype == b.dtype and a.size == b.size
    out = np.empty_like(a)
    _check(lib().orc_binary(_opcode(op), dtype_code(a), ctypes.c_uint64(a.size), _p(a), _p(b), _p(out)), op)
    return out


def nary(op, args):
    args = [_flat(a) for a in args]
    out = np.empty_like(args[0])
    ptrs = (ctypes.c_void_p * len(args))(*[a.ctypes.data for a in args])
    _check(lib().orc_nary(_opcode(op), dtype_code(args[0]), ctypes.c_uint64(out.size), len(args), ptrs, _p(out)), op)
    return out


def select(cond, then, otherwise):
    c, a, b = _flat(cond), _flat(then), _flat(otherwise)
    out = np.empty_like(a)
    _check(lib().orc_select(dtype_code(a), ctypes.c_uint64(a.size), _p(c), _p(a), _p(b), _p(out)), "SELECT")
    return out


def cast(x, out_dtype):
    x = _flat(x)
    out = np.empty(x.size, dtype=NP_OF[out_dtype])
    _check(lib().orc_cast(out_dtype, dtype_code(x), ctypes.c_uint64(x.size), _p(x), _p(out)), "CAST")
    return out


def assign(op, target, source):
    """In place on ``target`` (a flat contiguous array); returns it."""
    s = _flat(source)
    assert target.flags["C_CONTIGUOUS"] and target.dtype == s.dtype
    _check(lib().orc_assign(_opcode(op), dtype_code(s), ctypes.c_uint64(s.size), _p(target), _p(s)), op)
    return target


def _mask(ranks):
    m = 0
    for r in ranks:
        m |= 1 << int(r)
    return m


def reduce(op, x, shape, rank_set, wide_acc=False):
    x = _flat(x)
    s = shape8(shape)
    oshape = [1 if i in set(rank_set) else d for i, d in enumerate(s)]
    out = np.empty(n_elems(oshape), dtype=x.dtype)
    _check(lib().orc_reduce(_opcode(op), dtype_code(x), _u64(s), _mask(rank_set), int(wide_acc),
                            _p(x), _p(out)), op)
    return out, oshape


def argmax(x, shape, return_dim):
    x = _flat(x)
    s = shape8(shape)
    oshape = [1] * 8 if return_dim >= 8 else [1 if i == return_dim else d for i, d in enumerate(s)]
    out = np.empty(n_elems(oshape), dtype=x.dtype)
    _check(lib().orc_argmax(dtype_code(x), _u64(s), int(return_dim), _p(x), _p(out)), "ARGMAX")
    return out, oshape


def extend(x, shape, bcast):
    x = _flat(x)
    s, b = shape8(shape), shape8(bcast)
    oshape = [d * f for d, f in zip(s, b)]
    out = np.empty(n_elems(oshape), dtype=x.dtype)
    _check(lib().orc_extend(dtype_code(x), _u64(s), _u64(b), _p(x), _p(out)), "EXTEND")
    return out, oshape


def full_order(order):
    """internal/eigen/operator.hpp:182-194: append the unvisited dims ascending."""
    order = [int(o) for o in order][:RANK_CAP]
    return order + [i for i in range(RANK_CAP) if i not in order]


def permute(x, shape, order):
    x = _flat(x)
    s, o = shape8(shape), full_order(order)
    oshape = [s[i] for i in o]
    out = np.empty(x.size, dtype=x.dtype)
    _check(lib().orc_permute(dtype_code(x), _u64(s), _u64(o), _p(x), _p(out)), "PERMUTE")
    return out, oshape


def slice_clamp(shape, pairs):
    """internal/eigen/operator.hpp:219-230: clamp (offset, extent) pairs."""
    s = shape8(shape)
    offs, exts = [0] * 8, list(s)
    for i, (o, e) in enumerate(pairs[:RANK_CAP]):
        off = min(int(o), s[i] - 1)
        offs[i] = off
        exts[i] = min(int(e), s[i] - off)
    return offs, exts


def slice_(x, shape, pairs):
    x = _flat(x)
    s = shape8(shape)
    offs, exts = slice_clamp(s, pairs)
    out = np.empty(n_elems(exts), dtype=x.dtype)
    _check(lib().orc_slice(dtype_code(x), _u64(s), _u64(offs), _u64(exts), _p(x), _p(out)), "SLICE")
    return out, exts


def pad(x, shape, pairs):
    x = _flat(x)
    s = shape8(shape)
    before = [0] * 8
    after = [0] * 8
    for i, (b, a) in enumerate(pairs[:RANK_CAP]):
        before[i], after[i] = int(b), int(a)
    oshape = [d + b + a for d, b, a in zip(s, before, after)]
    out = np.empty(n_elems(oshape), dtype=x.dtype)
    _check(lib().orc_pad(dtype_code(x), _u64(s), _u64(before), _u64(after), _p(x), _p(out)), "PAD")
    return out, oshape


def reverse(x, shape, rank_set):
    x = _flat(x)
    s = shape8(shape)
    out = np.empty(x.size, dtype=x.dtype)
    _check(lib().orc_reverse(dtype_code(x), _u64(s), _mask(rank_set), _p(x), _p(out)), "REVERSE")
    return out, s


def stride(x, shape, incrs):
    x = _flat(x)
    s, inc = shape8(shape), shape8(incrs)
    # cfg/ops.yml:433-437: std::round(dim / incr), half away from zero
    oshape = list(s)
    for i in range(min(len(incrs), RANK_CAP)):
        oshape[i] = int(np.floor(s[i] / inc[i] + 0.5))
    out = np.empty(n_elems(oshape), dtype=x.dtype)
    _check(lib().orc_stride(dtype_code(x), _u64(s), _u64(inc), _u64(oshape), _p(x), _p(out)), "STRIDE")
    return out, oshape


def scatter(x, shape, incrs, outshape):
    x = _flat(x)
    s, inc, oshape = shape8(shape), shape8(incrs), shape8(outshape)
    out = np.empty(n_elems(oshape), dtype=x.dtype)
    _check(lib().orc_scatter(dtype_code(x), _u64(s), _u64(inc), _u64(oshape), _p(x), _p(out)), "SCATTER")
    return out, oshape


def concat(xs, shapes, axis):
    xs = [_flat(x) for x in xs]
    shapes = [shape8(s) for s in shapes]
    oshape = list(shapes[0])
    oshape[axis] = sum(s[axis] for s in shapes)
    out = np.empty(n_elems(oshape), dtype=xs[0].dtype)
    flat_shapes = [d for s in shapes for d in s]
    ptrs = (ctypes.c_void_p * len(xs))(*[x.ctypes.data for x in xs])
    _check(lib().orc_concat(dtype_code(xs[0]), int(axis), len(xs), _u64(flat_shapes), ptrs, _p(out)), "CONCAT")
    return out, oshape


def matmul(a, ashape, b, bshape, wide_acc=False):
    a, b = _flat(a), _flat(b)
    sa, sb = shape8(ashape), shape8(bshape)
    oshape = [sb[0], sa[1]] + sa[2:]
    out = np.empty(n_elems(oshape), dtype=a.dtype)
    _check(lib().orc_matmul(dtype_code(a), _u64(sa), _u64(sb), int(wide_acc), _p(a), _p(b), _p(out)), "MATMUL")
    return out, oshape


def contract_shape(ashape, bshape, pairs):
    """cfg/ops.yml:547-565: b's free dims (of its narrowed shape) then a's."""
    sa, sb = shape8(ashape), shape8(bshape)

    def narrow(s):
        s = list(s)
        while len(s) > 0 and s[-1] == 1:
            s.pop()
        return s

    acom = {int(p[0]) for p in pairs}
    bcom = {int(p[1]) for p in pairs}
    outlist = [d for i, d in enumerate(narrow(sb)) if i not in bcom]
    outlist += [d for i, d in enumerate(narrow(sa)) if i not in acom]
    return shape8(outlist)


def contract(a, ashape, b, bshape, pairs, wide_acc=False):
    a, b = _flat(a), _flat(b)
    sa, sb = shape8(ashape), shape8(bshape)
    oshape = contract_shape(sa, sb, pairs)
    out = np.empty(n_elems(oshape), dtype=a.dtype)
    flat_pairs = [int(v) for p in pairs for v in p]
    _check(lib().orc_contract(dtype_code(a), _u64(sa), _u64(sb), len(pairs), _u64(flat_pairs),
                              int(wide_acc), _p(a), _p(b), _p(out)), "CONTRACT")
    return out, oshape


def conv_shape(imgshape, kshape, ranks):
    """cfg/ops.yml:584-607."""
    si, sk = shape8(imgshape), shape8(kshape)
    oshape = list(si)
    for i, r in enumerate(list(ranks)[:RANK_CAP]):
        oshape[int(r)] -= sk[i] - 1
    return oshape


def conv(img, imgshape, kernel, kshape, ranks, wide_acc=False):
    img, kernel = _flat(img), _flat(kernel)
    si, sk = shape8(imgshape), shape8(kshape)
    oshape = conv_shape(si, sk, ranks)
    out = np.empty(n_elems(oshape), dtype=img.dtype)
    r = [int(v) for v in ranks][:RANK_CAP]
    _check(lib().orc_conv(dtype_code(img), _u64(si), _u64(sk), len(r), _u64(r if r else [0]), int(wide_acc),
                          _p(img), _p(kernel), _p(out)), "CONV")
    return out, oshape


def philox4x32_10(counter, key):
    """Philox4x32-10 of four counter words under two key words."""
    c = (ctypes.c_uint32 * 4)(*[int(v) for v in counter])
    k = (ctypes.c_uint32 * 2)(*[int(v) for v in key])
    out = (ctypes.c_uint32 * 4)()
    lib().orc_philox4x32_10(c, k, out)
    return [int(v) for v in out]


def rand_uniform(lo, hi, seed, first_block=0):
    """The device RAND_UNIF stream for bounds `lo`, `hi` (same dtype)."""
    lo, hi = _flat(lo), _flat(hi)
    assert lo.dtype == hi.dtype and lo.size == hi.size
    out = np.empty(lo.size, dtype=lo.dtype)
    _check(lib().orc_rand_uniform(dtype_code(lo), ctypes.c_uint64(lo.size), ctypes.c_uint64(seed),
                                  ctypes.c_uint64(first_block), _p(lo), _p(hi), _p(out)), "RAND_UNIF")
    return out
