"""Operator functions over device tensors, named and parameterised like the
reference's ``eigen::`` operator factories (internal/eigen/operator.hpp) and
following the shape rules of cfg/ops.yml.  Each call is one launch through the
C ABI; nothing here computes on the host.
"""
import numpy as np

from . import capi

RANK_CAP = capi.RANK_CAP


class Tens:
    """A device tensor: buffer + tenncor shape (dim 0 fastest) + dtype code."""

    def __init__(self, ctx, buf, shape):
        self.ctx = ctx
        self.buf = buf
        self.shape = capi.shape8(shape)
        self.dtype = buf.dtype

    @property
    def ptr(self):
        return self.buf.ptr

    @property
    def n(self):
        return capi.n_elems(self.shape)

    def get(self):
        return self.buf.get()[:self.n]

    def release(self):
        self.buf.release()


def from_host(ctx, data, shape):
    data = np.ascontiguousarray(data).reshape(-1)
    assert data.size == capi.n_elems(shape), "data does not fill shape"
    return Tens(ctx, ctx.upload(data), shape)


def _new(ctx, shape, like):
    return Tens(ctx, ctx.empty(capi.n_elems(shape), like.buf.np_dtype), shape)


def _same_shape(op, args):
    for a in args[1:]:
        if a.shape != args[0].shape:
            # cfg/ops.yml:35-41
            raise ValueError("cannot %s with incompatible shapes %s and %s" % (op, a.shape, args[0].shape))


def unary(op, x):
    out = _new(x.ctx, x.shape, x)
    x.ctx.ew_unary(op, x.dtype, x.n, x.ptr, out.ptr)
    return out


def binary(op, a, b):
    _same_shape(op, [a, b])
    out = _new(a.ctx, a.shape, a)
    a.ctx.ew_binary(op, a.dtype, a.n, a.ptr, b.ptr, out.ptr)
    return out


def nary(op, args):
    """eigen::add / eigen::mul over a group (internal/eigen/operator.hpp:694-795)."""
    _same_shape(op, args)
    out = _new(args[0].ctx, args[0].shape, args[0])
    if len(args) == 2:
        args[0].ctx.ew_binary(op, out.dtype, out.n, args[0].ptr, args[1].ptr, out.ptr)
    else:
        args[0].ctx.ew_nary(op, out.dtype, out.n, [a.ptr for a in args], out.ptr)
    return out


def select(cond, then, otherwise):
    _same_shape("SELECT", [cond, then, otherwise])
    out = _new(then.ctx, then.shape, then)
    then.ctx.ew_select(then.dtype, then.n, cond.ptr, then.ptr, otherwise.ptr, out.ptr)
    return out


def cast(x, out_dtype):
    out = Tens(x.ctx, x.ctx.empty(x.n, capi.NP_OF[out_dtype]), x.shape)
    x.ctx.cast(out_dtype, x.dtype, x.n, x.ptr, out.ptr)
    return out


def assign(op, target, source):
    _same_shape(op, [target, source])
    target.ctx.assign(op, target.dtype, target.n, target.ptr, source.ptr)
    return target


def reduce(op, x, rank_set):
    """cfg/ops.yml:123-139: reduced dims become 1."""
    ranks = sorted(set(int(r) for r in rank_set))
    oshape = [1 if i in ranks else d for i, d in enumerate(x.shape)]
    out = _new(x.ctx, oshape, x)
    x.ctx.reduce(op, x.dtype, x.shape, ranks, x.ptr, out.ptr)
    return out


def argmax(x, return_dim):
    oshape = [1] * 8 if return_dim >= RANK_CAP else [1 if i == return_dim else d for i, d in enumerate(x.shape)]
    out = _new(x.ctx, oshape, x)
    x.ctx.argmax(x.dtype, x.shape, return_dim, x.ptr, out.ptr)
    return out


def extend(x, bcast):
    """cfg/ops.yml:256-283."""
    b = capi.shape8(bcast)
    if any(d == 0 for d in b):
        raise ValueError("cannot extend using zero dimensions %s" % b)
    for i in range(RANK_CAP):
        if b[i] > 1 and x.shape[i] > 1:
            raise ValueError("cannot extend non-singular dimension %d of shape %s: bcast=%s" % (i, x.shape, b))
    oshape = [d * f for d, f in zip(x.shape, b)]
    out = _new(x.ctx, oshape, x)
    x.ctx.extend(x.dtype, x.shape, b, x.ptr, out.ptr)
    return out


def full_order(order):
    """internal/eigen/operator.hpp:182-194; cfg/ops.yml:213-231."""
    order = [int(o) for o in order][:RANK_CAP]
    if len(set(order)) != len(order):
        raise ValueError("permute does not support repeated orders (order=%s)" % order)
    return order + [i for i in range(RANK_CAP) if i not in order]


def permute(x, order):
    o = full_order(order)
    oshape = [x.shape[i] for i in o]
    out = _new(x.ctx, oshape, x)
    x.ctx.permute(x.dtype, x.shape, o, x.ptr, out.ptr)
    return out


def slice_(x, pairs):
    """internal/eigen/operator.hpp:219-230 clamping; a real copy is always made
    here (the reference aliases the last-dim case, which a caller can do with a
    pointer offset)."""
    offs, exts = [0] * 8, list(x.shape)
    for i, (o, e) in enumerate(list(pairs)[:RANK_CAP]):
        if e == 0:
            raise ValueError("cannot create slice with 0 dimensions (second value of extents)")
        off = min(int(o), x.shape[i] - 1)
        offs[i] = off
        exts[i] = min(int(e), x.shape[i] - off)
    out = _new(x.ctx, exts, x)
    x.ctx.slice(x.dtype, x.shape, offs, exts, x.ptr, out.ptr)
    return out


def pad(x, pairs):
    before, after = [0] * 8, [0] * 8
    for i, (b, a) in enumerate(list(pairs)[:RANK_CAP]):
        before[i], after[i] = int(b), int(a)
    oshape = [d + b + a for d, b, a in zip(x.shape, before, after)]
    out = _new(x.ctx, oshape, x)
    x.ctx.pad(x.dtype, x.shape, before, after, x.ptr, out.ptr)
    return out


def reverse(x, rank_set):
    out = _new(x.ctx, x.shape, x)
    x.ctx.reverse(x.dtype, x.shape, rank_set, x.ptr, out.ptr)
    return out


def stride(x, incrs):
    inc = capi.shape8(incrs)
    oshape = list(x.shape)
    for i in range(min(len(incrs), RANK_CAP)):
        # cfg/ops.yml:433-437: std::round(dim / incr)
        oshape[i] = int(np.floor(x.shape[i] / inc[i] + 0.5))
    out = _new(x.ctx, oshape, x)
    x.ctx.stride(x.dtype, x.shape, inc, oshape, x.ptr, out.ptr)
    return out


def scatter(x, incrs, outshape):
    oshape = capi.shape8(outshape)
    out = _new(x.ctx, oshape, x)
    x.ctx.scatter(x.dtype, x.shape, capi.shape8(incrs), oshape, x.ptr, out.ptr)
    return out


def concat(args, axis):
    """cfg/ops.yml:613-653."""
    first = args[0].shape
    for a in args[1:]:
        if any(a.shape[d] != first[d] for d in range(RANK_CAP) if d != axis):
            raise ValueError("cannot group concat incompatible shapes %s and %s along axis %d" % (first, a.shape, axis))
    if len(args) > 2 and any(a.shape[axis] != 1 for a in args):
        raise ValueError("cannot group concat shapes with dimension that is not one")
    oshape = list(first)
    oshape[axis] = sum(a.shape[axis] for a in args)
    out = _new(args[0].ctx, oshape, args[0])
    args[0].ctx.concat(out.dtype, axis, [a.shape for a in args], [a.ptr for a in args], out.ptr)
    return out


def matmul(a, b):
    """cfg/ops.yml:496-514."""
    if a.shape[2:] != b.shape[2:]:
        raise ValueError("invalid shapes %s and %s do not match for dimensions 2+" % (a.shape, b.shape))
    if a.shape[0] != b.shape[1]:
        raise ValueError("invalid shapes %s and %s have mismatch common dimension 0,1" % (a.shape, b.shape))
    oshape = [b.shape[0], a.shape[1]] + a.shape[2:]
    out = _new(a.ctx, oshape, a)
    a.ctx.matmul(a.dtype, a.shape, b.shape, a.ptr, b.ptr, out.ptr)
    return out


def _narrow(shape):
    s = list(shape)
    while s and s[-1] == 1:
        s.pop()
    return s


def contract(a, b, pairs):
    """cfg/ops.yml:517-565: out = b's free dims then a's."""
    acom = {int(p[0]) for p in pairs}
    bcom = {int(p[1]) for p in pairs}
    outlist = [d for i, d in enumerate(_narrow(b.shape)) if i not in bcom]
    outlist += [d for i, d in enumerate(_narrow(a.shape)) if i not in acom]
    out = _new(a.ctx, capi.shape8(outlist), a)
    a.ctx.contract(a.dtype, a.shape, b.shape, pairs, a.ptr, b.ptr, out.ptr)
    return out


def convolution(img, kernel, ranks):
    """cfg/ops.yml:568-607."""
    r = [int(v) for v in ranks][:RANK_CAP]
    if any(d > 1 for d in kernel.shape[len(r):]):
        raise ValueError("cannot have ambiguous ranks not specified in kernelshape %s (ranks=%s)" % (kernel.shape, r))
    oshape = list(img.shape)
    for i, d in enumerate(r):
        if kernel.shape[i] > oshape[d]:
            raise ValueError("cannot convolve a kernel of shape %s against smaller image of shape %s" % (kernel.shape, img.shape))
        oshape[d] -= kernel.shape[i] - 1
    out = _new(img.ctx, oshape, img)
    img.ctx.conv(img.dtype, img.shape, kernel.shape, r, img.ptr, kernel.ptr, out.ptr)
    return out
