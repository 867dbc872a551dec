"""tcg_conv_views: the correlation of tcg_conv_dense_box over operands and a
result that lie in memory permuted and reversed, as the PERMUTE and REVERSE
nodes round tenncor's convolutions leave them (cfg/tenncor/nn.yml:88-93,
tenncor/eteq/backprop.hpp:372-439).  Checked against tcg_conv_dense_box with
the direct kernels on the materialised operands (which tests/test_gpu_ops.py
ties to the oracle): bit for bit in int32 by every route, 1e-4 / 1e-12 in
fp32 / fp64.  The layouts of conv2d and its two gradients are among the cases:
there the kernel or the result already is the matrix of the product and is
used in place.
"""
import os
import zlib

import numpy as np
import pytest

from test_gpu_ops import ACC_RTOL, assert_acc_close, conv2d_idiom_cases

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from tenncor_amd import capi
    c = capi.Context(0)
    yield c
    c.close()


def seed_of(*parts):
    return zlib.crc32(repr(parts).encode())


def lay_out(logical, shape, perm, flips):
    """Memory holding the tensor `logical` (flat, dim 0 fastest, extents `shape`)
    with memory dim j = logical dim perm[j], the dims in `flips` running
    backwards: (flat memory, element stride per logical dim, offset of element 0)."""
    lt = np.asarray(logical).reshape(shape[::-1]).transpose(range(7, -1, -1))  # lt[c0..c7]
    mt = lt.transpose(perm)
    stride = [0] * 8
    run = 1
    for j, d in enumerate(perm):
        stride[d] = run
        run *= shape[d]
    offset = 0
    for d in flips:
        mt = np.flip(mt, axis=perm.index(d))
        offset += (shape[d] - 1) * stride[d]
        stride[d] = -stride[d]
    return np.ascontiguousarray(mt.flatten(order="F")), stride, offset


def read_back(memory, shape, perm, flips):
    """Inverse of lay_out: the flat logical tensor (dim 0 fastest)."""
    mt = np.asarray(memory).reshape([shape[d] for d in perm], order="F")
    for d in flips:
        mt = np.flip(mt, axis=perm.index(d))
    inverse = [perm.index(d) for d in range(8)]
    return np.ascontiguousarray(mt.transpose(inverse).flatten(order="F"))


def identity():
    return list(range(8))


def idiom_layouts(which):
    """(image perm/flips, kernel perm/flips, result perm/flips) as conv2d and
    its gradients meet them: the upstream gradient {O,OW,OH,B} is read where
    PERMUTE would put it as {1,OW,OH,B,O}; the kernel {O,C,KW,KH} is read
    through REVERSE{0}; results {.,.,.,.,O} land as PERMUTE{4,1,2,3,0} wants them."""
    front = [4, 1, 2, 3, 0, 5, 6, 7]  # memory dim 0 = logical dim 4
    if which == "forward":
        return (identity(), []), (identity(), [0]), (front, [])
    if which == "image_gradient":
        return (front, []), (identity(), [1, 2, 3]), (identity(), [])
    # kernel gradient: the "kernel" is the upstream gradient; the result {C,KW,KH,1,O} becomes {O,C,KW,KH} reversed in O
    return (identity(), []), (front, []), ([4, 0, 1, 2, 3, 5, 6, 7], [4])


def scrambled_layouts(rng):
    def one():
        perm = [int(v) for v in rng.permutation(5)] + [5, 6, 7]
        flips = [d for d in range(5) if rng.uniform() < 0.4]
        return perm, flips
    return one(), one(), one()


@pytest.mark.parametrize("layout", ["idiom", "scrambled"])
@pytest.mark.parametrize("which", ["forward", "image_gradient", "kernel_gradient"])
def test_conv_over_permuted_and_reversed_operands(ctx, oracle, which, layout):
    from tenncor_amd import capi
    # channel counts that are multiples of four let the fp32 product read the image in place too
    ishape, kshape, ranks, ibox, obox = conv2d_idiom_cases(C=12, W=15, H=13, B=12, O=24, KW=3, KH=4)[which]
    rng = np.random.default_rng(seed_of("convviews", which, layout))
    oshape = oracle.conv_shape(ishape, kshape, ranks)
    lo, hi = ibox
    boxshape = [hi[d] - lo[d] for d in range(8)]
    olo, ohi = obox if obox is not None else ([0] * 8, oshape)
    wshape = [ohi[d] - olo[d] for d in range(8)]
    kshape8 = oracle.shape8(kshape)
    (iperm, iflips), (kperm, kflips), (operm, oflips) = idiom_layouts(which) if layout == "idiom" else scrambled_layouts(rng)
    for np_dtype in (np.int32, np.float32, np.float64):
        if np_dtype == np.int32:
            box = rng.integers(-40, 41, oracle.n_elems(boxshape)).astype(np.int32)
            ker = rng.integers(-40, 41, oracle.n_elems(kshape)).astype(np.int32)
        else:
            box = rng.uniform(-1, 1, oracle.n_elems(boxshape)).astype(np_dtype)
            ker = rng.uniform(-1, 1, oracle.n_elems(kshape)).astype(np_dtype)
        dt = capi.dtype_code(np_dtype)
        esz = np.dtype(np_dtype).itemsize
        # the reference: dense operands, direct kernels, the whole result tensor; its window cut out on the host
        os.environ["TCG_CONV_GEMM"] = "0"
        try:
            full = ctx.upload(np.full(oracle.n_elems(oshape), 777, dtype=np_dtype))
            dbox, dker = ctx.upload(box), ctx.upload(ker)
            ctx.conv_dense_box(dt, ishape, kshape, ranks, ibox, obox, dbox.ptr, dker.ptr, full.ptr)
            ref, _ = oracle.slice_(full.get(), oshape, [[olo[d], wshape[d]] for d in range(8)])
        finally:
            os.environ.pop("TCG_CONV_GEMM", None)
        box_mem, box_stride, box_off = lay_out(box, boxshape, iperm, iflips)
        ker_mem, ker_stride, ker_off = lay_out(ker, kshape8, kperm, kflips)
        _, out_stride, out_off = lay_out(np.zeros(oracle.n_elems(wshape), np_dtype), wshape, operm, oflips)
        dbox, dker = ctx.upload(box_mem), ctx.upload(ker_mem)
        routes = (("direct", {"TCG_CONV_GEMM": "0"}), ("product", {}), ("product_copies", {"TCG_CONV_IN_PLACE": "0"}),
                  ("product_materialised_chunks", {"TCG_CONV_IMPLICIT": "0", "TCG_CONV_CHUNK_ROWS": "128"}))
        for route, env in routes:
            os.environ.update(env)
            try:
                # a guard band either side shows writes that leave the window
                guard = 64
                mem = ctx.upload(np.full(oracle.n_elems(wshape) + 2 * guard, 777, dtype=np_dtype))
                ctx.conv_views(dt, ishape, kshape, ranks, ibox, obox,
                               dbox.ptr + box_off * esz, box_stride, dker.ptr + ker_off * esz, ker_stride,
                               mem.ptr + (guard + out_off) * esz, out_stride)
                got_mem = mem.get()
            finally:
                for key in env:
                    os.environ.pop(key, None)
            assert (got_mem[:guard] == 777).all() and (got_mem[-guard:] == 777).all(), route
            got = read_back(got_mem[guard:-guard], wshape, operm, oflips)
            if np_dtype == np.int32:
                np.testing.assert_array_equal(got, ref, err_msg=route)
            else:
                assert_acc_close(got, ref, ACC_RTOL if np_dtype == np.float32 else 1e-12)
            mem.release()


def test_conv_views_refuses_missing_strides(ctx):
    from tenncor_amd import capi
    a = ctx.upload(np.zeros(64, np.float32))
    lib = ctx.lib
    shape = (capi.ctypes.c_uint64 * 8)(4, 4, 1, 1, 1, 1, 1, 1)
    kshape = (capi.ctypes.c_uint64 * 8)(2, 2, 1, 1, 1, 1, 1, 1)
    ranks = (capi.ctypes.c_uint64 * 2)(0, 1)
    rc = lib.tcg_conv_views(ctx.handle, capi.FLOAT, shape, kshape, 2, ranks, None, None, None, None,
                            a.ptr, None, a.ptr, None, a.ptr, None)
    assert rc != 0 and b"stride" in lib.tcg_last_error(ctx.handle)
