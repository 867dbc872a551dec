"""The convolution as a matrix product that reads the image out of a patch held in
LDS (tenncor_amd/csrc/conv_patch.hip): the forward pass and the image gradient of
a conv2d layer (cfg/tenncor/nn.yml:48-98, tenncor/eteq/backprop.hpp:360-401) in the
layouts the evaluator hands them over in, at sizes where that route is taken.

Checked against the direct kernels (which tests/test_gpu_ops.py ties to the
oracle) at 1e-4, and against the product that reads the image through its
tables (TCG_CONV_PATCH=0) -- the two products sum in different orders.  The
counter of the route says which one ran; shapes the route does not take (a
summed index that is no multiple of 32) must leave it alone.  Also here: the
one-launch route for a short summed index (the CNN's first layer) and the
route for few rows under a long summed index (that layer's kernel gradient).
"""
import os

import numpy as np
import pytest

from test_gpu_conv_views import idiom_layouts, lay_out, read_back, seed_of
from test_gpu_ops import ACC_RTOL, assert_acc_close, conv2d_idiom_cases

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from tenncor_amd import capi
    c = capi.Context(0)
    yield c
    c.close()


def run_views(ctx, oracle, which, dims, env):
    """One convolution of the conv2d idiom through tcg_conv_views; returns the logical result window."""
    from tenncor_amd import capi
    ishape, kshape, ranks, ibox, obox = conv2d_idiom_cases(**dims)[which]
    rng = np.random.default_rng(seed_of("convpatch", which, sorted(dims.items())))
    oshape = oracle.conv_shape(ishape, kshape, ranks)
    lo, hi = ibox
    boxshape = [hi[d] - lo[d] for d in range(8)]
    olo, ohi = obox if obox is not None else ([0] * 8, oshape)
    wshape = [ohi[d] - olo[d] for d in range(8)]
    kshape8 = oracle.shape8(kshape)
    (iperm, iflips), (kperm, kflips), (operm, oflips) = idiom_layouts(which)
    box = rng.uniform(-1, 1, oracle.n_elems(boxshape)).astype(np.float32)
    ker = rng.uniform(-1, 1, oracle.n_elems(kshape)).astype(np.float32)
    box_mem, box_stride, box_off = lay_out(box, boxshape, iperm, iflips)
    ker_mem, ker_stride, ker_off = lay_out(ker, kshape8, kperm, kflips)
    _, out_stride, out_off = lay_out(np.zeros(oracle.n_elems(wshape), np.float32), wshape, operm, oflips)
    dbox, dker = ctx.upload(box_mem), ctx.upload(ker_mem)
    guard = 64
    mem = ctx.upload(np.full(oracle.n_elems(wshape) + 2 * guard, 777, dtype=np.float32))
    os.environ.update(env)
    try:
        ctx.conv_views(capi.FLOAT, ishape, kshape, ranks, ibox, obox,
                       dbox.ptr + box_off * 4, box_stride, dker.ptr + ker_off * 4, ker_stride,
                       mem.ptr + (guard + out_off) * 4, out_stride)
        got_mem = mem.get()
    finally:
        for key in env:
            os.environ.pop(key, None)
    assert (got_mem[:guard] == 777).all() and (got_mem[-guard:] == 777).all()
    mem.release()
    return read_back(got_mem[guard:-guard], wshape, operm, oflips)


CASES = [
    # the second layer of the reference's CNN at a batch of 16: 6400 x 64 x 800 and 9216 x 32 x 1600
    ("forward", dict(C=32, W=24, H=24, B=16, O=64, KW=5, KH=5)),
    ("image_gradient", dict(C=32, W=24, H=24, B=16, O=64, KW=5, KH=5)),
    # rows that do not fill the last tile, images that are not square, a 3 x 4 window
    ("forward", dict(C=32, W=26, H=21, B=15, O=64, KW=5, KH=5)),
    ("image_gradient", dict(C=32, W=22, H=26, B=11, O=64, KW=5, KH=5)),
    ("forward", dict(C=64, W=19, H=17, B=24, O=128, KW=3, KH=4)),
    ("image_gradient", dict(C=64, W=19, H=17, B=36, O=32, KW=3, KH=4)),
    # a window one row high: only one dim of the image gradient meets a zero border
    ("image_gradient", dict(C=32, W=40, H=12, B=64, O=64, KW=5, KH=1)),
]


def test_a_patch_of_more_than_64_kib(ctx, oracle):
    """Ten rows of 26 pixels x 64 channels under a tile of 144 rows: 78 KiB of LDS, which a kernel has to ask for.
    (The tile is forced: left alone, this size takes the tile of 96 rows, which fills more CUs.)"""
    dims = dict(C=32, W=30, H=20, B=16, O=64, KW=5, KH=5)
    before = ctx.conv_route_counts()["patch"]
    got = run_views(ctx, oracle, "image_gradient", dims, {"TCG_CONV_PATCH_SHAPE": "0"})
    assert ctx.conv_route_counts()["patch"] == before + 1, "the route under test was not taken"
    assert_acc_close(got, run_views(ctx, oracle, "image_gradient", dims, {"TCG_CONV_GEMM": "0"}), ACC_RTOL)


@pytest.mark.parametrize("which,dims", CASES, ids=["%s-%s" % (w, "x".join(str(v) for v in d.values())) for w, d in CASES])
def test_product_over_a_patch_in_lds_equals_the_direct_kernels(ctx, oracle, which, dims):
    before = ctx.conv_route_counts()["patch"]
    got = run_views(ctx, oracle, which, dims, {})
    assert ctx.conv_route_counts()["patch"] == before + 1, "the route under test was not taken"
    tables = run_views(ctx, oracle, which, dims, {"TCG_CONV_PATCH": "0"})
    assert ctx.conv_route_counts()["patch"] == before + 1
    direct = run_views(ctx, oracle, which, dims, {"TCG_CONV_GEMM": "0"})
    assert_acc_close(got, direct, ACC_RTOL)
    assert_acc_close(got, tables, ACC_RTOL)
    # the same call again gives the same bits (fixed order of the partial sums)
    np.testing.assert_array_equal(run_views(ctx, oracle, which, dims, {}), got)


def test_shapes_the_route_does_not_take_leave_it_alone(ctx, oracle):
    before = ctx.conv_route_counts()["patch"]
    # 16 channels: the summed index (5 x 5 x 16 = 400) is no multiple of 32
    dims = dict(C=16, W=24, H=24, B=32, O=64, KW=5, KH=5)
    got = run_views(ctx, oracle, "forward", dims, {})
    assert ctx.conv_route_counts()["patch"] == before
    assert_acc_close(got, run_views(ctx, oracle, "forward", dims, {"TCG_CONV_GEMM": "0"}), ACC_RTOL)


@pytest.mark.parametrize("dims", [dict(C=1, W=28, H=28, B=32, O=32, KW=5, KH=5), dict(C=2, W=17, H=23, B=37, O=64, KW=4, KH=3),
                                  dict(C=1, W=20, H=20, B=50, O=16, KW=5, KH=5)],
                         ids=["cnn_first_layer", "two_channels_64_filters", "16_filters"])
def test_short_summed_index_in_one_launch_equals_the_direct_kernels(ctx, oracle, dims):
    """The first layer of the reference's CNN (one channel, a 5x5 window: 25 summed indices): gather, product and the
    layout of the kernel as one launch, against the direct kernels and against gather + product."""
    before = ctx.conv_route_counts()["short_sum"]
    got = run_views(ctx, oracle, "forward", dims, {})
    assert ctx.conv_route_counts()["short_sum"] == before + 1, "the route under test was not taken"
    two = run_views(ctx, oracle, "forward", dims, {"TCG_CONV_SHORT": "0"})
    assert ctx.conv_route_counts()["short_sum"] == before + 1
    direct = run_views(ctx, oracle, "forward", dims, {"TCG_CONV_GEMM": "0"})
    assert_acc_close(got, direct, ACC_RTOL)
    assert_acc_close(got, two, ACC_RTOL)
    np.testing.assert_array_equal(run_views(ctx, oracle, "forward", dims, {}), got)


@pytest.mark.parametrize("seed", range(10))
def test_seeded_layers_on_the_patch_route(ctx, oracle, seed):
    """Random conv2d layers whose forward pass or image gradient is large enough for the route: channel counts that make
    32, 64, 96 or 128 columns (one, two or three columns of tiles), windows of 1..5 x 1..5, images that are not square,
    batches that leave the last tile ragged."""
    rng = np.random.default_rng(seed_of("convpatch-random", seed))
    which = "forward" if seed % 2 == 0 else "image_gradient"
    KW, KH = int(rng.integers(1, 6)), int(rng.integers(1, 6))
    if KW * KH < 4:
        KW, KH = 3, 3
    W, H = int(rng.integers(KW + 8, 31)), int(rng.integers(KH + 8, 31))
    if which == "forward":
        C, O = 32 * int(rng.integers(1, 3)), 32 * int(rng.integers(1, 5))      # summed: KW KH C, columns: O
        rows_per_image, cols, sums = (W - KW + 1) * (H - KH + 1), O, KW * KH * C
    else:
        C, O = 32 * int(rng.integers(1, 5)), 32 * int(rng.integers(1, 3))      # summed: KW KH O, columns: C
        rows_per_image, cols, sums = W * H, C, KW * KH * O
    B = int(-(-(1 << 28) // (rows_per_image * cols * sums))) + int(rng.integers(0, 3))
    dims = dict(C=C, W=W, H=H, B=B, O=O, KW=KW, KH=KH)
    before = ctx.conv_route_counts()["patch"]
    got = run_views(ctx, oracle, which, dims, {})
    assert ctx.conv_route_counts()["patch"] == before + 1, "the route under test was not taken: %r" % (dims,)
    assert_acc_close(got, run_views(ctx, oracle, which, dims, {"TCG_CONV_GEMM": "0"}), ACC_RTOL)


@pytest.mark.parametrize("dims", [dict(C=1, W=28, H=28, B=32, O=32, KW=5, KH=5), dict(C=2, W=17, H=23, B=40, O=64, KW=4, KH=3),
                                  dict(C=1, W=20, H=21, B=90, O=16, KW=3, KH=3)],
                         ids=["cnn_first_layer", "two_channels_64_filters", "nine_rows_16_filters"])
def test_few_rows_under_a_long_summed_index_equal_the_direct_kernels(ctx, oracle, dims):
    """The kernel gradient of the reference's first CNN layer (25 x 32 results, each a sum over every pixel of the batch):
    A gathered while it is multiplied, stretches of the summed index added up by a second launch, against the direct
    kernels and against gather + product."""
    before = ctx.conv_route_counts()["few_rows"]
    got = run_views(ctx, oracle, "kernel_gradient", dims, {})
    assert ctx.conv_route_counts()["few_rows"] == before + 1, "the route under test was not taken"
    two = run_views(ctx, oracle, "kernel_gradient", dims, {"TCG_CONV_FEWROWS": "0"})
    assert ctx.conv_route_counts()["few_rows"] == before + 1
    direct = run_views(ctx, oracle, "kernel_gradient", dims, {"TCG_CONV_GEMM": "0"})
    assert_acc_close(got, direct, ACC_RTOL)
    assert_acc_close(got, two, ACC_RTOL)
    np.testing.assert_array_equal(run_views(ctx, oracle, "kernel_gradient", dims, {}), got)
