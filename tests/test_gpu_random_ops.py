"""Seeded random shapes and attributes for every operator family, each launch
through the C ABI held against the CPU oracle on the same inputs.  The fixed
cases of tests/test_gpu_ops.py pin the shapes the reference's tests use and the
full sizes; the sweeps here look for what a fixed list misses: odd extents
beside aligned ones (the kernels choose 128-bit or scalar lanes, tiled or
strided copies, one pass or several by shape and alignment), singleton dims in
the middle, rank sets and orders of every kind.  int32 and data movement: bit
for bit.  fp32 sums and products: 1e-4 of the oracle's double accumulation
(the bar of every fp32 reduction and contraction in this suite); fp64: 1e-12.
"""
import zlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

DTYPES = [np.float32, np.int32, np.float64]


@pytest.fixture(scope="module")
def ctx():
    from tenncor_amd import capi
    c = capi.Context(0)
    yield c
    c.close()


def seed_of(*parts):
    return zlib.crc32(repr(parts).encode())


def random_shape(rng, max_elems=6000, rank=None):
    """1..5 significant dims, odd and aligned extents mixed, sometimes a singleton in between."""
    rank = int(rng.integers(1, 6)) if rank is None else rank
    pool = [1, 2, 3, 4, 5, 7, 8, 12, 16, 17, 31, 32, 33, 64]
    while True:
        shape = [int(rng.choice(pool)) for _ in range(rank)]
        if int(np.prod(shape)) <= max_elems:
            return shape


def draw(rng, n, np_dtype, lo=-9, hi=9):
    if np_dtype == np.int32:
        return rng.integers(lo, hi + 1, n).astype(np.int32)
    return rng.uniform(lo, hi, n).astype(np_dtype)


def close(got, ref, np_dtype, exact=False):
    if np_dtype == np.int32 or exact:
        np.testing.assert_array_equal(got, ref)
    else:
        ref = np.asarray(ref, np.float64)
        bar = (1e-4 if np_dtype == np.float32 else 1e-12) * max(float(np.abs(ref).max()), 1e-30)
        assert float(np.abs(np.asarray(got, np.float64) - ref).max()) <= bar


@pytest.mark.parametrize("np_dtype", DTYPES, ids=lambda t: np.dtype(t).name)
def test_reductions_over_random_rank_sets(ctx, oracle, np_dtype):
    from tenncor_amd import ops
    rng = np.random.default_rng(seed_of("reduce", np.dtype(np_dtype).name))
    for case in range(60):
        shape = random_shape(rng)
        rank = len(shape)
        ranks = sorted(set(int(r) for r in rng.integers(0, rank, int(rng.integers(1, rank + 1)))))
        op = str(rng.choice(["REDUCE_SUM", "REDUCE_PROD", "REDUCE_MIN", "REDUCE_MAX"]))
        x = draw(rng, int(np.prod(shape)), np_dtype, -2, 2) if op == "REDUCE_PROD" else draw(rng, int(np.prod(shape)), np_dtype)
        if op == "REDUCE_PROD" and np_dtype != np.int32:
            x = (np.sign(x) * (0.8 + 0.4 * np.abs(x) / 2)).astype(np_dtype)   # products stay in range
        t = ops.from_host(ctx, x, shape)
        got = ops.reduce(op, t, ranks).get()
        ref, _ = oracle.reduce(op, x, shape, ranks, wide_acc=np_dtype == np.float32)
        close(got, ref, np_dtype, exact=op in ("REDUCE_MIN", "REDUCE_MAX"))
        t.release()
    for case in range(20):
        shape = random_shape(rng, rank=int(rng.integers(1, 4)))
        x = rng.permutation(int(np.prod(shape))).astype(np_dtype)     # no ties: one largest per slice
        dim = int(rng.integers(0, len(shape) + 1))
        dim = 8 if dim == len(shape) else dim                         # 8: over the whole tensor
        t = ops.from_host(ctx, x, shape)
        np.testing.assert_array_equal(ops.argmax(t, dim).get(), oracle.argmax(x, shape, dim)[0])
        t.release()


@pytest.mark.parametrize("np_dtype", DTYPES, ids=lambda t: np.dtype(t).name)
def test_data_movement_with_random_attributes(ctx, oracle, np_dtype):
    from tenncor_amd import ops
    rng = np.random.default_rng(seed_of("move", np.dtype(np_dtype).name))
    for case in range(80):
        shape = random_shape(rng)
        rank = len(shape)
        n = int(np.prod(shape))
        x = draw(rng, n, np_dtype)
        t = ops.from_host(ctx, x, shape)
        kind = case % 8
        if kind == 0:
            order = [int(v) for v in rng.permutation(rank)]
            got, ref = ops.permute(t, order).get(), oracle.permute(x, shape, order)[0]
        elif kind == 1:
            pairs = []
            for d in shape:
                off = int(rng.integers(0, d))
                pairs.append([off, int(rng.integers(1, d - off + 1))])
            got, ref = ops.slice_(t, pairs).get(), oracle.slice_(x, shape, pairs)[0]
        elif kind == 2:
            pairs = [[int(rng.integers(0, 4)), int(rng.integers(0, 4))] for _ in shape]
            got, ref = ops.pad(t, pairs).get(), oracle.pad(x, shape, pairs)[0]
        elif kind == 3:
            ranks = sorted(set(int(r) for r in rng.integers(0, rank, rank)))
            got, ref = ops.reverse(t, ranks).get(), oracle.reverse(x, shape, ranks)[0]
        elif kind == 4:
            # EXTEND multiplies singleton dims only: a shape with some dims set to one
            src_shape = [d if rng.uniform() < 0.5 else 1 for d in shape]
            bcast = [1 if s > 1 else int(rng.integers(1, 6)) for s in src_shape] + [int(rng.integers(1, 4))]
            xs = draw(rng, int(np.prod(src_shape)), np_dtype)
            ts = ops.from_host(ctx, xs, src_shape)
            got, ref = ops.extend(ts, bcast).get(), oracle.extend(xs, src_shape, bcast)[0]
            ts.release()
        elif kind == 5:
            # (extent / step rounds to at least one: a step above twice the extent would leave nothing)
            incrs = [int(rng.integers(1, min(3, d) + 1)) for d in shape]
            got, ref = ops.stride(t, incrs).get(), oracle.stride(x, shape, incrs)[0]
        elif kind == 6:
            incrs = [int(rng.integers(1, 4)) for _ in shape]
            outshape = [(d - 1) * i + 1 + int(rng.integers(0, i)) for d, i in zip(shape, incrs)]
            got, ref = ops.scatter(t, incrs, outshape).get(), oracle.scatter(x, shape, incrs, outshape)[0]
        else:
            axis = int(rng.integers(0, rank))
            other = list(shape)
            other[axis] = int(rng.choice([1, 3, 8, 17]))
            y = draw(rng, int(np.prod(other)), np_dtype)
            ty = ops.from_host(ctx, y, other)
            got, ref = ops.concat([t, ty], axis).get(), oracle.concat([x, y], [shape, other], axis)[0]
            ty.release()
        np.testing.assert_array_equal(got, ref, err_msg="case %d kind %d shape %s" % (case, kind, shape))
        t.release()


@pytest.mark.parametrize("np_dtype", DTYPES, ids=lambda t: np.dtype(t).name)
def test_products_with_random_shapes_and_pairs(ctx, oracle, np_dtype):
    from tenncor_amd import ops
    rng = np.random.default_rng(seed_of("products", np.dtype(np_dtype).name))
    extents = [1, 2, 3, 4, 5, 8, 12, 16, 20, 33, 48, 64]
    for case in range(40):
        m, k, n = (int(rng.choice(extents)) for _ in range(3))
        batch = [int(rng.choice([1, 2, 3]))] if rng.uniform() < 0.4 else []
        ashape, bshape = [k, m] + batch, [n, k] + batch
        a, b = draw(rng, int(np.prod(ashape)), np_dtype, -3, 3), draw(rng, int(np.prod(bshape)), np_dtype, -3, 3)
        ta, tb = ops.from_host(ctx, a, ashape), ops.from_host(ctx, b, bshape)
        close(ops.matmul(ta, tb).get(), oracle.matmul(a, ashape, b, bshape, wide_acc=np_dtype == np.float32)[0], np_dtype)
        ta.release()
        tb.release()
    for case in range(40):
        # operands of rank 2..4 sharing one or two contracted extents at random positions
        npairs = int(rng.integers(1, 3))
        shared = [int(rng.choice([2, 3, 4, 8, 16, 17])) for _ in range(npairs)]
        afree = [int(rng.choice([1, 2, 3, 5, 8, 16, 33])) for _ in range(int(rng.integers(1, 3)))]
        bfree = [int(rng.choice([1, 2, 3, 5, 8, 16, 33])) for _ in range(int(rng.integers(1, 3)))]
        adims = [("s", i) for i in range(npairs)] + [("f", e) for e in afree]
        bdims = [("s", i) for i in range(npairs)] + [("f", e) for e in bfree]
        adims = [adims[i] for i in rng.permutation(len(adims))]
        bdims = [bdims[i] for i in rng.permutation(len(bdims))]
        # a trailing extent of one would be narrowed away (cfg/ops.yml:547-565): keep the last dim above one
        ashape = [shared[v] if kind == "s" else v for kind, v in adims]
        bshape = [shared[v] if kind == "s" else v for kind, v in bdims]
        if ashape[-1] == 1 or bshape[-1] == 1:
            continue
        pairs = []
        for i in range(npairs):
            pairs.append((adims.index(("s", i)), bdims.index(("s", i))))
        a, b = draw(rng, int(np.prod(ashape)), np_dtype, -3, 3), draw(rng, int(np.prod(bshape)), np_dtype, -3, 3)
        ta, tb = ops.from_host(ctx, a, ashape), ops.from_host(ctx, b, bshape)
        got = ops.contract(ta, tb, pairs).get()
        ref, _ = oracle.contract(a, ashape, b, bshape, pairs, wide_acc=np_dtype == np.float32)
        close(got, ref, np_dtype)
        ta.release()
        tb.release()


@pytest.mark.parametrize("np_dtype", DTYPES, ids=lambda t: np.dtype(t).name)
def test_convolutions_with_random_ranks(ctx, oracle, np_dtype):
    from tenncor_amd import ops
    rng = np.random.default_rng(seed_of("conv", np.dtype(np_dtype).name))
    for case in range(40):
        rank = int(rng.integers(1, 5))
        shape = [int(rng.choice([1, 2, 3, 5, 8, 9, 16])) for _ in range(rank)]
        nk = int(rng.integers(1, rank + 1))
        ranks = [int(v) for v in rng.permutation(rank)[:nk]]
        kshape = [int(rng.integers(1, shape[r] + 1)) for r in ranks]
        x, k = draw(rng, int(np.prod(shape)), np_dtype, -3, 3), draw(rng, int(np.prod(kshape)), np_dtype, -3, 3)
        tx, tk = ops.from_host(ctx, x, shape), ops.from_host(ctx, k, kshape)
        got = ops.convolution(tx, tk, ranks).get()
        ref, _ = oracle.conv(x, shape, k, kshape, ranks, wide_acc=np_dtype == np.float32)
        close(got, ref, np_dtype)
        tx.release()
        tk.release()


@pytest.mark.parametrize("np_dtype", DTYPES, ids=lambda t: np.dtype(t).name)
def test_elementwise_at_random_lengths_and_alignments(ctx, oracle, np_dtype):
    """Lengths around the lane and unroll boundaries, operands that start off
    a 16-byte boundary (a SLICE alias of the last dim does)."""
    from tenncor_amd import capi
    rng = np.random.default_rng(seed_of("ew", np.dtype(np_dtype).name))
    dt = capi.dtype_code(np_dtype)
    esz = np.dtype(np_dtype).itemsize
    unary = ["NEG", "ABS", "SQUARE", "CUBE"] + ([] if np_dtype == np.int32 else ["TANH", "SIGMOID", "EXP", "SIN"])
    binary = ["ADD", "SUB", "MUL", "MIN", "MAX", "LT", "GT", "EQ", "NEQ"]
    for case in range(60):
        n = int(rng.choice([1, 3, 4, 5, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 4099, 70001]))
        shift_a, shift_b, shift_o = (int(v) for v in rng.integers(0, 4, 3))
        a, b = draw(rng, n + 8, np_dtype, -2, 2), draw(rng, n + 8, np_dtype, -2, 2)
        da, db = ctx.upload(a), ctx.upload(b)
        out = ctx.upload(np.full(n + 8, 77, np_dtype))
        if case % 2:
            op = str(rng.choice(unary))
            ctx.ew_unary(op, dt, n, da.ptr + shift_a * esz, out.ptr + shift_o * esz)
            ref = oracle.unary(op, a[shift_a:shift_a + n])
        else:
            op = str(rng.choice(binary))
            ctx.ew_binary(op, dt, n, da.ptr + shift_a * esz, db.ptr + shift_b * esz, out.ptr + shift_o * esz)
            ref = oracle.binary(op, a[shift_a:shift_a + n], b[shift_b:shift_b + n])
        got = out.get()
        assert (got[:shift_o] == 77).all() and (got[shift_o + n:] == 77).all(), (op, n)
        res = got[shift_o:shift_o + n]
        if np_dtype == np.int32 or op not in ("TANH", "SIGMOID", "EXP", "SIN"):
            np.testing.assert_array_equal(res, ref, err_msg="%s n=%d" % (op, n))
        else:
            np.testing.assert_allclose(res, ref, rtol=2e-6 if np_dtype == np.float32 else 1e-14, atol=1e-30)
        for buf in (da, db, out):
            buf.release()


@pytest.mark.parametrize("np_dtype", DTYPES, ids=lambda t: np.dtype(t).name)
def test_medium_sizes_reach_the_tiled_kernels(ctx, oracle, np_dtype):
    """The same sweeps at a few hundred thousand to a few million elements, where
    transposes go through LDS tiles, reductions split a dim over workgroups and
    products run on the matrix cores with edge tiles, K ranges or waves that
    share K: extents that are multiples of the tile sizes, one off either way,
    and odd."""
    from tenncor_amd import ops
    rng = np.random.default_rng(seed_of("medium", np.dtype(np_dtype).name))
    edge = [31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 250, 256, 257, 500, 512, 513]
    # PERMUTE: two or three significant dims, every order
    for case in range(18):
        rank = int(rng.choice([2, 3]))
        shape = [int(rng.choice(edge)) for _ in range(rank)]
        if rank == 3:
            shape[int(rng.integers(0, 3))] = int(rng.choice([2, 3, 5, 8]))
        order = [int(v) for v in rng.permutation(rank)]
        x = draw(rng, int(np.prod(shape)), np_dtype)
        t = ops.from_host(ctx, x, shape)
        np.testing.assert_array_equal(ops.permute(t, order).get(), oracle.permute(x, shape, order)[0],
                                      err_msg="permute %s %s" % (shape, order))
        t.release()
    # reductions of each dim and of pairs of dims
    for case in range(18):
        shape = [int(rng.choice(edge)), int(rng.choice(edge)), int(rng.choice([1, 2, 3, 7]))]
        ranks = [[0], [1], [2], [0, 1], [1, 2], [0, 2], [0, 1, 2]][case % 7]
        op = str(rng.choice(["REDUCE_SUM", "REDUCE_MAX", "REDUCE_MIN"]))
        x = draw(rng, int(np.prod(shape)), np_dtype)
        t = ops.from_host(ctx, x, shape)
        got = ops.reduce(op, t, ranks).get()
        ref, _ = oracle.reduce(op, x, shape, ranks, wide_acc=np_dtype == np.float32)
        close(got, ref, np_dtype, exact=op != "REDUCE_SUM")
        t.release()
    # products: [k, m] x [n, k], sometimes batched; long K over few results among them
    for case in range(18):
        m, n = int(rng.choice(edge)), int(rng.choice(edge))
        k = int(rng.choice([16, 64, 100, 256, 1000, 2048, 4100])) if case % 3 else int(rng.choice(edge))
        if m * n * k > 60_000_000:
            k = max(16, 60_000_000 // (m * n))
        batch = [int(rng.choice([2, 3]))] if case % 5 == 0 else []
        ashape, bshape = [k, m] + batch, [n, k] + batch
        a, b = draw(rng, int(np.prod(ashape)), np_dtype, -2, 2), draw(rng, int(np.prod(bshape)), np_dtype, -2, 2)
        ta, tb = ops.from_host(ctx, a, ashape), ops.from_host(ctx, b, bshape)
        got = ops.matmul(ta, tb).get()
        ref, _ = oracle.matmul(a, ashape, b, bshape, wide_acc=np_dtype == np.float32)
        close(got, ref, np_dtype)
        # the four operand layouts of a contraction over one pair
        if case % 2 == 0 and not batch:
            for pairs, sa, sb in ((((0, 0),), [k, m], [k, n]), (((1, 0),), [m, k], [k, n]), (((1, 1),), [m, k], [n, k])):
                ta2, tb2 = ops.from_host(ctx, a, sa), ops.from_host(ctx, b, sb)
                got = ops.contract(ta2, tb2, pairs).get()
                ref, _ = oracle.contract(a, sa, b, sb, pairs, wide_acc=np_dtype == np.float32)
                close(got, ref, np_dtype)
                ta2.release()
                tb2.release()
        ta.release()
        tb.release()
