"""The integer element types of the reference's full type configuration
(cfg/fulltype.yml:11-34: INT8, UINT8, INT16, UINT16, UINT32, INT64, UINT64)
through every kernel family of the C ABI, bit-exact against the CPU oracle
(which tests/test_oracle_int_widths.py pins against numpy's fixed-width
arithmetic).  Integer results have no tolerance: sums and products wrap modulo
2^width, so they do not depend on the order of accumulation.
"""
import zlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

WIDTHS = [np.int8, np.uint8, np.int16, np.uint16, np.uint32, np.int64, np.uint64]
ids = lambda t: np.dtype(t).name


def seed_of(*parts):
    return zlib.crc32(repr(parts).encode())


@pytest.fixture(scope="module")
def ctx():
    from tenncor_amd import capi
    c = capi.Context(0)
    yield c
    c.close()


@pytest.fixture(scope="module")
def ops():
    from tenncor_amd import ops as o
    return o


def full_range(rng, t, n):
    info = np.iinfo(t)
    x = rng.integers(info.min, info.max, n, dtype=t, endpoint=True)
    edge = [info.min, info.max, 0, 1][:n]
    x[:len(edge)] = edge
    return x


def small(rng, t, n, lo, hi):
    info = np.iinfo(t)
    return rng.integers(max(lo, info.min), min(hi, info.max), n, endpoint=True).astype(t)


@pytest.mark.parametrize("t", WIDTHS, ids=ids)
def test_unary(ctx, ops, oracle, t):
    rng = np.random.default_rng(seed_of("unary", ids(t)))
    n = 200003  # odd: vector body and scalar tail
    x = full_range(rng, t, n)
    tx = ops.from_host(ctx, x, [n])
    for op in ("ABS", "NEG", "ROUND", "SQUARE", "CUBE"):
        np.testing.assert_array_equal(ops.unary(op, tx).get(), oracle.unary(op, x), err_msg=op)
    # through double-precision libm and truncated back: values whose results fit the type
    # (a negative result has no unsigned counterpart in C: unsigned types keep to arguments in [0, 1] for those)
    unsigned = np.iinfo(t).min == 0
    for op in ("SIN", "COS", "TAN", "EXP", "TANH", "SIGMOID"):
        v = small(rng, t, n, 0, 1) if unsigned and op in ("SIN", "COS", "TAN") else small(rng, t, n, -4, 4)
        got, ref = ops.unary(op, ops.from_host(ctx, v, [n])).get(), oracle.unary(op, v)
        assert np.mean(got != ref) < 1e-4, op  # can differ only within an ulp of an integer
    # up to the last arguments whose exponential still fits the integer the double is converted
    # to (32 bits, 64 for the 64-bit types; beyond them C++ leaves the conversion undefined)
    wide = np.dtype(t).itemsize == 8
    reach = (44 if wide else 22) if unsigned else (43 if wide else 21)
    edge = np.arange(0 if unsigned else -reach, reach + 1).astype(t)
    for op in ("EXP", "SIGMOID"):
        got, ref = ops.unary(op, ops.from_host(ctx, edge, [edge.size])).get(), oracle.unary(op, edge)
        assert (got != ref).sum() <= 1, (op, edge[got != ref], got[got != ref], ref[got != ref])
    p = small(rng, t, n, 1, 120)
    tp = ops.from_host(ctx, p, [n])
    for op in ("LOG", "SQRT"):
        got, ref = ops.unary(op, tp).get(), oracle.unary(op, p)
        assert np.mean(got != ref) < 1e-4, op


@pytest.mark.parametrize("t", WIDTHS, ids=ids)
def test_binary_select_assign(ctx, ops, oracle, t):
    rng = np.random.default_rng(seed_of("binary", ids(t)))
    n = 150001
    a, b = full_range(rng, t, n), full_range(rng, t, n)[::-1].copy()
    b[::7] = a[::7]
    ta, tb = ops.from_host(ctx, a, [n]), ops.from_host(ctx, b, [n])
    for op in ("ADD", "SUB", "MUL", "MIN", "MAX", "EQ", "NEQ", "LT", "GT"):
        np.testing.assert_array_equal(ops.binary(op, ta, tb).get(), oracle.binary(op, a, b), err_msg=op)
    # division: zero divisors and lowest / -1 included (the CPU traps there; 0, or the wrapped quotient of narrow types)
    d = b.copy()
    d[5::11] = 0
    if np.iinfo(t).min < 0:
        d[0] = -1  # a[0] is the lowest value
    np.testing.assert_array_equal(ops.binary("DIV", ta, ops.from_host(ctx, d, [n])).get(), oracle.binary("DIV", a, d))
    base, expo = small(rng, t, n, -3, 3), small(rng, t, n, 0, 4)
    np.testing.assert_array_equal(ops.binary("POW", ops.from_host(ctx, base, [n]), ops.from_host(ctx, expo, [n])).get(),
                                  oracle.binary("POW", base, expo))
    cond = (rng.uniform(size=n) < 0.5).astype(t)
    np.testing.assert_array_equal(ops.select(ops.from_host(ctx, cond, [n]), ta, tb).get(), oracle.select(cond, a, b))
    xs = [full_range(rng, t, n) for _ in range(5)]
    ts = [ops.from_host(ctx, x, [n]) for x in xs]
    for op in ("ADD", "MUL"):
        np.testing.assert_array_equal(ops.nary(op, ts).get(), oracle.nary(op, xs), err_msg=op)
    for op in ("ASSIGN", "ASSIGN_ADD", "ASSIGN_SUB", "ASSIGN_MUL", "ASSIGN_DIV"):
        target = ops.from_host(ctx, a, [n])
        ops.assign(op, target, ops.from_host(ctx, d, [n]))
        np.testing.assert_array_equal(target.get(), oracle.assign(op, a.copy(), d), err_msg=op)


def test_casts_between_every_pair(ctx, ops, oracle):
    from tenncor_amd import capi
    rng = np.random.default_rng(3)
    n = 50001
    for code, src in capi.NP_OF.items():
        if np.dtype(src).kind == "f":
            x = rng.uniform(-100, 100, n).astype(src)
        else:
            x = full_range(rng, src, n)
        for out_code, dst in capi.NP_OF.items():
            v = x
            if np.dtype(src).kind == "f" and np.dtype(dst).kind == "u":
                v = np.abs(x)  # a negative value has no unsigned counterpart in C
            got = ops.cast(ops.from_host(ctx, v, [n]), out_code).get()
            np.testing.assert_array_equal(got, oracle.cast(v, out_code), err_msg="%s -> %s" % (ids(src), ids(dst)))


REDUCE_CASES = [([2048, 64], [0]), ([2048, 64], [1]), ([2048, 64], [0, 1]), ([5, 7, 3, 4], [0, 2]),
                ([3, 50000], [1]), ([100003], [0]), ([6, 5, 4, 3, 2, 2, 3, 2], [1, 3, 5, 7])]


@pytest.mark.parametrize("t", WIDTHS, ids=ids)
def test_reductions_and_argmax(ctx, ops, oracle, t):
    rng = np.random.default_rng(seed_of("reduce", ids(t)))
    for shape, ranks in REDUCE_CASES:
        x = full_range(rng, t, oracle.n_elems(shape))
        tx = ops.from_host(ctx, x, shape)
        for op in ("REDUCE_SUM", "REDUCE_PROD", "REDUCE_MIN", "REDUCE_MAX"):
            out = ops.reduce(op, tx, ranks)
            ref, oshape = oracle.reduce(op, x, shape, ranks)
            assert out.shape == oshape
            np.testing.assert_array_equal(out.get(), ref, err_msg="%s %s %s" % (op, shape, ranks))
    shape = [7, 50, 9]
    x = small(rng, t, oracle.n_elems(shape), -50, 50)  # ties on purpose
    tx = ops.from_host(ctx, x, shape)
    for rd in (0, 1, 2, 8):
        np.testing.assert_array_equal(ops.argmax(tx, rd).get(), oracle.argmax(x, shape, rd)[0])


@pytest.mark.parametrize("t", WIDTHS, ids=ids)
def test_data_movement(ctx, ops, oracle, t):
    from test_gpu_ops import movement_cases
    rng = np.random.default_rng(seed_of("move", ids(t)))
    for name, shape, gfn, ofn in movement_cases(oracle, ops, rng):
        x = full_range(rng, t, oracle.n_elems(shape))
        out = gfn(ops.from_host(ctx, x, shape))
        ref, oshape = ofn(x, shape)
        assert out.shape == oracle.shape8(oshape), name
        np.testing.assert_array_equal(out.get(), ref, err_msg=name)
    shapes = [[5, 3, 4], [7, 3, 4]]
    xs = [full_range(rng, t, oracle.n_elems(s)) for s in shapes]
    out = ops.concat([ops.from_host(ctx, x, s) for x, s in zip(xs, shapes)], 0)
    np.testing.assert_array_equal(out.get(), oracle.concat(xs, shapes, 0)[0])
    # a transposing permute large enough for the tiled kernels
    shape = [1030, 515]
    x = full_range(rng, t, oracle.n_elems(shape))
    np.testing.assert_array_equal(ops.permute(ops.from_host(ctx, x, shape), [1, 0]).get(), oracle.permute(x, shape, [1, 0])[0])


@pytest.mark.parametrize("t", WIDTHS, ids=ids)
def test_products(ctx, ops, oracle, t):
    from tenncor_amd import capi
    rng = np.random.default_rng(seed_of("products", ids(t)))
    for ashape, bshape in (([10, 3], [9, 10]), ([100, 37], [53, 100]), ([32, 48, 5], [40, 32, 5]), ([256, 128], [192, 256])):
        a, b = full_range(rng, t, oracle.n_elems(ashape)), full_range(rng, t, oracle.n_elems(bshape))
        out = ops.matmul(ops.from_host(ctx, a, ashape), ops.from_host(ctx, b, bshape))
        ref, oshape = oracle.matmul(a, ashape, b, bshape)
        assert out.shape == oshape
        np.testing.assert_array_equal(out.get(), ref, err_msg=str(ashape))
    for ashape, bshape, pairs in (([4, 2, 3], [2, 4, 2], [[0, 1], [1, 2]]), ([12, 7], [12, 9], [[0, 0]]),
                                  ([5, 6, 7], [7, 3, 5], [[0, 2], [2, 0]]), ([768, 1, 8], [64, 768], [[0, 1]])):
        a, b = full_range(rng, t, oracle.n_elems(ashape)), full_range(rng, t, oracle.n_elems(bshape))
        out = ops.contract(ops.from_host(ctx, a, ashape), ops.from_host(ctx, b, bshape), pairs)
        np.testing.assert_array_equal(out.get(), oracle.contract(a, ashape, b, bshape, pairs)[0], err_msg=str(ashape))
    for ishape, kshape, ranks in (([3, 3], [2], [1]), ([2, 4, 3, 3], [1, 2, 2, 1], list(range(8))),
                                  ([1, 12, 12, 4, 5], [3, 1, 5, 5], [4, 0, 1, 2]), ([4, 10, 9, 2, 5], [1, 6, 4, 2, 3], list(range(8)))):
        img, ker = full_range(rng, t, oracle.n_elems(ishape)), full_range(rng, t, oracle.n_elems(kshape))
        out = ops.convolution(ops.from_host(ctx, img, ishape), ops.from_host(ctx, ker, kshape), ranks)
        np.testing.assert_array_equal(out.get(), oracle.conv(img, ishape, ker, kshape, ranks)[0], err_msg=str(ishape))
    # transposed operands and a long K through tcg_gemm
    for M, N, K, batch, ta, tb in ((20, 12, 300, 5, 1, 1), (7, 9, 33, 3, 0, 1), (128, 10, 64, 1, 0, 0), (130, 70, 65, 2, 1, 0)):
        a, b = full_range(rng, t, batch * M * K), full_range(rng, t, batch * K * N)
        a_can = a if not ta else oracle.permute(a, [M, K, batch], [1, 0, 2])[0]
        b_can = b if not tb else oracle.permute(b, [K, N, batch], [1, 0, 2])[0]
        ref, _ = oracle.matmul(a_can, [K, M, batch], b_can, [N, K, batch])
        da, db, dc = ctx.upload(a), ctx.upload(b), ctx.empty(batch * M * N, t)
        ctx.gemm(capi.dtype_code(t), M, N, K, batch, da.ptr, M if ta else K, M * K, ta,
                 db.ptr, K if tb else N, K * N, tb, dc.ptr, N, M * N)
        np.testing.assert_array_equal(dc.get(), ref, err_msg=str((M, N, K, batch, ta, tb)))
        for buf in (da, db, dc):
            buf.release()


@pytest.mark.parametrize("t", WIDTHS, ids=ids)
def test_fused_chain_equals_node_by_node(ctx, ops, oracle, t):
    """tcg_ew_fused compiles its program for the element type at hand."""
    from tenncor_amd import capi
    rng = np.random.default_rng(seed_of("fused", ids(t)))
    n = 70001
    a, b = full_range(rng, t, n), full_range(rng, t, n)
    da, db, out = ctx.upload(a), ctx.upload(b), ctx.empty(n, t)
    L = capi.OPD_LEAF0
    ctx.ew_fused(capi.dtype_code(t), n, [da.ptr, db.ptr],
                 [("ADD", L, L + 1, capi.OPD_ACC), ("MUL", capi.OPD_ACC, L + 1, capi.OPD_ACC), ("CUBE", capi.OPD_ACC, 0, capi.OPD_ACC),
                  ("MAX", capi.OPD_ACC, L, capi.OPD_ACC)], out.ptr)
    ref = oracle.binary("MAX", oracle.unary("CUBE", oracle.binary("MUL", oracle.binary("ADD", a, b), b)), a)
    np.testing.assert_array_equal(out.get(), ref)


@pytest.mark.parametrize("t", WIDTHS, ids=ids)
def test_device_generator(ctx, oracle, t):
    rng = np.random.default_rng(seed_of("rand", ids(t)))
    info = np.iinfo(t)
    seed = 0xabcdef12345
    ctx.rand_seed(seed)
    per = 2 if np.dtype(t).itemsize == 8 else 4
    drawn = 0
    for n in (1, 5, 64, 300007):
        lo = small(rng, t, n, -1000, 1000)
        hi = (lo.astype(np.int64) + rng.integers(0, 100, n)).clip(info.min, min(info.max, 2 ** 62)).astype(t)
        if n > 4:
            lo[1], hi[1] = info.min, info.max  # the whole range
            lo[2], hi[2] = 9, 3                # empty: the lower bound
        dlo, dhi, out = ctx.upload(lo), ctx.upload(hi), ctx.empty(n, t)
        ctx.rand_uniform(out.dtype, n, dlo.ptr, dhi.ptr, out.ptr)
        np.testing.assert_array_equal(out.get(), oracle.rand_uniform(lo, hi, seed, first_block=drawn))
        drawn += (n + per - 1) // per
        assert ctx.rand_state() == (seed, drawn)
        for buf in (dlo, dhi, out):
            buf.release()
