"""GPU parity: every entry point of the C ABI against the CPU oracle on the
same seeded inputs, and against the reference's golden vectors.

Bars: bit-exact for int32 ops and PERMUTE / SLICE / EXTEND
(and the other pure data movement), 1e-5 relative for fp32 elementwise, 1e-4
relative for fp32 reductions and contractions.  fp32 reductions/contractions are
compared with the oracle accumulating in fp64, relative to max(|ref|, floor)
where floor = mean |ref| of the output (individual sums of signed values can be
arbitrarily close to zero).
"""
import json
import os
import zlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
with open(os.path.join(GOLDEN, "operator_goldens.json")) as f:
    OPG = json.load(f)
with open(os.path.join(GOLDEN, "equation_vectors.json")) as f:
    EQV = json.load(f)

def seed_of(*parts):
    """Deterministic per-case seed (hash() of str is salted per process)."""
    return zlib.crc32(repr(parts).encode())


EW_RTOL = 1e-5
ACC_RTOL = 1e-4


@pytest.fixture(scope="module")
def ctx():
    from tenncor_amd import capi
    c = capi.Context(0)
    assert c.arch.startswith("gfx9"), c.arch
    yield c
    c.close()


@pytest.fixture(scope="module")
def ops():
    from tenncor_amd import ops as o
    return o


def assert_acc_close(got, ref, rtol=ACC_RTOL):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    floor = np.mean(np.abs(ref)) if ref.size else 0.0
    denom = np.maximum(np.abs(ref), floor)
    denom[denom == 0] = 1.0
    err = np.abs(got - ref) / denom
    assert err.max() <= rtol, "max rel err %.3g at %d (got %r ref %r)" % (
        err.max(), err.argmax(), got.flat[err.argmax()], ref.flat[err.argmax()])


def gpu_case(ops, ctx, case, np_dtype=np.float64):
    op = case["op"]
    args = [ops.from_host(ctx, np.asarray(a["data"], dtype=np_dtype), a["shape"]) for a in case["args"]]
    if op in ("REDUCE_SUM", "REDUCE_PROD", "REDUCE_MIN", "REDUCE_MAX"):
        out = ops.reduce(op, args[0], case["rank_set"])
    elif op == "ARGMAX":
        out = ops.argmax(args[0], case["rank"])
    elif op == "EXTEND":
        out = ops.extend(args[0], case["dimensions"])
    elif op == "PERMUTE":
        out = ops.permute(args[0], case["ranks"])
    elif op == "SLICE":
        out = ops.slice_(args[0], case["dimension_pairs"])
    elif op == "PAD":
        out = ops.pad(args[0], case["dimension_pairs"])
    elif op == "STRIDE":
        out = ops.stride(args[0], case["dimensions"])
    elif op == "SCATTER":
        out = ops.scatter(args[0], case["dimensions"], case["outshape"])
    elif op == "REVERSE":
        out = ops.reverse(args[0], case["rank_set"])
    elif op == "CONCAT":
        out = ops.concat(args, case["rank"])
    elif op == "SELECT":
        out = ops.select(*args)
    elif op == "CONTRACT":
        out = ops.contract(args[0], args[1], case["rank_pairs"])
    elif op == "CONV":
        out = ops.convolution(args[0], args[1], case["ranks"])
    elif op in ("ADD", "MUL"):
        out = ops.nary(op, args)
    else:
        out = ops.binary(op, args[0], args[1])
    return out.get(), out.shape


@pytest.mark.parametrize("case", OPG["cases"], ids=[c["name"] for c in OPG["cases"]])
def test_reference_goldens_on_gpu(ctx, ops, oracle, case):
    """internal/eigen/test/test_operator.cpp vectors, evaluated in double."""
    got, shape = gpu_case(ops, ctx, case)
    assert list(shape) == oracle.shape8(case["outshape"])
    expect = np.asarray(case["expect"], dtype=np.float64)
    if "tol" in case or case["op"] in ("POW", "DIV"):
        np.testing.assert_allclose(got, expect, rtol=1e-13, atol=0)
    else:
        np.testing.assert_array_equal(got, expect)


UNARY = ["ABS", "NEG", "SIN", "COS", "TAN", "EXP", "LOG", "SQRT", "ROUND", "SIGMOID", "TANH", "SQUARE", "CUBE"]
BINARY = ["POW", "ADD", "SUB", "MUL", "DIV", "MIN", "MAX", "EQ", "NEQ", "LT", "GT"]


@pytest.mark.parametrize("op", UNARY)
@pytest.mark.parametrize("np_dtype", [np.float32, np.float64, np.int32])
def test_unary_vs_oracle(ctx, ops, oracle, op, np_dtype):
    rng = np.random.default_rng(seed_of(op, str(np_dtype)))
    n = 1000003  # odd: exercises the vector body and the scalar tail
    if np_dtype == np.int32:
        x = rng.integers(-30, 30, n).astype(np.int32)
        if op in ("LOG", "SQRT"):
            x = np.abs(x) + 1
        if op in ("EXP",):
            x = rng.integers(-5, 20, n).astype(np.int32)
    else:
        x = rng.uniform(-4, 4, n).astype(np_dtype)
        if op in ("LOG", "SQRT"):
            x = np.abs(x) + np_dtype(0.01)
        if op == "TAN":
            x = rng.uniform(-1.4, 1.4, n).astype(np_dtype)
    t = ops.from_host(ctx, x, [n])
    got = ops.unary(op, t).get()
    ref = oracle.unary(op, x)
    if np_dtype == np.int32:
        if op in ("SIN", "COS", "TAN", "EXP", "LOG", "SQRT", "TANH"):
            # double-precision libm on both sides, truncated: the integer part can
            # differ only when the value sits within an ulp of an integer
            assert np.mean(got != ref) < 1e-4
        else:
            np.testing.assert_array_equal(got, ref)
    elif op in ("ABS", "NEG", "ROUND", "SQUARE", "CUBE", "SQRT"):
        np.testing.assert_array_equal(got, ref)  # exactly rounded operations
    else:
        rtol = EW_RTOL if np_dtype == np.float32 else 1e-13
        np.testing.assert_allclose(got, ref, rtol=rtol, atol=0)


@pytest.mark.parametrize("op", ["TANH", "SIGMOID"])
def test_fp32_tanh_and_sigmoid_over_their_whole_range(ctx, ops, oracle, op):
    """fp32 TANH is the rational approximation the reference itself computes
    with (Eigen 3.3.7's generic_fast_tanh_float) and SIGMOID ends in a 1-ulp
    reciprocal: against the libm oracle at 1e-5 relative from 1e-30 to
    saturation, exactly at 0, the limits at infinity, NaN stays NaN."""
    mags = np.logspace(-30, 2, 40001).astype(np.float32)
    x = np.concatenate([mags, -mags, np.linspace(-12, 12, 200001).astype(np.float32)])
    got = ops.unary(op, ops.from_host(ctx, x, [x.size])).get()
    ref = oracle.unary(op, x)
    tiny = np.abs(ref) < 1e-30   # sigmoid of large negative arguments underflows: compare absolutely there
    np.testing.assert_allclose(got[~tiny], ref[~tiny], rtol=EW_RTOL, atol=0)
    assert np.all(np.abs(got[tiny]) < 1e-30)
    assert np.all(np.abs(got) <= 1)
    edge = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 9.0, -9.0, 88.0, -88.0, 104.0, -104.0], np.float32)
    got = ops.unary(op, ops.from_host(ctx, edge, [edge.size])).get()
    want = np.tanh(edge.astype(np.float64)) if op == "TANH" else 1 / (1 + np.exp(-edge.astype(np.float64)))
    assert np.isnan(got[4])
    np.testing.assert_allclose(np.delete(got, 4), np.delete(want, 4), rtol=EW_RTOL, atol=1e-37)
    if op == "TANH":
        # saturation is the value of the approximation at its clamp, one ulp inside (-1, 1)
        assert got[0] == 0 and got[1] == 0 and np.signbit(got[1]) and got[2] == -got[3] and 1 - 1e-7 <= got[2] <= 1
    else:
        assert got[0] == 0.5 and got[2] == 1 and got[3] == 0


@pytest.mark.parametrize("op", BINARY)
@pytest.mark.parametrize("np_dtype", [np.float32, np.float64, np.int32])
def test_binary_vs_oracle(ctx, ops, oracle, op, np_dtype):
    rng = np.random.default_rng(seed_of(op, str(np_dtype), 2))
    n = 777777
    if np_dtype == np.int32:
        a = rng.integers(-1000, 1000, n).astype(np.int32)
        b = rng.integers(-1000, 1000, n).astype(np.int32)
        if op == "MUL":
            a = rng.integers(-2 ** 31, 2 ** 31 - 1, n).astype(np.int32)  # wraps
        if op == "DIV":
            b[b == 0] = 7
        if op == "POW":
            a = rng.integers(-9, 9, n).astype(np.int32)
            b = rng.integers(0, 9, n).astype(np.int32)
    else:
        a = rng.uniform(-3, 3, n).astype(np_dtype)
        b = rng.uniform(-3, 3, n).astype(np_dtype)
        if op == "POW":
            a = np.abs(a) + np_dtype(0.1)
        b[::7] = a[::7]  # some equal pairs for EQ/NEQ/MIN/MAX
    ta, tb = ops.from_host(ctx, a, [n]), ops.from_host(ctx, b, [n])
    got = ops.binary(op, ta, tb).get()
    ref = oracle.binary(op, a, b)
    if np_dtype == np.int32 or op not in ("POW",):
        np.testing.assert_array_equal(got, ref)
    else:
        np.testing.assert_allclose(got, ref, rtol=EW_RTOL if np_dtype == np.float32 else 1e-13, atol=0)


@pytest.mark.parametrize("np_dtype", [np.float32, np.int32])
@pytest.mark.parametrize("nargs", [3, 8, 11])
def test_nary_left_fold(ctx, ops, oracle, np_dtype, nargs):
    rng = np.random.default_rng(nargs)
    n = 300001
    if np_dtype == np.int32:
        xs = [rng.integers(-2 ** 30, 2 ** 30, n).astype(np.int32) for _ in range(nargs)]
    else:
        xs = [rng.uniform(-1, 1, n).astype(np.float32) for _ in range(nargs)]
    ts = [ops.from_host(ctx, x, [n]) for x in xs]
    for op in ("ADD", "MUL"):
        got = ops.nary(op, ts).get()
        np.testing.assert_array_equal(got, oracle.nary(op, xs))  # same fold order: bit-exact


def test_select_cast_assign(ctx, ops, oracle):
    from tenncor_amd import capi
    rng = np.random.default_rng(5)
    n = 100003
    c = (rng.uniform(size=n) < 0.5).astype(np.float32)
    a = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    tc, ta, tb = (ops.from_host(ctx, v, [n]) for v in (c, a, b))
    np.testing.assert_array_equal(ops.select(tc, ta, tb).get(), oracle.select(c, a, b))
    x = (a * 100).astype(np.float32)
    for out_dtype in (capi.INT32, capi.DOUBLE, capi.FLOAT):
        np.testing.assert_array_equal(ops.cast(ops.from_host(ctx, x, [n]), out_dtype).get(), oracle.cast(x, out_dtype))
    xi = rng.integers(-10 ** 6, 10 ** 6, n).astype(np.int32)
    np.testing.assert_array_equal(ops.cast(ops.from_host(ctx, xi, [n]), capi.FLOAT).get(), oracle.cast(xi, capi.FLOAT))
    for op in ("ASSIGN", "ASSIGN_ADD", "ASSIGN_SUB", "ASSIGN_MUL", "ASSIGN_DIV"):
        t = ops.from_host(ctx, a, [n])
        ops.assign(op, t, tb)
        ref = oracle.assign(op, a.copy(), b)
        np.testing.assert_array_equal(t.get(), ref)


def test_assign_and_cast_goldens(ctx, ops):
    """internal/eigen/test/test_operator.cpp:2647-2879: the reference's vectors
    for ASSIGN .. ASSIGN_DIV (in place on the target) and CAST."""
    from tenncor_amd import capi
    goldens = {"ASSIGN": [1, 0, 3, 9, 10, 11], "ASSIGN_ADD": [3, 8, 7, 14, 16, 18], "ASSIGN_SUB": [1, 8, 1, -4, -4, -4],
               "ASSIGN_MUL": [2, 0, 12, 45, 60, 77], "ASSIGN_DIV": [2, 4, 4. / 3, 5. / 9, 0.6, 7. / 11]}
    for op, want in goldens.items():
        target = ops.from_host(ctx, np.array([2, 8, 4, 5, 6, 7], np.float64), [2, 3])
        source = ops.from_host(ctx, np.array([1, 2 if op == "ASSIGN_DIV" else 0, 3, 9, 10, 11], np.float64), [2, 3])
        ops.assign(op, target, source)
        np.testing.assert_allclose(target.get(), want, rtol=4e-16, err_msg=op)
    x = ops.from_host(ctx, np.array([2.1, 8.5, 4.3, 5.2, 6.1, 7.2], np.float64), [2, 3])
    np.testing.assert_array_equal(ops.cast(x, capi.INT32).get(), np.array([2, 8, 4, 5, 6, 7], np.int32))


def test_unaligned_operands_take_the_scalar_path(ctx, ops, oracle):
    """Aliased last-dim slices give pointers that are not 16-byte aligned
    (internal/eigen/operator.hpp:231-248)."""
    from tenncor_amd import capi
    rng = np.random.default_rng(9)
    n = 4099
    a = rng.standard_normal(n + 3).astype(np.float32)
    b = rng.standard_normal(n + 3).astype(np.float32)
    da, db = ctx.upload(a), ctx.upload(b)
    out = ctx.empty(n + 3, np.float32)
    ctx.ew_binary("ADD", capi.FLOAT, n, da.ptr + 4, db.ptr + 8, out.ptr + 12)
    np.testing.assert_array_equal(out.get()[3:], oracle.binary("ADD", a[1:n + 1], b[2:n + 2]))
    ctx.ew_unary("EXP", capi.FLOAT, n, da.ptr + 4, out.ptr)
    np.testing.assert_allclose(out.get()[:n], oracle.unary("EXP", a[1:n + 1]), rtol=EW_RTOL)
    ctx.reduce("REDUCE_SUM", capi.FLOAT, [n], [0], da.ptr + 4, out.ptr)
    assert_acc_close(out.get()[:1], oracle.reduce("REDUCE_SUM", a[1:n + 1], [n], [0], wide_acc=True)[0])


def test_fused_chain_equals_node_by_node(ctx, ops, oracle):
    """config 2's chain ADD, MUL, EXP, TANH, SIGMOID in one pass over memory."""
    from tenncor_amd import capi
    rng = np.random.default_rng(2)
    n = 1 << 20
    a, b, c = (rng.uniform(-1, 1, n).astype(np.float32) for _ in range(3))
    ta, tb, tc = (ops.from_host(ctx, v, [n]) for v in (a, b, c))
    L = capi.OPD_LEAF0
    prog = [("ADD", L + 0, L + 1, capi.OPD_ACC), ("MUL", capi.OPD_ACC, L + 2, capi.OPD_ACC),
            ("EXP", capi.OPD_ACC, 0, capi.OPD_ACC), ("TANH", capi.OPD_ACC, 0, capi.OPD_ACC),
            ("SIGMOID", capi.OPD_ACC, 0, capi.OPD_ACC)]
    out = ctx.empty(n, np.float32)
    ctx.ew_fused(capi.FLOAT, n, [ta.ptr, tb.ptr, tc.ptr], prog, out.ptr)
    unfused = ops.unary("SIGMOID", ops.unary("TANH", ops.unary("EXP", ops.binary("MUL", ops.binary("ADD", ta, tb), tc))))
    np.testing.assert_array_equal(out.get(), unfused.get())
    ref = oracle.unary("SIGMOID", oracle.unary("TANH", oracle.unary("EXP", oracle.binary("MUL", oracle.binary("ADD", a, b), c))))
    np.testing.assert_allclose(out.get(), ref, rtol=EW_RTOL)
    # registers and immediates: sigmoid gradient  s * (1 - s) * g  with s = sigmoid(a)
    prog = [("SIGMOID", L + 0, 0, capi.OPD_T0), ("SUB", capi.OPD_IMM, capi.OPD_T0, capi.OPD_ACC, 1.0),
            ("MUL", capi.OPD_T0, capi.OPD_ACC, capi.OPD_ACC), ("MUL", capi.OPD_ACC, L + 1, capi.OPD_ACC)]
    ctx.ew_fused(capi.FLOAT, n, [ta.ptr, tb.ptr], prog, out.ptr)
    s = oracle.unary("SIGMOID", a)
    ref = oracle.binary("MUL", oracle.binary("MUL", s, oracle.binary("SUB", np.ones(n, np.float32), s)), b)
    np.testing.assert_allclose(out.get(), ref, rtol=EW_RTOL, atol=1e-12)
    # int32 chain is bit-exact
    ai, bi = (rng.integers(-1000, 1000, n).astype(np.int32) for _ in range(2))
    tai, tbi = ops.from_host(ctx, ai, [n]), ops.from_host(ctx, bi, [n])
    outi = ctx.empty(n, np.int32)
    ctx.ew_fused(capi.INT32, n, [tai.ptr, tbi.ptr], [("ADD", L, L + 1, capi.OPD_ACC), ("MUL", capi.OPD_ACC, L + 1, capi.OPD_ACC),
                                                      ("CUBE", capi.OPD_ACC, 0, capi.OPD_ACC)], outi.ptr)
    np.testing.assert_array_equal(outi.get(), oracle.unary("CUBE", oracle.binary("MUL", oracle.binary("ADD", ai, bi), bi)))


REDUCE_CASES = [
    ([2048, 512], [0]), ([2048, 512], [1]), ([2048, 512], [0, 1]),
    ([64, 20, 20, 16], [1, 2]), ([5, 7, 3, 4], [0, 2]), ([5, 7, 3, 4], [1, 3]), ([5, 7, 3, 4], [0, 1, 2, 3]),
    ([3, 100000], [1]), ([100003], [0]), ([9, 3], [1]), ([1, 1, 300, 1, 77], [2]), ([33, 1, 17], [0, 2]),
    ([1 << 22], [0]), ([6, 5, 4, 3, 2, 2, 3, 2], [0, 2, 4, 6]), ([6, 5, 4, 3, 2, 2, 3, 2], [1, 3, 5, 7]),
]


@pytest.mark.parametrize("shape,ranks", REDUCE_CASES, ids=[str(c) for c in REDUCE_CASES])
def test_reduce_vs_oracle(ctx, ops, oracle, shape, ranks):
    rng = np.random.default_rng(seed_of(shape, ranks))
    n = oracle.n_elems(shape)
    xf = rng.uniform(-1, 1, n).astype(np.float32)
    xi = rng.integers(-1000, 1000, n).astype(np.int32) * rng.integers(-1000, 1000, n).astype(np.int32)
    tf, ti = ops.from_host(ctx, xf, shape), ops.from_host(ctx, xi, shape)
    for op in ("REDUCE_SUM", "REDUCE_MAX", "REDUCE_MIN"):
        out = ops.reduce(op, tf, ranks)
        ref, oshape = oracle.reduce(op, xf, shape, ranks, wide_acc=True)
        assert out.shape == oshape
        if op == "REDUCE_SUM":
            assert_acc_close(out.get(), ref)
        else:
            np.testing.assert_array_equal(out.get(), ref)
        # int32: wrap-around sums are order independent, so bit-exact
        np.testing.assert_array_equal(ops.reduce(op, ti, ranks).get(), oracle.reduce(op, xi, shape, ranks)[0])
    xd = rng.uniform(0.999, 1.001, n)  # keeps products of millions of values in range
    got = ops.reduce("REDUCE_PROD", ops.from_host(ctx, xd, shape), ranks).get()
    np.testing.assert_allclose(got, oracle.reduce("REDUCE_PROD", xd, shape, ranks)[0], rtol=1e-9)


def test_argmax_vs_oracle(ctx, ops, oracle):
    rng = np.random.default_rng(4)
    shape = [7, 50, 9]
    x = rng.integers(-50, 50, oracle.n_elems(shape)).astype(np.float32)  # ties on purpose
    t = ops.from_host(ctx, x, shape)
    for rd in (0, 1, 2, 8):
        np.testing.assert_array_equal(ops.argmax(t, rd).get(), oracle.argmax(x, shape, rd)[0])


def movement_cases(oracle, ops, rng):
    """(name, gpu thunk, oracle thunk) over int32 payloads: all bit-exact."""
    cases = []

    def add(name, shape, gfn, ofn):
        cases.append((name, shape, gfn, ofn))

    add("permute_2d", [300, 200], lambda t: ops.permute(t, [1, 0]), lambda x, s: oracle.permute(x, s, [1, 0]))
    add("permute_batched", [70, 130, 5], lambda t: ops.permute(t, [1, 0, 2]), lambda x, s: oracle.permute(x, s, [1, 0, 2]))
    add("permute_rot", [20, 30, 40], lambda t: ops.permute(t, [2, 0, 1]), lambda x, s: oracle.permute(x, s, [2, 0, 1]))
    add("permute_inner_kept", [64, 5, 7, 3], lambda t: ops.permute(t, [0, 2, 1, 3]), lambda x, s: oracle.permute(x, s, [0, 2, 1, 3]))
    add("permute_conv2d", [1, 20, 18, 6, 32], lambda t: ops.permute(t, [4, 1, 2, 3]), lambda x, s: oracle.permute(x, s, [4, 1, 2, 3]))
    add("permute_wide_tiles", [132, 68, 3], lambda t: ops.permute(t, [1, 0, 2]), lambda x, s: oracle.permute(x, s, [1, 0, 2]))
    add("permute_wide_batched", [64, 6, 128], lambda t: ops.permute(t, [2, 1, 0]), lambda x, s: oracle.permute(x, s, [2, 1, 0]))
    add("permute_narrow_odd", [66, 35], lambda t: ops.permute(t, [1, 0]), lambda x, s: oracle.permute(x, s, [1, 0]))
    add("permute_small", [3, 4, 5], lambda t: ops.permute(t, [2, 1, 0]), lambda x, s: oracle.permute(x, s, [2, 1, 0]))
    add("extend_bias", [9, 1], lambda t: ops.extend(t, [1, 300]), lambda x, s: oracle.extend(x, s, [1, 300]))
    add("extend_scalar", [1], lambda t: ops.extend(t, [32, 24, 24, 8]), lambda x, s: oracle.extend(x, s, [32, 24, 24, 8]))
    add("extend_mid", [16, 1, 5, 1], lambda t: ops.extend(t, [1, 33, 1, 4]), lambda x, s: oracle.extend(x, s, [1, 33, 1, 4]))
    add("extend_inner", [1, 77], lambda t: ops.extend(t, [130]), lambda x, s: oracle.extend(x, s, [130]))
    add("slice_seq", [256, 64, 16], lambda t: ops.slice_(t, [[0, 256], [5, 1]]), lambda x, s: oracle.slice_(x, s, [[0, 256], [5, 1]]))
    add("slice_gate", [2048, 1, 16], lambda t: ops.slice_(t, [[512, 512]]), lambda x, s: oracle.slice_(x, s, [[512, 512]]))
    add("slice_odd", [37, 11, 5], lambda t: ops.slice_(t, [[3, 30], [2, 100], [1, 3]]), lambda x, s: oracle.slice_(x, s, [[3, 30], [2, 100], [1, 3]]))
    add("pad_dim4", [4, 10, 9, 2], lambda t: ops.pad(t, [[0, 0]] * 4 + [[2, 2]]), lambda x, s: oracle.pad(x, s, [[0, 0]] * 4 + [[2, 2]]))
    add("pad_inner", [16, 7], lambda t: ops.pad(t, [[4, 8], [1, 0]]), lambda x, s: oracle.pad(x, s, [[4, 8], [1, 0]]))
    add("pad_odd", [5, 6, 3], lambda t: ops.pad(t, [[1, 2], [0, 3], [2, 0]]), lambda x, s: oracle.pad(x, s, [[1, 2], [0, 3], [2, 0]]))
    add("reverse_0", [32, 4, 5, 6], lambda t: ops.reverse(t, [0]), lambda x, s: oracle.reverse(x, s, [0]))
    add("reverse_all", [8, 4, 5, 6], lambda t: ops.reverse(t, [0, 1, 2, 3]), lambda x, s: oracle.reverse(x, s, [0, 1, 2, 3]))
    add("stride", [17, 9, 4], lambda t: ops.stride(t, [2, 3]), lambda x, s: oracle.stride(x, s, [2, 3]))
    add("scatter", [9, 3, 4], lambda t: ops.scatter(t, [2, 3], [17, 9, 4]), lambda x, s: oracle.scatter(x, s, [2, 3], [17, 9, 4]))
    return cases


def test_data_movement_bit_exact(ctx, ops, oracle):
    rng = np.random.default_rng(12)
    for name, shape, gfn, ofn in movement_cases(oracle, ops, rng):
        n = oracle.n_elems(shape)
        for np_dtype in (np.int32, np.float64):
            x = rng.integers(-2 ** 31, 2 ** 31 - 1, n).astype(np.int32)
            if np_dtype == np.float64:
                x = rng.standard_normal(n)
            out = gfn(ops.from_host(ctx, x, shape))
            ref, oshape = ofn(x, shape)
            assert out.shape == oracle.shape8(oshape), name
            np.testing.assert_array_equal(out.get(), ref, err_msg=name)


@pytest.mark.parametrize("np_dtype", [np.float32, np.int32, np.float64])
def test_transposing_permutes_with_wide_and_narrow_accesses(ctx, ops, oracle, np_dtype):
    """PERMUTE that moves the contiguous dim: tiles through LDS with 128-bit
    accesses when extents, strides and addresses allow it, element by element
    otherwise (odd extents, an operand at an odd element offset) -- every case
    bit-exact against the oracle and against numpy's transpose."""
    from tenncor_amd import capi
    rng = np.random.default_rng(seed_of("transpose", np_dtype.__name__))
    cases = [([64, 64], [1, 0]), ([128, 68], [1, 0]), ([260, 132, 3], [1, 0, 2]), ([512, 512, 5], [1, 0, 2]),
             ([66, 35], [1, 0]), ([130, 62, 2], [1, 0, 2]), ([64, 6, 128], [2, 1, 0]), ([4, 1028], [1, 0]),
             ([1028, 4], [1, 0]), ([16, 16, 16, 4], [1, 0, 3, 2])]
    for shape, order in cases:
        n = int(np.prod(shape))
        x = rng.integers(-10 ** 6, 10 ** 6, n).astype(np_dtype)
        got = ops.permute(ops.from_host(ctx, x, shape), order)
        ref, oshape = oracle.permute(x, shape, order)
        assert got.shape == oracle.shape8(oshape)
        np.testing.assert_array_equal(got.get(), ref, err_msg=str((shape, order)))
        nd = len(shape)
        axes = [nd - 1 - order[nd - 1 - k] for k in range(nd)]
        np.testing.assert_array_equal(ref, x.reshape(shape[::-1]).transpose(axes).reshape(-1))
    # the same tile shapes from a source and into a destination that are not 16-byte aligned
    shape, order = [128, 68], [1, 0]
    n = 128 * 68
    x = rng.integers(-10 ** 6, 10 ** 6, n + 1).astype(np_dtype)
    src = ctx.upload(x)
    dst = ctx.empty(n + 1, np_dtype)
    item = np.dtype(np_dtype).itemsize
    ctx.permute(capi.dtype_code(np_dtype), shape, order + list(range(2, 8)), src.ptr + item, dst.ptr + item)
    np.testing.assert_array_equal(dst.get()[1:], oracle.permute(x[1:], shape, order)[0])


def test_column_reductions_with_few_columns_take_one_launch(ctx, ops, oracle):
    """[A, R] -> [A] with too few columns to fill the chip at full tile width:
    narrower tiles in one pass (config 2's dim-1 reduction is the case that
    matters: np[4096,16384] -> [16384]); values against the oracle in all
    three dtypes, with column counts that leave partial tiles."""
    rng = np.random.default_rng(seed_of("wide columns"))
    for np_dtype in (np.float32, np.int32, np.float64):
        for shape in ([16384, 1030], [4096 + 64, 1500], [20000, 1024], [8192, 2048, 2]):
            n = int(np.prod(shape))
            x = rng.integers(-1000, 1001, n).astype(np_dtype) if np_dtype == np.int32 else rng.uniform(-1, 1, n).astype(np_dtype)
            t = ops.from_host(ctx, x, shape)
            for op in ("REDUCE_SUM", "REDUCE_MAX", "REDUCE_MIN"):
                got = ops.reduce(op, t, [1]).get()
                ref = oracle.reduce(op, x, shape, [1], wide_acc=np_dtype != np.int32)[0]
                if np_dtype == np.int32 or op != "REDUCE_SUM":
                    np.testing.assert_array_equal(got, ref, err_msg=str((np_dtype.__name__, shape, op)))
                else:
                    assert_acc_close(got, ref)


def test_sum_of_contractions(ctx, ops, oracle):
    """tcg_contract_sum against the oracle's contractions added up in fp64:
    the LSTM weight-gradient shape family (operands {F,1,B} x {G,1,B} summed over
    the batch, one term per time step) on the matrix cores, both operand orders,
    int32 and odd shapes through the term-by-term route (bit-exact there)."""
    from tenncor_amd import capi
    rng = np.random.default_rng(seed_of("contract_sum"))
    cases = [
        (np.float32, [96, 1, 64], [160, 1, 64], [[1, 1], [2, 2]], 9),     # K = 64 per term: one product over 576
        (np.float32, [64, 48], [64, 80], [[0, 0]], 5),                    # K contiguous in both operands
        (np.float32, [40, 1, 6], [24, 1, 6], [[1, 1], [2, 2]], 4),        # K = 6: term by term
        (np.int32, [32, 1, 16], [48, 1, 16], [[1, 1], [2, 2]], 6),
        (np.float64, [32, 1, 16], [48, 1, 16], [[1, 1], [2, 2]], 3),
    ]
    for np_dtype, ashape, bshape, pairs, nterms in cases:
        na, nb = int(np.prod(ashape)), int(np.prod(bshape))
        draw = (lambda n: rng.integers(-50, 51, n).astype(np.int32)) if np_dtype == np.int32 else \
            (lambda n: rng.uniform(-1, 1, n).astype(np_dtype))
        xs, ys = [draw(na) for _ in range(nterms)], [draw(nb) for _ in range(nterms)]
        refs = [oracle.contract(x, ashape, y, bshape, pairs, wide_acc=np_dtype != np.int32)[0] for x, y in zip(xs, ys)]
        da, db = [ctx.upload(x) for x in xs], [ctx.upload(y) for y in ys]
        out = ctx.empty(refs[0].size, np_dtype)
        ctx.contract_sum(capi.dtype_code(np_dtype), ashape, bshape, pairs, [d.ptr for d in da], [d.ptr for d in db], out.ptr)
        got = out.get()[:refs[0].size]
        if np_dtype == np.int32:
            total = refs[0].copy()
            for r in refs[1:]:
                total = (total.astype(np.int64) + r).astype(np.int32)
            np.testing.assert_array_equal(got, total)
        else:
            assert_acc_close(got, np.sum(np.asarray(refs, dtype=np.float64), axis=0), rtol=ACC_RTOL if np_dtype == np.float32 else 1e-12)
        # one term is the contraction itself
        ctx.contract_sum(capi.dtype_code(np_dtype), ashape, bshape, pairs, [da[0].ptr], [db[0].ptr], out.ptr)
        single = ctx.empty(refs[0].size, np_dtype)
        ctx.contract(capi.dtype_code(np_dtype), ashape, bshape, pairs, da[0].ptr, db[0].ptr, single.ptr)
        np.testing.assert_array_equal(out.get(), single.get())
        for d in da + db + [out, single]:
            d.release()


def test_concat_bit_exact(ctx, ops, oracle):
    rng = np.random.default_rng(13)
    sa, sb = [256, 1, 16], [512, 1, 16]
    a = rng.standard_normal(oracle.n_elems(sa)).astype(np.float32)
    b = rng.standard_normal(oracle.n_elems(sb)).astype(np.float32)
    out = ops.concat([ops.from_host(ctx, a, sa), ops.from_host(ctx, b, sb)], 0)
    ref, oshape = oracle.concat([a, b], [sa, sb], 0)
    assert out.shape == oshape
    np.testing.assert_array_equal(out.get(), ref)
    # n-ary form along the sequence dim
    shapes = [[48, 1, 5]] * 9
    xs = [rng.integers(-99, 99, 240).astype(np.int32) for _ in shapes]
    out = ops.concat([ops.from_host(ctx, x, s) for x, s in zip(xs, shapes)], 1)
    ref, oshape = oracle.concat(xs, shapes, 1)
    assert out.shape == oshape
    np.testing.assert_array_equal(out.get(), ref)


@pytest.mark.parametrize("np_dtype", [np.float32, np.float64, np.int32])
def test_concat_of_many_operands_is_one_pass(ctx, ops, oracle, np_dtype):
    """Three operands and more are gathered by one launch through a table of
    where each starts along the axis: equal and ragged extents, the axis first,
    in the middle and last, rows that allow 16-byte accesses and rows that do not."""
    rng = np.random.default_rng(seed_of("concat_many", str(np_dtype)))
    cases = [
        (1, [[512, 1, 6]] * 64),                                   # the outputs of 64 steps of a recurrent layer
        (0, [[3, 5, 2], [1, 5, 2], [7, 5, 2], [4, 5, 2]]),         # ragged along the fastest dim
        (2, [[6, 5, 1], [6, 5, 4], [6, 5, 2]]),                    # along the slowest dim
        (1, [[8, 2, 3], [8, 1, 3], [8, 9, 3], [8, 1, 3], [8, 1, 3]]),
        (1, [[5, k + 1, 3, 2] for k in range(17)]),                # odd rows: element by element
    ]
    for axis, shapes in cases:
        from tenncor_amd import capi
        xs = [(rng.integers(-1000, 1000, oracle.n_elems(s))).astype(np_dtype) for s in shapes]
        ref, oshape = oracle.concat(xs, shapes, axis)
        # (the node API only groups operands of extent 1 along the axis, cfg/ops.yml:613-653; the kernel takes any)
        bufs = [ctx.upload(x) for x in xs]
        out = ctx.empty(ref.size, np_dtype)
        ctx.concat(capi.dtype_code(np_dtype), axis, [oracle.shape8(s) for s in shapes], [b.ptr for b in bufs], out.ptr)
        np.testing.assert_array_equal(out.get(), ref, err_msg=str((axis, shapes[:2])))
        for b in bufs + [out]:
            b.release()


MATMUL_CASES = [
    ([10, 3], [9, 10]), ([64, 64], [64, 64]), ([100, 37], [53, 100]), ([256, 128], [192, 256]),
    ([768, 256], [2048, 768]), ([32, 48, 5], [40, 32, 5]), ([128, 128, 3, 2], [128, 128, 3, 2]),
    ([513, 130], [259, 513]), ([1024, 512], [512, 1024]),
]


@pytest.mark.parametrize("ashape,bshape", MATMUL_CASES, ids=[str(c) for c in MATMUL_CASES])
def test_matmul_vs_oracle(ctx, ops, oracle, ashape, bshape):
    rng = np.random.default_rng(seed_of(ashape, bshape))
    a = rng.standard_normal(oracle.n_elems(ashape)).astype(np.float32)
    b = (rng.standard_normal(oracle.n_elems(bshape)) / np.sqrt(ashape[0])).astype(np.float32)
    out = ops.matmul(ops.from_host(ctx, a, ashape), ops.from_host(ctx, b, bshape))
    ref, oshape = oracle.matmul(a, ashape, b, bshape, wide_acc=True)
    assert out.shape == oshape
    assert_acc_close(out.get(), ref)
    if oracle.n_elems(ashape) <= 1 << 16:
        ai = rng.integers(-2 ** 15, 2 ** 15, oracle.n_elems(ashape)).astype(np.int32)
        bi = rng.integers(-2 ** 15, 2 ** 15, oracle.n_elems(bshape)).astype(np.int32)
        outi = ops.matmul(ops.from_host(ctx, ai, ashape), ops.from_host(ctx, bi, bshape))
        np.testing.assert_array_equal(outi.get(), oracle.matmul(ai, ashape, bi, bshape)[0])  # wraps, exact
        ad, bd = a.astype(np.float64), b.astype(np.float64)
        outd = ops.matmul(ops.from_host(ctx, ad, ashape), ops.from_host(ctx, bd, bshape))
        np.testing.assert_allclose(outd.get(), oracle.matmul(ad, ashape, bd, bshape)[0], rtol=1e-10, atol=1e-12)


GEMM_CASES = [
    # (M, N, K, batch, trans_a, trans_b): sizes on the matrix-core path (multiples of 4, >= 32)
    (128, 128, 64, 1, 0, 0), (128, 128, 64, 1, 1, 0), (128, 128, 64, 1, 0, 1), (128, 128, 64, 1, 1, 1),
    (100, 36, 40, 1, 0, 0), (100, 36, 40, 3, 1, 1), (260, 132, 72, 2, 1, 0), (260, 132, 72, 2, 0, 1),
    (512, 384, 200, 1, 0, 0), (2048, 256, 768, 1, 1, 0), (768, 2048, 256, 1, 0, 1),
    # few tiles, long K: several workgroups share a tile (K split in ranges, last one ragged)
    (256, 768, 2048, 1, 0, 1), (256, 2048, 768, 1, 0, 0), (64, 96, 1000, 2, 1, 0), (36, 44, 4100, 1, 0, 0),
    (12, 32, 2048, 1, 0, 0), (24, 8, 1024, 1, 1, 0), (8, 20, 600, 3, 0, 1),
    # tall with few columns (a convolution lowered to a product): tiles 32 or 64 columns wide
    (33000, 32, 40, 1, 0, 0), (33000, 24, 40, 1, 1, 0), (131300, 32, 24, 1, 0, 1), (2100, 28, 52, 16, 1, 1),
    (33000, 64, 40, 1, 0, 0), (33000, 40, 36, 1, 1, 1), (4200, 64, 72, 8, 0, 1),
    # K a whole number of 16-slabs: operands go from memory straight into LDS; ragged M and N in every
    # layout, for the 128 x 128 tiles (one round, and K ranges), the 128 x 64 ones and the 64 x 64 ones
    (2052, 2052, 32, 1, 0, 0), (2052, 2052, 32, 1, 1, 0), (2052, 2052, 32, 1, 0, 1), (2052, 2052, 32, 1, 1, 1),
    (516, 644, 1600, 1, 0, 0), (516, 644, 1600, 1, 1, 1), (644, 516, 1616, 1, 1, 0), (644, 516, 1616, 1, 0, 1),
    (33000, 60, 48, 1, 0, 0), (33000, 60, 48, 1, 1, 0), (4200, 64, 80, 8, 0, 1), (4200, 44, 80, 8, 1, 1),
    (100, 36, 48, 3, 1, 1), (260, 132, 80, 2, 0, 1), (260, 132, 80, 2, 1, 0), (68, 68, 16, 5, 0, 0),
    # ... and the 128 x 32 tiles of a tall result with few columns (waves 4 x 1)
    (33000, 32, 48, 1, 0, 0), (33000, 24, 48, 1, 1, 0), (131300, 32, 32, 1, 0, 1), (2100, 28, 64, 16, 1, 1),
    (33000, 32, 1024, 1, 0, 0),
    # off the matrix-core path: odd extents
    (33, 35, 17, 2, 0, 0), (33, 35, 17, 2, 1, 1),
]


@pytest.mark.parametrize("M,N,K,batch,ta,tb", GEMM_CASES, ids=[str(c) for c in GEMM_CASES])
def test_gemm_transposed_operands_vs_oracle(ctx, oracle, M, N, K, batch, ta, tb):
    """tcg_gemm with every operand layout a contraction can lower to."""
    from tenncor_amd import capi
    rng = np.random.default_rng(seed_of(M, N, K, batch, ta, tb))
    a = rng.standard_normal(batch * M * K).astype(np.float32)
    b = (rng.standard_normal(batch * K * N) / np.sqrt(K)).astype(np.float32)
    # oracle works on the canonical layout a{K,M,batch}, b{N,K,batch}
    a_can = a if not ta else oracle.permute(a, [M, K, batch], [1, 0, 2])[0]
    b_can = b if not tb else oracle.permute(b, [K, N, batch], [1, 0, 2])[0]
    ref, _ = oracle.matmul(a_can, [K, M, batch], b_can, [N, K, batch], wide_acc=True)
    da, db = ctx.upload(a), ctx.upload(b)
    dc = ctx.empty(batch * M * N, np.float32)
    ctx.gemm(capi.FLOAT, M, N, K, batch, da.ptr, M if ta else K, M * K, ta,
             db.ptr, K if tb else N, K * N, tb, dc.ptr, N, M * N)
    assert_acc_close(dc.get(), ref)


@pytest.mark.parametrize("np_dtype,K", [(np.float64, 32), (np.float64, 8), (np.float32, 64), (np.float32, 16)])
def test_gemm_infinity_in_the_last_slab_stays_an_infinity(ctx, np_dtype, K):
    """The matrix-core kernels fetch slabs past the end of K again to keep their
    loads countable; what those steps multiply must not reach the result (an
    infinity times a zero would be a NaN)."""
    from tenncor_amd import capi
    M = N = 256
    A, B = np.ones((M, K), np_dtype), np.ones((K, N), np_dtype)
    B[K - 1, 5] = np.inf
    a, b, c = ctx.upload(A.ravel()), ctx.upload(B.ravel()), ctx.empty(M * N, np_dtype)
    ctx.gemm(capi.dtype_code(np_dtype), M, N, K, 1, a.ptr, K, 0, 0, b.ptr, N, 0, 0, c.ptr, N, 0)
    out = c.get().reshape(M, N)
    assert np.isposinf(out[:, 5]).all() and not np.isnan(out).any()
    assert (np.delete(out, 5, axis=1) == K).all()


GEMM_F64_CASES = [
    # on the fp64 matrix-core path: even extents, enough tiles to fill the chip
    (1024, 1024, 64, 1, 0, 0), (1024, 1024, 64, 1, 1, 0), (1024, 1024, 64, 1, 0, 1), (1024, 1024, 64, 1, 1, 1),
    (1500, 1100, 42, 1, 0, 0), (1500, 1100, 42, 1, 1, 1), (2048, 2050, 130, 1, 1, 0), (2050, 2048, 130, 1, 0, 1),
    (260, 132, 72, 24, 0, 0), (260, 132, 72, 24, 1, 0), (132, 260, 10, 24, 0, 1), (100, 36, 40, 80, 1, 1),
    # off it: odd extents, few tiles
    (1025, 1023, 33, 1, 0, 0), (128, 128, 64, 1, 0, 0), (33, 35, 17, 2, 1, 1),
]


@pytest.mark.parametrize("M,N,K,batch,ta,tb", GEMM_F64_CASES, ids=[str(c) for c in GEMM_F64_CASES])
def test_gemm_f64_transposed_operands_vs_oracle(ctx, oracle, M, N, K, batch, ta, tb):
    """tcg_gemm in double: the matrix-core kernel and the generic one sum over k in ascending order."""
    from tenncor_amd import capi
    rng = np.random.default_rng(seed_of(M, N, K, batch, ta, tb, 64))
    a = rng.standard_normal(batch * M * K)
    b = rng.standard_normal(batch * K * N) / np.sqrt(K)
    a_can = a if not ta else oracle.permute(a, [M, K, batch], [1, 0, 2])[0]
    b_can = b if not tb else oracle.permute(b, [K, N, batch], [1, 0, 2])[0]
    ref, _ = oracle.matmul(a_can, [K, M, batch], b_can, [N, K, batch])
    da, db = ctx.upload(a), ctx.upload(b)
    dc = ctx.empty(batch * M * N, np.float64)
    ctx.gemm(capi.DOUBLE, M, N, K, batch, da.ptr, M if ta else K, M * K, ta,
             db.ptr, K if tb else N, K * N, tb, dc.ptr, N, M * N)
    assert_acc_close(dc.get(), ref, rtol=1e-12)


SMALL_GEMM_CASES = [(128, 10, 64, 1, 0, 0), (64, 10, 128, 1, 1, 0), (20, 12, 300, 5, 1, 1), (7, 9, 33, 3, 0, 1),
                    (1, 1, 4000, 1, 0, 0), (128, 128, 32, 1, 0, 0)]


@pytest.mark.parametrize("np_dtype", [np.float32, np.float64, np.int32])
@pytest.mark.parametrize("M,N,K,batch,ta,tb", SMALL_GEMM_CASES, ids=[str(c) for c in SMALL_GEMM_CASES])
def test_small_products_with_a_long_k(ctx, oracle, M, N, K, batch, ta, tb, np_dtype):
    """Few results, K of 32 or more: every lane owns one result and walks K in
    ascending order (int32 exact; fp32 against the oracle accumulating in
    double at 1e-4 of the largest entry, fp64 at 1e-12)."""
    from tenncor_amd import capi
    rng = np.random.default_rng(seed_of(M, N, K, batch, ta, tb, str(np_dtype)))
    if np_dtype == np.int32:
        a = rng.integers(-2000, 2000, batch * M * K).astype(np.int32)
        b = rng.integers(-2000, 2000, batch * K * N).astype(np.int32)
    else:
        a = rng.standard_normal(batch * M * K).astype(np_dtype)
        b = (rng.standard_normal(batch * K * N) / np.sqrt(K)).astype(np_dtype)
    a_can = a if not ta else oracle.permute(a, [M, K, batch], [1, 0, 2])[0]
    b_can = b if not tb else oracle.permute(b, [K, N, batch], [1, 0, 2])[0]
    ref, _ = oracle.matmul(a_can, [K, M, batch], b_can, [N, K, batch], wide_acc=(np_dtype == np.float32))
    da, db = ctx.upload(a), ctx.upload(b)
    dc = ctx.empty(batch * M * N, np_dtype)
    ctx.gemm(capi.dtype_code(np.dtype(np_dtype)), M, N, K, batch, da.ptr, M if ta else K, M * K, ta,
             db.ptr, K if tb else N, K * N, tb, dc.ptr, N, M * N)
    if np_dtype == np.int32:
        np.testing.assert_array_equal(dc.get(), ref)
    else:
        assert_acc_close(dc.get(), ref, rtol=ACC_RTOL if np_dtype == np.float32 else 1e-12)


CONTRACT_CASES = [
    ([10, 3], [9, 10], [[0, 1]]),                      # dense layer (config 1)
    ([768, 1, 64], [512, 768], [[0, 1]]),              # LSTM gate product (config 4)
    ([64, 1, 1, 32], [10, 64], [[0, 1]]),              # CNN dense head (config 5)
    ([4, 2, 3], [2, 4, 2], [[0, 1], [1, 2]]),          # reference golden shape
    ([12, 7], [12, 9], [[0, 0]]),                      # both contracted-inner
    ([7, 12], [9, 12], [[1, 1]]),                      # both contracted-outer
    ([7, 12], [12, 9], [[1, 0]]),
    ([5, 6, 7], [6, 4], [[1, 0]]),                     # a needs repacking
    ([5, 6, 7], [7, 3, 5], [[0, 2], [2, 0]]),          # b's order differs
    ([3, 4, 5, 6], [5, 2, 3], [[0, 2], [2, 0]]),
]


@pytest.mark.parametrize("ashape,bshape,pairs", CONTRACT_CASES, ids=[str(c) for c in CONTRACT_CASES])
def test_contract_vs_oracle(ctx, ops, oracle, ashape, bshape, pairs):
    rng = np.random.default_rng(seed_of(ashape, bshape))
    a = rng.standard_normal(oracle.n_elems(ashape)).astype(np.float32)
    b = rng.standard_normal(oracle.n_elems(bshape)).astype(np.float32)
    out = ops.contract(ops.from_host(ctx, a, ashape), ops.from_host(ctx, b, bshape), pairs)
    ref, oshape = oracle.contract(a, ashape, b, bshape, pairs, wide_acc=True)
    assert out.shape == oshape
    assert_acc_close(out.get(), ref)
    ai = rng.integers(-999, 999, a.size).astype(np.int32)
    bi = rng.integers(-999, 999, b.size).astype(np.int32)
    outi = ops.contract(ops.from_host(ctx, ai, ashape), ops.from_host(ctx, bi, bshape), pairs)
    np.testing.assert_array_equal(outi.get(), oracle.contract(ai, ashape, bi, bshape, pairs)[0])


CONV_CASES = [
    ([3, 3], [2], [1]),
    ([2, 4, 3, 3], [1, 2, 2, 1], list(range(8))),            # tenncor/test/test_api.cpp:2265
    ([1, 12, 12, 4, 5], [3, 1, 5, 5], [4, 0, 1, 2]),          # conv2d idiom, small
    ([4, 10, 9, 2, 5], [3, 4, 5, 6], [4, 0, 1, 2]),           # tenncor/test/test_api.cpp:2505 shapes
    ([4, 10, 9, 2, 5], [1, 6, 4, 2, 3], list(range(8))),      # kernel-gradient form
    ([20, 16], [5, 3], [0, 1]),
]


@pytest.mark.parametrize("ishape,kshape,ranks", CONV_CASES, ids=[str(c) for c in CONV_CASES])
def test_conv_vs_oracle(ctx, ops, oracle, ishape, kshape, ranks):
    rng = np.random.default_rng(seed_of(ishape, kshape))
    img = rng.uniform(-1, 1, oracle.n_elems(ishape)).astype(np.float32)
    ker = rng.uniform(-1, 1, oracle.n_elems(kshape)).astype(np.float32)
    out = ops.convolution(ops.from_host(ctx, img, ishape), ops.from_host(ctx, ker, kshape), ranks)
    ref, oshape = oracle.conv(img, ishape, ker, kshape, ranks, wide_acc=True)
    assert out.shape == oshape
    assert_acc_close(out.get(), ref)
    ii = rng.integers(-99, 99, img.size).astype(np.int32)
    ki = rng.integers(-99, 99, ker.size).astype(np.int32)
    outi = ops.convolution(ops.from_host(ctx, ii, ishape), ops.from_host(ctx, ki, kshape), ranks)
    np.testing.assert_array_equal(outi.get(), oracle.conv(ii, ishape, ki, kshape, ranks)[0])


def test_conv_boxed_skips_padding_and_unread_outputs(ctx, ops, oracle):
    """The conv2d idiom and its image-gradient idiom: an image that is zero
    outside a box, and an output of which only a window is read.  Inside the
    window the result must equal the plain correlation bit for bit in int32
    (skipped terms are exact zeros) and to 1e-4 in fp32."""
    from tenncor_amd import capi
    rng = np.random.default_rng(77)
    C, W, H, B, O, KW, KH = 3, 7, 6, 2, 4, 3, 2
    for np_dtype in (np.int32, np.float32):
        if np_dtype == np.int32:
            x = rng.integers(-50, 50, C * W * H * B).astype(np.int32)
            k = rng.integers(-50, 50, O * C * KW * KH).astype(np.int32)
        else:
            x = rng.uniform(-1, 1, C * W * H * B).astype(np.float32)
            k = rng.uniform(-1, 1, O * C * KW * KH).astype(np.float32)
        dt = capi.dtype_code(np_dtype)
        # forward idiom: PAD dim 4 by (O-1, O-1), kernel dims -> image dims {4,0,1,2}
        padded, pshape = oracle.pad(x, [C, W, H, B], [[0, 0]] * 4 + [[O - 1, O - 1]])
        ref, oshape = oracle.conv(padded, pshape, k, [O, C, KW, KH], [4, 0, 1, 2], wide_acc=np_dtype == np.float32)
        dimg, dker = ctx.upload(padded), ctx.upload(k)
        out = ctx.empty(oracle.n_elems(oshape), np_dtype)
        lo = [0, 0, 0, 0, O - 1, 0, 0, 0]
        hi = [C, W, H, B, O, 1, 1, 1]
        ctx.conv_boxed(dt, pshape, [O, C, KW, KH], [4, 0, 1, 2], (lo, hi), None, dimg.ptr, dker.ptr, out.ptr)
        if np_dtype == np.int32:
            np.testing.assert_array_equal(out.get(), ref)
        else:
            assert_acc_close(out.get(), ref)
        # output window: only index 1 of dim 4 is asked for; the rest stays as it was
        sentinel = np.full(oracle.n_elems(oshape), 12345, dtype=np_dtype)
        ctx.h2d(out.ptr, sentinel)
        wlo = [0, 0, 0, 0, 1, 0, 0, 0]
        whi = list(oshape)
        whi[4] = 2
        ctx.conv_boxed(dt, pshape, [O, C, KW, KH], [4, 0, 1, 2], (lo, hi), (wlo, whi), dimg.ptr, dker.ptr, out.ptr)
        got = out.get().reshape(oshape[::-1])
        want = ref.reshape(oshape[::-1])
        if np_dtype == np.int32:
            np.testing.assert_array_equal(got[:, :, :, 1], want[:, :, :, 1])
        else:
            assert_acc_close(got[:, :, :, 1], want[:, :, :, 1])
        assert (got[:, :, :, 0] == 12345).all() and (got[:, :, :, 2:] == 12345).all()


def conv2d_idiom_cases(C, W, H, B, O, KW, KH):
    """(image shape, kernel shape, ranks, image box, output window) of conv2d's
    forward, image-gradient and kernel-gradient convolutions
    (cfg/tenncor/nn.yml:48-98 and the CONV rules of tenncor/eteq/backprop.hpp)."""
    OW, OH = W - KW + 1, H - KH + 1
    one = [1, 1, 1]
    fwd = ([C, W, H, B, 2 * O - 1] + one, [O, C, KW, KH], [4, 0, 1, 2],
           ([0, 0, 0, 0, O - 1, 0, 0, 0], [C, W, H, B, O] + one), None)
    # gradient of the padded image: supgrad {1,OW,OH,B,O} padded by K-1 on every kernel dim
    gshape = [2 * C - 1, OW + 2 * (KW - 1), OH + 2 * (KH - 1), B, 3 * O - 2] + one
    dgrad = (gshape, [O, C, KW, KH], [4, 0, 1, 2],
             ([C - 1, KW - 1, KH - 1, 0, O - 1, 0, 0, 0], [C, KW - 1 + OW, KH - 1 + OH, B, 2 * O - 1] + one),
             ([0, 0, 0, 0, O - 1, 0, 0, 0], [C, W, H, B, O] + one))
    # gradient of the kernel: the padded image correlated with supgrad as the kernel
    wgrad = ([C, W, H, B, 2 * O - 1] + one, [1, OW, OH, B, O], list(range(8)),
             ([0, 0, 0, 0, O - 1, 0, 0, 0], [C, W, H, B, O] + one), None)
    return {"forward": fwd, "image_gradient": dgrad, "kernel_gradient": wgrad}


@pytest.mark.parametrize("which", ["forward", "image_gradient", "kernel_gradient"])
def test_conv_as_matrix_product_equals_direct_kernels(ctx, oracle, which):
    """The three convolutions of a conv2d layer at a size where tcg_conv_boxed
    takes the matrix-product route (with a small row chunk, so that several
    passes are made), against the direct kernels: equal bit for bit in int32
    (both sum exact products, the skipped terms are zeros), 1e-4 in fp32."""
    from tenncor_amd import capi
    ishape, kshape, ranks, ibox, obox = conv2d_idiom_cases(C=12, W=15, H=13, B=12, O=24, KW=3, KH=4)[which]
    rng = np.random.default_rng(seed_of("convgemm", which))
    n_img, n_ker = oracle.n_elems(ishape), oracle.n_elems(kshape)
    oshape = oracle.conv_shape(ishape, kshape, ranks)
    n_out = oracle.n_elems(oshape)
    lo, hi = ibox
    # zero outside the box, as PAD leaves it... except where nothing may look
    inside = np.ones(ishape[::-1], dtype=bool)
    for d in range(8):
        idx = np.arange(ishape[d])
        keep = (idx >= lo[d]) & (idx < hi[d])
        shape = [1] * 8
        shape[7 - d] = ishape[d]
        inside &= keep.reshape(shape)
    inside = inside.reshape(-1)
    for np_dtype in (np.int32, np.float32, np.float64):
        if np_dtype == np.int32:
            img = rng.integers(-40, 41, n_img).astype(np.int32)
            ker = rng.integers(-40, 41, n_ker).astype(np.int32)
        else:
            img = rng.uniform(-1, 1, n_img).astype(np_dtype)
            ker = rng.uniform(-1, 1, n_ker).astype(np_dtype)
        img[~inside] = 12345  # garbage outside the box must never be read
        dt = capi.dtype_code(np_dtype)
        dimg, dker = ctx.upload(img), ctx.upload(ker)
        results = {}
        for route, env in (("direct", {"TCG_CONV_GEMM": "0"}), ("product", {"TCG_CONV_GEMM": "1", "TCG_CONV_CHUNK_ROWS": "128"})):
            os.environ.update(env)
            try:
                out = ctx.upload(np.full(n_out, 777, dtype=np_dtype))
                ctx.conv_boxed(dt, ishape, kshape, ranks, ibox, obox, dimg.ptr, dker.ptr, out.ptr)
                results[route] = out.get()
            finally:
                for key in env:
                    os.environ.pop(key, None)
        if np_dtype == np.int32:
            np.testing.assert_array_equal(results["product"], results["direct"])
        else:
            assert_acc_close(results["product"], results["direct"], ACC_RTOL if np_dtype == np.float32 else 1e-12)
        if obox is not None:
            # outside the window the destination keeps what it held
            untouched = results["direct"] == 777
            assert untouched.any() and (results["product"][untouched] == 777).all()
        # the same correlations from the box alone (the image never laid out
        # with its border): the same bits as from the padded image, by either route
        box, _ = oracle.slice_(img, ishape, [[lo[d], hi[d] - lo[d]] for d in range(8)])
        dbox = ctx.upload(box)
        for route, env in (("direct", {"TCG_CONV_GEMM": "0"}), ("product", {"TCG_CONV_GEMM": "1", "TCG_CONV_CHUNK_ROWS": "128"})):
            os.environ.update(env)
            try:
                out = ctx.upload(np.full(n_out, 777, dtype=np_dtype))
                ctx.conv_dense_box(dt, ishape, kshape, ranks, ibox, obox, dbox.ptr, dker.ptr, out.ptr)
                np.testing.assert_array_equal(out.get(), results[route])
            finally:
                for key in env:
                    os.environ.pop(key, None)


def test_kept_convolution_tables_are_counted_and_found_again():
    """The row / summed-index tables of a convolution lowered to a product stay
    with the context (outside its pool): tcg_mem_stats_kept counts them, a second
    correlation of the same plan finds them again instead of adding to them,
    and neither call leaves anything handed out."""
    from tenncor_amd import capi
    from oracle import oracle as orc
    own = capi.Context(0)
    try:
        ishape, kshape, ranks, ibox, obox = conv2d_idiom_cases(C=12, W=15, H=13, B=12, O=24, KW=3, KH=4)["forward"]
        rng = np.random.default_rng(seed_of("kept tables"))
        img = rng.uniform(-1, 1, orc.n_elems(ishape)).astype(np.float32)
        ker = rng.uniform(-1, 1, orc.n_elems(kshape)).astype(np.float32)
        n_out = orc.n_elems(orc.conv_shape(ishape, kshape, ranks))
        dimg, dker, out = own.upload(img), own.upload(ker), own.empty(n_out, np.float32)
        assert own.mem_stats_kept() == 0
        in_use = own.mem_stats()[0]
        own.conv_boxed(capi.FLOAT, ishape, kshape, ranks, ibox, obox, dimg.ptr, dker.ptr, out.ptr)
        first = out.get().copy()
        kept = own.mem_stats_kept()
        assert 0 < kept <= 256 << 20
        own.conv_boxed(capi.FLOAT, ishape, kshape, ranks, ibox, obox, dimg.ptr, dker.ptr, out.ptr)
        np.testing.assert_array_equal(out.get(), first)
        assert own.mem_stats_kept() == kept
        assert own.mem_stats()[0] == in_use
    finally:
        own.close()


@pytest.mark.parametrize("which", ["forward", "image_gradient", "kernel_gradient"])
@pytest.mark.parametrize("channels", [(8, 32), (6, 36)], ids=["groups_of_four", "element_by_element"])
def test_conv_product_reading_the_image_in_place(ctx, oracle, which, channels):
    """fp32 convolutions whose matrix product gathers its left operand from the
    image while multiplying (nothing materialised), with channel counts that
    allow 128-bit gathers and ones that do not, against the same product with
    the operand materialised first and against the direct kernels (1e-4).
    Elements outside the box hold garbage that must never be read."""
    from tenncor_amd import capi
    C, O = channels
    ishape, kshape, ranks, ibox, obox = conv2d_idiom_cases(C=C, W=15, H=13, B=12, O=O, KW=3, KH=4)[which]
    rng = np.random.default_rng(seed_of("convimplicit", which, C))
    n_img, n_ker = oracle.n_elems(ishape), oracle.n_elems(kshape)
    n_out = oracle.n_elems(oracle.conv_shape(ishape, kshape, ranks))
    lo, hi = ibox
    img = rng.uniform(-1, 1, n_img).astype(np.float32)
    ker = rng.uniform(-1, 1, n_ker).astype(np.float32)
    box, _ = oracle.slice_(img, ishape, [[lo[d], hi[d] - lo[d]] for d in range(8)])
    inside = np.ones(ishape[::-1], dtype=bool)
    for d in range(8):
        idx = np.arange(ishape[d])
        shape = [1] * 8
        shape[7 - d] = ishape[d]
        inside &= ((idx >= lo[d]) & (idx < hi[d])).reshape(shape)
    img[~inside.reshape(-1)] = 12345
    dimg, dbox, dker = ctx.upload(img), ctx.upload(box), ctx.upload(ker)
    results = {}
    # (operands whose groups of four are not aligned are materialised by either product route)
    routes = (("direct", {"TCG_CONV_GEMM": "0"}), ("materialised", {"TCG_CONV_IMPLICIT": "0"}), ("in_place", {}),
              ("in_place_chunked", {"TCG_CONV_CHUNK_ROWS": "192"}))
    for route, env in routes:
        os.environ.update(env)
        try:
            out = ctx.upload(np.full(n_out, 777, dtype=np.float32))
            ctx.conv_boxed(capi.FLOAT, ishape, kshape, ranks, ibox, obox, dimg.ptr, dker.ptr, out.ptr)
            results[route] = out.get()
            out = ctx.upload(np.full(n_out, 777, dtype=np.float32))
            ctx.conv_dense_box(capi.FLOAT, ishape, kshape, ranks, ibox, obox, dbox.ptr, dker.ptr, out.ptr)
            np.testing.assert_array_equal(out.get(), results[route])
        finally:
            for key in env:
                os.environ.pop(key, None)
    for route in ("materialised", "in_place", "in_place_chunked"):
        assert_acc_close(results[route], results["direct"])


@pytest.mark.parametrize("np_dtype", [np.float32, np.int32, np.float64])
def test_pad_interior_writes_the_operand_and_nothing_else(ctx, oracle, np_dtype):
    """tcg_pad_interior against PAD: equal to the oracle's padded tensor inside
    the operand's box, the destination's earlier content everywhere else; a
    convolution clipped to the box then gives the PAD + CONV result."""
    from tenncor_amd import capi
    rng = np.random.default_rng(1234)
    dt = capi.dtype_code(np_dtype)
    for shape, pads in (([8, 5, 3], [[4, 4], [0, 2], [1, 0]]), ([3, 7, 6, 2], [[0, 0]] * 4 + [[3, 3]]),
                        ([5], [[2, 6]]), ([4, 4], [[0, 0], [0, 0]])):
        n = oracle.n_elems(shape)
        x = rng.integers(1, 90, n).astype(np_dtype)
        ref, pshape = oracle.pad(x, shape, pads)
        before = [p[0] for p in pads]
        after = [p[1] for p in pads]
        sentinel = np.full(oracle.n_elems(pshape), 77777, dtype=np_dtype)
        out, src = ctx.upload(sentinel), ctx.upload(x)
        ctx.pad_interior(dt, shape, before, after, src.ptr, out.ptr)
        got = out.get()
        # the oracle's padding is zero and the operand is >= 1: zeros mark the border
        inside = ref != 0
        np.testing.assert_array_equal(got[inside], ref[inside])
        assert (got[~inside] == 77777).all()
        assert inside.sum() == n


def test_api_convolution_golden_on_gpu(ctx, ops):
    fx = EQV["api_convolution"]
    out = ops.convolution(ops.from_host(ctx, np.array(fx["data"]), fx["alist"]),
                          ops.from_host(ctx, np.array(fx["data2"]), fx["blist"]), list(range(8)))
    assert out.shape == fx["expectslist"]
    np.testing.assert_array_equal(out.get(), np.array(fx["expect_out"]))


def test_matmul_chain_golden_on_gpu(ctx, ops):
    """tenncor/test/test_equation.cpp:26-87 in double."""
    fx = EQV["matmul_complex"]
    a, b, c = (ops.from_host(ctx, np.array(fx[k]), fx[s]) for k, s in (("data", "alist"), ("data2", "blist"), ("data3", "clist")))
    d = ops.matmul(a, b)
    e = ops.matmul(c, d)
    f = ops.matmul(ops.permute(d, [1, 0]), ops.permute(c, [1, 0]))
    dest = ops.matmul(e, f)
    np.testing.assert_allclose(dest.get(), np.array(fx["expect_dest"]), rtol=1e-14)


def test_errors_are_reported_not_thrown_across_the_abi(ctx, ops):
    from tenncor_amd import capi
    a = ops.from_host(ctx, np.zeros(12, np.float32), [4, 3])
    with pytest.raises(capi.TcgError) as info:
        ctx.extend(capi.FLOAT, [4, 3], [2, 1], a.ptr, a.ptr)
    assert "non-singular" in str(info.value)
    with pytest.raises(capi.TcgError):
        ctx.permute(capi.FLOAT, [4, 3], [0, 0, 2, 3, 4, 5, 6, 7], a.ptr, a.ptr)
    with pytest.raises(capi.TcgError):
        ctx.ew_unary("ADD", capi.FLOAT, 12, a.ptr, a.ptr)
    with pytest.raises(capi.TcgError):
        ctx.ew_unary("EXP", 99, 12, a.ptr, a.ptr)  # no such element type


def test_pool_recycles_blocks(ctx):
    in_use0, _ = ctx.mem_stats()
    p = ctx.alloc(1 << 20)
    ctx.free(p, 1 << 20)
    q = ctx.alloc(1 << 20)
    assert q == p  # stream-ordered reuse without going back to the driver
    ctx.free(q, 1 << 20)
    assert ctx.mem_stats()[0] == in_use0


def test_full_size_properties_config2(ctx, ops):
    """[4096,16384] tensors: properties that need no CPU pass over 256 MiB."""
    from tenncor_amd import capi
    rng = np.random.default_rng(2)
    shape = [16384, 4096]
    n = 16384 * 4096
    xi = rng.integers(-1000, 1001, n, dtype=np.int32)
    yi = rng.integers(-1000, 1001, n, dtype=np.int32)
    tx, ty = ops.from_host(ctx, xi, shape), ops.from_host(ctx, yi, shape)
    prod = ops.binary("MUL", ops.binary("ADD", tx, ty), ty)
    # checksum of checksums: reducing dim 0 then dim 1 == reducing dim 1 then dim 0 == all at once
    r0 = ops.reduce("REDUCE_SUM", ops.reduce("REDUCE_SUM", prod, [0]), [1]).get()
    r1 = ops.reduce("REDUCE_SUM", ops.reduce("REDUCE_SUM", prod, [1]), [0]).get()
    rall = ops.reduce("REDUCE_SUM", prod, [0, 1]).get()
    want = np.int64(((xi.astype(np.int64) + yi) * yi).sum()).astype(np.int32)  # mod 2^32
    assert r0[0] == r1[0] == rall[0] == want
    m0 = ops.reduce("REDUCE_MAX", ops.reduce("REDUCE_MAX", prod, [0]), [1]).get()
    assert m0[0] == ops.reduce("REDUCE_MAX", prod, [0, 1]).get()[0] == ((xi.astype(np.int64) + yi) * yi).max()
    # row sums against numpy on the first and last rows
    rows = ops.reduce("REDUCE_SUM", prod, [0]).get()
    p_host = ((xi.astype(np.int64) + yi) * yi).astype(np.int32).reshape(4096, 16384)
    np.testing.assert_array_equal(rows, p_host.sum(axis=1, dtype=np.int32))
    cols = ops.reduce("REDUCE_SUM", prod, [1]).get()
    np.testing.assert_array_equal(cols, p_host.sum(axis=0, dtype=np.int32))
    # PERMUTE twice is the identity; a transposed row is a column
    tt = ops.permute(ops.permute(prod, [1, 0]), [1, 0])
    np.testing.assert_array_equal(tt.get(), p_host.reshape(-1))
    np.testing.assert_array_equal(ops.permute(prod, [1, 0]).get().reshape(16384, 4096)[5], p_host[:, 5])


def test_full_size_config2_fp32_chain_and_reductions(ctx, ops, oracle):
    """configs[1] in fp32 at np[4096,16384]: ADD, MUL, EXP, TANH, SIGMOID node by
    node, every intermediate against the oracle on 256 seeded rows and 256 seeded
    columns at 1e-5 (the oracle runs on the slices: elementwise results do not
    depend on their neighbours), then REDUCE_SUM / REDUCE_MAX over each dim
    against an fp64 sum of the chain result the device itself produced, at 1e-4
    of max(|ref|, mean|ref|) -- 16384-long fp32 row sums are the case where a
    sequential fp32 accumulation would fail that bar -- and the same reductions
    of the oracle's own chain result over the checked rows and columns."""
    rng = np.random.default_rng(2)
    shape = [16384, 4096]
    rows_n, cols_n = 4096, 16384
    n = rows_n * cols_n
    a, b, c = (rng.uniform(-1, 1, n).astype(np.float32) for _ in range(3))
    ta, tb, tc = (ops.from_host(ctx, v, shape) for v in (a, b, c))
    t1 = ops.binary("ADD", ta, tb)
    t2 = ops.binary("MUL", t1, tc)
    t3 = ops.unary("EXP", t2)
    t4 = ops.unary("TANH", t3)
    t5 = ops.unary("SIGMOID", t4)
    rsel = np.sort(rng.choice(rows_n, 256, replace=False))
    csel = np.sort(rng.choice(cols_n, 256, replace=False))

    def pick(flat):
        m = flat.reshape(rows_n, cols_n)
        return np.ascontiguousarray(m[rsel]).reshape(-1), np.ascontiguousarray(m[:, csel]).reshape(-1)

    sa, sb, sc = pick(a), pick(b), pick(c)
    chain_ref = []
    for k in range(2):  # rows, then columns
        r1 = oracle.binary("ADD", sa[k], sb[k])
        r2 = oracle.binary("MUL", r1, sc[k])
        r3 = oracle.unary("EXP", r2)
        r4 = oracle.unary("TANH", r3)
        r5 = oracle.unary("SIGMOID", r4)
        chain_ref.append((r1, r2, r3, r4, r5))
    final = None
    for idx, t in enumerate((t1, t2, t3, t4, t5)):
        got = t.get()
        for k in range(2):
            ref = chain_ref[k][idx]
            sel = pick(got)[k]
            if idx < 2:
                np.testing.assert_array_equal(sel, ref)  # one rounding each: the same bits
            else:
                np.testing.assert_allclose(sel, ref, rtol=EW_RTOL, atol=0)
        final = got
    assert np.isfinite(final).all()
    # the chain as one group launch (at this size: non-temporal operand loads, two
    # indices in flight per lane) gives the bits of the five separate launches
    from tenncor_amd import capi
    L, R, NONE = capi.FX_LEAF0, capi.FX_REG0, capi.FX_NONE
    group = [("ADD", L, L + 1, NONE, R), ("MUL", R, L + 2, NONE, R), ("EXP", R, NONE, NONE, R),
             ("TANH", R, NONE, NONE, R), ("SIGMOID", R, NONE, NONE, R), ("STORE", R, NONE, NONE, 0)]
    fused = ctx.empty(n, np.float32)
    ctx.ew_fusedx(capi.FLOAT, shape, [{"ptr": v.buf.ptr} for v in (ta, tb, tc)], group, [fused.ptr])
    np.testing.assert_array_equal(fused.get(), final)
    # ... also when the extent leaves a tail behind the whole tiles
    odd = [16384, 4095]
    ctx.fill_zero(fused.ptr, 4 * n)
    ctx.ew_fusedx(capi.FLOAT, odd, [{"ptr": v.buf.ptr} for v in (ta, tb, tc)], group, [fused.ptr])
    np.testing.assert_array_equal(fused.get()[:16384 * 4095], final[:16384 * 4095])
    assert not fused.get()[16384 * 4095:].any()
    fused.release()
    m64 = final.reshape(rows_n, cols_n).astype(np.float64)
    for rank_set, axis in (([0], 1), ([1], 0)):
        got_sum = ops.reduce("REDUCE_SUM", t5, rank_set).get()
        assert_acc_close(got_sum, m64.sum(axis=axis))
        got_max = ops.reduce("REDUCE_MAX", t5, rank_set).get()
        np.testing.assert_array_equal(got_max, final.reshape(rows_n, cols_n).max(axis=axis))
    # the same against the oracle's chain: row sums of the checked rows, and the
    # oracle's own reduction (fp64 accumulation) of those rows
    got_rows = ops.reduce("REDUCE_SUM", t5, [0]).get()[rsel]
    ref_rows, _ = oracle.reduce("REDUCE_SUM", chain_ref[0][4], [cols_n, 256], [0], wide_acc=True)
    assert_acc_close(got_rows, ref_rows)
    got_cols = ops.reduce("REDUCE_SUM", t5, [1]).get()[csel]
    ref_cols, _ = oracle.reduce("REDUCE_SUM", chain_ref[1][4], [256, rows_n], [1], wide_acc=True)
    assert_acc_close(got_cols, ref_cols)
    ref_max, _ = oracle.reduce("REDUCE_MAX", chain_ref[0][4], [cols_n, 256], [0])
    np.testing.assert_allclose(ops.reduce("REDUCE_MAX", t5, [0]).get()[rsel], ref_max, rtol=EW_RTOL)
    # inputs whose sums do not hide errors behind a large mean: the signed product t2
    # (row sums are O(sqrt(n)) around zero), relative to max(|ref|, mean|ref|)
    p64 = t2.get().reshape(rows_n, cols_n).astype(np.float64)
    for rank_set, axis in (([0], 1), ([1], 0)):
        assert_acc_close(ops.reduce("REDUCE_SUM", t2, rank_set).get(), p64.sum(axis=axis))
        np.testing.assert_array_equal(ops.reduce("REDUCE_MIN", t2, rank_set).get(),
                                      t2.get().reshape(rows_n, cols_n).min(axis=axis))


def test_full_size_properties_config3(ctx, ops):
    """4096^3 fp32 MATMUL and the batched [64,512,512] product at full size,
    checked without a CPU product: C r against A (B r) in fp64 for a random
    vector r (Freivalds), at the 1e-4 bar relative to the largest entry; the
    int32 product of the same shape exactly (mod 2^32); PERMUTE of the result
    is an involution and moves rows to columns; the 4096^3 product in double
    by Freivalds at 1e-12."""
    rng = np.random.default_rng(3)
    n = 4096
    a = (rng.standard_normal(n * n) / 64).astype(np.float32)
    b = (rng.standard_normal(n * n) / 64).astype(np.float32)
    ta, tb = ops.from_host(ctx, a, [n, n]), ops.from_host(ctx, b, [n, n])
    c = ops.matmul(ta, tb)
    got = c.get().reshape(n, n).astype(np.float64)
    r = rng.standard_normal(n)
    want = a.reshape(n, n).astype(np.float64) @ (b.reshape(n, n).astype(np.float64) @ r)
    assert np.abs(got @ r - want).max() <= ACC_RTOL * np.abs(want).max()
    rt = rng.standard_normal(n)   # and from the left: r^T C = (r^T A) B
    want = (rt @ a.reshape(n, n).astype(np.float64)) @ b.reshape(n, n).astype(np.float64)
    assert np.abs(rt @ got - want).max() <= ACC_RTOL * np.abs(want).max()
    ct = ops.permute(c, [1, 0])
    np.testing.assert_array_equal(ops.permute(ct, [1, 0]).get(), c.get())
    np.testing.assert_array_equal(ct.get().reshape(n, n)[7], c.get().reshape(n, n)[:, 7])
    # int32: exact modulo 2^32 whatever the order of summation
    ai = rng.integers(-1000, 1001, n * n, dtype=np.int32)
    bi = rng.integers(-1000, 1001, n * n, dtype=np.int32)
    ci = ops.matmul(ops.from_host(ctx, ai, [n, n]), ops.from_host(ctx, bi, [n, n])).get().reshape(n, n)
    ri = rng.integers(-3, 4, n).astype(np.int64)
    want = ai.reshape(n, n).astype(np.int64) @ (bi.reshape(n, n).astype(np.int64) @ ri)
    np.testing.assert_array_equal((ci.astype(np.int64) @ ri).astype(np.int32), want.astype(np.int32))
    # the same product in double on the fp64 matrix cores: Freivalds in extended
    # precision, at 1e-12 relative to the largest entry
    ad, bd = a.astype(np.float64), b.astype(np.float64)
    cd = ops.matmul(ops.from_host(ctx, ad, [n, n]), ops.from_host(ctx, bd, [n, n])).get().reshape(n, n)
    rl = r.astype(np.longdouble)
    want = ad.reshape(n, n).astype(np.longdouble) @ (bd.reshape(n, n).astype(np.longdouble) @ rl)
    assert np.abs(cd.astype(np.longdouble) @ rl - want).max() <= 1e-12 * np.abs(want).max()
    want = (rl @ ad.reshape(n, n).astype(np.longdouble)) @ bd.reshape(n, n).astype(np.longdouble)
    assert np.abs(rl @ cd.astype(np.longdouble) - want).max() <= 1e-12 * np.abs(want).max()
    # batched: np[64,512,512] x np[64,512,512], every batch by Freivalds
    m, nb = 512, 64
    a3 = (rng.standard_normal(nb * m * m) / 22).astype(np.float32)
    b3 = (rng.standard_normal(nb * m * m) / 22).astype(np.float32)
    c3 = ops.matmul(ops.from_host(ctx, a3, [m, m, nb]), ops.from_host(ctx, b3, [m, m, nb]))
    got = c3.get().reshape(nb, m, m).astype(np.float64)
    r = rng.standard_normal(m)
    want = np.einsum("bij,bj->bi", a3.reshape(nb, m, m).astype(np.float64),
                     np.einsum("bij,j->bi", b3.reshape(nb, m, m).astype(np.float64), r))
    assert np.abs(got @ r - want).max() <= ACC_RTOL * np.abs(want).max()
    swapped = ops.permute(c3, [1, 0, 2]).get().reshape(nb, m, m)
    np.testing.assert_array_equal(swapped, got.astype(np.float32).transpose(0, 2, 1))


@pytest.mark.parametrize("config", ["lstm", "cnn"])
def test_full_size_recordings_equal_the_walk(config):
    """configs[3] and configs[4] at their full sizes: the recorded pass (shared
    launches, exchanged products, convolutions reading their operands in
    place) against the node-by-node walk on the same input, bit for bit --
    except where a sum of products runs as one product, where a product reads
    the parts of a concatenation instead of its laid-out copy (K in chunks of
    the parts), and where a convolution reads an operand through the PERMUTE in
    front of it (its sums then run along the operand's memory): other orders of
    the same fp32 additions, held to 1e-5 of the largest entry."""
    from tenncor_amd import graph, configs
    results = {}
    for kind in ("plain", "replay_launches"):
        graph.set_evaluator(kind)
        g = graph.Graph()
        try:
            targets = (configs.config4_lstm if config == "lstm" else configs.config5_cnn)(g)[0]
            for _ in range(3):  # walked, recorded, replayed
                g.evaluate(targets)
            results[kind] = [t.get().copy() for t in targets]
            if kind != "plain":
                st = graph.evaluator_stats()
                assert st["recorded"] == 1 and st["launches"] < 0.4 * g.count_functors(targets) + 40
        finally:
            g.close()
            graph.set_evaluator("default")
    for k, (a, b) in enumerate(zip(results["plain"], results["replay_launches"])):
        assert np.isfinite(a).all()
        if config == "lstm":
            # the walk computes the weight gradient as 64 products and adds them up, the
            # recording as one product per block over the concatenated summed index; the
            # products of a step sum over the parts of [x_t, h] and of the gate gradients
            # in chunks -- the bar of a contraction, against the largest entry
            assert np.abs(a - b).max() <= 1e-5 * np.abs(a).max()
            continue
        if config == "cnn":
            # the image gradient of the second layer sums over (channel, kx, ky) with the
            # channel first in the recording and last in the walk; the first layer's kernel
            # gradient is computed from it
            assert np.abs(a - b).max() <= 1e-5 * np.abs(a).max()
            continue
        np.testing.assert_array_equal(a, b)


@pytest.mark.parametrize("np_dtype", [np.float32, np.int32, np.float64])
def test_fused_group_with_views_and_several_outputs(ctx, oracle, np_dtype):
    """tcg_ew_fusedx against the same nodes evaluated one by one by the oracle:
    an LSTM-cell shaped group reading four SLICE views of one matrix, an
    EXTEND view of a bias row and a PAD view, storing three results.  The
    fused kernel uses the scalar routines of the one-node kernels, so fp32
    results are held to the elementwise bar and int32 ones to bit equality."""
    from tenncor_amd import capi
    rng = np.random.default_rng(seed_of("fusedx", str(np_dtype)))
    dt = capi.dtype_code(np_dtype)
    for H, B in ((8, 5), (7, 3), (64, 12)):
        if np_dtype == np.int32:
            draw = lambda n: rng.integers(-9, 10, n).astype(np.int32)
        else:
            draw = lambda n: rng.uniform(-1, 1, n).astype(np_dtype)
        gates = draw(4 * H * B)          # teq shape [4H, B]
        state = draw(H * B)              # [H, B]
        bias = draw(H)                   # [H] extended over B
        small = draw((H - 2) * B)        # [H-2, B] padded by (1, 1) along dim 0
        # the graph, node by node on the oracle
        sl = [oracle.slice_(gates, [4 * H, B], [[k * H, H]])[0] for k in range(4)]
        bext = oracle.extend(bias, [H], [1, B])[0]
        padded = oracle.pad(small, [H - 2, B], [[1, 1]])[0]
        g = oracle.unary("TANH", oracle.binary("ADD", sl[0], bext))
        i = oracle.unary("SIGMOID", sl[1])
        f = oracle.unary("SIGMOID", sl[2])
        o = oracle.unary("ABS", sl[3])
        new_state = oracle.nary("ADD", [oracle.binary("MUL", g, i), oracle.binary("MUL", state, f), padded])
        hidden = oracle.binary("MUL", new_state, o)
        picked = oracle.select(oracle.binary("GT", hidden, np.full(H * B, 0.25).astype(np_dtype)), hidden,
                               oracle.binary("MUL", hidden, np.full(H * B, 2).astype(np_dtype)))
        dg, ds, db, dp = ctx.upload(gates), ctx.upload(state), ctx.upload(bias), ctx.upload(small)
        L, R = capi.FX_LEAF0, capi.FX_REG0
        leaves = [{"ptr": dg.ptr, "offset": k * H, "stride": [1, 4 * H] + [4 * H * B] * 6} for k in range(4)]
        leaves.append({"ptr": ds.ptr})
        leaves.append({"ptr": db.ptr, "stride": [1, 0, 0, 0, 0, 0, 0, 0]})
        leaves.append({"ptr": dp.ptr, "offset": -1, "stride": [1, H - 2] + [(H - 2) * B] * 6,
                       "lo": [1, 0, 0, 0, 0, 0, 0, 0], "hi": [H - 1, B, 1, 1, 1, 1, 1, 1]})
        N = capi.FX_NONE
        prog = [
            ("ADD", L + 0, L + 5, N, R + 0),
            ("TANH", R + 0, N, N, R + 0),
            ("SIGMOID", L + 1, N, N, R + 1),
            ("SIGMOID", L + 2, N, N, R + 2),
            ("ABS", L + 3, N, N, R + 3),
            ("MUL", R + 0, R + 1, N, R + 4),
            ("MUL", L + 4, R + 2, N, R + 5),
            ("ADD", R + 4, R + 5, N, R + 6),
            ("ADD", R + 6, L + 6, N, R + 6),
            ("STORE", R + 6, N, N, 0),
            ("MUL", R + 6, R + 3, N, R + 7),
            ("STORE", R + 7, N, N, 1),
            ("GT", R + 7, capi.FX_IMM, N, R + 8, 0.25),
            ("MUL", R + 7, capi.FX_IMM, N, R + 9, 2.0),
            ("SELECT", R + 8, R + 7, R + 9, R + 10),
            ("STORE", R + 10, N, N, 2),
        ]
        outs = [ctx.empty(H * B, np_dtype) for _ in range(3)]
        ctx.ew_fusedx(dt, [H, B], leaves, prog, [o_.ptr for o_ in outs])
        for got, want in zip(outs, (new_state, hidden, picked)):
            if np_dtype == np.int32:
                np.testing.assert_array_equal(got.get(), want)
            else:
                np.testing.assert_allclose(got.get(), want, rtol=EW_RTOL, atol=1e-7)


def test_fused_group_rejects_malformed_programs(ctx):
    from tenncor_amd import capi
    x = ctx.upload(np.ones(16, np.float32))
    out = ctx.empty(16, np.float32)
    L, R, N = capi.FX_LEAF0, capi.FX_REG0, capi.FX_NONE
    bad = [
        [("NEG", L + 1, N, N, R + 0), ("STORE", R + 0, N, N, 0)],      # leaf that does not exist
        [("NEG", R + 3, N, N, R + 0), ("STORE", R + 0, N, N, 0)],      # register never written
        [("NEG", L + 0, N, N, R + 0)],                                 # output never stored
        [("MATMUL", L + 0, L + 0, N, R + 0), ("STORE", R + 0, N, N, 0)],
        [("NEG", L + 0, N, N, R + 16), ("STORE", R + 0, N, N, 0)],
    ]
    for prog in bad:
        with pytest.raises(capi.TcgError):
            ctx.ew_fusedx(capi.FLOAT, [16], [{"ptr": x.ptr}], prog, [out.ptr])


def test_interpreted_groups_match_too():
    """TCG_FX_JIT=0 sends fused groups to the interpreting kernel instead of a
    kernel compiled for the program; the switch is read once per process, so the
    group tests and the LSTM replay test are run again in a child process."""
    import subprocess
    import sys
    here = os.path.dirname(os.path.abspath(__file__))
    env = dict(os.environ, TCG_FX_JIT="0")
    cmd = [sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider",
           os.path.join(here, "test_gpu_ops.py"), os.path.join(here, "test_gpu_replay.py"),
           "-k", "fused_group_with_views or fused_lstm or fused_views"]
    done = subprocess.run(cmd, env=env, cwd=os.path.dirname(here), stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True, timeout=300)
    assert done.returncode == 0, done.stdout[-3000:]
    assert " passed" in done.stdout


# ---- device RAND_UNIF --------------------------------------------------------

@pytest.mark.parametrize("np_dtype", [np.float32, np.float64, np.int32])
def test_device_generator_is_bit_exact_with_the_restated_stream(ctx, oracle, np_dtype):
    """Bit-exact against the CPU restatement of Philox4x32-10 (itself pinned by
    the published known-answer vectors): ragged sizes, consecutive draws that
    continue one stream, a restart under a new seed."""
    rng = np.random.default_rng(11)
    seed = 0x5eed0000cafe
    ctx.rand_seed(seed)
    assert ctx.rand_state() == (seed, 0)
    per = 2 if np_dtype == np.float64 else 4
    drawn = 0
    for n in (1, 3, 5, 64, 1000003):
        if np_dtype == np.int32:
            lo = rng.integers(-1000, 1000, n).astype(np.int32)
            hi = (lo + rng.integers(0, 5000, n)).astype(np.int32)
            if n > 4:
                lo[1], hi[1] = -2 ** 31, 2 ** 31 - 1
                lo[2], hi[2] = 9, 3
        else:
            lo = rng.uniform(-3, 1, n).astype(np_dtype)
            hi = (lo + rng.uniform(0, 4, n)).astype(np_dtype)
        dlo, dhi, out = ctx.upload(lo), ctx.upload(hi), ctx.empty(n, np_dtype)
        ctx.rand_uniform(out.dtype, n, dlo.ptr, dhi.ptr, out.ptr)
        got = out.get()
        np.testing.assert_array_equal(got, oracle.rand_uniform(lo, hi, seed, first_block=drawn))
        drawn += (n + per - 1) // per
        assert ctx.rand_state() == (seed, drawn)
        if np_dtype != np.int32:
            assert np.all(got >= lo) and np.all(got <= hi)
        for buf in (dlo, dhi, out):
            buf.release()
    ctx.rand_seed(77)
    lo, hi = np.zeros(10, np_dtype), np.full(10, 100, np_dtype)
    dlo, dhi, out = ctx.upload(lo), ctx.upload(hi), ctx.empty(10, np_dtype)
    ctx.rand_uniform(out.dtype, 10, dlo.ptr, dhi.ptr, out.ptr)
    np.testing.assert_array_equal(out.get(), oracle.rand_uniform(lo, hi, 77))


def test_device_generator_draws_anew_at_every_launch_of_a_recording(ctx, oracle):
    n, seed = 1000, 2024
    lo, hi = np.full(n, -1, np.float32), np.full(n, 1, np.float32)
    dlo, dhi, out = ctx.upload(lo), ctx.upload(hi), ctx.empty(n, np.float32)
    ctx.rand_seed(seed)
    ctx.sync()
    ctx.capture_begin()
    ctx.rand_uniform(out.dtype, n, dlo.ptr, dhi.ptr, out.ptr)
    graph = ctx.capture_end()
    for launch in range(4):
        ctx.graph_launch(graph)
        np.testing.assert_array_equal(out.get(), oracle.rand_uniform(lo, hi, seed, first_block=launch * 250))
    assert ctx.rand_state() == (seed, 1000)
    ctx.graph_destroy(graph)


@pytest.mark.parametrize("np_dtype", [np.float32, np.int32, np.float64])
@pytest.mark.parametrize("case", ["forward", "transposed_weight", "weight_gradient_block", "odd"])
def test_sum_of_products_over_parts_of_tensors(ctx, oracle, case, np_dtype):
    """tcg_gemm_terms: a contraction over a dim along which an operand is a
    concatenation, computed from the parts where they lie -- each term with its
    own leading dim (a row slice of a [batch, seq, n] input has rows seq * n
    apart), the other operand's rows taken by pointer offset, the result
    written into a block of a wider matrix.  Against the product of the
    materialised concatenation (int32 exactly; fp32 at 1e-4 of the oracle
    accumulating in double; fp64 at 1e-12)."""
    from tenncor_amd import capi
    rng = np.random.default_rng(seed_of("gemm_terms", case, str(np_dtype)))
    esz = np.dtype(np_dtype).itemsize

    def draw(n):
        if np_dtype == np.int32:
            return rng.integers(-2000, 2000, n).astype(np.int32)
        return (rng.standard_normal(n) / 8).astype(np_dtype)

    if case == "forward":
        # [x_t, h] . W with x_t a slice of x[batch][seq][nin]: three terms of K = 128
        # (enough 32x32 blocks for the kernel whose waves share K)
        batch, seq, nin, hid, N, t = 256, 5, 128, 256, 2048, 3
        x, h, w = draw(batch * seq * nin), draw(batch * hid), draw((nin + hid) * N)
        xt = x.reshape(batch, seq, nin)[:, t, :]
        ref = np.concatenate([xt, h.reshape(batch, hid)], axis=1).astype(np.float64) @ w.reshape(nin + hid, N).astype(np.float64)
        dx, dh, dw = ctx.upload(x), ctx.upload(h), ctx.upload(w)
        K = 128
        a = [dx.ptr + t * nin * esz, dh.ptr, dh.ptr + K * esz]
        lda = [seq * nin, hid, hid]
        b = [dw.ptr, dw.ptr + K * N * esz, dw.ptr + 2 * K * N * esz]
        M, ldb, ta, tb, ldc, coff, cols = batch, [N] * 3, 0, 0, N, 0, N
    elif case == "transposed_weight":
        # sum_g dgate_g . W[:, g-th block]^T, only the columns 64.. of the result, into a wider buffer
        batch, hid, rows = 64, 128, 192
        gates = [draw(batch * hid) for _ in range(4)]
        w = draw(rows * 4 * hid)
        full = np.concatenate([g.reshape(batch, hid) for g in gates], axis=1).astype(np.float64) @ w.reshape(rows, 4 * hid).astype(np.float64).T
        n0 = 64
        ref = full[:, n0:]
        dg = [ctx.upload(g) for g in gates]
        dw = ctx.upload(w)
        K, M, cols = hid, batch, rows - n0
        a, lda = [d.ptr for d in dg], [hid] * 4
        b = [dw.ptr + (n0 * 4 * hid + g * hid) * esz for g in range(4)]
        ldb, ta, tb, ldc, coff = [4 * hid] * 4, 0, 1, rows, n0
    elif case == "weight_gradient_block":
        # sum_t h_t^T . dgate_t into the block (rows 32.., columns 128..) of dW
        steps, batch, hid, gate = 6, 64, 96, 128
        hs, gs = [draw(batch * hid) for _ in range(steps)], [draw(batch * gate) for _ in range(steps)]
        ref = sum(h.reshape(batch, hid).astype(np.float64).T @ g.reshape(batch, gate).astype(np.float64) for h, g in zip(hs, gs))
        dh, dgt = [ctx.upload(h) for h in hs], [ctx.upload(g) for g in gs]
        K, M, cols = batch, hid, gate
        a, lda, b, ldb = [d.ptr for d in dh], [hid] * steps, [d.ptr for d in dgt], [gate] * steps
        ta, tb, ldc, coff = 1, 0, 384, 32 * 384 + 128
    else:
        # nothing aligned: term by term on the generic kernels
        M, cols, K = 7, 9, 5
        As, Bs = [draw(M * K) for _ in range(3)], [draw(K * cols) for _ in range(3)]
        ref = sum(x.reshape(M, K).astype(np.float64) @ y.reshape(K, cols).astype(np.float64) for x, y in zip(As, Bs))
        da, db = [ctx.upload(x) for x in As], [ctx.upload(y) for y in Bs]
        a, lda, b, ldb, ta, tb, ldc, coff = [d.ptr for d in da], [K] * 3, [d.ptr for d in db], [cols] * 3, 0, 0, cols + 3, 1
    rows_c = M + (2 if case == "weight_gradient_block" else 0) + 40
    out = ctx.upload(np.full(rows_c * ldc + 8, 777, dtype=np_dtype))
    ctx.gemm_terms(capi.dtype_code(np_dtype), M, cols, K, a, lda, ta, b, ldb, tb, out.ptr + coff * esz, ldc)
    got = out.get()
    block = np.array([got[coff + m * ldc: coff + m * ldc + cols] for m in range(M)])
    if np_dtype == np.int32:
        np.testing.assert_array_equal(block, ref.astype(np.int64).astype(np.int32))
    else:
        assert_acc_close(block, ref, ACC_RTOL if np_dtype == np.float32 else 1e-12)
    # nothing outside the block was written
    mask = np.ones(got.size, bool)
    for m in range(M):
        mask[coff + m * ldc: coff + m * ldc + cols] = False
    assert (got[mask] == 777).all()


@pytest.mark.parametrize("jit", ["1", "0"])
def test_product_ranges_are_added_by_the_launch_that_reads_them(ctx, jit):
    """tcg_gemm_terms_ranges leaves the K ranges of a sum of products side by
    side and a tcg_ew_fusedx operand with nsum > 1 adds them in range order
    while it loads: the product backwards through a recurrent step
    (cfg/tenncor/layer.yml:716-768, tenncor/eteq/backprop.hpp:269-359: the four
    gate gradients times the transposed weight, few results under a long K) then
    needs no launch of its own for the sum.  The ranges added on the host in
    fp32, in order, fix every bit of what the reading launch must see; their sum
    is held against the product in double at 1e-4.  The run-time compiled kernel
    (both lane widths, a boxed operand) and the interpreter are covered; the
    interpreter runs in a process of its own, the switch being read once."""
    import subprocess
    import sys
    if jit == "0":
        if os.environ.get("TCG_FX_JIT") != "0":
            env = dict(os.environ, TCG_FX_JIT="0")
            here = os.path.abspath(__file__)
            res = subprocess.run([sys.executable, "-m", "pytest", "-q", "-x", here + "::" +
                                  "test_product_ranges_are_added_by_the_launch_that_reads_them"],
                                 env=env, capture_output=True, text=True, timeout=600)
            assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-2000:]
            return
    from tenncor_amd import capi
    rng = np.random.default_rng(seed_of("ranges", jit))
    batch, hid, rows, n0, R = 64, 128, 192, 64, 8
    gates = [(rng.standard_normal(batch * hid) / 8).astype(np.float32) for _ in range(4)]
    w = (rng.standard_normal(rows * 4 * hid) / 8).astype(np.float32)
    full = np.concatenate([g.reshape(batch, hid) for g in gates], axis=1).astype(np.float64) @ w.reshape(rows, 4 * hid).astype(np.float64).T
    ref = full[:, n0:]
    M, N, K = batch, rows - n0, hid
    dg = [ctx.upload(g) for g in gates]
    dw = ctx.upload(w)
    a, lda = [d.ptr for d in dg], [hid] * 4
    b, ldb = [dw.ptr + (n0 * 4 * hid + g * hid) * 4 for g in range(4)], [4 * hid] * 4
    guard = 64
    parts = ctx.upload(np.full(R * M * N + 2 * guard, 777, np.float32))
    ctx.gemm_terms_ranges(capi.FLOAT, M, N, K, a, lda, 0, b, ldb, 1, R, parts.ptr + guard * 4)
    got = parts.get()
    assert (got[:guard] == 777).all() and (got[-guard:] == 777).all()
    ranges = got[guard:-guard].reshape(R, M, N)
    want = ranges[0].copy()
    for r in range(1, R):
        want = want + ranges[r]  # fp32, in range order
    assert_acc_close(want, ref, ACC_RTOL)
    # every range is the product over its part of K
    for r in (0, R - 1):
        k0, k1 = r * 4 * K // R, (r + 1) * 4 * K // R
        cat = np.concatenate([g.reshape(batch, hid) for g in gates], axis=1).astype(np.float64)
        piece = cat[:, k0:k1] @ w.reshape(rows, 4 * hid).astype(np.float64).T[k0:k1, n0:]
        assert_acc_close(ranges[r], piece, ACC_RTOL)
    other = (rng.standard_normal(M * N) / 8).astype(np.float32)
    dother = ctx.upload(other)
    # out0 = sum of the ranges * other; out1 = sum of the ranges (128-bit lanes)
    out0, out1 = ctx.empty(M * N, np.float32), ctx.empty(M * N, np.float32)
    leaf = {"ptr": parts.ptr, "offset": guard, "nsum": R, "sum_stride": M * N}
    prog = [("MUL", capi.FX_LEAF0, capi.FX_LEAF0 + 1, capi.FX_NONE, capi.FX_REG0), ("STORE", capi.FX_REG0, capi.FX_NONE, capi.FX_NONE, 0),
            ("STORE", capi.FX_LEAF0, capi.FX_NONE, capi.FX_NONE, 1)]
    ctx.ew_fusedx(capi.FLOAT, [N, M], [leaf, {"ptr": dother.ptr}], prog, [out0.ptr, out1.ptr])
    np.testing.assert_array_equal(out1.get().reshape(M, N), want)
    np.testing.assert_array_equal(out0.get().reshape(M, N), want * other.reshape(M, N))
    # a window of the sums read through a border of zeros, one element per lane:
    # rows 3.. and columns 5.. of the result, shifted by (2, 1) into a [N - 4, M - 2] box
    shape = [N - 4, M - 2]
    view = {"ptr": parts.ptr, "offset": guard + 3 * N + 5 - (2 * N + 1), "stride": [1, N] + [0] * 6,
            "lo": [1, 2] + [0] * 6, "hi": [N - 5 + 1, M - 3 + 2] + [1] * 6, "nsum": R, "sum_stride": M * N}
    out2 = ctx.empty(shape[0] * shape[1], np.float32)
    ctx.ew_fusedx(capi.FLOAT, shape, [view], [("NEG", capi.FX_LEAF0, capi.FX_NONE, capi.FX_NONE, capi.FX_REG0),
                                              ("STORE", capi.FX_REG0, capi.FX_NONE, capi.FX_NONE, 0)], [out2.ptr])
    expect = np.zeros((shape[1], shape[0]), np.float32)
    hi_m, hi_n = min(shape[1], M - 3 + 2), min(shape[0], N - 5 + 1)
    expect[2:hi_m, 1:hi_n] = want[3:3 + hi_m - 2, 5:5 + hi_n - 1]
    np.testing.assert_array_equal(out2.get().reshape(shape[1], shape[0]), -expect)
    # shapes the matrix cores do not take are refused, not approximated
    with pytest.raises(RuntimeError, match="tcg_gemm_terms_ranges"):
        ctx.gemm_terms_ranges(capi.FLOAT, M, N, K, a, lda, 0, b, ldb, 1, 3, parts.ptr + guard * 4)
    with pytest.raises(RuntimeError, match="tcg_gemm_terms_ranges"):
        ctx.gemm_terms_ranges(capi.INT32, M, N, K, a, lda, 0, b, ldb, 1, R, parts.ptr + guard * 4)


@pytest.mark.parametrize("np_dtype", [np.float32, np.int32])
@pytest.mark.parametrize("case", ["one_product", "block_by_block"])
def test_blocks_of_a_sum_of_products_over_concatenated_operands(ctx, oracle, case, np_dtype):
    """tcg_gemm_terms_grid: dW = sum_t [x_t, h_t]^T [g0_t .. g3_t], the weight
    gradient of a recurrent cell (tenncor/eteq/backprop.hpp:269-359 over the
    CONCAT and the ADD of PADs of cfg/tenncor/layer.yml:716-768), from the
    parts where they lie.  With parts of whole 128-row / column tiles the fp32
    blocks run as one matrix-core product; other extents and int32 go block by
    block.  Against the sum of products of the laid-out concatenations (fp32
    at 1e-4 of a double accumulation, int32 exactly), with a guard band round
    the result in a wider matrix."""
    from tenncor_amd import capi
    rng = np.random.default_rng(seed_of("grid", case, str(np_dtype)))
    esz = 4
    steps, batch = 5, 64
    if case == "one_product":
        Mp, Np = [128, 256], [128, 128, 256]
    else:
        Mp, Np = [96, 40], [128, 72]

    def draw(n):
        if np_dtype == np.int32:
            return rng.integers(-50, 51, n).astype(np.int32)
        return (rng.standard_normal(n) / 4).astype(np.float32)

    # x parts live in one [batch][steps][Mp0] tensor (rows steps * Mp0 apart), h parts are tensors of their own
    x = draw(batch * steps * Mp[0])
    hs = [draw(batch * Mp[1]) for _ in range(steps)]
    gs = [[draw(batch * n) for _ in range(steps)] for n in Np]
    dx, dh = ctx.upload(x), [ctx.upload(h) for h in hs]
    dg = [[ctx.upload(v) for v in part] for part in gs]
    a_ptrs = [[dx.ptr + t * Mp[0] * esz for t in range(steps)], [d.ptr for d in dh]]
    lda = [steps * Mp[0], Mp[1]]
    b_ptrs = [[d.ptr for d in part] for part in dg]
    ldb = list(Np)
    M, N = sum(Mp), sum(Np)
    ldc, guard = N + 12, 64
    out = ctx.upload(np.full(guard + M * ldc + guard, 777, np_dtype))
    ctx.gemm_terms_grid(capi.dtype_code(np_dtype), Mp, Np, batch, a_ptrs, lda, 1, b_ptrs, ldb, 0,
                        out.ptr + guard * esz, ldc)
    got = out.get()
    assert (got[:guard] == 777).all() and (got[-guard:] == 777).all()
    C = got[guard:-guard].reshape(M, ldc)
    assert (C[:, N:] == 777).all()
    want = np.zeros((M, N), np.float64)
    x3 = x.reshape(batch, steps, Mp[0])
    for t in range(steps):
        left = np.concatenate([x3[:, t, :], hs[t].reshape(batch, Mp[1])], axis=1).astype(np.float64)
        right = np.concatenate([gs[j][t].reshape(batch, Np[j]) for j in range(len(Np))], axis=1).astype(np.float64)
        want += left.T @ right
    if np_dtype == np.int32:
        np.testing.assert_array_equal(C[:, :N], want.astype(np.int64).astype(np.int32))
    else:
        assert_acc_close(C[:, :N], want, ACC_RTOL)
