"""Pins the CPU oracle against the vectors the reference's own tests hold
(tests/golden/*.json), against numpy library routines and against brute force.
A mistake in the oracle (dropped term, wrong index, transposed operand) must
fail at least one of these."""
import json
import math
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

with open(os.path.join(GOLDEN, "operator_goldens.json")) as f:
    OPG = json.load(f)
with open(os.path.join(GOLDEN, "equation_vectors.json")) as f:
    EQV = json.load(f)


def run_case(orc, case, dtype=np.float64):
    """Evaluate one golden case with the oracle; returns (flat data, shape)."""
    op = case["op"]
    args = [np.asarray(a["data"], dtype=dtype) for a in case["args"]]
    shapes = [a["shape"] for a in case["args"]]
    if op in ("REDUCE_SUM", "REDUCE_PROD", "REDUCE_MIN", "REDUCE_MAX"):
        return orc.reduce(op, args[0], shapes[0], case["rank_set"])
    if op == "ARGMAX":
        return orc.argmax(args[0], shapes[0], case["rank"])
    if op == "EXTEND":
        return orc.extend(args[0], shapes[0], case["dimensions"])
    if op == "PERMUTE":
        return orc.permute(args[0], shapes[0], case["ranks"])
    if op == "SLICE":
        return orc.slice_(args[0], shapes[0], case["dimension_pairs"])
    if op == "PAD":
        return orc.pad(args[0], shapes[0], case["dimension_pairs"])
    if op == "STRIDE":
        return orc.stride(args[0], shapes[0], case["dimensions"])
    if op == "SCATTER":
        return orc.scatter(args[0], shapes[0], case["dimensions"], case["outshape"])
    if op == "REVERSE":
        return orc.reverse(args[0], shapes[0], case["rank_set"])
    if op == "CONCAT":
        return orc.concat(args, shapes, case["rank"])
    if op == "SELECT":
        return orc.select(*args), orc.shape8(shapes[0])
    if op == "CONTRACT":
        return orc.contract(args[0], shapes[0], args[1], shapes[1], case["rank_pairs"])
    if op == "CONV":
        return orc.conv(args[0], shapes[0], args[1], shapes[1], case["ranks"])
    if op in ("ADD", "MUL") and len(args) != 2:
        return orc.nary(op, args), orc.shape8(shapes[0])
    return orc.binary(op, args[0], args[1]), orc.shape8(shapes[0])


@pytest.mark.parametrize("case", OPG["cases"], ids=[c["name"] for c in OPG["cases"]])
def test_operator_goldens(oracle, case):
    got, shape = run_case(oracle, case)
    assert list(shape) == oracle.shape8(case["outshape"])
    expect = np.asarray(case["expect"], dtype=np.float64)
    if "tol" in case:
        np.testing.assert_allclose(got, expect, rtol=case["tol"], atol=0)
    else:
        # EXPECT_VECEQ / EXPECT_EQ in the reference: exact
        np.testing.assert_array_equal(got, expect)


CLOSED = {
    "abs": abs, "neg": lambda e: -e, "sin": math.sin, "cos": math.cos, "tan": math.tan,
    "exp": math.exp, "log": math.log, "sqrt": math.sqrt,
    "round_half_away": lambda e: math.copysign(math.floor(abs(e) + 0.5), e),
    "sigmoid": lambda e: 1. / (1. + math.exp(-e)), "tanh": math.tanh,
    "square": lambda e: e * e, "cube": lambda e: e * e * e,
}


@pytest.mark.parametrize("op", sorted(OPG["unary"]["ops"]))
def test_unary_closed_forms(oracle, op):
    spec = OPG["unary"]["ops"][op]
    data = spec.get("input", OPG["unary"]["default_input"])
    expect = np.array([CLOSED[spec["closed_form"]](e) for e in data])
    got = oracle.unary(op, np.asarray(data, dtype=np.float64))
    np.testing.assert_allclose(got, expect, rtol=1e-15, atol=0)
    got32 = oracle.unary(op, np.asarray(data, dtype=np.float32))
    expect32 = np.array([CLOSED[spec["closed_form"]](float(np.float32(e))) for e in data])
    np.testing.assert_allclose(got32, expect32.astype(np.float32), rtol=2e-7, atol=0)


def test_int32_wraps_like_twos_complement(oracle):
    a = np.array([2147483647, -2147483648, 65536, -7, 123456789], dtype=np.int32)
    b = np.array([1, -1, 65536, 3, 987654321], dtype=np.int32)
    wide = a.astype(np.int64)
    np.testing.assert_array_equal(oracle.binary("ADD", a, b), (wide + b).astype(np.int32))
    np.testing.assert_array_equal(oracle.binary("SUB", a, b), (wide - b).astype(np.int32))
    np.testing.assert_array_equal(oracle.binary("MUL", a, b), (wide * b).astype(np.int32))
    got, _ = oracle.reduce("REDUCE_SUM", a, [5], [0])
    assert got[0] == np.int64(wide.sum()).astype(np.int32)
    # truncating division and comparisons, as for C++ int
    np.testing.assert_array_equal(oracle.binary("DIV", np.array([7, -7, 9], np.int32), np.array([2, 2, -4], np.int32)),
                                  np.array([3, -3, -2], np.int32))


def np_view(flat, shape):
    """numpy array of the same memory: numpy shape = reversed tenncor shape."""
    return np.asarray(flat).reshape([d for d in reversed(shape)])


def test_reduce_matches_numpy_on_reversed_axes(oracle):
    rng = np.random.default_rng(7)
    shape = [5, 3, 4, 2]
    x = rng.standard_normal(120)
    xi = rng.integers(-1000, 1000, 120).astype(np.int32)
    for ranks in ([0], [1], [3], [0, 2], [1, 2], [0, 1, 2, 3]):
        axes = tuple(len(shape) - 1 - r for r in ranks)
        for op, fn in (("REDUCE_SUM", np.sum), ("REDUCE_MAX", np.max), ("REDUCE_MIN", np.min), ("REDUCE_PROD", np.prod)):
            got, oshape = oracle.reduce(op, x, shape, ranks)
            want = fn(np_view(x, shape), axis=axes, keepdims=True)
            np.testing.assert_allclose(np_view(got, oshape[:4]), want, rtol=1e-12)
        got, oshape = oracle.reduce("REDUCE_SUM", xi, shape, ranks)
        np.testing.assert_array_equal(np_view(got, oshape[:4]),
                                      np.sum(np_view(xi, shape), axis=axes, keepdims=True, dtype=np.int32))


def test_data_movement_matches_numpy(oracle):
    rng = np.random.default_rng(11)
    shape = [4, 3, 5]
    x = rng.integers(-99, 99, 60).astype(np.int32)
    v = np_view(x, shape)
    # PERMUTE: out dim i = in dim order[i]  <=> numpy transpose with reversed bookkeeping
    for order in ([1, 0, 2], [2, 0, 1], [2, 1, 0], [0, 2, 1], [1, 2]):
        got, oshape = oracle.permute(x, shape, order)
        full = oracle.full_order(order)[:3]
        n = len(shape)
        axes = [n - 1 - full[n - 1 - j] for j in range(n)]
        np.testing.assert_array_equal(np_view(got, oshape[:3]), v.transpose(axes))
    # EXTEND = numpy tile
    got, oshape = oracle.extend(x[:12], [4, 1, 3], [1, 5, 1, 2])
    want = np.tile(np_view(x[:12], [4, 1, 3, 1]), (2, 1, 5, 1))
    np.testing.assert_array_equal(np_view(got, oshape[:4]), want)
    # SLICE / PAD / REVERSE / STRIDE
    got, oshape = oracle.slice_(x, shape, [[1, 2], [0, 9], [2, 2]])
    np.testing.assert_array_equal(np_view(got, oshape[:3]), v[2:4, :, 1:3])
    got, oshape = oracle.pad(x, shape, [[1, 0], [0, 2], [3, 1]])
    np.testing.assert_array_equal(np_view(got, oshape[:3]), np.pad(v, ((3, 1), (0, 2), (1, 0))))
    got, oshape = oracle.reverse(x, shape, [0, 2])
    np.testing.assert_array_equal(np_view(got, oshape[:3]), v[::-1, :, ::-1])
    got, oshape = oracle.stride(x, shape, [2, 1, 2])
    assert oshape[:3] == [2, 3, 3]  # round(5/2) = 3 (half away from zero)
    np.testing.assert_array_equal(np_view(got, oshape[:3]), v[::2, :, ::2])
    # SCATTER is the inverse of STRIDE on the touched positions
    sc, sshape = oracle.scatter(got, oshape, [2, 1, 2], shape)
    want = np.zeros_like(v)
    want[::2, :, ::2] = v[::2, :, ::2]
    np.testing.assert_array_equal(np_view(sc, sshape[:3]), want)
    # CONCAT along each axis
    for axis in range(3):
        got, oshape = oracle.concat([x, x[::-1].copy()], [shape, shape], axis)
        np.testing.assert_array_equal(np_view(got, oshape[:3]),
                                      np.concatenate([v, np_view(x[::-1].copy(), shape)], axis=2 - axis))


def test_matmul_contract_match_einsum(oracle):
    rng = np.random.default_rng(3)
    # MATMUL: a{K,M}, b{N,K} -> {N,M}; row-major C[M,N] = A[M,K] B[K,N]
    K, M, N, B = 7, 5, 6, 3
    a = rng.standard_normal(K * M * B)
    b = rng.standard_normal(N * K * B)
    got, oshape = oracle.matmul(a, [K, M, B], b, [N, K, B])
    assert oshape[:3] == [N, M, B]
    want = np.einsum("bmk,bkn->bmn", np_view(a, [K, M, B]), np_view(b, [N, K, B]))
    np.testing.assert_allclose(np_view(got, oshape[:3]), want, rtol=1e-12)
    # CONTRACT with two pairs, a{4,2,3} b{2,4,2}, pairs (a0,b1),(a1,b2): golden shape {2,3}
    a = rng.standard_normal(24)
    b = rng.standard_normal(16)
    got, oshape = oracle.contract(a, [4, 2, 3], b, [2, 4, 2], [[0, 1], [1, 2]])
    want = np.einsum("mjk,jkn->mn", np_view(a, [4, 2, 3]), np_view(b, [2, 4, 2]))
    np.testing.assert_allclose(np_view(got, oshape[:2]), want, rtol=1e-12)
    # free dims on both sides: out = b free (dims 0) then a free (dims 1, 2)
    a = rng.standard_normal(4 * 3 * 2)
    b = rng.standard_normal(5 * 4)
    got, oshape = oracle.contract(a, [4, 3, 2], b, [5, 4], [[0, 1]])
    assert oshape[:3] == [5, 3, 2]
    want = np.einsum("cbk,kn->cbn", np_view(a, [4, 3, 2]), np_view(b, [5, 4]))
    np.testing.assert_allclose(np_view(got, oshape[:3]), want, rtol=1e-12)
    # int32 contraction is exact
    ai = rng.integers(-50, 50, 12).astype(np.int32)
    bi = rng.integers(-50, 50, 20).astype(np.int32)
    got, oshape = oracle.matmul(ai, [4, 3], bi, [5, 4])
    np.testing.assert_array_equal(np_view(got, oshape[:2]), np_view(ai, [4, 3]) @ np_view(bi, [5, 4]))


def test_api_convolution_golden(oracle):
    """tenncor/test/test_api.cpp:2265-2339: forward values of a 4-D correlation."""
    fx = EQV["api_convolution"]
    got, oshape = oracle.conv(np.array(fx["data"]), fx["alist"], np.array(fx["data2"]), fx["blist"], list(range(8)))
    assert oshape == fx["expectslist"]
    np.testing.assert_array_equal(got, np.array(fx["expect_out"]))


def test_conv_matches_scipy_correlate(oracle):
    from scipy.signal import correlate
    rng = np.random.default_rng(5)
    img = rng.standard_normal(6 * 7 * 3)
    ker = rng.standard_normal(2 * 3 * 3)
    got, oshape = oracle.conv(img, [6, 7, 3], ker, [2, 3, 3], [0, 1, 2])
    want = correlate(np_view(img, [6, 7, 3]), np_view(ker, [2, 3, 3]), mode="valid")
    np.testing.assert_allclose(np_view(got, oshape[:3]), want, rtol=1e-12, atol=1e-12)
    # kernel dim 0 slides along image dim 2, kernel dim 1 along image dim 0
    ker2 = rng.standard_normal(2 * 3)
    got, oshape = oracle.conv(img, [6, 7, 3], ker2, [2, 3], [2, 0])
    assert oshape[:3] == [4, 7, 2]
    iv, kv = np_view(img, [6, 7, 3]), np_view(ker2, [2, 3])  # iv[d2,d1,d0], kv[k1,k0]
    want = np.zeros((2, 7, 4))
    for k1 in range(3):
        for k0 in range(2):
            want += iv[k0:k0 + 2, :, k1:k1 + 4] * kv[k1, k0]
    np.testing.assert_allclose(np_view(got, oshape[:3]), want, rtol=1e-12, atol=1e-12)


def test_matmul_chain_golden(oracle):
    """tenncor/test/test_equation.cpp:26-87: dest = (c.d).(d^T.c^T), d = a.b."""
    fx = EQV["matmul_complex"]
    a, b, c = (np.array(fx[k]) for k in ("data", "data2", "data3"))
    d, ds = oracle.matmul(a, fx["alist"], b, fx["blist"])
    e, es = oracle.matmul(c, fx["clist"], d, ds)
    dt, dts = oracle.permute(d, ds, [1, 0])
    ct, cts = oracle.permute(c, fx["clist"], [1, 0])
    f, fs = oracle.matmul(dt, dts, ct, cts)
    dest, _ = oracle.matmul(e, es, f, fs)
    np.testing.assert_allclose(dest, np.array(fx["expect_dest"]), rtol=4e-16 * 8)


def test_cast_and_assign(oracle):
    x = np.array([-2.7, -0.5, 0.5, 2.7, 1e3], dtype=np.float64)
    np.testing.assert_array_equal(oracle.cast(x, oracle.INT32), np.array([-2, 0, 0, 2, 1000], np.int32))
    np.testing.assert_array_equal(oracle.cast(x, oracle.FLOAT), x.astype(np.float32))
    t = np.array([1., 2., 3.], dtype=np.float32)
    oracle.assign("ASSIGN_SUB", t, np.array([.5, .5, 4.], np.float32))
    np.testing.assert_array_equal(t, np.array([.5, 1.5, -1.], np.float32))


# internal/eigen/test/test_operator.cpp:2647-2818 (Assign .. AssignDiv) and
# :2821-2879 (Cast): the reference's own vectors
ASSIGN_GOLDENS = {
    "ASSIGN": [1, 0, 3, 9, 10, 11],
    "ASSIGN_ADD": [3, 8, 7, 14, 16, 18],
    "ASSIGN_SUB": [1, 8, 1, -4, -4, -4],
    "ASSIGN_MUL": [2, 0, 12, 45, 60, 77],
    "ASSIGN_DIV": [2, 4, 4. / 3, 5. / 9, 0.6, 7. / 11],
}
ASSIGN_TARGET = [2, 8, 4, 5, 6, 7]
ASSIGN_SOURCE = [1, 0, 3, 9, 10, 11]
ASSIGN_DIV_SOURCE = [1, 2, 3, 9, 10, 11]   # :2789 divides by {1, 2, 3, 9, 10, 11}
CAST_SOURCE = [2.1, 8.5, 4.3, 5.2, 6.1, 7.2]
CAST_INT32 = [2, 8, 4, 5, 6, 7]


@pytest.mark.parametrize("op", sorted(ASSIGN_GOLDENS))
def test_assign_goldens(oracle, op):
    target = np.array(ASSIGN_TARGET, np.float64)
    source = np.array(ASSIGN_DIV_SOURCE if op == "ASSIGN_DIV" else ASSIGN_SOURCE, np.float64)
    oracle.assign(op, target, source)
    np.testing.assert_allclose(target, ASSIGN_GOLDENS[op], rtol=4e-16)


def test_cast_golden(oracle):
    x = np.array(CAST_SOURCE, np.float64)
    np.testing.assert_array_equal(oracle.cast(x, oracle.DOUBLE), x)
    np.testing.assert_array_equal(oracle.cast(x, oracle.INT32), np.array(CAST_INT32, np.int32))


# ---- the device RAND_UNIF stream -------------------------------------------

# Known-answer vectors of the Random123 distribution (kat_vectors, philox4x32
# with 10 rounds): counter words, key words, expected output words
PHILOX_KAT = [
    ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
    ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
    ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
     [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
]


@pytest.mark.parametrize("counter,key,expect", PHILOX_KAT, ids=["zeros", "ones", "pi"])
def test_philox_known_answers(oracle, counter, key, expect):
    assert oracle.philox4x32_10(counter, key) == expect


def test_rand_uniform_is_the_documented_function_of_the_generator_words(oracle):
    """Element i takes word i%4 of block first+i/4 (double: two words of block
    first+i/2); real results are the correctly rounded lo + u*(hi-lo); int32
    results lo + ((word*(hi-lo+1)) >> 32).  Worked in exact rational /
    integer arithmetic from the generator words."""
    from fractions import Fraction
    seed, first, n = 0x0123456789abcdef, (1 << 32) - 2, 23  # the block counter carries into its high word
    key = [seed & 0xffffffff, seed >> 32]
    rng = np.random.default_rng(0)

    def words(block):
        return oracle.philox4x32_10([block & 0xffffffff, block >> 32, 0, 0], key)

    lo = rng.uniform(-3, 1, n).astype(np.float32)
    hi = (lo + rng.uniform(0.5, 4, n)).astype(np.float32)
    got = oracle.rand_uniform(lo, hi, seed, first)
    for i in range(n):
        u = Fraction(words(first + i // 4)[i % 4] >> 8, 1 << 24)
        # fl(hi-lo) is what the multiply-add sees
        exact = Fraction(float(lo[i])) + u * Fraction(float(np.float32(hi[i] - lo[i])))
        assert abs(Fraction(float(got[i])) - exact) <= Fraction(float(np.spacing(np.abs(got[i])))) / 2

    lo64 = rng.uniform(-3, 1, n)
    hi64 = lo64 + rng.uniform(0.5, 4, n)
    got = oracle.rand_uniform(lo64, hi64, seed, first)
    for i in range(n):
        w = words(first + i // 2)
        u = Fraction(((w[2 * (i % 2) + 1] << 32) | w[2 * (i % 2)]) >> 11, 1 << 53)
        exact = Fraction(float(lo64[i])) + u * Fraction(float(hi64[i] - lo64[i]))
        assert abs(Fraction(float(got[i])) - exact) <= Fraction(float(np.spacing(np.abs(got[i])))) / 2

    ilo = rng.integers(-2 ** 31, 2 ** 31 - 1, n).astype(np.int32)
    ihi = np.maximum(ilo, rng.integers(-2 ** 31, 2 ** 31 - 1, n).astype(np.int32))
    ilo[0], ihi[0] = -2 ** 31, 2 ** 31 - 1   # the whole range
    ilo[1], ihi[1] = 7, 7                    # one value
    ilo[2], ihi[2] = 5, 4                    # empty range: lo
    got = oracle.rand_uniform(ilo, ihi, seed, first)
    for i in range(n):
        if ihi[i] < ilo[i]:
            assert got[i] == ilo[i]
            continue
        span = int(ihi[i]) - int(ilo[i]) + 1
        assert int(got[i]) == int(ilo[i]) + ((words(first + i // 4)[i % 4] * span) >> 32)


def test_rand_uniform_stream_properties(oracle):
    n = 200000
    lo, hi = np.full(n, -2.0, np.float32), np.full(n, 6.0, np.float32)
    x = oracle.rand_uniform(lo, hi, 42)
    assert x.min() >= -2.0 and x.max() < 6.0
    # uniform on [-2, 6): mean 2, variance 64/12; 5 sigma of the estimators
    assert abs(x.mean() - 2.0) < 5 * np.sqrt(64 / 12 / n)
    assert abs(x.var() - 64 / 12) < 5 * np.sqrt(0.8 * (64 / 12) ** 2 / n)
    # a later start continues the same stream; another seed is another stream
    tail = oracle.rand_uniform(lo[:4000], hi[:4000], 42, first_block=1000)
    np.testing.assert_array_equal(tail, x[4000:8000])
    assert not np.array_equal(oracle.rand_uniform(lo, hi, 43), x)
    dice = oracle.rand_uniform(np.full(n, 1, np.int32), np.full(n, 6, np.int32), 7)
    counts = np.bincount(dice, minlength=7)
    assert counts[0] == 0 and counts[1:].sum() == n
    assert np.all(np.abs(counts[1:] - n / 6) < 5 * np.sqrt(n * 5 / 36))
