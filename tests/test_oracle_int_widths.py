"""The oracle's integer element types beyond INT32 (cfg/fulltype.yml:11-34:
INT8, UINT8, INT16, UINT16, UINT32, INT64, UINT64), pinned against numpy's own
fixed-width arithmetic: numpy wraps modulo 2^width in its array operations,
orders signed and unsigned values by their own rules and truncates casts the
way C does, and none of that shares code with the oracle's macros.  A wrong
width (a sum carried in 32 bits for an 8-bit type), a sign mix-up (unsigned
values compared as signed) or a dropped wrap fails here.  The products are
checked against Python's unbounded integers reduced modulo 2^width.
"""
import numpy as np
import pytest

INT_TYPES = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64]


def full_range(rng, t, n):
    info = np.iinfo(t)
    x = rng.integers(info.min, info.max, n, dtype=t, endpoint=True)
    edge = [info.min, info.max, 0, 1][:n]
    x[:len(edge)] = edge
    return x


def wrap(values, t):
    """Python integers reduced to the two's-complement range of t."""
    bits = 8 * np.dtype(t).itemsize
    out = []
    for v in values:
        v = int(v) % (1 << bits)
        if np.issubdtype(t, np.signedinteger) and v >= 1 << (bits - 1):
            v -= 1 << bits
        out.append(v)
    return np.array(out, dtype=t)


@pytest.mark.parametrize("t", INT_TYPES, ids=lambda t: t.__name__)
def test_elementwise_arithmetic_wraps_like_numpy(oracle, t):
    rng = np.random.default_rng(np.dtype(t).num)
    n = 5000
    a, b = full_range(rng, t, n), full_range(rng, t, n)[::-1].copy()
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(oracle.binary("ADD", a, b), a + b)
        np.testing.assert_array_equal(oracle.binary("SUB", a, b), a - b)
        np.testing.assert_array_equal(oracle.binary("MUL", a, b), a * b)
        np.testing.assert_array_equal(oracle.unary("NEG", a), (0 - a.astype(np.uint64)).astype(t) if t == np.uint64 else (-a))
        np.testing.assert_array_equal(oracle.unary("SQUARE", a), a * a)
        np.testing.assert_array_equal(oracle.unary("CUBE", a), a * a * a)
    # against unbounded integers: the wrap is modulo 2^width of THIS type
    np.testing.assert_array_equal(oracle.binary("MUL", a[:300], b[:300]), wrap([int(x) * int(y) for x, y in zip(a[:300], b[:300])], t))
    np.testing.assert_array_equal(oracle.binary("ADD", a[:300], b[:300]), wrap([int(x) + int(y) for x, y in zip(a[:300], b[:300])], t))
    np.testing.assert_array_equal(oracle.binary("MIN", a, b), np.minimum(a, b))
    np.testing.assert_array_equal(oracle.binary("MAX", a, b), np.maximum(a, b))
    for op, fn in (("EQ", np.equal), ("NEQ", np.not_equal), ("LT", np.less), ("GT", np.greater)):
        b2 = b.copy()
        b2[::5] = a[::5]
        np.testing.assert_array_equal(oracle.binary(op, a, b2), fn(a, b2).astype(t))
    np.testing.assert_array_equal(oracle.unary("ROUND", a), a)
    if np.issubdtype(t, np.signedinteger):
        with np.errstate(over="ignore"):
            np.testing.assert_array_equal(oracle.unary("ABS", a), np.abs(a))  # |lowest| wraps to lowest in both
    else:
        np.testing.assert_array_equal(oracle.unary("ABS", a), a)


@pytest.mark.parametrize("t", INT_TYPES, ids=lambda t: t.__name__)
def test_division_truncates_and_the_trapping_cases_give_zero(oracle, t):
    rng = np.random.default_rng(100 + np.dtype(t).num)
    n = 5000
    a, b = full_range(rng, t, n), full_range(rng, t, n)[::-1].copy()
    b[b == 0] = 3
    info = np.iinfo(t)
    signed = info.min < 0
    if signed:
        b[(a == info.min) & (b == -1)] = 2
    want = wrap([abs(int(x)) // abs(int(y)) * (1 if (x < 0) == (y < 0) else -1) for x, y in zip(a, b)], t)  # C truncation
    np.testing.assert_array_equal(oracle.binary("DIV", a, b), want)
    zero = np.zeros(4, t)
    np.testing.assert_array_equal(oracle.binary("DIV", a[:4], zero), zero)
    if signed:
        lowest = np.array([info.min], t)
        got = oracle.binary("DIV", lowest, np.array([-1], t))
        # 32 and 64 bits trap on the CPU (0 here); narrower types divide as int and wrap back
        assert got[0] == (0 if np.dtype(t).itemsize >= 4 else info.min)


@pytest.mark.parametrize("t", INT_TYPES, ids=lambda t: t.__name__)
def test_reductions_products_and_movement(oracle, t):
    rng = np.random.default_rng(200 + np.dtype(t).num)
    shape = [7, 5, 6]
    x = full_range(rng, t, 7 * 5 * 6)
    x3 = x.reshape(6, 5, 7)  # numpy order is the reverse of the tenncor shape
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(oracle.reduce("REDUCE_SUM", x, shape, [1])[0], x3.sum(axis=1, dtype=t).reshape(-1))
        np.testing.assert_array_equal(oracle.reduce("REDUCE_PROD", x, shape, [0, 2])[0], x3.prod(axis=(0, 2), dtype=t).reshape(-1))
    np.testing.assert_array_equal(oracle.reduce("REDUCE_MIN", x, shape, [0])[0], x3.min(axis=2).reshape(-1))
    np.testing.assert_array_equal(oracle.reduce("REDUCE_MAX", x, shape, [0, 1, 2])[0], [x.max()])
    # argmax: the index of the first largest value, in the element type
    small = rng.integers(0, 100, 7 * 5 * 6).astype(t)
    got, _ = oracle.argmax(small, shape, 1)
    np.testing.assert_array_equal(got, small.reshape(6, 5, 7).argmax(axis=1).astype(t).reshape(-1))
    # matrix product modulo 2^width
    a, b = full_range(rng, t, 4 * 3), full_range(rng, t, 5 * 4)
    got, oshape = oracle.matmul(a, [4, 3], b, [5, 4])
    A = [[int(v) for v in row] for row in a.reshape(3, 4)]
    B = [[int(v) for v in row] for row in b.reshape(4, 5)]
    want = wrap([sum(A[i][k] * B[k][j] for k in range(4)) for i in range(3) for j in range(5)], t)
    assert oshape[:2] == [5, 3]
    np.testing.assert_array_equal(got, want)
    # movement moves bytes whatever the type
    np.testing.assert_array_equal(oracle.permute(x, shape, [2, 0, 1])[0], x3.transpose(1, 2, 0).reshape(-1))
    np.testing.assert_array_equal(oracle.reverse(x, shape, [1])[0], x3[:, ::-1, :].reshape(-1))
    np.testing.assert_array_equal(oracle.concat([x, x], [shape, shape], 0)[0], np.concatenate([x3, x3], axis=2).reshape(-1))


def test_casts_between_every_pair_of_types(oracle):
    from oracle.oracle import NP_OF, dtype_code
    rng = np.random.default_rng(7)
    for src in INT_TYPES:
        x = full_range(rng, src, 400)
        for code, dst in NP_OF.items():
            with np.errstate(over="ignore"):
                want = x.astype(dst)  # C conversion: modulo 2^width between integers, nearest for floating point
            np.testing.assert_array_equal(oracle.cast(x, code), want, err_msg="%s -> %s" % (src.__name__, np.dtype(dst).name))
    for src in (np.float32, np.float64):
        x = (rng.uniform(-100, 100, 400)).astype(src)
        for code, dst in NP_OF.items():
            lo = 0 if np.dtype(dst).kind == "u" else -100
            v = np.clip(x, lo, 100)
            np.testing.assert_array_equal(oracle.cast(v, code), v.astype(dst), err_msg="%s -> %s" % (src.__name__, np.dtype(dst).name))
    assert dtype_code(np.zeros(1, np.uint16)) == 7


@pytest.mark.parametrize("t", INT_TYPES, ids=lambda t: t.__name__)
def test_generator_stays_in_range_and_covers_it(oracle, t):
    info = np.iinfo(t)
    n = 4000
    lo = np.full(n, max(info.min, -50), t)
    hi = np.full(n, 50, t)
    got = oracle.rand_uniform(lo, hi, 99)
    assert got.dtype == t and got.min() >= lo[0] and got.max() <= 50
    assert len(np.unique(got)) == int(hi[0]) - int(lo[0]) + 1  # 4000 draws over at most 101 values
    assert abs(float(got.astype(np.float64).mean()) - (float(lo[0]) + 50) / 2) < 3
    # the whole range of the type, an empty range and a single value
    lo[:], hi[:] = info.min, info.max
    lo[1], hi[1] = 9, 3
    lo[2], hi[2] = 17, 17
    got = oracle.rand_uniform(lo, hi, 5)
    assert got[1] == 9 and got[2] == 17
    spread = got.astype(np.float64)
    assert spread.std() > 0.2 * (float(info.max) - float(info.min))  # uniform: 0.289 of the range


def test_one_numbering_in_the_device_header_the_bindings_and_the_oracle():
    import os
    import re
    from oracle import oracle as orc
    from tenncor_amd import capi
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    names = ["DOUBLE", "FLOAT", "INT32", "INT8", "UINT8", "INT16", "UINT16", "UINT32", "INT64", "UINT64"]
    with open(os.path.join(root, "include", "tcg.h")) as f:
        header = f.read()
    with open(os.path.join(root, "oracle", "tc_oracle.h")) as f:
        oracle_header = f.read()
    for code, name in enumerate(names, start=1):
        assert re.search(r"TCG_%s = %d\b" % (name, code), header), name
        assert re.search(r"ORC_%s = %d\b" % (name, code), oracle_header), name
        assert getattr(capi, name) == code and getattr(orc, name) == code
        numpy_name = {"DOUBLE": "float64", "FLOAT": "float32"}.get(name, name.lower())
        assert capi.NP_OF[code] == orc.NP_OF[code] and np.dtype(capi.NP_OF[code]).name == numpy_name
