"""Forward values and gradients of every elementwise operator on the data and
against the closed forms of the reference's API tests
(tenncor/test/test_api.cpp:132-216 unary helper with its data :217-235,
:236-380 binary helper with its data :347-380, :382-516 the int32 helper for
comparisons; the closed forms at :882-1187 and :1367-1460), on the GPU in
double (comparisons in int32).

For an operator f(a, b) the reference checks the gradient of f(a, a) with
respect to a, and of f(a, b) with respect to each side; all three here.
Tolerance: the reference asks for 4 ulp (EXPECT_DOUBLE_EQ) against the host's
libm; the GPU's libm differs from it in the last place, so transcendental
results are compared at 1e-14 relative, everything else exactly.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

DATA = np.array([59, 10, 28, 10, 67, 62, 23, 4, 55, 77, 28, 16, 82, 52, 47, 16, 7, 85, 37, 2, 8, 52, 62, 43], np.float64)
BDATA = np.array([
    0.0919361505, 0.5135099474, 0.3147548326, 0.0281299379, 0.3705218798, 0.6808164860,
    0.1933972592, 0.2326945471, 0.4600163558, 0.1600801317, 0.9942654588, 0.8739832345,
    0.9664644529, 0.6152766955, 0.8795922916, 0.6384690466, 0.3922073677, 0.5979097486,
    0.0425608731, 0.1178122813, 0.1594330664, 0.0926580999, 0.9309809737, 0.2119471989])
BDATA2 = np.array([
    0.2547977589, 0.8808089905, 0.4323663340, 0.5710527217, 0.6207772267, 0.8574923091,
    0.2315629833, 0.8740258926, 0.9239905856, 0.0346148639, 0.3255387878, 0.7443564112,
    0.0930828560, 0.9324878301, 0.6552622891, 0.8305292319, 0.9515416240, 0.3653033185,
    0.0504231590, 0.8494357051, 0.0908431573, 0.1567913571, 0.1211327459, 0.5269402648])
CST = 0.7819955055
IDATA = np.array([1, 2, 3, 0, 1, 2, 2, 1, 1, 3, 3, 1, 2, 2, 3, 0, 1, 3, 3, 1, 2, 0, 0, 2], np.int32)
IDATA2 = np.array([0, 0, 2, 1, 3, 3, 2, 2, 3, 1, 2, 3, 1, 3, 1, 3, 1, 0, 2, 1, 2, 2, 0, 1], np.int32)
ICST = 2


@pytest.fixture()
def env():
    from tenncor_amd import graph
    g = graph.Graph()
    yield g, graph.Api(g)
    g.close()


def sig(d):
    return 1 / (1 + np.exp(-d))


def tanh_e2d(d):
    e2d = np.exp(2 * d)
    return (e2d - 1) / (e2d + 1)


# opcode -> (forward, backward, exact)
UNARY = {
    "ABS": (np.abs, lambda d: d / np.abs(d), True),
    "NEG": (np.negative, lambda d: -np.ones_like(d), True),
    "SIN": (np.sin, np.cos, False),
    "COS": (np.cos, lambda d: -np.sin(d), False),
    "TAN": (np.tan, lambda d: 1.0 / np.cos(d) / np.cos(d), False),
    "EXP": (np.exp, np.exp, False),
    "LOG": (np.log, lambda d: 1.0 / d, False),
    "SQRT": (np.sqrt, lambda d: 1.0 / (2 * np.sqrt(d)), False),
    "ROUND": (np.round, np.ones_like, True),
    "SIGMOID": (sig, lambda d: sig(d) * (1 - sig(d)), False),
    "TANH": (np.tanh, lambda d: 1 - np.tanh(d) ** 2, False),
    "SQUARE": (lambda d: d * d, lambda d: 2 * d, True),
    "CUBE": (lambda d: d * d * d, lambda d: 3 * d * d, False),
}


def check(got, want, exact, what):
    if exact:
        np.testing.assert_array_equal(got, want, err_msg=what)
    else:
        # the derivative of tanh at 85 is 1 - (1 - 2e-74)^2 = 0 in double on both sides
        np.testing.assert_allclose(got, want, rtol=1e-14, atol=1e-300, err_msg=what)


@pytest.mark.parametrize("op", sorted(UNARY))
@pytest.mark.parametrize("shape", [[2, 3, 4], [2, 3]], ids=["tensor", "matrix"])
def test_unary_forward_and_gradient(env, op, shape):
    from tenncor_amd import capi
    g, api = env
    fwd, bwd, exact = UNARY[op]
    data = DATA[:int(np.prod(shape))]
    src = g.constant(data, shape)
    dest = api.unary(op, src)
    g.evaluate([dest])
    g.evaluate([dest])  # idempotency check, as the reference does
    assert dest.shape[:len(shape)] == shape
    check(dest.get(), fwd(data), exact, op)
    grad = g.functor("CAST", [g.derive(api.unary(op, src), [src])[0]], dtype=capi.DOUBLE)
    g.evaluate([grad])
    g.evaluate([grad])
    assert grad.shape[:len(shape)] == shape
    check(grad.get(), bwd(data), exact and op != "ABS", op + " gradient")


def minmax_bwd(pick_left):
    def bwd(a, b, lg, rg):
        left = pick_left(a, b)
        right = pick_left(b, a)
        return np.where(left, lg, np.where(right, rg, lg + rg))
    return bwd


BINARY = {
    "POW": (np.power, lambda a, b, lg, rg: lg * b * np.power(a, b - 1) + rg * np.power(a, b) * np.log(a), False),
    "ADD": (np.add, lambda a, b, lg, rg: lg + rg + 0 * a, True),
    "SUB": (np.subtract, lambda a, b, lg, rg: lg - rg + 0 * a, True),
    "MUL": (np.multiply, lambda a, b, lg, rg: lg * b + rg * a, True),
    "DIV": (np.divide, lambda a, b, lg, rg: (lg * b - rg * a) / (b * b), False),
    "MIN": (np.minimum, minmax_bwd(lambda a, b: b > a), True),
    "MAX": (np.maximum, minmax_bwd(lambda a, b: a > b), True),
}


@pytest.mark.parametrize("op", sorted(BINARY))
@pytest.mark.parametrize("shape", [[3, 2, 4], [3, 2]], ids=["tensor", "matrix"])
def test_binary_forward_and_gradients(env, op, shape):
    from tenncor_amd import capi
    g, api = env
    fwd, bwd, exact = BINARY[op]
    n = int(np.prod(shape))
    data, data2 = BDATA[:n], BDATA2[:n]
    src, src2 = g.constant(data, shape), g.constant(data2, shape)
    dest = api.binary(op, src, src2)
    clhs = api.binary(op, src, CST)       # tensor op scalar
    crhs = api.binary(op, CST, src2)      # scalar op tensor
    g.evaluate([dest])
    g.evaluate([dest])
    check(dest.get(), fwd(data, data2), exact, op)
    g.evaluate([clhs, crhs])
    check(clhs.get(), fwd(data, np.full(n, CST)), exact, op + " with a scalar on the right")
    check(crhs.get(), fwd(np.full(n, CST), data2), exact, op + " with a scalar on the left")

    def gradient(root, wrt):
        node = g.functor("CAST", [g.derive(root, [wrt])[0]], dtype=capi.DOUBLE)
        g.evaluate([node])
        g.evaluate([node])
        assert node.shape[:len(shape)] == shape
        return node.get()

    check(gradient(api.binary(op, src, src), src), bwd(data, data, 1.0, 1.0), False, op + " of (a, a)")
    check(gradient(dest, src), bwd(data, data2, 1.0, 0.0), False, op + " left gradient")
    check(gradient(dest, src2), bwd(data, data2, 0.0, 1.0), False, op + " right gradient")


COMPARE = {"EQ": np.equal, "NEQ": np.not_equal, "LT": np.less, "GT": np.greater}


@pytest.mark.parametrize("op", sorted(COMPARE))
@pytest.mark.parametrize("shape", [[4, 3, 2], [4, 2]], ids=["tensor", "matrix"])
def test_comparisons_in_int32_have_zero_gradients(env, op, shape):
    from tenncor_amd import capi
    g, api = env
    n = int(np.prod(shape))
    data, data2 = IDATA[:n], IDATA2[:n]
    src, src2 = g.constant(data, shape), g.constant(data2, shape)
    dest = api.binary(op, src, src2)
    clhs = api.binary(op, src, ICST)
    crhs = api.binary(op, ICST, src2)
    g.evaluate([dest, clhs, crhs])
    g.evaluate([dest, clhs, crhs])
    assert dest.dtype == capi.INT32
    np.testing.assert_array_equal(dest.get(), COMPARE[op](data, data2).astype(np.int32))
    np.testing.assert_array_equal(clhs.get(), COMPARE[op](data, ICST).astype(np.int32))
    np.testing.assert_array_equal(crhs.get(), COMPARE[op](ICST, data2).astype(np.int32))
    for root, wrt in ((api.binary(op, src, src), src), (dest, src), (dest, src2)):
        grad = g.functor("CAST", [g.derive(root, [wrt])[0]], dtype=capi.INT32)
        g.evaluate([grad])
        np.testing.assert_array_equal(grad.get(), np.zeros(n, np.int32))


# ---- reductions (test_api.cpp:1540-1873) --------------------------------------

RDATA = np.array([22, 15, 74, 38, 61, 95, 62, 81, 99, 76, 7, 22, 56, 50, 19, 13, 12, 10, 31, 40, 60, 54, 6, 83], np.float64)
RSHAPE = [2, 3, 4]


def np_view(flat, shape):
    return np.asarray(flat).reshape(shape[::-1])


@pytest.mark.parametrize("op,npf", [("REDUCE_SUM", np.sum), ("REDUCE_MIN", np.min), ("REDUCE_MAX", np.max)])
def test_reductions_and_their_gradients(env, op, npf):
    from tenncor_amd import capi
    g, api = env
    src = g.constant(RDATA, RSHAPE)
    full = api.reduce(op, src)              # over every dim
    along = api.reduce(op, src, 1, 1)       # over dim 1
    g.evaluate([full, along])
    g.evaluate([full, along])
    view = np_view(RDATA, RSHAPE)           # np[4,3,2]
    np.testing.assert_array_equal(full.get(), [npf(RDATA)])
    assert along.shape[:3] == [2, 1, 4]
    np.testing.assert_array_equal(np_view(along.get(), [2, 1, 4]), npf(view, axis=1, keepdims=True))
    gfull = g.functor("CAST", [g.derive(full, [src])[0]], dtype=capi.DOUBLE)
    galong = g.functor("CAST", [g.derive(along, [src])[0]], dtype=capi.DOUBLE)
    g.evaluate([gfull, galong])
    g.evaluate([gfull, galong])
    if op == "REDUCE_SUM":
        np.testing.assert_array_equal(gfull.get(), np.ones(24))
        np.testing.assert_array_equal(galong.get(), np.ones(24))
    else:
        # one at the extreme of each reduced group, zero elsewhere
        np.testing.assert_array_equal(gfull.get(), (RDATA == npf(RDATA)).astype(np.float64))
        want = (view == npf(view, axis=1, keepdims=True)).astype(np.float64)
        np.testing.assert_array_equal(np_view(galong.get(), RSHAPE), want)


def test_reduce_prod_in_int32_and_its_gradient(env):
    from tenncor_amd import capi
    g, api = env
    data = np.array([2, 1, 7, 3, 6, 9, 6, 8, 9, 7, 7, 2], np.int32)
    shape = [2, 2, 3]
    src = g.constant(data, shape)
    full = api.reduce("REDUCE_PROD", src)
    along = api.reduce("REDUCE_PROD", src, 1, 1)
    g.evaluate([full, along])
    g.evaluate([full, along])
    assert full.get()[0] == np.prod(data.astype(np.int64))
    view = np_view(data, shape)
    np.testing.assert_array_equal(np_view(along.get(), [2, 1, 3]), np.prod(view, axis=1, keepdims=True))
    gfull = g.functor("CAST", [g.derive(full, [src])[0]], dtype=capi.INT32)
    galong = g.functor("CAST", [g.derive(along, [src])[0]], dtype=capi.INT32)
    g.evaluate([gfull, galong])
    g.evaluate([gfull, galong])
    np.testing.assert_array_equal(gfull.get(), np.prod(data.astype(np.int64)) // data)
    # the reference's expected values, test_api.cpp:1693-1700
    np.testing.assert_array_equal(galong.get(), [7, 3, 2, 1, 6, 8, 6, 9, 7, 2, 9, 7])


# ---- data movement and selection (test_api.cpp:1189-1364, 1506-1537, 1876-1983)

def test_slice_and_its_gradient(env):
    from tenncor_amd import capi
    g, api = env
    shape = [3, 2, 4]
    src = g.constant(BDATA, shape)
    dest = g.functor("SLICE", [src], dimension_pairs=[0, 3, 1, 1])   # slice(src, {{0,3},{1,1}})
    g.evaluate([dest])
    g.evaluate([dest])
    assert dest.shape[:3] == [3, 1, 4]
    np.testing.assert_array_equal(dest.get(), np_view(BDATA, shape)[:, 1:2, :].reshape(-1))
    grad = g.functor("CAST", [g.derive(dest, [src])[0]], dtype=capi.DOUBLE)
    g.evaluate([grad])
    g.evaluate([grad])
    assert grad.shape[:3] == shape
    np.testing.assert_array_equal(grad.get(), [0, 0, 0, 1, 1, 1] * 4)  # test_api.cpp:1343-1348


def test_permute_and_its_gradient(env):
    from tenncor_amd import capi
    g, api = env
    shape, order = [4, 3, 2], [2, 0, 1]
    data = np.array([70, 36, 93, 50, 59, 98, 39, 5, 54, 84, 100, 94, 75, 64, 30, 17, 90, 79, 21, 54, 6, 7, 69, 53], np.float64)
    src = g.constant(data, shape)
    dest = api.permute(src, order)
    g.evaluate([dest])
    g.evaluate([dest])
    oshape = dest.shape[:3]
    assert oshape == [shape[o] for o in order]
    got = dest.get()
    # out coordinate j is in coordinate order[j] (test_api.cpp:1901-1909)
    for i in range(24):
        c = [i % 4, (i // 4) % 3, i // 12]
        oc = [c[order[j]] for j in range(3)]
        assert got[oc[0] + oshape[0] * (oc[1] + oshape[1] * oc[2])] == data[i]
    grad = g.functor("CAST", [g.derive(dest, [src])[0]], dtype=capi.DOUBLE)
    g.evaluate([grad])
    assert grad.shape[:3] == shape
    np.testing.assert_array_equal(grad.get(), np.ones(24))


def test_extend_and_its_gradient(env):
    from tenncor_amd import capi
    g, api = env
    data = np.array([51, 42, 9, 43, 37, 36, 65, 95, 10, 33], np.float64)
    src = g.constant(data, [2, 5])
    dest = api.extend(src, 2, [1, 3])
    g.evaluate([dest])
    g.evaluate([dest])
    assert dest.shape[:4] == [2, 5, 1, 3]
    np.testing.assert_array_equal(dest.get(), np.tile(data, 3))
    grad = g.functor("CAST", [g.derive(dest, [src])[0]], dtype=capi.DOUBLE)
    g.evaluate([grad])
    assert grad.shape[:2] == [2, 5]
    np.testing.assert_array_equal(grad.get(), np.full(10, 3.0))


@pytest.mark.parametrize("shape", [[3, 2, 4], [3, 2]], ids=["tensor", "matrix"])
def test_select_and_its_gradients(env, shape):
    from tenncor_amd import capi
    g, api = env
    n = int(np.prod(shape))
    cond = (np.arange(n) % 3 != 1).astype(np.float64)
    data, data2 = BDATA[:n], BDATA2[:n]
    csrc, src, src2 = g.constant(cond, shape), g.constant(data, shape), g.constant(data2, shape)
    dest = api.if_then_else(csrc, src, src2)
    g.evaluate([dest])
    g.evaluate([dest])
    np.testing.assert_array_equal(dest.get(), np.where(cond != 0, data, data2))
    # choosing between a tensor and itself is that tensor (test_api.cpp:1253-1254)
    assert api.if_then_else(csrc, src, src).id == src.id
    gl = g.functor("CAST", [g.derive(dest, [src])[0]], dtype=capi.DOUBLE)
    gr = g.functor("CAST", [g.derive(dest, [src2])[0]], dtype=capi.DOUBLE)
    g.evaluate([gl, gr])
    g.evaluate([gl, gr])
    np.testing.assert_array_equal(gl.get(), cond)
    np.testing.assert_array_equal(gr.get(), (cond == 0).astype(np.float64))


def test_argmax_over_everything_and_no_gradient(env):
    from tenncor_amd import graph
    g, api = env
    src = g.constant(RDATA, RSHAPE)
    dest = g.functor("ARGMAX", [src], rank=8)
    g.evaluate([dest])
    g.evaluate([dest])
    assert dest.shape == [1] * 8
    assert dest.get()[0] == 8          # the flat index of 99
    with pytest.raises(graph.GraphError, match="cannot derive ARGMAX"):
        g.derive(dest, [src])
