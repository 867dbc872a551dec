"""Gradients against central differences.  tests/test_host_backprop.py pins the
GRAPHS teq::derive builds to the reference's expected printouts
(tenncor/eteq/test/test_backprop.cpp); here the VALUES those graphs compute are
held against what the mathematics fixes: for loss = sum(op(x, ...) * r) with a
fixed random r, d loss / d x_i = (loss(x + h e_i) - loss(x - h e_i)) / 2h up to
O(h^2).  Double precision on the GPU, h = 1e-5, bar 1e-6 of the gradient's
largest entry plus 1e-8 (truncation ~ h^2 f''' ~ 1e-10, rounding ~ 1e-16 / h).
A rule of tenncor/eteq/backprop.hpp:18-542 restated with a dropped factor, a
wrong sign, a transposed operand or a reduction over the wrong dims fails here
whatever graph it prints.  Operands stay away from kinks (|x| at 0, ties of
MIN / MAX) so that the derivative exists where it is probed.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture()
def g():
    from tenncor_amd import graph
    graph.set_evaluator("plain")
    gr = graph.Graph()
    yield gr
    gr.close()


def distinct(rng, n, lo=0.5, hi=2.0):
    """n values at least (hi - lo) / (4 n) apart, in random order: no ties for MIN / MAX."""
    base = np.linspace(lo, hi, n) + rng.uniform(-1, 1, n) * (hi - lo) / (8 * n)
    return rng.permutation(base)


def check(g, api, build, shapes, positive=False, signs=False, wrt=None, seed=0):
    """build(nodes) -> y; checks d sum(y * r) / d operand for every operand in `wrt`."""
    rng = np.random.default_rng(seed)
    values, nodes = [], []
    for k, shape in enumerate(shapes):
        n = int(np.prod(shape))
        v = distinct(rng, n)
        if signs:
            v = v * rng.choice([-1.0, 1.0], n)
        values.append(v.astype(np.float64))
        nodes.append(g.variable(values[-1], list(shape), "x%d" % k))
    y = build(nodes)
    ny = int(np.prod(y.shape))
    r = g.variable(rng.uniform(0.5, 1.5, ny) * rng.choice([-1.0, 1.0], ny), list(y.shape), "r")
    loss = api.reduce_sum(api.mul(y, r))
    which = list(range(len(nodes))) if wrt is None else list(wrt)
    grads = g.derive(loss, [nodes[k] for k in which])
    g.evaluate(grads)
    analytic = [gr.get().astype(np.float64).copy() for gr in grads]
    h = 1e-5
    for gi, k in enumerate(which):
        numeric = np.zeros_like(values[k])
        for i in range(values[k].size):
            for sign in (1.0, -1.0):
                moved = values[k].copy()
                moved[i] += sign * h
                g.assign(nodes[k], moved)
                g.evaluate([loss])
                numeric[i] += sign * float(loss.get()[0]) / (2 * h)
        g.assign(nodes[k], values[k])
        scale = max(float(np.abs(numeric).max()), 1.0)
        err = float(np.abs(analytic[gi].reshape(-1) - numeric).max())
        assert err <= 1e-6 * scale + 1e-8, "operand %d: %g off (gradient up to %g)\n%s\n%s" % (
            k, err, scale, analytic[gi].reshape(-1)[:8], numeric[:8])


UNARY = ["ABS", "NEG", "SIN", "COS", "TAN", "EXP", "LOG", "SQRT", "SIGMOID", "TANH", "SQUARE", "CUBE"]


@pytest.mark.parametrize("op", UNARY)
def test_unary(g, op):
    from tenncor_amd import graph
    api = graph.Api(g)
    # TAN away from its poles, LOG and SQRT on positive values, ABS on both signs away from 0
    check(g, api, lambda xs: api.unary(op, xs[0]), [(4, 3)], signs=op in ("ABS", "NEG", "SIN", "COS", "SQUARE", "CUBE", "TANH", "SIGMOID"))
    # composed with itself: the chain rule through two nodes of the kind
    if op not in ("LOG", "SQRT", "TAN", "EXP"):
        check(g, api, lambda xs: api.unary(op, api.unary(op, xs[0])), [(5, 2)], seed=1)


@pytest.mark.parametrize("op", ["ADD", "SUB", "MUL", "DIV", "POW", "MIN", "MAX"])
def test_binary_both_operands(g, op):
    from tenncor_amd import graph
    api = graph.Api(g)
    check(g, api, lambda xs: api.binary(op, xs[0], xs[1]), [(4, 3), (4, 3)])
    # one operand used twice, once through another node
    check(g, api, lambda xs: api.binary(op, xs[0], api.unary("SQUARE", xs[0])), [(3, 4)], seed=2)


def test_nary_add_and_mul(g):
    from tenncor_amd import graph
    api = graph.Api(g)
    check(g, api, lambda xs: g.functor("ADD", xs), [(3, 2)] * 4)
    check(g, api, lambda xs: g.functor("MUL", xs), [(3, 2)] * 4, seed=3)
    check(g, api, lambda xs: g.functor("MUL", [xs[0], xs[1], xs[0]]), [(3, 2)] * 2, seed=4)


def test_select_passes_the_gradient_to_the_chosen_side(g):
    from tenncor_amd import graph
    api = graph.Api(g)
    mask = g.variable(np.array([1, 0, 0, 1, 1, 0, 1, 0], np.float64), [4, 2], "mask")
    check(g, api, lambda xs: api.if_then_else(mask, api.mul(xs[0], xs[1]), api.neg(xs[1])), [(4, 2), (4, 2)])


@pytest.mark.parametrize("op", ["REDUCE_SUM", "REDUCE_PROD"])
@pytest.mark.parametrize("dims", [(0, 1), (1, 1), (0, 2), (1, 2), (0, 3)], ids=lambda d: "offset%d_n%d" % d)
def test_reductions(g, op, dims):
    from tenncor_amd import graph
    api = graph.Api(g)
    check(g, api, lambda xs: api.square(api.reduce(op, xs[0], dims[0], dims[1])), [(3, 4, 2)])


@pytest.mark.parametrize("op", ["REDUCE_MIN", "REDUCE_MAX"])
def test_extremum_reductions_follow_the_reference_rule_not_the_derivative(g, op):
    """tenncor/eteq/backprop.hpp:208-217 passes EQ(extend(out), arg * extend(supgrad))
    down from REDUCE_MIN / REDUCE_MAX: a 0/1 mask that compares the extremum
    with the operand TIMES the incoming gradient, which is the derivative only
    where that gradient is one.  The graphs are pinned to the reference's
    printouts in tests/test_host_backprop.py; here the values: the rule as the
    reference states it, evaluated by numpy."""
    from tenncor_amd import graph
    api = graph.Api(g)
    rng = np.random.default_rng(5)
    x = distinct(rng, 24).astype(np.float64)
    r = np.where(rng.uniform(size=8) < 0.5, 1.0, 2.0)   # incoming gradient: one for some rows, two for others
    vx, vr = g.variable(x, [3, 4, 2], "x"), g.variable(r, [1, 4, 2], "r")
    out = api.reduce(op, vx, 0, 1)
    loss = api.reduce_sum(api.mul(out, vr))
    (grad,) = g.derive(loss, [vx])
    g.evaluate([grad])
    x3 = x.reshape(2, 4, 3)
    extremum = (x3.min if op == "REDUCE_MIN" else x3.max)(axis=2, keepdims=True)
    want = (extremum == x3 * r.reshape(2, 4, 1)).astype(np.float64)
    np.testing.assert_array_equal(grad.get().reshape(2, 4, 3), want)
    assert want.sum() == (r == 1.0).sum()       # the rows whose incoming gradient is one get their mask


def test_data_movement(g):
    from tenncor_amd import graph
    api = graph.Api(g)
    shape = (3, 4, 2)
    w = lambda y: api.mul(y, api.tanh(y))   # a reader whose derivative depends on the value
    check(g, api, lambda xs: w(api.permute(xs[0], [2, 0, 1])), [shape])
    check(g, api, lambda xs: w(api.extend(xs[0], 2, [3])), [(3, 4)], seed=1)
    check(g, api, lambda xs: w(api.extend(api.reduce_sum(xs[0], 1, 1), 1, [4])), [(3, 4)], seed=2)
    check(g, api, lambda xs: w(api.slice(xs[0], 1, 2, 1)), [shape], seed=3)
    check(g, api, lambda xs: w(api.slice(api.slice(xs[0], 1, 2, 0), 0, 1, 2)), [shape], seed=4)
    check(g, api, lambda xs: w(api.pad(xs[0], [[1, 2], [0, 1]])), [(3, 2)], seed=5)
    check(g, api, lambda xs: w(api.reverse(xs[0], [0, 2])), [shape], seed=6)
    check(g, api, lambda xs: w(api.concat([xs[0], xs[1]], 1)), [(3, 2), (3, 3)], seed=7)
    check(g, api, lambda xs: w(api.concat([xs[0], xs[1], xs[0]], 0)), [(1, 3), (1, 3)], seed=8)
    check(g, api, lambda xs: w(g.functor("STRIDE", [xs[0]], dimensions=[2, 1, 2])), [(5, 3, 4)], seed=9)
    # (STRIDE rounds extent / step, cfg/ops.yml:425-438: the gradient of a SCATTER has the
    # operand's shape when the scattered extents round back to it, 5 / 2 -> 3 and 6 / 3 -> 2)
    check(g, api, lambda xs: w(g.functor("SCATTER", [xs[0]], dimensions=[2, 3], shape=[5, 6, 1, 1, 1, 1, 1, 1])), [(3, 2)], seed=10)
    check(g, api, lambda xs: w(g.functor("RESHAPE", [xs[0]], shape=[6, 4, 1, 1, 1, 1, 1, 1])), [shape], seed=11)
    check(g, api, lambda xs: w(api.identity(api.neg(xs[0]))), [(3, 2)], seed=12)


def test_products(g):
    from tenncor_amd import graph
    api = graph.Api(g)
    check(g, api, lambda xs: api.matmul(xs[0], xs[1]), [(4, 3), (5, 4)])
    check(g, api, lambda xs: api.matmul(xs[0], xs[1]), [(4, 3, 2), (5, 4, 2)], seed=1)          # batched
    check(g, api, lambda xs: api.contract(xs[0], xs[1], ((0, 1),)), [(4, 3), (5, 4)], seed=2)
    check(g, api, lambda xs: api.contract(xs[0], xs[1], ((0, 0),)), [(4, 3), (4, 5)], seed=3)
    check(g, api, lambda xs: api.contract(xs[0], xs[1], ((1, 0),)), [(3, 4), (4, 5)], seed=4)
    # (several pairs: listed with the dims of both operands ascending, the order in which
    # tenncor/eteq/backprop.hpp:269-359 takes the product it builds to list them)
    check(g, api, lambda xs: api.contract(xs[0], xs[1], ((0, 1), (2, 2))), [(4, 3, 2), (5, 4, 2)], seed=5)
    check(g, api, lambda xs: api.contract(xs[0], xs[1], ((1, 1), (2, 2))), [(3, 1, 4), (5, 1, 4)], seed=6)
    # the same tensor on both sides
    check(g, api, lambda xs: api.matmul(xs[0], api.permute(xs[0], [1, 0])), [(4, 3)], seed=7)


def test_convolutions(g):
    from tenncor_amd import graph
    api = graph.Api(g)
    check(g, api, lambda xs: api.convolution(xs[0], xs[1], [0, 1]), [(6, 5), (3, 2)])
    check(g, api, lambda xs: api.convolution(xs[0], xs[1], [1, 0]), [(6, 5), (3, 2)], seed=1)
    check(g, api, lambda xs: api.convolution(xs[0], xs[1], [0, 2]), [(5, 2, 4), (2, 3)], seed=2)
    check(g, api, lambda xs: api.conv2d(xs[0], xs[1]), [(2, 5, 4, 3), (3, 2, 2, 3)], seed=3)
    check(g, api, lambda xs: api.conv2d(xs[0], xs[1], zero_padding=((1, 0), (1, 2))), [(2, 4, 3, 2), (3, 2, 2, 2)], seed=4)


def test_layers_of_several_rules(g):
    """softmax + cross entropy over a dense layer: EXTEND of reductions, DIV, LOG and a product in one chain."""
    from tenncor_amd import graph
    api = graph.Api(g)
    labels = g.variable(np.eye(4, dtype=np.float64)[[1, 3, 0]].reshape(-1), [4, 3], "labels")
    check(g, api, lambda xs: api.cross_entropy(labels, api.softmax(api.dense(xs[0], xs[1], xs[2]), 0, 1)),
          [(5, 3), (4, 5), (4,)])
