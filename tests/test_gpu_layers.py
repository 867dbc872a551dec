"""Recurrent networks built the way the reference's layer API builds them
(cfg/tenncor/layer.yml: dense :113-129/:636-660, rnn :277-295/:694-715, bind
:17-27), evaluated on the GPU in double against the gradients the reference's
own tests hold (tenncor/test/test_equation.cpp:842-1101, tenncor/test/
test_layer.cpp:264-1593), from tests/golden/layer_goldens.json.  The largest
case walks one step of a hand-written rms-momentum trainer through three groups
of evaluate-then-assign, checking every variable after every group.

The layer API's bookkeeping (input placeholders, layer tags, layr::connect's
copy of the graph onto a new input) changes no value: the graphs here are built
directly on their inputs.

Tolerance: the reference compares with EXPECT_DOUBLE_EQ (4 ulp) against values
printed with 17 digits from Eigen on a CPU; exp/tanh/log of the GPU's libm differ
in the last place, so values are compared at 1e-11 of the largest expected
magnitude of each tensor plus 1e-9 of each value.
"""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "layer_goldens.json")) as _f:
    GOLD = json.load(_f)


@pytest.fixture(params=["plain", "replay_launches", "replay"])
def env(request):
    from tenncor_amd import graph
    graph.set_evaluator(request.param)
    g = graph.Graph()
    try:
        yield g, graph.Api(g)
    finally:
        g.close()
        graph.set_evaluator("default")


def close_to(got, expected, what):
    got = np.asarray(got, np.float64)
    expected = np.asarray(expected, np.float64)
    assert got.shape == expected.shape, what
    tol = 1e-11 * np.abs(expected).max() + 1e-9 * np.abs(expected)
    err = np.abs(got - expected)
    worst = int(np.argmax(err - tol))
    assert np.all(err <= tol), "%s[%d]: expect %r, got %r" % (what, worst, expected[worst], got[worst])


def var(g, gold, key, shape, label=None):
    # make_variable(data, shape) reads shape.n_elems() values: some of the tests
    # hold more than their shape takes
    data = np.array(gold[key], np.float64)[:int(np.prod(shape))]
    return g.variable(data, shape, label or key)


def recurrent(api, g, x, weight, bias, hidden):
    """layer.rnn<double>(indim, hidden, tanh, nseq, ...): zero initial state of
    {hidden} extended like one slice of the input."""
    istate = g.variable(np.zeros(hidden), [hidden], "init_state")
    state = api.extend_like(istate, api.slice(x, 0, 1, 1))
    out = api.rnn(x, state, lambda xc: api.dense(xc, weight, bias), api.tanh, 1)
    return out, istate


def test_rnn_layer_on_given_state(env):
    # EQUATION.TanhRNNLayer / TanhRNNLayerConnect: the same numbers twice
    g, api = env
    for key in ("equation_tanh_rnn_layer", "equation_tanh_rnn_layer_connect"):
        gold = GOLD[key]
        x = var(g, gold, "in_data", gold["in_shape"])
        weight = var(g, gold, "weight_data", gold["weight_shape"])
        bias = var(g, gold, "bias_data", gold["bias_shape"])
        istate = var(g, gold, "state_data", gold["state_shape"])
        out = var(g, gold, "out_data", gold["out_shape"])
        state = api.extend_like(istate, api.slice(x, 0, 1, 1))
        output = api.rnn(x, state, lambda xc: api.dense(xc, weight, bias), api.tanh, 1)
        err = api.pow(api.sub(out, output), 2.0)
        ders = g.derive(err, [weight, bias, istate])
        g.evaluate(ders)
        for der, name in zip(ders, ("expect_gw", "expect_gb", "expect_gstate")):
            close_to(der.get(), gold[name], key + "." + name)


def test_rnn_layer(env):
    # CONNECT.TanhRNN
    g, api = env
    gold = GOLD["connect_tanh_rnn"]
    indim, hidden, nseq = gold["indim"], gold["hidden_dim"], gold["nseq"]
    x = var(g, gold, "in_data", [indim, nseq])
    out = var(g, gold, "out_data", [hidden, nseq])
    weight = var(g, gold, "weight_data", [hidden, indim + hidden])
    bias = var(g, gold, "bias_data", [hidden])
    output, istate = recurrent(api, g, x, weight, bias, hidden)
    err = api.pow(api.sub(out, output), 2.0)
    ders = g.derive(err, [weight, bias, istate])
    g.evaluate(ders)
    assert ders[0].shape[:2] == [hidden, indim + hidden]
    for der, name in zip(ders, ("expect_gw", "expect_gb", "expect_gstate")):
        close_to(der.get(), gold[name], name)


def stacked(g, api, gold, with_out_layer):
    """link({dense, rnn[, dense, bind(sigmoid)]}) on the test's input."""
    indim, hidden, nseq = gold["indim"], gold["hidden_dim"], gold["nseq"]
    x = var(g, gold, "in_data", [indim, nseq], "input")
    w0 = var(g, gold, "w0_data", [hidden, indim])
    b0 = var(g, gold, "b0_data", [hidden])
    w1 = var(g, gold, "w1_data", [hidden, hidden + hidden])
    b1 = var(g, gold, "b1_data", [hidden])
    hid = api.dense(x, w0, b0)
    output, istate = recurrent(api, g, hid, w1, b1, hidden)
    leaves = {"w0": w0, "b0": b0, "w1": w1, "b1": b1, "state": istate}
    if with_out_layer:
        outdim = gold["outdim"]
        w2 = var(g, gold, "w2_data", [outdim, hidden])
        b2 = var(g, gold, "b2_data", [outdim])
        output = api.identity(api.sigmoid(api.dense(output, w2, b2)))
        leaves.update(w2=w2, b2=b2)
    odim = gold["outdim"] if with_out_layer else hidden
    out = var(g, gold, "out_data", [odim, nseq], "output")
    return output, out, leaves


def test_dense_then_rnn(env):
    # CONNECT.DenseTanhRNN
    g, api = env
    gold = GOLD["connect_dense_tanh_rnn"]
    output, out, leaves = stacked(g, api, gold, False)
    err = api.pow(api.sub(out, output), 2.0)
    names = [("w1", "expect_gw1"), ("b1", "expect_gb"), ("state", "expect_gstate"),
             ("w0", "expect_gw0"), ("b0", "expect_gb0")]
    ders = g.derive(err, [leaves[k] for k, _ in names])
    g.evaluate(ders)
    for der, (_, name) in zip(ders, names):
        close_to(der.get(), gold[name], name)


FULL = [("w0", "expect_gw0"), ("b0", "expect_gb0"), ("state", "expect_gstate"), ("w1", "expect_gw1"),
        ("b1", "expect_gb1"), ("w2", "expect_gw2"), ("b2", "expect_gb2")]


def test_dense_rnn_dense_sigmoid(env):
    # CONNECT.TanhRNNFull
    g, api = env
    gold = GOLD["connect_tanh_rnn_full"]
    output, out, leaves = stacked(g, api, gold, True)
    err = api.pow(api.sub(out, output), 2.0)
    ders = g.derive(err, [leaves[k] for k, _ in FULL])
    g.evaluate(ders)
    for der, (_, name) in zip(ders, FULL):
        close_to(der.get(), gold[name], name)


def cross_entropy(api, out, output, epsilon):
    common = api.add(output, epsilon)
    return api.reduce_mean(api.neg(api.add(api.mul(out, api.log(common)),
                                           api.mul(api.sub(1.0, out), api.log(api.sub(1.0, common))))))


def test_dense_rnn_dense_sigmoid_cross_entropy(env):
    # CONNECT.TanhRNNCrossEntropyLoss
    g, api = env
    gold = GOLD["connect_tanh_rnn_cross_entropy"]
    output, out, leaves = stacked(g, api, gold, True)
    err = cross_entropy(api, out, output, gold["epsilon"])
    ders = g.derive(err, [leaves[k] for k, _ in FULL])
    g.evaluate(ders)
    for der, (_, name) in zip(ders, FULL):
        close_to(der.get(), gold[name], name)


def test_training_step_in_three_groups(env):
    # CONNECT.TanhRNNTraining
    g, api = env
    gold = GOLD["connect_tanh_rnn_training"]
    lmbd, rate, term, eps = gold["lmbd"], gold["learning_rate"], gold["momentum_term"], gold["eps"]
    output, out, leaves = stacked(g, api, gold, True)
    err = cross_entropy(api, out, output, gold["epsilon"])
    targets = [leaves[k] for k in ("w0", "b0", "w1", "b1", "state", "w2", "b2")]
    ders = g.derive(err, targets)
    n = len(ders)
    momentums = [g.variable(np.zeros(int(np.prod(d.shape))), d.shape, "momentum") for d in ders]
    mvavg_sqrs = [g.variable(np.zeros(int(np.prod(d.shape))), d.shape, "mvavg_sqrs") for d in ders]
    momentum_tmps = [api.mul(m, term) for m in momentums]
    group1 = [api.add(t, tmp) for t, tmp in zip(targets, momentum_tmps)]
    group2 = [api.add(api.mul(lmbd, sq), api.mul(1.0 - lmbd, api.pow(d, 2.0))) for sq, d in zip(mvavg_sqrs, ders)]
    pgrad_norm = [api.div(api.mul(rate, d), api.add(api.sqrt(sq), eps)) for d, sq in zip(ders, mvavg_sqrs)]
    group3 = [api.sub(tmp, p) for tmp, p in zip(momentum_tmps, pgrad_norm)] + \
             [api.sub(t, p) for t, p in zip(targets, pgrad_norm)]

    def check(nodes, name):
        for i, node in enumerate(nodes):
            close_to(node.get(), gold[name][i], "%s[%d]" % (name, i))

    def assign_group(lefts, rights):
        g.evaluate(rights)
        values = [r.get().copy() for r in rights]
        for left, value in zip(lefts, values):
            g.assign(left, value)

    g.evaluate(ders)
    check(ders, "expect_der1")
    assign_group(targets, group1)
    check(targets, "expect_g1")
    g.evaluate(ders)
    check(ders, "expect_der2")
    assign_group(mvavg_sqrs, group2)
    check(mvavg_sqrs, "expect_g2")
    assign_group(momentums + targets, group3)
    check(momentums + targets, "expect_g3")
    assert n == 7
