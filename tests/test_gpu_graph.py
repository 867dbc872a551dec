"""GPU parity of whole graphs built through the host layer (Functor nodes, the
gradient builder, teq::Evaluator + eigen::Device): the reference's own
whole-graph golden vectors (tenncor/test/test_equation.cpp, test_api.cpp) in
double, and the benchmark configurations 1, 4 and 5 at reduced size against
PyTorch's CPU autograd as an independent library routine.

Tolerances: goldens are compared at 1e-12 relative (the reference asserts
EXPECT_DOUBLE_EQ against Eigen; device libm differs from it in the last bits);
fp32 graphs at the 1e-4 relative bar of the north star, relative to
max(|ref|, mean |ref|).
"""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
with open(os.path.join(GOLDEN, "equation_vectors.json")) as f:
    EQV = json.load(f)


@pytest.fixture(autouse=True)
def plain_evaluator_afterwards():
    """Set up before the graph of a test, so that it runs after the graph is
    closed: a test that installs another evaluator leaves the default behind."""
    yield
    from tenncor_amd import graph
    graph.set_evaluator("default")


@pytest.fixture()
def g():
    from tenncor_amd import graph
    gr = graph.Graph()
    yield gr
    gr.close()


@pytest.fixture()
def api(g):
    from tenncor_amd import graph
    return graph.Api(g)


def close(got, ref, rtol):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    floor = np.mean(np.abs(ref)) if ref.size else 0.0
    denom = np.maximum(np.abs(ref), floor)
    denom[denom == 0] = 1.0
    err = np.abs(got - ref) / denom
    assert err.max() <= rtol, "max rel err %.3g at %d: got %r ref %r" % (
        err.max(), err.argmax(), got.flat[err.argmax()], ref.flat[err.argmax()])


def npv(flat, shape):
    """numpy view of a tenncor tensor: reversed dims."""
    return np.asarray(flat).reshape([d for d in reversed(shape)])


@pytest.mark.parametrize("optimized", [False, True], ids=["as_built", "optimized"])
def test_matmul_chain_golden(g, api, optimized):
    """tenncor/test/test_equation.cpp:26-136, forward and three gradients."""
    for key, mm in (("matmul_complex", api.matmul), ("contract_equivalent", api.contract)):
        fx = EQV[key]
        a = g.variable(np.array(fx["data"]), fx["alist"], "a")
        b = g.variable(np.array(fx["data2"]), fx["blist"], "b")
        c = g.variable(np.array(fx["data3"]), fx["clist"], "c")
        d = mm(a, b)
        e = mm(c, d)
        f = mm(api.transpose(d), api.transpose(c))
        dest = mm(e, f)
        da, db, dc = g.derive(dest, [a, b, c])
        if optimized:  # EQUATION.OptimizedMatmulComplex, test_equation.cpp:1146-1154
            (dest, da, db, dc), _ = g.optimize([dest, da, db, dc])
        g.evaluate([dest, da, db, dc])
        np.testing.assert_allclose(dest.get(), fx["expect_dest"], rtol=1e-13)
        np.testing.assert_allclose(da.get(), fx["expect_ga"], rtol=1e-13)
        np.testing.assert_allclose(db.get(), fx["expect_gb"], rtol=1e-13)
        np.testing.assert_allclose(dc.get(), fx["expect_gc"], rtol=1e-13)
        g.evaluate([dest, da, db, dc])  # idempotency check, as the reference does
        np.testing.assert_allclose(da.get(), fx["expect_ga"], rtol=1e-13)


def mlp_graph(g, api, fx, np_dtype, slow):
    leaf = lambda k, s: g.variable(np.array(fx[k], dtype=np_dtype), fx[s], k)
    x, w0, b0 = leaf("in_data", "in_shape"), leaf("w0_data", "weight0_shape"), leaf("b0_data", "bias0_shape")
    w1, b1, out = leaf("w1_data", "weight1_shape"), leaf("b1_data", "bias1_shape"), leaf("out_data", "out_shape")

    def sig(v):
        if slow:  # 1 / (1 + exp(-x)) spelled out, test_equation.cpp:413-417
            return api.div(1.0, api.add(1.0, api.exp(api.neg(v))))
        return api.sigmoid(v)

    sig0 = sig(api.add(api.matmul(x, w0), api.extend(b0, 1, [3])))
    sig1 = sig(api.add(api.matmul(sig0, w1), api.extend(b1, 1, [3])))
    err = api.pow(api.sub(out, sig1), 2.0)
    return err, [w0, b0, w1, b1], x


@pytest.mark.parametrize("optimized", [False, True], ids=["as_built", "optimized"])
@pytest.mark.parametrize("slow", [False, True], ids=["sigmoid_op", "spelled_out"])
def test_config1_mlp_gradients_golden(g, api, slow, optimized):
    """tenncor/test/test_equation.cpp:252-706: exactly the config-1 shapes
    (x{10,3}, W0{9,10}, b0{9}, W1{5,9}, b1{5}) with 17-digit goldens."""
    fx = EQV["sigmoid_mlp_slow" if slow else "sigmoid_mlp_fast"]
    err, params, _ = mlp_graph(g, api, fx, np.float64, slow)
    grads = g.derive(err, params)
    if optimized:  # EQUATION.OptimizedSlow/FastSigmoidMLP, test_equation.cpp:1157-1176
        grads, _ = g.optimize(grads)
    g.evaluate(grads)
    for grad, key, shp in zip(grads, ("expect_gw0", "expect_gb0", "expect_gw1", "expect_gb1"),
                              ("weight0_shape", "bias0_shape", "weight1_shape", "bias1_shape")):
        assert grad.shape[:len(fx[shp])] == fx[shp]
        np.testing.assert_allclose(grad.get(), fx[key], rtol=1e-12)


def test_config1_mlp_fp32_and_reassignment(g, api):
    """fp32 (the config's dtype) within 1e-4 of the double goldens; assigning a
    new input recomputes, assigning the old one back reproduces the values."""
    fx = EQV["sigmoid_mlp_fast"]
    err, params, x = mlp_graph(g, api, fx, np.float32, False)
    grads = g.derive(err, params)
    g.evaluate(grads)
    first = [gr.get() for gr in grads]
    for got, key in zip(first, ("expect_gw0", "expect_gb0", "expect_gw1", "expect_gb1")):
        close(got, fx[key], 1e-4)
    versions = [g.version(gr) for gr in grads]
    g.assign(x, np.array(fx["in_data"], np.float32)[::-1].copy())
    g.evaluate(grads)
    assert all(g.version(gr) > v for gr, v in zip(grads, versions))
    assert not np.allclose(grads[0].get(), first[0])
    g.assign(x, np.array(fx["in_data"], np.float32))
    g.evaluate(grads)
    for got, want in zip([gr.get() for gr in grads], first):
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("optimized", [False, True], ids=["as_built", "optimized"])
def test_tanh_rnn_golden(g, api, optimized):
    """tenncor/test/test_equation.cpp:709-839: unrolled tanh RNN (SLICE, CONCAT,
    CONTRACT, n-ary CONCAT and their gradients) with golden gradients."""
    fx = EQV["tanh_rnn"]
    leaf = lambda k, s: g.variable(np.array(fx[k]), fx[s], k)
    x, weight, bias = leaf("in_data", "in_shape"), leaf("weight_data", "weight_shape"), leaf("bias_data", "bias_shape")
    istate, out = leaf("state_data", "state_shape"), leaf("out_data", "out_shape")
    state, states = istate, []
    for i in range(x.shape[1]):
        inslice = api.slice(x, i, 1, 1)
        fc = api.contract(api.concat([inslice, state], 0), weight)
        state = api.tanh(api.add(fc, api.extend_like(bias, fc)))
        states.append(state)
    output = api.concat(states, 1)
    err = api.pow(api.sub(out, output), 2.0)
    dw, db, dstate = g.derive(err, [weight, bias, istate])
    if optimized:  # EQUATION.OptimizedTanhRNN, test_equation.cpp:1179-1187
        (dw, db, dstate), _ = g.optimize([dw, db, dstate])
    g.evaluate([dw, db, dstate])
    np.testing.assert_allclose(dw.get(), fx["expect_gw"], rtol=1e-12)
    np.testing.assert_allclose(db.get(), fx["expect_gb"], rtol=1e-12)
    np.testing.assert_allclose(dstate.get(), fx["expect_gstate"], rtol=1e-12)


def test_api_convolution_gradients_golden(g, api):
    """tenncor/test/test_api.cpp:2265-2373: forward, image and kernel gradients."""
    fx = EQV["api_convolution"]
    img = g.constant(np.array(fx["data"]), fx["alist"])
    ker = g.constant(np.array(fx["data2"]), fx["blist"])
    dest = api.convolution(img, ker, list(range(8)))
    gl, gr = g.derive(dest, [img, ker])
    g.evaluate([dest, gl, gr])
    assert dest.shape == fx["expectslist"]
    np.testing.assert_array_equal(dest.get(), fx["expect_out"])
    np.testing.assert_array_equal(gl.get(), fx["expect_ga"])
    np.testing.assert_array_equal(gr.get(), fx["expect_gb"])


def test_api_matmul_int32_gradients_golden(g, api):
    """tenncor/test/test_api.cpp:1986-2085 (int32 data, exact gradients)."""
    fx = EQV["api_matmul"]
    a = g.constant(np.array(fx["data"], np.int32), fx["alist"])
    b = g.constant(np.array(fx["data2"], np.int32), fx["blist"])
    dest = api.matmul(a, b)
    gl, gr = g.derive(dest, [a, b])
    g.evaluate([dest, gl, gr])
    np.testing.assert_array_equal(npv(dest.get(), [4, 2]),
                                  npv(fx["data"], [3, 2]) @ npv(fx["data2"], [4, 3]))
    np.testing.assert_array_equal(gl.get(), fx["expect_ga"])
    np.testing.assert_array_equal(gr.get(), fx["expect_gb"])


def test_api_contract_int32_gradients_golden(g, api):
    """tenncor/test/test_api.cpp:2089-2190: a{3,1,2} and b{4,1,3} contracted
    over a's dim 0 and b's dim 2 in int32; forward against numpy, both
    gradients exact, and the gradient of contracting a tensor with itself."""
    fx = EQV["api_contract"]
    a = g.constant(np.array(fx["data"], np.int32), fx["alist"])
    b = g.constant(np.array(fx["data2"], np.int32), fx["blist"])
    dest = api.contract(a, b, [(0, 2)])
    assert dest.shape[:4] == [4, 1, 1, 2]
    (gl,), (gr,) = g.derive(dest, [a]), g.derive(dest, [b])
    g.evaluate([dest, gl, gr])
    g.evaluate([dest, gl, gr])  # idempotency check, as the reference does
    av, bv = npv(fx["data"], fx["alist"]), npv(fx["data2"], fx["blist"])  # np[2,1,3], np[3,1,4]
    np.testing.assert_array_equal(npv(dest.get(), [4, 1, 1, 2]).reshape(2, 4), av.reshape(2, 3) @ bv.reshape(3, 4))
    np.testing.assert_array_equal(gl.get(), fx["expect_ga"])
    np.testing.assert_array_equal(gr.get(), fx["expect_gb"])
    c = g.constant(np.array(fx["data3"], np.int32), fx["sqrlist"])
    (gs,) = g.derive(api.contract(c, c, [(0, 0)]), [c])
    g.evaluate([gs])
    assert gs.shape[:2] == fx["sqrlist"]


def test_group_sum_and_buffers_return_to_the_pool(g, api):
    """tenncor/test/test_api.cpp:2376-2414 (4-argument ADD) and the TTL
    protocol: after an evaluation only leaves and targets hold device memory."""
    from tenncor_amd import capi
    fx = EQV["api_group_sum"]
    xs = [g.variable(np.array(fx[k]), fx["slist"], k) for k in ("data", "data2", "data3", "data4")]
    total = g.functor("ADD", xs)
    sq = api.square(api.exp(total))
    out = api.reduce_sum(sq, 0, 2)
    g.evaluate([out])
    want = np.exp(sum(np.array(fx[k]) for k in ("data", "data2", "data3", "data4"))) ** 2
    np.testing.assert_allclose(out.get(), npv(want, fx["slist"]).sum(axis=(1, 2)), rtol=1e-12)
    # intermediates (total, exp, square) expired: asking for their data fails
    from tenncor_amd import graph
    for node in (total, sq):
        with pytest.raises(graph.GraphError):
            node.get()
    assert out.get().shape == (4,)


def torch_reference():
    """PyTorch's CPU autograd in fp64 is the independent reference of configs 4
    and 5: a box without it must fail these cases, not skip them."""
    try:
        import torch
    except ImportError as err:
        pytest.fail("torch is needed as the reference of this case and cannot be imported: %s" % err)
    torch.set_num_threads(4)
    return torch


def evaluate_under(g, evaluator, targets, fed, fed_value):
    """One evaluation under the walk, or three under the replaying evaluator
    with the input assigned anew before each (walked, recorded, replayed):
    the values the targets hold afterwards come from the recording."""
    from tenncor_amd import graph
    if evaluator == "plain":
        g.evaluate(targets)
        return
    graph.set_evaluator(evaluator)  # until the end of the test (plain_evaluator_afterwards)
    for _ in range(3):
        g.assign(fed, fed_value)
        g.evaluate(targets)
    stats = graph.evaluator_stats()
    assert stats["recorded"] == 1 and stats["replayed"] >= 1, stats


@pytest.mark.parametrize("evaluator", ["plain", "replay"])
@pytest.mark.parametrize("seq,batch,nin,hid,np_dtype,rtol", [
    (6, 5, 7, 8, np.float32, 1e-4), (64, 256, 256, 512, np.float32, 1e-4), (8, 256, 256, 512, np.float64, 1e-10)],
    ids=["reduced", "full_size", "double_on_matrix_cores"])
def test_config4_lstm_forward_and_gradient(g, api, seq, batch, nin, hid, np_dtype, rtol, evaluator):
    """config 4 at reduced size (seq 6, batch 5, in 7, hidden 8) and at its
    full size: the layer.yml lstm recipe with one fused gate weight {4h, in+h}
    cut by SLICEs, loss = sum(h^2) over the concatenated hidden outputs,
    against torch autograd in fp64.  The third case is the graph in double at
    the full widths (its 256x768x2048 products run on the fp64 matrix cores),
    eight steps long, at 1e-10.  Under "replay" the values compared are those
    of the third evaluation, which a recording serves: the launches the
    benchmark times (shared launches, products over parts of concatenations,
    products with their reading group as epilogue) are held to torch
    directly, at the same bar."""
    torch = torch_reference()
    if batch > 16:
        torch.set_num_threads(16)
    rng = np.random.default_rng(4)
    w_np = rng.normal(0, 0.05, (nin + hid, 4 * hid)).astype(np_dtype)   # np[768,2048] in the config
    x_np = rng.uniform(-1, 1, (batch, seq, nin)).astype(np_dtype)       # np[batch,seq,in]
    x = g.variable(x_np, [nin, seq, batch], "x")
    w = g.variable(w_np, [4 * hid, nin + hid], "w")
    zeros = np.zeros(hid * batch, np_dtype)
    state0 = g.constant(zeros, [hid, 1, batch])
    hidden0 = g.constant(zeros, [hid, 1, batch])

    def gate(k):
        def fn(xc):
            full = api.contract(xc, w)                      # {4h, 1, batch}
            return api.slice(full, k * hid, hid, 0)         # gate k's columns
        return fn

    out = api.lstm(x, state0, hidden0, {"g": gate(0), "i": gate(1), "f": gate(2), "o": gate(3)}, seq_dim=1)
    loss = api.reduce_sum(api.square(out))
    (dw,) = g.derive(loss, [w])
    evaluate_under(g, evaluator, [out, loss, dw], x, x_np)

    xt = torch.tensor(x_np, dtype=torch.float64)
    wt = torch.tensor(w_np, dtype=torch.float64, requires_grad=True)
    state = torch.zeros(batch, hid, dtype=torch.float64)
    hidden = torch.zeros(batch, hid, dtype=torch.float64)
    hs = []
    for t in range(seq):
        xc = torch.cat([xt[:, t, :], hidden], dim=1)
        full = xc @ wt
        gg, ii, ff, oo = (full[:, k * hid:(k + 1) * hid] for k in range(4))
        state = torch.tanh(gg) * torch.sigmoid(ii) + state * torch.sigmoid(ff)
        hidden = state * torch.sigmoid(oo)
        hs.append(hidden)
    h_all = torch.stack(hs, dim=1)  # [batch, seq, hid]
    loss_t = (h_all ** 2).sum()
    loss_t.backward()
    assert out.shape[:3] == [hid, seq, batch]
    close(out.get(), h_all.detach().numpy().reshape(-1), rtol)
    close(loss.get(), [loss_t.item()], rtol)
    close(dw.get(), wt.grad.numpy().reshape(-1), rtol)


@pytest.mark.parametrize("batch,hw,c1,c2,ncls,np_dtype,rtol", [
    (3, 12, 4, 6, 5, np.float32, 1e-4), (16, 20, 8, 32, 10, np.float32, 1e-4), (128, 28, 32, 64, 10, np.float32, 1e-4),
    (16, 20, 8, 32, 10, np.float64, 1e-10)],
    ids=["direct_kernels", "matrix_products", "full_size", "double"])
@pytest.mark.parametrize("evaluator", ["plain", "replay"])
def test_config5_cnn_forward_and_gradient(g, api, batch, hw, c1, c2, ncls, np_dtype, rtol, evaluator):
    """config 5 at reduced size (5x5 kernels 1->c1->c2, dense c2->ncls): the
    nn.yml conv2d idiom and its gradient idioms (PAD / REVERSE / CONV / PERMUTE
    / SLICE), softmax cross-entropy, against torch.  The first size stays on
    the direct convolution kernels; at the second the second layer's forward,
    image-gradient and kernel-gradient convolutions run as matrix products.
    Under "replay" the values compared are those of the third evaluation,
    served by a recording (convolutions over views, shared launches)."""
    torch = torch_reference()
    if batch > 16:
        torch.set_num_threads(16)
    F = torch.nn.functional
    rng = np.random.default_rng(5)
    x_np = rng.uniform(0, 1, (batch, hw, hw, 1)).astype(np_dtype)
    k1_np = rng.normal(0, 0.2, (5, 5, 1, c1)).astype(np_dtype)          # np[kh,kw,in,out]
    k2_np = rng.normal(0, 0.4 / np.sqrt(c1), (5, 5, c1, c2)).astype(np_dtype)
    # logits of order one: a saturated softmax makes the comparison with fp64 meaningless
    wd_std = 0.3 if hw <= 12 else 2.0 / ((hw - 8) ** 2 * np.sqrt(c2))
    wd_np = rng.normal(0, wd_std, (c2, ncls)).astype(np_dtype)
    labels = rng.integers(0, ncls, batch)
    y_np = np.eye(ncls, dtype=np_dtype)[labels]
    x = g.variable(x_np, [1, hw, hw, batch], "x")
    k1 = g.variable(k1_np, [c1, 1, 5, 5], "k1")
    k2 = g.variable(k2_np, [c2, c1, 5, 5], "k2")
    wd = g.variable(wd_np, [ncls, c2], "wd")
    y = g.variable(y_np, [ncls, 1, 1, batch], "y")
    h1 = api.relu(api.conv2d(x, k1))
    h2 = api.relu(api.conv2d(h1, k2))
    pooled = api.reduce_sum(h2, 1, 2)                                     # {c2,1,1,batch}
    logits = api.contract(pooled, wd)                                     # {ncls,1,1,batch}
    probs = api.softmax(logits, 0, 1)
    loss = api.reduce_sum(api.cross_entropy(y, probs))
    grads = g.derive(loss, [k1, k2, wd])
    evaluate_under(g, evaluator, [loss] + grads, x, x_np)

    xt = torch.tensor(x_np, dtype=torch.float64).permute(0, 3, 1, 2)
    k1t = torch.tensor(k1_np, dtype=torch.float64, requires_grad=True)
    k2t = torch.tensor(k2_np, dtype=torch.float64, requires_grad=True)
    wdt = torch.tensor(wd_np, dtype=torch.float64, requires_grad=True)
    yt = torch.tensor(y_np, dtype=torch.float64)
    eps = float(np.finfo(np.float32).eps)
    a1 = F.relu(F.conv2d(xt, k1t.permute(3, 2, 0, 1)))
    a2 = F.relu(F.conv2d(a1, k2t.permute(3, 2, 0, 1)))
    pooled_t = a2.sum(dim=(2, 3))
    logits_t = pooled_t @ wdt
    # the reference's gradient of REDUCE_MAX is EQ(extend(max), arg * extend(gradient))
    # (tenncor/eteq/backprop.hpp:208-217), which is zero wherever arg * gradient differs
    # from the maximum, i.e. nothing flows back through the shift of the softmax: detached here.
    # (With the epsilon in the denominator that path would carry about 1e-8 of the gradient.)
    ex = torch.exp(logits_t - logits_t.max(dim=1, keepdim=True).values.detach())
    probs_t = ex / (ex.sum(dim=1, keepdim=True) + eps)
    inp = probs_t + eps
    loss_t = -(yt * torch.log(inp) + (1 - yt) * torch.log(1 - inp)).sum()
    loss_t.backward()
    close(loss.get(), [loss_t.item()], rtol)
    close(grads[2].get(), wdt.grad.numpy().reshape(-1), rtol)
    close(grads[1].get(), k2t.grad.numpy().reshape(-1), rtol)
    close(grads[0].get(), k1t.grad.numpy().reshape(-1), rtol)


def test_assign_sub_updates_the_leaf_in_place(g, api):
    """sgd step (cfg/tenncor/approx.yml:52): ASSIGN_SUB(w, lr * grad); the
    leaf's host view follows the device copy and its version moves on."""
    w = g.variable(np.array([1.0, 2.0, 3.0, 4.0], np.float32), [4], "w")
    x = g.variable(np.array([0.5, -1.0, 2.0, 0.0], np.float32), [4], "x")
    loss = api.reduce_sum(api.square(api.mul(w, x)))
    (dw,) = g.derive(loss, [w])
    step = g.functor("ASSIGN_SUB", [w, api.mul(0.1, dw)])
    v0 = g.version(w)
    g.evaluate([step])
    want = np.array([1.0, 2.0, 3.0, 4.0]) - 0.1 * 2 * np.array([1.0, 2.0, 3.0, 4.0]) * np.array([0.5, -1.0, 2.0, 0.0]) ** 2
    np.testing.assert_allclose(w.get(), want, rtol=1e-6)
    np.testing.assert_allclose(step.get(), want, rtol=1e-6)
    assert g.version(w) > v0
    g.evaluate([loss])
    np.testing.assert_allclose(loss.get(), [np.sum((want * np.array([0.5, -1.0, 2.0, 0.0])) ** 2)], rtol=1e-5)


def test_aliases_casts_and_rand(g, api):
    """Zero-copy nodes (IDENTITY, RESHAPE, last-dim SLICE), CAST and RAND_UNIF."""
    from tenncor_amd import capi
    data = np.arange(24, dtype=np.float32)
    x = g.variable(data, [3, 2, 4], "x")
    ident = api.identity(x)
    resh = g.functor("RESHAPE", [api.neg(x)], shape=[6, 4, 1, 1, 1, 1, 1, 1])
    last = api.slice(api.neg(x), 2, 1, 2)          # alias at element offset 12
    mid = api.slice(x, 1, 1, 1)                    # real copy
    casted = g.functor("CAST", [api.mul(x, 0.5)], dtype=capi.INT32)
    doubled = api.mul(last, 2.0)
    g.evaluate([ident, resh, last, mid, casted, doubled])
    np.testing.assert_array_equal(ident.get(), data)
    np.testing.assert_array_equal(resh.get(), -data)
    assert resh.shape[:2] == [6, 4]
    np.testing.assert_array_equal(last.get(), -data[12:18])
    np.testing.assert_array_equal(mid.get(), npv(data, [3, 2, 4])[:, 1:2, :].reshape(-1))
    np.testing.assert_array_equal(casted.get(), (data * 0.5).astype(np.int32))
    np.testing.assert_array_equal(doubled.get(), -2 * data[12:18])
    lo = g.scalar(0.25, np.float64, [31, 21])
    hi = g.scalar(3.2, np.float64, [31, 21])
    r = g.functor("RAND_UNIF", [lo, hi])
    g.evaluate([r])
    first = r.get()
    assert first.min() > 0.25 and first.max() < 3.2
    g.evaluate([r])  # not idempotent: a new draw every evaluation
    assert not np.array_equal(first, r.get())


def test_padded_image_read_by_convolutions_and_by_others(g, api, oracle):
    """A PAD node whose only readers are CONV nodes has its border left
    unwritten; as soon as anything else reads it (an evaluation target, another
    operator) it must hold the zeros PAD defines (internal/eigen/operator.hpp:
    257-275).  The buffer is dirtied first so that a missing border would show."""
    rng = np.random.default_rng(5)
    C, W, H, B, O, KW, KH = 2, 6, 5, 2, 3, 3, 2
    xv = rng.integers(1, 9, C * W * H * B).astype(np.float32)
    kv = rng.integers(-4, 5, O * C * KW * KH).astype(np.float32)
    padded_ref, pshape = oracle.pad(xv, [C, W, H, B], [[0, 0]] * 4 + [[O - 1, O - 1]])
    conv_ref, oshape = oracle.conv(padded_ref, pshape, kv, [O, C, KW, KH], [4, 0, 1, 2])
    n_pad = oracle.n_elems(pshape)
    # leave non-zero garbage of the padded size in the pool
    junk = g.variable(np.full(n_pad, 7.0, np.float32), pshape[:5], "junk")
    dirty = api.reduce_sum(api.add(junk, 1.0))
    g.evaluate([dirty])
    x = g.variable(xv, [C, W, H, B], "x")
    k = g.variable(kv, [O, C, KW, KH], "k")
    pad = api.pad(x, [[0, 0]] * 4 + [[O - 1, O - 1]])
    conv = api.convolution(pad, k, [4, 0, 1, 2])
    g.evaluate([conv])
    np.testing.assert_array_equal(conv.get(), conv_ref)
    # now the padded image itself is asked for too
    total = api.reduce_sum(pad)
    g.assign(junk, np.full(n_pad, 5.0, np.float32))
    g.assign(x, xv)
    g.evaluate([dirty])
    g.evaluate([conv, pad, total])
    np.testing.assert_array_equal(conv.get(), conv_ref)
    np.testing.assert_array_equal(pad.get(), padded_ref)
    np.testing.assert_array_equal(total.get(), [xv.sum()])


# ---- optimiser steps on the device (cfg/tenncor/approx.yml) -------------------

def numpy_optimisers(rule, w, grad_fn, steps, **kw):
    """The update rules restated in numpy (fp64), one trajectory of `steps`."""
    eps = float(np.finfo(np.float32).eps)
    state = {}
    traj = []
    w = w.astype(np.float64).copy()
    for _ in range(steps):
        g = grad_fn(w)
        if rule == "sgd":
            w = w - kw.get("learning_rate", 0.5) * g
        elif rule == "adagrad":
            state["m"] = state.get("m", np.ones_like(w)) + g * g
            w = w - kw.get("learning_rate", 0.5) * g / (np.sqrt(state["m"]) + eps)
        elif rule == "rms_momentum":
            d = kw.get("discount_factor", 0.99)
            state["m"] = d * state.get("m", np.ones_like(w)) + (1 - d) * g * g
            w = w - kw.get("learning_rate", 0.5) * g / (np.sqrt(state["m"]) + eps)
        elif rule == "adam":
            b1, b2, lr = kw.get("decay1", 0.9), kw.get("decay2", 0.999), kw.get("step_rate", 0.001)
            state["m"] = b1 * state.get("m", np.zeros_like(w)) + (1 - b1) * g
            state["v"] = b2 * state.get("v", np.zeros_like(w)) + (1 - b2) * g * g
            state["t"] = state.get("t", 0) + 1
            mc = state["m"] / (1 - b1 ** state["t"])
            vc = state["v"] / (1 - b2 ** state["t"])
            w = w - lr * mc / (np.sqrt(vc) + eps)
        elif rule == "adadelta":
            d, off, lr = kw.get("decay", 0.9), kw.get("offset", 0.0001), kw.get("step_rate", 1.0)
            state["msg"] = d * state.get("msg", np.zeros_like(w)) + (1 - d) * g * g
            delta = lr * np.sqrt(state.get("msd", np.zeros_like(w)) + off) / (np.sqrt(state["msg"] + off) + eps) * g
            state["msd"] = d * state.get("msd", np.zeros_like(w)) + (1 - d) * delta * delta
            w = w - delta
        traj.append(w.copy())
    return traj


@pytest.mark.parametrize("evaluator", ["plain", "replay"])
@pytest.mark.parametrize("rule,kw", [("sgd", {"learning_rate": 0.05}), ("adagrad", {"learning_rate": 0.1}),
                                     ("rms_momentum", {"learning_rate": 0.01}), ("adam", {"step_rate": 0.01}),
                                     ("adadelta", {})])
def test_optimiser_steps_stay_on_the_device(rule, kw, evaluator):
    """Five steps of every ApproxAPI rule on a least-squares problem: the
    variable (and the rule's state variables) are updated in place by ASSIGN*
    nodes; the host view of the weights after each step follows numpy's
    trajectory of the same rule to fp32 accuracy."""
    from tenncor_amd import graph
    rng = np.random.default_rng(31)
    xv = rng.uniform(-1, 1, (6, 4)).astype(np.float32)     # np[batch, in]
    yv = rng.uniform(-1, 1, (6, 3)).astype(np.float32)
    w0 = rng.uniform(-0.5, 0.5, (4, 3)).astype(np.float32)

    def grad_fn(w):
        r = xv.astype(np.float64) @ w - yv
        return 2 * xv.astype(np.float64).T @ r

    want = numpy_optimisers(rule, w0, grad_fn, 5, **kw)
    graph.set_evaluator(evaluator)
    g = graph.Graph()
    try:
        api = graph.Api(g)
        x = g.variable(xv, [4, 6], "x")
        y = g.variable(yv, [3, 6], "y")
        w = g.variable(w0, [3, 4], "w")
        err = api.reduce_sum(api.square(api.sub(api.matmul(x, w), y)))
        updates = getattr(graph.Approx(api), rule)(err, [w], **kw)
        step = graph.Approx(api).apply_update(err, updates)
        for i in range(5):
            g.evaluate([step])
            np.testing.assert_allclose(w.get().reshape(4, 3), want[i], rtol=2e-4, atol=2e-6)
        r = xv.astype(np.float64) @ want[3] - yv
        np.testing.assert_allclose(step.get(), [np.sum(r * r)], rtol=1e-4)   # error at the weights the step began with
        if evaluator == "replay":
            assert graph.evaluator_stats()["replayed"] >= 3
    finally:
        g.close()
        graph.set_evaluator("default")


def test_prefetch_uploads_a_leaf_ahead_of_the_evaluation(g, api):
    """tcr_prefetch: the device copy of a re-assigned leaf is brought up to date at the call;
    the evaluation that follows computes from the new value either way, and a functor is refused."""
    from tenncor_amd import graph
    x = g.variable(np.arange(12, dtype=np.float32), [4, 3], "x")
    y = api.square(x)
    for i in range(4):
        v = np.arange(12, dtype=np.float32) + i
        g.assign(x, v)
        if i % 2:
            g.prefetch(x)
            g.prefetch(x)  # nothing left to copy
        g.evaluate([y])
        np.testing.assert_array_equal(y.get(), v * v)
    with pytest.raises(graph.GraphError):
        g.prefetch(y)
