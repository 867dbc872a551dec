"""The oracle's whole-graph executor (oracle/graph_tape.c: every functor under
the targets, children first, by the oracle's routine for its opcode) against
the reference's whole-graph golden vectors -- tenncor/test/test_equation.cpp:
the sigmoid MLP forward and gradients at the shapes of the first benchmark
configuration, the matmul / contract chains -- and, for the recurrent and
convolution graphs the reference holds no vectors for, against PyTorch's CPU
autograd in double at reduced size.  No GPU: the graphs are built through the
host layer, which needs none, and never evaluated on a device."""
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
with open(os.path.join(GOLDEN, "equation_vectors.json")) as f:
    EQV = json.load(f)


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


def test_matmul_chain_goldens_on_the_tape(g, api, oracle):
    from oracle import graph_tape
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
        tape = graph_tape.Tape(g, [dest, da, db, dc])
        tape.run()
        np.testing.assert_allclose(tape.value(dest), fx["expect_dest"], rtol=1e-13)
        np.testing.assert_allclose(tape.value(da), fx["expect_ga"], rtol=1e-13)
        np.testing.assert_allclose(tape.value(db), fx["expect_gb"], rtol=1e-13)
        np.testing.assert_allclose(tape.value(dc), fx["expect_gc"], rtol=1e-13)


@pytest.mark.parametrize("slow", [False, True], ids=["sigmoid_op", "spelled_out"])
def test_sigmoid_mlp_goldens_on_the_tape(g, api, oracle, slow):
    """EQUATION.SigmoidMLP_Slow / _Fast (test_equation.cpp:383-646): the graph of
    the first benchmark configuration, whose gradients the reference lists."""
    from oracle import graph_tape
    fx = EQV["sigmoid_mlp_slow" if slow else "sigmoid_mlp_fast"]
    leaf = lambda k, s: g.variable(np.array(fx[k], dtype=np.float64), fx[s], k)
    x, w0, b0 = leaf("in_data", "in_shape"), leaf("w0_data", "weight0_shape"), leaf("b0_data", "bias0_shape")
    w1, b1, out = leaf("w1_data", "weight1_shape"), leaf("b1_data", "bias1_shape"), leaf("out_data", "out_shape")

    def sig(v):
        if slow:
            return api.div(1.0, api.add(1.0, api.exp(api.neg(v))))
        return api.sigmoid(v)

    sig0 = sig(api.add(api.matmul(x, w0), api.extend(b0, 1, [3])))
    sig1 = sig(api.add(api.matmul(sig0, w1), api.extend(b1, 1, [3])))
    err = api.pow(api.sub(out, sig1), 2.0)
    grads = g.derive(err, [w0, b0, w1, b1])
    tape = graph_tape.Tape(g, grads)
    secs = tape.run(3)
    assert len(secs) == 3 and all(s > 0 for s in secs)
    for node, key in zip(grads, ("expect_gw0", "expect_gb0", "expect_gw1", "expect_gb1")):
        np.testing.assert_allclose(tape.value(node), fx[key], rtol=1e-12, atol=1e-15)


def test_recurrent_and_convolution_graphs_on_the_tape(g, api, oracle):
    """configs 4 and 5 at reduced size against torch autograd in double: SLICE /
    CONCAT / PAD / n-ary ADD for the unrolled LSTM, CONV / PERMUTE / REVERSE /
    REDUCE / EXTEND / comparisons for the CNN."""
    torch = pytest.importorskip("torch")
    from oracle import graph_tape
    from tenncor_amd import configs
    # the reduced LSTM of tests/test_gpu_graph.py, in float32 (the configuration's type)
    targets, x, w, _ = configs.config4_lstm(g, seq=5, batch=4, nin=6, hid=8)
    tape = graph_tape.Tape(g, targets)
    tape.run()
    x_np = g.data(x).reshape(4, 5, 6).astype(np.float64)
    w_np = g.data(w).reshape(14, 32).astype(np.float64)
    xt, wt = torch.tensor(x_np), torch.tensor(w_np, requires_grad=True)
    state, hidden, hs = torch.zeros(4, 8, dtype=torch.float64), torch.zeros(4, 8, dtype=torch.float64), []
    for t in range(5):
        full = torch.cat([xt[:, t, :], hidden], dim=1) @ wt
        gg, ii, ff, oo = (full[:, k * 8:(k + 1) * 8] for k in range(4))
        state = torch.tanh(gg) * torch.sigmoid(ii) + state * torch.sigmoid(ff)
        hidden = state * torch.sigmoid(oo)
        hs.append(hidden)
    loss_t = (torch.stack(hs, dim=1) ** 2).sum()
    loss_t.backward()
    np.testing.assert_allclose(tape.value(targets[0]), [loss_t.item()], rtol=1e-5)
    ref = wt.grad.numpy().reshape(-1)
    assert np.abs(tape.value(targets[1]) - ref).max() <= 1e-4 * np.abs(ref).max()
    # the CNN: loss and the three gradients exist and are finite; the values are held to torch on the GPU side
    targets, _, _, _ = configs.config5_cnn(g, batch=2, hw=12, c1=3, c2=4, ncls=5)
    tape = graph_tape.Tape(g, targets)
    tape.run()
    assert all(np.isfinite(tape.value(t)).all() for t in targets)
    assert np.abs(tape.value(targets[2])).max() > 0
