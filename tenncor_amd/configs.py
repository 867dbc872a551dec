"""The five benchmark configurations as tenncor graphs, built through the host
layer exactly as a tenncor user would build them (cfg/tenncor/*.yml recipes in
``graph.Api``), at full or reduced size.  Data is synthetic and seeded.
"""
import numpy as np

from . import graph as tg


def config1_mlp(g, seed=1, batch=3, np_dtype=np.float32):
    """Dense MLP forward+gradient (demo/gd_demo.cpp:104-168): x[batch,10],
    target[batch,5], 10 -> 9 -> 5 with sigmoids, MSE loss, gradients w.r.t.
    W0, b0, W1, b1.  Returns (targets, x variable, parameter variables)."""
    api = tg.Api(g)
    rng = np.random.default_rng(seed)
    lim = np.sqrt(6.0 / 19.0)
    x = g.variable(rng.uniform(-1, 1, (batch, 10)).astype(np_dtype), [10, batch], "x")
    y = g.variable(rng.uniform(0, 1, (batch, 5)).astype(np_dtype), [5, batch], "target")
    w0 = g.variable(rng.uniform(-lim, lim, (10, 9)).astype(np_dtype), [9, 10], "w0")
    b0 = g.variable(np.zeros(9, np_dtype), [9], "b0")
    w1 = g.variable(rng.uniform(-lim, lim, (9, 5)).astype(np_dtype), [5, 9], "w1")
    b1 = g.variable(np.zeros(5, np_dtype), [5], "b1")
    h = api.sigmoid(api.dense(x, w0, b0))
    out = api.sigmoid(api.dense(h, w1, b1))
    diff = api.sub(y, out)
    loss = api.div(api.reduce_sum(api.square(diff)), float(batch * 5))
    grads = g.derive(loss, [w0, b0, w1, b1])
    return [loss] + grads, x, [w0, b0, w1, b1]


def config4_lstm(g, seed=4, seq=64, batch=256, nin=256, hid=512):
    """LSTM unrolled over `seq` steps (cfg/tenncor/layer.yml:716-768) with one
    fused gate weight np[in+hid, 4*hid] cut into the four gates by SLICEs;
    loss = sum of squared hidden outputs; gradient w.r.t. the weight."""
    api = tg.Api(g)
    rng = np.random.default_rng(seed)
    w = g.variable(rng.normal(0, 0.05, (nin + hid, 4 * hid)).astype(np.float32), [4 * hid, nin + hid], "w")
    x = g.variable(rng.uniform(-1, 1, (batch, seq, nin)).astype(np.float32), [nin, seq, batch], "x")
    zeros = np.zeros(hid * batch, np.float32)
    state0 = g.constant(zeros, [hid, 1, batch])
    hidden0 = g.constant(zeros, [hid, 1, batch])
    cache = {}

    def gate(k):
        def fn(xc):
            # the four gates of a step share one product with the fused weight
            if xc.id not in cache:
                cache[xc.id] = api.contract(xc, w)
            return api.slice(cache[xc.id], k * hid, hid, 0)
        return fn

    out = api.lstm(x, state0, hidden0, {"g": gate(0), "i": gate(1), "f": gate(2), "o": gate(3)}, seq_dim=1)
    loss = api.reduce_sum(api.square(out))
    (dw,) = g.derive(loss, [w])
    gemm_flops = 3 * seq * 2.0 * batch * (nin + hid) * 4 * hid
    return [loss, dw], x, w, gemm_flops


def config5_cnn(g, seed=5, batch=128, hw=28, c1=32, c2=64, ncls=10):
    """Small CNN forward+gradient: conv 5x5 1->c1 valid, ReLU, conv 5x5 c1->c2
    valid, ReLU, REDUCE_SUM spatial, dense c2->ncls, softmax cross-entropy
    against seeded one-hot labels; gradients w.r.t. both kernels and the dense
    weight (cfg/tenncor/nn.yml:48-98, core.yml:1232-1267, loss.yml:40-59)."""
    api = tg.Api(g)
    rng = np.random.default_rng(seed)
    x = g.variable(rng.uniform(0, 1, (batch, hw, hw, 1)).astype(np.float32), [1, hw, hw, batch], "x")
    k1 = g.variable(rng.normal(0, 0.05, (5, 5, 1, c1)).astype(np.float32), [c1, 1, 5, 5], "k1")
    k2 = g.variable(rng.normal(0, 0.05, (5, 5, c1, c2)).astype(np.float32), [c2, c1, 5, 5], "k2")
    wd = g.variable(rng.normal(0, 0.05, (c2, ncls)).astype(np.float32), [ncls, c2], "wd")
    labels = rng.integers(0, ncls, batch)
    y = g.variable(np.eye(ncls, dtype=np.float32)[labels], [ncls, 1, 1, batch], "y")
    h1 = api.relu(api.conv2d(x, k1))
    h2 = api.relu(api.conv2d(h1, k2))
    pooled = api.reduce_sum(h2, 1, 2)
    logits = api.contract(pooled, wd)
    probs = api.softmax(logits, 0, 1)
    loss = api.reduce_sum(api.cross_entropy(y, probs))
    grads = g.derive(loss, [k1, k2, wd])
    o1, o2 = hw - 4, hw - 8
    useful_flops = 3 * 2.0 * batch * (o1 * o1 * 25 * 1 * c1 + o2 * o2 * 25 * c1 * c2)
    return [loss] + grads, x, [k1, k2, wd], useful_flops
