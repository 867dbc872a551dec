"""Recorded launch sequences (tcg_capture_* / tcg_graph_*) and the evaluator
built on them (eigen::ReplayEvaluator, the replacement for the node-by-node
walk of internal/teq/evaluator.hpp:11-61).

A replay must give what issuing the same calls one by one gives, bit for bit:
the same kernels run with the same arguments ("replay_launches").  The default
kind ("replay") also records the pass of a graph of small tensors as ONE
kernel whose sums run in index order: those are checked at the tolerance of
reductions and contractions.  Every test replays several
times, with ordinary launches and synchronisations of the same context between
the replays, and checks every replay against the eagerly computed result.
"""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
with open(os.path.join(GOLDEN, "equation_vectors.json")) as f:
    EQV = json.load(f)


@pytest.fixture()
def ctx():
    from tenncor_amd import capi
    c = capi.Context(0)
    yield c
    c.close()


def chain(ctx, capi, M, K, N, a, b, bias, work, out_sum, out_max):
    """matmul -> + bias row -> tanh -> reductions; uses pool temporaries inside
    tcg_reduce and tcg_extend targets allocated by the caller."""
    ctx.matmul(capi.FLOAT, [K, M], [N, K], a, b, work[0])
    ctx.extend(capi.FLOAT, [N], [1, M], bias, work[1])
    ctx.ew_binary("ADD", capi.FLOAT, M * N, work[0], work[1], work[2])
    ctx.ew_unary("TANH", capi.FLOAT, M * N, work[2], work[0])
    ctx.reduce("REDUCE_SUM", capi.FLOAT, [N, M], [1], work[0], out_sum)
    ctx.reduce("REDUCE_MAX", capi.FLOAT, [N, M], [0, 1], work[0], out_max)


def test_recorded_sequence_replays_bit_exact(ctx):
    from tenncor_amd import capi
    rng = np.random.default_rng(11)
    M, K, N = 96, 200, 160
    av = rng.uniform(-1, 1, M * K).astype(np.float32)
    bv = rng.uniform(-1, 1, K * N).astype(np.float32)
    cv = rng.uniform(-1, 1, N).astype(np.float32)
    a, b, bias = ctx.upload(av), ctx.upload(bv), ctx.upload(cv)
    # eager pass, ordinary pool memory
    work = [ctx.empty(M * N, np.float32) for _ in range(3)]
    s_eager, m_eager = ctx.empty(N, np.float32), ctx.empty(1, np.float32)
    chain(ctx, capi, M, K, N, a.ptr, b.ptr, bias.ptr, [w.ptr for w in work], s_eager.ptr, m_eager.ptr)
    want_s, want_m = s_eager.get(), m_eager.get()
    in_use_before, _ = ctx.mem_stats()

    # recorded pass: buffers allocated while recording belong to the recording
    ctx.capture_begin()
    rwork = [ctx.alloc(M * N * 4) for _ in range(3)]
    rs, rm = ctx.alloc(N * 4), ctx.alloc(4)
    chain(ctx, capi, M, K, N, a.ptr, b.ptr, bias.ptr, rwork, rs, rm)
    for p in rwork:
        ctx.free(p, M * N * 4)
    with pytest.raises(capi.TcgError):
        ctx.sync()              # refused while recording
    with pytest.raises(capi.TcgError):
        ctx.d2h(rs, N, np.float32)
    graph = ctx.capture_end()
    nodes, nbytes = ctx.graph_stats(graph)
    assert nodes >= 6 and nbytes >= 3 * M * N * 4
    # recording runs nothing
    for rep in range(4):
        ctx.graph_launch(graph)
        np.testing.assert_array_equal(ctx.d2h(rs, N, np.float32), want_s)
        np.testing.assert_array_equal(ctx.d2h(rm, 1, np.float32), want_m)
        # ordinary work and a new input between replays
        av = rng.uniform(-1, 1, M * K).astype(np.float32)
        ctx.h2d(a.ptr, av)
        scratch = ctx.empty(M * N, np.float32)
        ctx.ew_unary("NEG", capi.FLOAT, M * N, work[0].ptr, scratch.ptr)
        chain(ctx, capi, M, K, N, a.ptr, b.ptr, bias.ptr, [w.ptr for w in work], s_eager.ptr, m_eager.ptr)
        ctx.sync()
        want_s, want_m = s_eager.get(), m_eager.get()
        scratch.release()
    # memory of the recording returns to the pool with it, claimed blocks stay
    ctx.graph_claim(graph, rs)
    ctx.graph_destroy(graph)
    ctx.free(rs, N * 4)
    ctx.free(rm, 4)  # given back after its graph is gone: ordinary pool block by now
    in_use_after, _ = ctx.mem_stats()
    assert in_use_after == in_use_before


def test_capture_abort_and_errors(ctx):
    from tenncor_amd import capi
    x = ctx.upload(np.ones(64, np.float32))
    ctx.capture_begin()
    with pytest.raises(capi.TcgError):
        ctx.capture_begin()
    tmp = ctx.alloc(256)
    ctx.ew_unary("NEG", capi.FLOAT, 64, x.ptr, tmp)
    ctx.capture_abort()
    # nothing ran, nothing leaked, the context still works
    y = ctx.empty(64, np.float32)
    ctx.ew_unary("NEG", capi.FLOAT, 64, x.ptr, y.ptr)
    np.testing.assert_array_equal(y.get(), -np.ones(64, np.float32))
    with pytest.raises(capi.TcgError):
        ctx.capture_end()


# ---- the evaluator ---------------------------------------------------------

@pytest.fixture()
def replay_graph():
    from tenncor_amd import graph
    graph.set_evaluator("replay_launches")
    g = graph.Graph()
    try:
        yield g, graph.Api(g), graph
    finally:
        g.close()
        graph.set_evaluator("default")


def mlp(g, api, fx, np_dtype):
    x = g.variable(np.array(fx["in_data"], np_dtype), [10, 3], "in")
    w0 = g.variable(np.array(fx["w0_data"], np_dtype), [9, 10], "w0")
    b0 = g.variable(np.array(fx["b0_data"], np_dtype), [9], "b0")
    w1 = g.variable(np.array(fx["w1_data"], np_dtype), [5, 9], "w1")
    b1 = g.variable(np.array(fx["b1_data"], np_dtype), [5], "b1")
    out = g.variable(np.array(fx["out_data"], np_dtype), [5, 3], "out")
    l0 = api.sigmoid(api.add(api.matmul(x, w0), api.extend(b0, 1, [3])))
    l1 = api.sigmoid(api.add(api.matmul(l0, w1), api.extend(b1, 1, [3])))
    err = api.pow(api.sub(out, l1), 2.0)
    grads = g.derive(err, [w0, b0, w1, b1])
    return x, [w0, b0, w1, b1], err, grads


def test_replayed_mlp_matches_golden_and_plain_walk(replay_graph):
    """tenncor/test/test_equation.cpp:482-706 evaluated five times with new
    inputs: passes 1 walks node by node, pass 2 records, later ones replay."""
    g, api, graph = replay_graph
    fx = EQV["sigmoid_mlp_fast"]
    x, leaves, err, grads = mlp(g, api, fx, np.float64)
    targets = [err] + grads
    rng = np.random.default_rng(3)
    x0 = np.array(fx["in_data"], np.float64)
    inputs = [x0, rng.uniform(-1, 1, 30), rng.uniform(-1, 1, 30), x0, rng.uniform(-1, 1, 30), x0]
    got = []
    for xv in inputs:
        g.assign(x, xv)
        g.evaluate(targets)
        got.append([t.get().copy() for t in targets])
    st = graph.evaluator_stats()
    assert st["plain"] == 1 and st["recorded"] == 1 and st["replayed"] == 5 and st["launches"] > 5
    for key, val in zip(("expect_gw0", "expect_gb0", "expect_gw1", "expect_gb1"), got[0][1:]):
        np.testing.assert_allclose(val, np.array(fx[key]), rtol=1e-12)
    # same inputs, same launches: identical bits whether walked or replayed
    for i in (3, 5):
        for a, b in zip(got[0], got[i]):
            np.testing.assert_array_equal(a, b)
    # nothing moved: nothing to do
    g.evaluate(targets)
    assert graph.evaluator_stats()["skipped"] == 1
    for a, t in zip(got[5], targets):
        np.testing.assert_array_equal(a, t.get())
    # the other inputs against the plain evaluator on a second graph
    graph.set_evaluator("plain")
    g2 = graph.Graph()
    api2 = graph.Api(g2)
    x2, _, err2, grads2 = mlp(g2, api2, fx, np.float64)
    for i in (1, 2, 4):
        g2.assign(x2, inputs[i])
        g2.evaluate([err2] + grads2)
        for a, t in zip(got[i], [err2] + grads2):
            np.testing.assert_array_equal(a, t.get())
    g2.close()


def test_replayed_training_loop_updates_leaves_in_place(replay_graph):
    """sgd (cfg/tenncor/approx.yml:52) through ASSIGN_SUB nodes: the recorded
    step must keep moving the weights, and the host view must follow."""
    g, api, graph = replay_graph
    rng = np.random.default_rng(8)
    wv = rng.uniform(-1, 1, 12).astype(np.float32)
    xs = [rng.uniform(-1, 1, 8).astype(np.float32) for _ in range(6)]
    def build(gr, ap):
        w = gr.variable(wv, [3, 4], "w")
        x = gr.variable(xs[0], [4, 2], "x")
        loss = ap.reduce_sum(ap.square(ap.tanh(ap.matmul(x, w))))
        (dw,) = gr.derive(loss, [w])
        step = gr.functor("ASSIGN_SUB", [w, ap.mul(0.05, dw)])
        return w, x, loss, step
    w, x, loss, step = build(g, api)
    seen = []
    for xv in xs:
        g.assign(x, xv)
        g.evaluate([step])
        seen.append(w.get().copy())
    st = graph.evaluator_stats()
    assert st["replayed"] >= 4
    graph.set_evaluator("default")
    g2 = graph.Graph()
    w2, x2, loss2, step2 = build(g2, graph.Api(g2))
    for i, xv in enumerate(xs):
        g2.assign(x2, xv)
        g2.evaluate([step2])
        np.testing.assert_array_equal(seen[i], w2.get())
    g2.close()
    graph.set_evaluator("replay_launches")
    # a different target set afterwards sees the updated weights
    g.evaluate([loss])
    g2 = None
    ref = np.sum(np.tanh(xs[-1].reshape(2, 4).astype(np.float64) @ seen[-1].reshape(4, 3).astype(np.float64)) ** 2)
    np.testing.assert_allclose(loss.get(), [ref], rtol=1e-5)


def test_replay_mixes_with_other_target_sets_and_aliases(replay_graph):
    """Recorded and walked passes interleaved on one graph: targets that are
    aliases, a padded image read only by a convolution, and a node read by a
    later, different target set."""
    g, api, graph = replay_graph
    rng = np.random.default_rng(21)
    C, W, H, B, O = 2, 6, 5, 2, 3
    xv = rng.integers(1, 9, C * W * H * B).astype(np.float32)
    kv = rng.integers(-4, 5, O * C * 3 * 2).astype(np.float32)
    x = g.variable(xv, [C, W, H, B], "x")
    k = g.variable(kv, [O, C, 3, 2], "k")
    conv = api.conv2d(x, k)
    act = api.relu(conv)
    alias = api.identity(act)
    total = api.reduce_sum(act)
    results = []
    for i in range(5):
        g.assign(x, xv + i)
        g.evaluate([alias, total])
        results.append((alias.get().copy(), total.get().copy()))
        if i == 2:
            # another target set in between, walked node by node
            g.evaluate([conv])
            mid = conv.get().copy()
    assert graph.evaluator_stats()["replayed"] >= 3
    graph.set_evaluator("default")
    g2 = graph.Graph()
    api2 = graph.Api(g2)
    x2 = g2.variable(xv, [C, W, H, B], "x")
    k2 = g2.variable(kv, [O, C, 3, 2], "k")
    conv2 = api2.conv2d(x2, k2)
    act2 = api2.relu(conv2)
    tot2 = api2.reduce_sum(act2)
    for i in range(5):
        g2.assign(x2, xv + i)
        g2.evaluate([act2, tot2, conv2])
        np.testing.assert_array_equal(results[i][0], act2.get())
        np.testing.assert_array_equal(results[i][1], tot2.get())
        if i == 2:
            np.testing.assert_array_equal(mid, conv2.get())
    g2.close()
    graph.set_evaluator("replay_launches")


def test_recordings_are_dropped_when_nodes_go_away():
    from tenncor_amd import graph
    graph.set_evaluator("replay_launches")
    try:
        g = graph.Graph()
        api = graph.Api(g)
        x = g.variable(np.arange(6, dtype=np.float32), [3, 2], "x")
        y = api.exp(api.neg(x))
        for i in range(3):
            g.assign(x, np.arange(6, dtype=np.float32) + i)
            g.evaluate([y])
        assert graph.evaluator_stats()["reserved_bytes"] > 0
        np.testing.assert_allclose(y.get(), np.exp(-(np.arange(6) + 2.0)), rtol=1e-6)
        g.close()
        # a new graph may reuse the node addresses: nothing of the old one may be replayed
        g = graph.Graph()
        api = graph.Api(g)
        x = g.variable(np.arange(6, dtype=np.float32), [3, 2], "x")
        y = api.square(x)
        for i in range(3):
            g.assign(x, np.arange(6, dtype=np.float32) + i)
            g.evaluate([y])
            np.testing.assert_array_equal(y.get(), (np.arange(6, dtype=np.float32) + i) ** 2)
        g.close()
    finally:
        graph.set_evaluator("default")


# ---- shared launches ---------------------------------------------------------

def run_both(build, feeds, kinds=("plain", "replay_launches", "replay_unfused")):
    """Evaluate the same graph under each evaluator over the same sequence of
    inputs; returns {kind: [[target values per pass]]} and the stats of each."""
    from tenncor_amd import graph
    results, stats = {}, {}
    for kind in kinds:
        graph.set_evaluator(kind)
        g = graph.Graph()
        try:
            targets, x = build(g, graph.Api(g))
            rows = []
            for feed in feeds:
                g.assign(x, feed)
                g.evaluate(targets)
                rows.append([t.get().copy() for t in targets])
            results[kind] = rows
            stats[kind] = graph.evaluator_stats()
        finally:
            g.close()
            graph.set_evaluator("default")
    return results, stats


def assert_same_bits(results):
    base = results["plain"]
    for kind, rows in results.items():
        for i, (row, ref) in enumerate(zip(rows, base)):
            for j, (a, b) in enumerate(zip(row, ref)):
                np.testing.assert_array_equal(a, b, err_msg="%s pass %d target %d" % (kind, i, j))


def test_fused_lstm_matches_the_walk_bit_for_bit():
    """configs[3] at reduced size (cfg/tenncor/layer.yml:716-768 unrolled, fused
    gate weight cut by SLICEs, loss and weight gradient): the recording with
    shared launches must reproduce the node-by-node results exactly, with far
    fewer launches than functors."""
    from tenncor_amd import configs
    rng = np.random.default_rng(17)
    seq, batch, nin, hid = 5, 6, 8, 12
    feeds = [rng.uniform(-1, 1, batch * seq * nin).astype(np.float32) for _ in range(4)]
    counts = {}

    def build(g, api):
        targets, x, w, _ = configs.config4_lstm(g, seq=seq, batch=batch, nin=nin, hid=hid)
        counts["functors"] = g.count_functors(targets)
        return targets, x

    results, stats = run_both(build, feeds)
    assert_same_bits(results)
    assert stats["replay_launches"]["replayed"] == 3 and stats["replay_unfused"]["replayed"] == 3
    assert stats["replay_launches"]["launches"] < 0.5 * stats["replay_unfused"]["launches"]


def assert_close_to_walk(results, tol=1e-5):
    base = results["plain"]
    for kind, rows in results.items():
        for i, (row, ref) in enumerate(zip(rows, base)):
            for j, (a, b) in enumerate(zip(row, ref)):
                assert np.isfinite(b).all()
                assert np.abs(a - b).max() <= tol * np.abs(b).max(), "%s pass %d target %d" % (kind, i, j)


def test_products_over_the_parts_of_concatenations_follow_the_walk():
    """configs[3] at sizes where the recording never lays out [x_t, h] or the
    joined gate gradients (cfg/tenncor/layer.yml:716-768,
    tenncor/eteq/backprop.hpp:269-359): the step's product runs as a sum of
    products over the parts, the product on the way back over the four gate
    gradients and only for the columns of h, the weight gradient block by block.
    The sums over K then come in another order than in the walk: 1e-5 of the
    largest entry, the bar of a contraction.  The second case has part extents
    with a small common divisor (12 and 20: chunks of 4), which the matrix
    cores do not take, so that the concatenations are laid out as before and
    the results of the recording without single-kernel runs are the walk's bit
    for bit (with them, the small steps of such a graph sum in another order)."""
    from tenncor_amd import configs, graph
    rng = np.random.default_rng(41)
    for (seq, batch, nin, hid), exact in (((6, 64, 32, 64), False), ((5, 48, 12, 20), True)):
        feeds = [rng.uniform(-1, 1, batch * seq * nin).astype(np.float32) for _ in range(3)]

        def build(g, api):
            targets, x, w, _ = configs.config4_lstm(g, seq=seq, batch=batch, nin=nin, hid=hid)
            lines = g.launch_plan(targets)
            assert any(l.startswith("parts") for l in lines) != exact, lines
            return targets, x

        results, stats = run_both(build, feeds, kinds=("plain", "replay_launches", "replay"))
        assert_close_to_walk(results)
        if exact:
            assert_same_bits({kind: results[kind] for kind in ("plain", "replay_launches")})
        assert stats["replay"]["replayed"] == 2 and stats["replay"]["record_failures"] == 0


def test_products_over_parts_read_each_part_where_the_walk_does():
    """Two products over one concatenation with an assignment to one of its
    parts between them in the walk's order: the concatenation holds the part's
    old value (internal/eigen/device.hpp:508-544 rewrites the variable's
    buffer only), so it is laid out and both products read that; a second
    concatenation, built over the assignment, is read part by part and sees the
    new value.  A concatenation that nothing rewrites is never laid out."""
    rng = np.random.default_rng(43)
    xs = [rng.uniform(-1, 1, 32 * 64).astype(np.float32) for _ in range(3)]
    hv, cv = rng.uniform(-1, 1, 48 * 64).astype(np.float32), rng.uniform(-1, 1, 32 * 64).astype(np.float32)
    w1v, w2v = (rng.uniform(-1, 1, 96 * 80).astype(np.float32) for _ in range(2))

    def build(g, api):
        x = g.variable(xs[0], [32, 64], "x")
        h = g.variable(hv, [48, 64], "h")
        c = g.variable(cv, [32, 64], "c")
        w1, w2 = g.variable(w1v, [96, 80], "w1"), g.variable(w2v, [96, 80], "w2")
        z = api.concat([x, h], 0)
        clean = api.add(api.matmul(api.concat([h, c], 0), w1), api.matmul(api.concat([h, c], 0), w2))
        upd = api.assign(x, c)
        q1, q2 = api.matmul(z, w1), api.matmul(z, w2)
        late = api.matmul(api.concat([upd, h], 0), w1)
        targets = [api.add(api.add(q1, late), q2), clean]
        lines = g.launch_plan(targets)
        assert sum(l.startswith("parts CONCAT+MATMUL") for l in lines) == 3, lines
        assert sum(l.startswith(("group CONCAT", "node CONCAT")) for l in lines) == 1, lines
        return targets, x

    results, stats = run_both(build, xs, kinds=("plain", "replay_launches", "replay"))
    assert_close_to_walk(results)
    # the first target depends on x's fed value through the laid-out concatenation only
    want = np.concatenate([xs[1].reshape(64, 32), hv.reshape(64, 48)], axis=1).astype(np.float64)
    new = np.concatenate([cv.reshape(64, 32), hv.reshape(64, 48)], axis=1).astype(np.float64)
    w1m, w2m = w1v.reshape(80, 96).astype(np.float64), w2v.reshape(80, 96).astype(np.float64)
    ref = want @ w1m + new @ w1m + want @ w2m
    got = results["replay"][1][0].reshape(64, 96)
    assert np.abs(got - ref).max() <= 1e-5 * np.abs(ref).max()


def test_groups_add_the_k_ranges_of_a_product_they_read():
    """A product with a transposed operand, few results and a long K runs as K
    ranges on separate workgroups.  Where elementwise groups reading through
    SLICEs are all that reads it, the recording never lays the result out: the
    ranges stay side by side (tcg_gemm_terms_ranges) and the groups add them up
    in range order while they load.  Against the walk (1e-5 of the largest
    entry) and against numpy in double (1e-4); the second reader goes through a
    PAD of a narrower SLICE, so its leaf starts off the window's first row."""
    rng = np.random.default_rng(47)
    g0s = [rng.uniform(-1, 1, 128 * 64).astype(np.float32) for _ in range(3)]
    g1v, sv = rng.uniform(-1, 1, 128 * 64).astype(np.float32), rng.uniform(-1, 1, 128 * 64).astype(np.float32)
    wv = rng.uniform(-1, 1, 256 * 192).astype(np.float32)

    def build(g, api):
        g0, g1 = g.variable(g0s[0], [128, 64], "g0"), g.variable(g1v, [128, 64], "g1")
        wt = g.variable(wv, [256, 192], "wt")
        scale = g.variable(sv, [128, 64], "scale")
        back = api.contract(api.concat([g0, g1], 0), wt, ((0, 0),))
        first = api.mul(api.slice(back, 64, 128, 0), scale)
        second = api.add(api.pad(api.slice(api.slice(back, 96, 64, 0), 8, 40, 1), [[32, 32], [8, 16]]), scale)
        lines = g.launch_plan([first, second])
        assert lines[0].startswith("parts CONCAT+CONTRACT x2+SLICE ranges="), lines
        return [first, second], g0

    results, stats = run_both(build, g0s, kinds=("plain", "replay_launches", "replay"))
    assert_close_to_walk(results)
    cat = np.concatenate([g0s[2].reshape(64, 128), g1v.reshape(64, 128)], axis=1).astype(np.float64)
    full = cat @ wv.reshape(192, 256).astype(np.float64).T        # [64, 192]
    want = full[:, 64:192] * sv.reshape(64, 128)
    got = results["replay"][2][0].reshape(64, 128)
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()
    padded = np.zeros((64, 128))
    padded[8:48, 32:96] = full[8:48, 96:160]
    want2 = padded + sv.reshape(64, 128)
    got2 = results["replay"][2][1].reshape(64, 128)
    assert np.abs(got2 - want2).max() <= 1e-4 * np.abs(want2).max()


def random_products_graph(g, api, seed, x0, with_updates=False):
    """Matrix products over concatenations, gate-like SLICEs of their results
    and gradients of it all, at sizes where the planner rewrites what it can
    (products over parts, windows, K ranges left to the groups, sums of
    products): returns (targets, fed variable, plan lines).  `with_updates`
    adds assignments to operands in between; everything then hangs under ONE
    root, a sum whose terms come in a seeded order, because the order in which
    an evaluator visits several targets is its own business
    (internal/teq/evaluator.hpp:33-45 walks a set) and with it which side of an
    assignment a read in another target falls on."""
    rng = np.random.default_rng(seed)
    batch = 64
    widths = [32, 48, 64, 96, 128]

    def variable(width, name, scale=1.0, rows=batch):
        data = rng.uniform(-scale, scale, width * rows).astype(np.float32)
        return g.variable(data, [width, rows], name)

    x = g.variable(x0, [64, batch], "x")
    pool = [x] + [variable(int(rng.choice(widths)), "v%d" % k) for k in range(3)]
    variables = list(pool)
    weights = []
    results = []
    updates = []
    for step in range(int(rng.integers(3, 6))):
        a, b = (pool[int(i)] for i in rng.choice(len(pool), 2, replace=False))
        z = api.concat([a, b], 0)
        k = z.shape[0]
        n = int(rng.choice([64, 128, 192, 256]))
        kind = int(rng.integers(0, 3))
        if kind == 0:
            w = variable(n, "w%d" % step, 0.2, rows=k)           # [n, k]
            p = api.matmul(z, w)
        elif kind == 1:
            w = variable(k, "w%d" % step, 0.2, rows=n)           # [k, n]: K along the memory of both
            p = api.contract(z, w, ((0, 0),))
        else:
            w = variable(n, "w%d" % step, 0.2, rows=k)
            p = api.contract(z, w, ((0, 1),))
        weights.append(w)
        # gates: halves of the result through SLICEs, recombined elementwise
        half = n // 2
        lo, hi = api.slice(p, 0, half, 0), api.slice(p, half, half, 0)
        h = api.mul(api.sigmoid(lo), api.tanh(hi))                # [half, batch]
        if rng.uniform() < 0.4:
            h = api.add(h, api.pad(api.slice(hi, 8, half - 24, 0), [[8, 16]]))
        results.append(h)
        pool.append(h)
        if with_updates and rng.uniform() < 0.5 and variables:
            # (each variable at most once: two assignments to one variable keep a pass on the walk)
            target = variables.pop(int(rng.integers(0, len(variables))))
            source = next((t for t in reversed(pool) if t.shape == target.shape and t is not target), None)
            if source is not None:
                updates.append(api.reduce_sum(api.assign(target, api.tanh(source))))
    loss = api.reduce_sum(api.square(results[0]))
    for r in results[1:]:
        loss = api.add(loss, api.reduce_sum(api.square(r)))
    grads = g.derive(loss, weights[:2] + [x])
    targets = [loss] + grads
    if with_updates:
        # (ASSIGN has no derivative: the updates stand beside the loss)
        terms = [loss] + [api.reduce_sum(api.square(gr)) for gr in grads] + updates
        order = rng.permutation(len(terms))
        root = terms[int(order[0])]
        for i in order[1:]:
            root = api.add(root, terms[int(i)])
        targets = [root]
    return targets, x, g.launch_plan(targets)


@pytest.mark.parametrize("with_updates", [False, True], ids=["pure", "updates"])
@pytest.mark.parametrize("seed", range(10))
def test_random_graphs_of_products_over_parts_follow_the_walk(seed, with_updates):
    """Seeded random graphs of the shapes the planner rewrites (products over
    CONCATs, SLICEd gates, their gradients: ADDs of PADs, sums of products,
    transposed weights; with assignments to operands in between in the second
    variant), three passes with new inputs each: the recording and its replays
    against the node-by-node walk at 1e-4 of each target's largest entry (sums
    over K come in another order where a rewrite applies; a read on the wrong
    side of an update, or of a value its own launch is still to write, is an
    error of order one)."""
    rng = np.random.default_rng(1000 + seed)
    feeds = [rng.uniform(-1, 1, 64 * 64).astype(np.float32) for _ in range(3)]
    seen = {}

    def build(g, api):
        targets, x, lines = random_products_graph(g, api, seed, feeds[0], with_updates)
        seen["lines"] = lines
        return targets, x

    results, stats = run_both(build, feeds, kinds=("plain", "replay_launches", "replay"))
    assert stats["replay"]["record_failures"] == 0 and stats["replay"]["replayed"] >= 1, stats
    assert_close_to_walk(results, tol=1e-4)


def test_random_graphs_exercise_the_rewrites():
    """The generator above reaches every rewrite at least once over its seeds
    (host logic only: the plans)."""
    from tenncor_amd import graph
    kinds = set()
    for seed in range(10):
        g = graph.Graph()
        try:
            _, _, lines = random_products_graph(g, graph.Api(g), seed, np.zeros(64 * 64, np.float32))
        finally:
            g.close()
        for line in lines:
            kinds.add(line.split(" ")[0])
            if " ranges=" in line:
                kinds.add("ranges")
            if line.startswith("parts") and "+SLICE" in line:
                kinds.add("window")
    assert {"parts", "ranges", "window", "group"} <= kinds, kinds


def test_a_view_of_a_group_result_is_read_after_the_group_has_stored_it():
    """h is computed by an elementwise group; y adds h and PAD(SLICE(h)) -- the
    shape the gradient of a SLICE added back onto its operand takes.  The view
    is read from memory, so y's launch must come after the one that stores h;
    in one launch it would read what the buffer held before."""
    rng = np.random.default_rng(53)
    feeds = [rng.uniform(-1, 1, 64 * 16).astype(np.float32) for _ in range(3)]
    bv = rng.uniform(-1, 1, 64 * 16).astype(np.float32)

    def build(g, api):
        a, b = g.variable(feeds[0], [64, 16], "a"), g.variable(bv, [64, 16], "b")
        h = api.mul(api.sigmoid(a), api.tanh(b))
        y = api.add(h, api.pad(api.slice(h, 8, 40, 0), [[8, 16]]))
        return [api.square(y), api.neg(h)], a

    results, _ = run_both(build, feeds, kinds=("plain", "replay_launches", "replay"))
    assert_same_bits(results)
    h = (1 / (1 + np.exp(-feeds[2].astype(np.float64)))) * np.tanh(bv.astype(np.float64))
    h = h.reshape(16, 64)
    y = h.copy()
    y[:, 8:48] += h[:, 8:48]
    assert np.abs(results["replay"][2][0].reshape(16, 64) - y * y).max() <= 1e-5


def test_a_recording_with_a_plain_assign_runs_at_every_pass():
    """ASSIGN leaves its target newer than itself (internal/eigen/device.hpp:508-544
    bumps the target's version; tenncor/eteq/functor.hpp:246-268 compares the
    operands' versions with the node's), so the walk runs it, and everything
    that reads the target, at every pass -- also when no input was fed in
    between.  A state that feeds back on itself then moves with every
    evaluation; the recording must do the same and not take the pass for
    unchanged."""
    from tenncor_amd import graph
    rng = np.random.default_rng(59)
    s0 = rng.uniform(-1, 1, 32 * 8).astype(np.float32)
    wv = rng.uniform(-0.5, 0.5, 32 * 32).astype(np.float32)
    seen = {}
    for kind in ("plain", "replay_launches", "replay"):
        graph.set_evaluator(kind)
        g = graph.Graph()
        try:
            api = graph.Api(g)
            state = g.variable(s0, [32, 8], "state")
            w = g.variable(wv, [32, 32], "w")
            nxt = api.tanh(api.matmul(state, w))
            root = api.reduce_sum(api.square(api.assign(state, nxt)))
            rows = []
            for _ in range(5):
                g.evaluate([root])
                rows.append(float(root.get()[0]))
            seen[kind] = rows
            if kind != "plain":
                st = graph.evaluator_stats()
                assert st["replayed"] >= 3 and st["skipped"] == 0, st
        finally:
            g.close()
            graph.set_evaluator("default")
    assert len(set(seen["plain"])) == 5          # the state moves
    x = s0.reshape(8, 32).astype(np.float64)
    for k in range(5):
        x = np.tanh(x @ wv.reshape(32, 32).astype(np.float64))
        assert abs(seen["plain"][k] - (x * x).sum()) <= 1e-4 * (x * x).sum()
    for kind in ("replay_launches", "replay"):
        assert np.allclose(seen[kind], seen["plain"], rtol=1e-5, atol=0), (kind, seen)


def random_elementwise_graph(g, api, seed, x0, shape, np_dtype, with_updates):
    """Elementwise nodes over views of each other (EXTEND of reduced rows,
    SLICE + PAD back to shape, transposes, CONCATs of halves, SELECT, IDENTITY)
    and, with `with_updates`, assignments to the variables in between, all
    under one root."""
    rng = np.random.default_rng(seed)
    a, b = shape
    integer = np.issubdtype(np_dtype, np.integer)

    def draw(n):
        if integer:
            return rng.integers(-9, 10, n).astype(np_dtype)
        return rng.uniform(-1, 1, n).astype(np_dtype)

    x = g.variable(x0, [a, b], "x")
    variables = [x] + [g.variable(draw(a * b), [a, b], "v%d" % k) for k in range(2)]
    row = g.variable(draw(a), [a], "row")
    pool = list(variables)
    unassigned = list(variables)
    unary = ["NEG", "SQUARE", "ABS"] + ([] if integer else ["TANH", "SIGMOID"])
    binary = ["ADD", "SUB", "MUL", "MIN", "MAX"]
    updates = []
    for step in range(int(rng.integers(8, 16))):
        kind = int(rng.integers(0, 11))
        p = pool[int(rng.integers(0, len(pool)))]
        q = pool[int(rng.integers(0, len(pool)))]
        if kind == 0:
            node = api.unary(str(rng.choice(unary)), p)
        elif kind == 1:
            node = api.binary(str(rng.choice(binary)), p, q)
        elif kind == 2:
            node = api.binary(str(rng.choice(binary)), p, api.extend(row, 1, [b]))
        elif kind == 3:
            lo = int(rng.integers(0, a // 2))
            ext = int(rng.integers(1, a - lo))
            node = api.add(q, api.pad(api.slice(p, lo, ext, 0), [[lo, a - lo - ext]]))
        elif kind == 4:
            node = api.sub(api.permute(api.mul(api.permute(p, [1, 0]), api.permute(q, [1, 0])), [1, 0]), p)
        elif kind == 5:
            summed = api.reduce_sum(p, 1, 1) if integer else api.tanh(api.reduce_sum(p, 1, 1))
            node = api.binary("ADD" if integer else "MUL", q, api.extend(summed, 1, [b]))
        elif kind == 6:
            half = a // 2
            node = api.concat([api.slice(p, half, a - half, 0), api.slice(q, 0, half, 0)], 0)
        elif kind == 7:
            node = api.if_then_else(api.binary("LT", p, q), api.identity(p), api.neg(q))
        elif kind == 8:
            node = api.binary("MAX", api.reverse(p, [0]), q)
        elif kind == 9:
            # a product of two nodes, its rows summed and spread back over the shape
            prod = api.matmul(p, api.permute(q, [1, 0]))                       # [b, b]
            if not integer:
                prod = api.tanh(prod)
            node = api.binary("ADD", p, api.extend(api.reduce_sum(prod, 0, 1), 0, [a]))
        else:
            node = api.binary("SUB", q, api.extend(api.reduce("REDUCE_MAX", api.contract(p, q, ((1, 1),)), 1, 1), 1, [b]))
        if not integer:
            node = api.tanh(node)    # keeps every value in (-1, 1)
        pool.append(node)
        if with_updates and rng.uniform() < 0.3 and unassigned:
            # (each variable at most once: two assignments to one variable keep a pass on the walk)
            target = unassigned.pop(int(rng.integers(0, len(unassigned))))
            updates.append(api.reduce_sum(api.assign(target, node)))
    terms = [api.reduce_sum(api.square(t)) for t in pool[len(variables):]] + updates
    order = rng.permutation(len(terms))
    root = terms[int(order[0])]
    for i in order[1:]:
        root = api.add(root, terms[int(i)])
    targets = [root] if with_updates else [root, pool[-1], pool[len(pool) // 2]]
    return targets, x


@pytest.mark.parametrize("with_updates", [False, True], ids=["pure", "updates"])
@pytest.mark.parametrize("np_dtype", [np.float32, np.int32], ids=["f32", "i32"])
@pytest.mark.parametrize("shape", [(12, 10), (96, 80)], ids=["one_kernel", "launches"])
@pytest.mark.parametrize("seed", range(6))
def test_random_elementwise_graphs_follow_the_walk(seed, shape, np_dtype, with_updates):
    """Seeded random graphs of elementwise nodes reading each other through
    views, at a size whose pass is recorded as the steps of one kernel and at
    one recorded launch by launch: int32 must equal the walk bit for bit
    (wrapping arithmetic does not depend on the order of a sum), fp32 launch by
    launch too (same scalar routines, same order), fp32 as one kernel within
    1e-5 of the largest entry (its reductions run in index order)."""
    rng = np.random.default_rng(2000 + seed)
    n = shape[0] * shape[1]
    if np_dtype == np.int32:
        feeds = [rng.integers(-9, 10, n).astype(np.int32) for _ in range(3)]
    else:
        feeds = [rng.uniform(-1, 1, n).astype(np.float32) for _ in range(3)]

    def build(g, api):
        return random_elementwise_graph(g, api, seed, feeds[0], shape, np_dtype, with_updates)

    results, stats = run_both(build, feeds, kinds=("plain", "replay_launches", "replay"))
    assert stats["replay"]["record_failures"] == 0 and stats["replay"]["replayed"] >= 1, stats
    if np_dtype == np.int32:
        assert_same_bits(results)
    else:
        assert_same_bits({k: v for k, v in results.items() if k != "replay"})
        assert_close_to_walk(results, tol=1e-5)


def test_two_assignments_to_one_variable_stay_with_the_walk():
    """Which of two ASSIGNs to one variable the walk runs at a later pass
    depends on the versions they left behind (tenncor/eteq/functor.hpp:246-268,
    eteq/variable.hpp:129-132): with nothing fed, the first runs again and the
    second, no older than the variable, does not, so the variable ends the
    pass with the first one's value.  A recording would run both; such passes
    are never recorded, and every evaluator gives what the walk gives."""
    from tenncor_amd import graph
    rng = np.random.default_rng(61)
    v0, cv, dv = (rng.uniform(-1, 1, 24).astype(np.float32) for _ in range(3))
    seen = {}
    for kind in ("plain", "replay_launches", "replay"):
        graph.set_evaluator(kind)
        g = graph.Graph()
        try:
            api = graph.Api(g)
            v = g.variable(v0, [6, 4], "v")
            c, d = g.variable(cv, [6, 4], "c"), g.variable(dv, [6, 4], "d")
            first = api.reduce_sum(api.assign(v, api.tanh(c)))
            second = api.reduce_sum(api.assign(v, api.neg(d)))
            root = api.add(api.add(first, second), api.reduce_sum(api.abs(v)) if hasattr(api, "abs") else api.reduce_sum(api.unary("ABS", v)))
            rows = []
            for _ in range(4):
                g.evaluate([root])
                rows.append((float(root.get()[0]), v.get().copy()))
            seen[kind] = rows
            if kind != "plain":
                st = graph.evaluator_stats()
                assert st["recorded"] == 0 and st["plain"] == 4, st
        finally:
            g.close()
            graph.set_evaluator("default")
    for kind in ("replay_launches", "replay"):
        for (a, va), (b, vb) in zip(seen[kind], seen["plain"]):
            assert a == b
            np.testing.assert_array_equal(va, vb)


def random_conv_graph(g, api, seed, x0, dims, np_dtype):
    """One or two conv2d layers (cfg/tenncor/nn.yml:48-98) with seeded channel
    counts, kernel extents and zero padding, a nonlinearity between them, the
    gradients with respect to image and kernels
    (tenncor/eteq/backprop.hpp:372-439), and an elementwise reader of the first
    layer's output beside the second layer: the PAD / PERMUTE / REVERSE nodes
    round every CONV are folded into its launch where convolutions are all
    that reads them and laid out where something else does."""
    rng = np.random.default_rng(seed)
    c, w, h, b = dims
    integer = np.issubdtype(np_dtype, np.integer)

    def draw(n, scale):
        if integer:
            return rng.integers(-3, 4, n).astype(np_dtype)
        return rng.uniform(-scale, scale, n).astype(np_dtype)

    x = g.variable(x0, [c, w, h, b], "x")
    o1 = int(rng.choice([4, 8, 12, 16]))
    k1w, k1h = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    k1 = g.variable(draw(o1 * c * k1w * k1h, 0.3), [o1, c, k1w, k1h], "k1")
    pad = ((int(rng.integers(0, 2)), int(rng.integers(0, 2))), (int(rng.integers(0, 2)), int(rng.integers(0, 2))))
    y1 = api.conv2d(x, k1, zero_padding=pad)
    act = api.relu(y1) if integer or rng.uniform() < 0.5 else api.tanh(y1)
    kernels = [k1]
    terms = [api.reduce_sum(api.square(act))]
    if rng.uniform() < 0.7:
        o2 = int(rng.choice([4, 8, 16]))
        k2w = int(rng.integers(1, min(3, act.shape[1]) + 1))
        k2h = int(rng.integers(1, min(3, act.shape[2]) + 1))
        k2 = g.variable(draw(o2 * o1 * k2w * k2h, 0.3), [o2, o1, k2w, k2h], "k2")
        y2 = api.conv2d(act, k2)
        kernels.append(k2)
        terms.append(api.reduce_sum(api.square(y2)))
    loss = terms[0]
    for t in terms[1:]:
        loss = api.add(loss, t)
    grads = g.derive(loss, [x] + kernels)
    return [loss] + grads, x


@pytest.mark.parametrize("np_dtype", [np.float32, np.int32], ids=["f32", "i32"])
@pytest.mark.parametrize("dims", [(4, 9, 8, 6), (8, 14, 12, 32)], ids=["direct", "products"])
@pytest.mark.parametrize("seed", range(6))
def test_random_conv_graphs_follow_the_walk(seed, dims, np_dtype):
    """Seeded convolution layers with their gradients, at a size the direct
    kernels take and at one where the correlations run as matrix products:
    int32 equals the walk bit for bit by every route (wrapping sums do not
    depend on their order), fp32 within 1e-5 of each target's largest entry
    (a convolution that reads an operand through a PERMUTE sums along the
    operand's memory: another order of the same additions)."""
    rng = np.random.default_rng(3000 + seed)
    n = dims[0] * dims[1] * dims[2] * dims[3]
    if np_dtype == np.int32:
        feeds = [rng.integers(-4, 5, n).astype(np.int32) for _ in range(3)]
    else:
        feeds = [rng.uniform(-1, 1, n).astype(np.float32) for _ in range(3)]

    def build(g, api):
        return random_conv_graph(g, api, seed, feeds[0], dims, np_dtype)

    results, stats = run_both(build, feeds, kinds=("plain", "replay_launches", "replay"))
    assert stats["replay"]["record_failures"] == 0 and stats["replay"]["replayed"] >= 1, stats
    if np_dtype == np.int32:
        assert_same_bits(results)
    else:
        assert_close_to_walk(results, tol=1e-5)


def test_fused_cnn_and_mlp_match_the_walk_bit_for_bit():
    from tenncor_amd import configs
    rng = np.random.default_rng(18)
    feeds = [rng.uniform(0, 1, 4 * 12 * 12).astype(np.float32) for _ in range(3)]

    def cnn(g, api):
        targets, x, _, _ = configs.config5_cnn(g, batch=4, hw=12, c1=4, c2=8, ncls=5)
        return targets, x

    results, stats = run_both(cnn, feeds)
    assert_same_bits(results)
    assert stats["replay_launches"]["launches"] < stats["replay_unfused"]["launches"]

    def mlp_cfg(g, api):
        targets, x, _ = configs.config1_mlp(g)
        return targets, x

    feeds = [rng.uniform(-1, 1, 30).astype(np.float32) for _ in range(4)]
    results, stats = run_both(mlp_cfg, feeds)
    assert_same_bits(results)
    assert stats["replay_launches"]["launches"] < stats["replay_unfused"]["launches"]


@pytest.mark.parametrize("np_dtype", [np.int32, np.float32])
def test_convolutions_over_views_follow_the_walk(np_dtype):
    """A conv2d layer with its two gradients at a size where the correlations
    run as matrix products (cfg/tenncor/nn.yml:88-93,
    tenncor/eteq/backprop.hpp:372-439), followed by an in-place update of the
    kernel.  The recording reads the operands through the PAD / PERMUTE /
    REVERSE nodes in front of each CONV and writes where the PERMUTE / REVERSE
    behind it would: in int32 every result equals the walk's bit for bit
    (wrapping sums do not depend on their order), in fp32 within 1e-5 of the
    largest entry; the kernel update must see the gradient of the old kernel."""
    rng = np.random.default_rng(31)
    C, W, H, B, O, K = 8, 14, 12, 32, 16, 3
    if np_dtype == np.int32:
        feeds = [rng.integers(-9, 10, C * W * H * B).astype(np.int32) for _ in range(4)]
        k0 = rng.integers(-5, 6, O * C * K * K).astype(np.int32)
    else:
        feeds = [rng.uniform(-1, 1, C * W * H * B).astype(np.float32) for _ in range(4)]
        k0 = rng.uniform(-0.3, 0.3, O * C * K * K).astype(np.float32)

    def build(g, api):
        x = g.variable(feeds[0], [C, W, H, B], "x")
        k = g.variable(k0, [O, C, K, K], "k")
        y = api.conv2d(x, k)
        loss = api.reduce_sum(api.square(y))
        dx, dk = g.derive(loss, [x, k])
        step = api.assign_sub(k, dk)  # the next pass convolves with the updated kernel
        return [loss, dx, dk, step], x

    results, stats = run_both(build, feeds, kinds=("plain", "replay_launches", "replay"))
    for kind in ("replay_launches", "replay"):
        assert stats[kind]["recorded"] == 1 and stats[kind]["replayed"] == len(feeds) - 1  # the recording pass launches it too
        for row, ref in zip(results[kind], results["plain"]):
            for got, want in zip(row, ref):
                if np_dtype == np.int32:
                    np.testing.assert_array_equal(got, want, err_msg=kind)
                else:
                    assert np.abs(got.astype(np.float64) - want).max() <= 1e-5 * max(np.abs(want).max(), 1e-30), kind
    from tenncor_amd import graph
    g = graph.Graph()
    try:
        targets, _ = build(g, graph.Api(g))
        lines = g.launch_plan(targets)
        # (a REVERSE of the kernel that a convolution behind the update still reads keeps its own launch)
        assert sum(1 for l in lines if l.startswith("viewed ")) == 3 and "node CONV" not in lines and "node PAD" not in lines
    finally:
        g.close()


@pytest.mark.parametrize("np_dtype", [np.float32, np.int32, np.float64])
def test_fused_views_diamonds_and_wide_groups(np_dtype):
    """Shapes the grouping has to get right: operands seen through SLICE, PAD,
    EXTEND and PERMUTE chains; a node read both inside its group and by a
    matmul outside it; a group fed by the result of a launch that itself reads
    the group's earlier output (must not be merged into one launch); n-ary
    sums with scalar constants; more live values and outputs than one launch
    holds."""
    rng = np.random.default_rng(seed=29)
    draw = (lambda n: rng.integers(-6, 7, n).astype(np.int32)) if np_dtype == np.int32 else \
        (lambda n: rng.uniform(-1, 1, n).astype(np_dtype))
    feeds = [draw(6 * 4) for _ in range(4)]
    consts = {"w": draw(6 * 6), "b": draw(6), "p": draw(4 * 4), "q": draw(4 * 6)}

    def build(g, api):
        x = g.variable(feeds[0], [6, 4], "x")
        w = g.variable(consts["w"], [6, 6], "w")
        b = g.variable(consts["b"], [6], "b")
        p = g.variable(consts["p"], [4, 4], "p")
        q = g.variable(consts["q"], [4, 6], "q")
        s = api.add(x, api.extend(b, 1, [4]))                  # reads b through EXTEND
        t = api.mul(api.square(s), api.neg(s))                 # s read by two nodes of its group
        m = api.matmul(t, w)                                   # t also read by a launch outside
        u = api.sub(api.add(t, m), api.mul(s, 2))              # must come after the matmul
        lo = api.slice(u, 1, 4, 0)                             # [4, 4] views of u
        padded = api.pad(api.mul(lo, p), [[1, 1]])             # back to [6, 4] with a zero border
        perm = api.permute(q, [1, 0])                          # [6, 4] seen through a transpose
        wide = g.functor("ADD", [u, padded, perm, api.extend(b, 1, [4]), api.mul(x, 3), s])
        outs = [api.mul(wide, k + 2) for k in range(6)]        # more outputs than one launch stores
        deep = x
        regs = []
        for k in range(20):                                    # more live values than registers
            deep = api.add(api.mul(deep, x), k + 1)
            regs.append(deep)
        tall = g.functor("ADD", regs)
        neg = api.neg(api.unary("ABS", tall))
        return [u, wide, tall, neg, padded] + outs, x

    results, stats = run_both(build, feeds, kinds=("plain", "replay_launches"))
    assert_same_bits(results)
    assert stats["replay_launches"]["replayed"] == 3


def test_reads_of_a_variable_stay_on_their_side_of_an_assignment():
    """ASSIGN* rewrites its target in place: a node that reads the variable before
    the assignment in the walk's order sees the old value, one after it the new
    value (internal/eigen/device.hpp:508-544).  The shared launches must keep
    that, whichever elementwise nodes they merge."""
    rng = np.random.default_rng(seed=31)
    feeds = [rng.uniform(-1, 1, 24).astype(np.float32) for _ in range(4)]
    v0 = rng.uniform(-1, 1, 24).astype(np.float32)
    w0 = rng.uniform(-1, 1, 6).astype(np.float32)

    def build(g, api):
        c = g.variable(feeds[0], [6, 4], "c")
        v = g.variable(v0, [6, 4], "v")
        w = g.variable(w0, [6], "w")
        x = api.neg(v)                                      # old v
        a = api.assign(v, c)
        y = api.mul(x, v)                                   # new v
        t = api.add(api.add(x, a), y)
        wide = api.extend(w, 1, [4])                        # old w, laid out before the update
        upd = api.assign_add(w, api.reduce_sum(api.mul(api.neg(wide), c), 1, 1))
        late = api.add(api.extend(upd, 1, [4]), api.mul(wide, c))  # wide: read after the update too
        mid = api.square(api.identity(a))
        second = api.assign_sub(v, mid)
        tail = api.add(api.neg(second), mid)
        # one target, so that the order of the walk is the order written here
        # (several targets are walked in the order of an unordered set)
        return [g.functor("ADD", [t, late, tail])], c

    results, stats = run_both(build, feeds, kinds=("plain", "replay_launches", "replay"))
    for kind in ("replay_launches", "replay"):
        for i, (row, ref) in enumerate(zip(results[kind], results["plain"])):
            if kind == "replay":
                np.testing.assert_allclose(row[0], ref[0], rtol=1e-5, atol=1e-6, err_msg="%s pass %d" % (kind, i))
            else:
                np.testing.assert_array_equal(row[0], ref[0], err_msg="%s pass %d" % (kind, i))
    assert stats["replay_launches"]["replayed"] == 3
    # and the walk itself computes what the order of the nodes says
    c0, vold, wold = feeds[0].reshape(4, 6).astype(np.float64), v0.reshape(4, 6).astype(np.float64), w0.astype(np.float64)
    t = -vold + c0 + (-vold) * c0
    wnew = wold + (-wold[None, :] * c0).sum(axis=0)
    late = wnew[None, :] + wold[None, :] * c0
    tail = -(c0 - c0 * c0) + c0 * c0
    np.testing.assert_allclose(results["plain"][0][0].reshape(4, 6), t + late + tail, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("np_dtype", [np.float32, np.int32, np.float64])
def test_fused_concat_keeps_every_bit(np_dtype):
    """CONCAT inside a group is an OR of zero-bordered operands: signed zeros,
    NaN payloads and every integer bit pattern must come through, also when the
    operands are seen through SLICE views and feed further elementwise nodes."""
    rng = np.random.default_rng(41)
    if np_dtype == np.int32:
        draw = lambda n: rng.integers(-2 ** 31, 2 ** 31 - 1, n).astype(np.int32)
    else:
        def draw(n):
            v = rng.uniform(-1, 1, n).astype(np_dtype)
            v[::7] = -0.0
            v[3::11] = np.nan
            return v
    feeds = [draw(5 * 4 * 3) for _ in range(4)]
    other = draw(7 * 3)

    def build(g, api):
        x = g.variable(feeds[0], [5, 4, 3], "x")
        y = g.variable(other, [7, 1, 3], "y")
        first = api.slice(x, 1, 1, 1)                    # [5, 1, 3] views of x
        last = api.slice(x, 3, 1, 1)
        along0 = api.concat([api.concat([first, y], 0), last], 0)   # [17, 1, 3], nested two-operand forms
        along1 = api.concat([first, last, api.slice(x, 0, 1, 1)], 1)   # [5, 3, 3]
        doubled = api.neg(api.neg(along0))               # elementwise readers in the same launch
        return [along0, along1, doubled, api.neg(along1)], x

    results, stats = run_both(build, feeds, kinds=("plain", "replay_launches"))
    for row, ref in zip(results["replay_launches"], results["plain"]):
        for a, b in zip(row, ref):
            assert a.tobytes() == b.tobytes()
    assert stats["replay_launches"]["replayed"] == 3


@pytest.mark.parametrize("evaluator", ["plain", "replay"])
def test_rand_unif_on_the_device_under_both_evaluators(evaluator):
    """RAND_UNIF with the device generator: non-idempotent (a new draw per
    evaluation, cfg/ops.yml:101-103), within its bounds, the restated stream in
    evaluation order, replayable, and restartable with seed()."""
    from tenncor_amd import graph
    from oracle import oracle
    graph.set_random("device")
    graph.set_evaluator(evaluator)
    try:
        g = graph.Graph()
        n = 4096
        lo_v, hi_v = np.linspace(-2, 0, n).astype(np.float32), np.linspace(1, 3, n).astype(np.float32)
        lo, hi = g.variable(lo_v, [64, 64], "lo"), g.variable(hi_v, [64, 64], "hi")
        noise = g.functor("RAND_UNIF", [lo, hi])
        root = g.functor("MUL", [noise, g.scalar(2.0, np.float32, [64, 64])])
        graph.seed(99)
        draws = []
        for _ in range(5):
            g.evaluate([root])
            draws.append(g.data(root).copy())
        for k, got in enumerate(draws):
            want = oracle.rand_uniform(lo_v, hi_v, 99, first_block=k * n // 4) * np.float32(2)
            np.testing.assert_array_equal(got, want)
        if evaluator == "replay":
            stats = graph.evaluator_stats()
            # walked once, then recorded; the recording serves that pass and the three after it
            assert stats["plain"] == 1 and stats["recorded"] == 1 and stats["replayed"] == 4
        graph.seed(99)
        g.evaluate([root])
        np.testing.assert_array_equal(g.data(root), draws[0])
        g.close()
    finally:
        graph.set_random("host")
        graph.set_evaluator("default")


# ---- a whole pass recorded as one kernel ---------------------------------------

@pytest.mark.parametrize("np_dtype", [np.float32, np.float64, np.int32])
def test_small_sequence_recorded_as_one_kernel(ctx, np_dtype):
    """tcg_capture_begin_small: elementwise, data-movement, contraction,
    reduction and in-place steps in one launch against the same calls issued
    one by one.  Elementwise and data-movement results are bit-identical;
    sums are compared at 1e-5 (fp32) / 1e-13 (fp64) relative to the largest
    value, exactly in int32 (ascending order here, a tree there)."""
    from tenncor_amd import capi
    rng = np.random.default_rng(5)
    dt = capi.dtype_code(np_dtype)
    M, K, N = 6, 10, 9
    if np_dtype == np.int32:
        draw = lambda n: rng.integers(-50, 50, n).astype(np.int32)
    else:
        draw = lambda n: rng.uniform(-1, 1, n).astype(np_dtype)
    av, bv, cv, tv = draw(M * K), draw(K * N), draw(N), draw(M * N)
    a, b, bias = ctx.upload(av), ctx.upload(bv), ctx.upload(cv)
    targets = [ctx.upload(tv), ctx.upload(tv)]

    def sequence(alloc, target):
        prod, ext, summed, act, perm, cut = (alloc(M * N) for _ in range(6))
        s0, s1, mx, outer = alloc(N), alloc(M), alloc(1), alloc(M * M)
        ctx.matmul(dt, [K, M], [N, K], a.ptr, b.ptr, prod)
        ctx.extend(dt, [N], [1, M], bias.ptr, ext)
        ctx.ew_binary("ADD", dt, M * N, prod, ext, summed)
        ctx.ew_unary("ABS", dt, M * N, summed, act)
        ctx.ew_nary("MUL", dt, M * N, [act, ext, summed], ext)
        ctx.permute(dt, [N, M], [1, 0, 2, 3, 4, 5, 6, 7], act, perm)                    # {M, N}
        ctx.slice(dt, [M, N], [1, 2], [4, 5], perm, cut)                # {4, 5}
        ctx.reduce("REDUCE_SUM", dt, [N, M], [1], act, s0)
        ctx.reduce("REDUCE_SUM", dt, [N, M], [0], act, s1)
        ctx.reduce("REDUCE_MAX", dt, [N, M], [0, 1], act, mx)
        ctx.contract(dt, [N, M], [N, M], [[0, 0]], act, summed, outer)  # act . summed^T -> {M, M}
        ctx.assign("ASSIGN_ADD", dt, M * N, target, ext)
        return {"act": (act, M * N), "ext": (ext, M * N), "perm": (perm, M * N), "cut": (cut, 20), "s0": (s0, N),
                "s1": (s1, M), "mx": (mx, 1), "outer": (outer, M * M), "target": (target, M * N)}

    esz = np.dtype(np_dtype).itemsize
    eager = sequence(lambda n: ctx.alloc(n * esz), targets[0].ptr)
    want = {k: ctx.d2h(p, n, np_dtype) for k, (p, n) in eager.items()}
    ctx.capture_begin(small=True)
    recorded = sequence(lambda n: ctx.alloc(n * esz), targets[1].ptr)
    graph = ctx.capture_end()
    assert ctx.graph_stats(graph)[0] == 1
    updated = tv.copy()
    for launch in range(3):
        ctx.graph_launch(graph)
        updated = updated + want["ext"]
        got = {k: ctx.d2h(p, n, np_dtype) for k, (p, n) in recorded.items() if k != "target"}
        for k in ("act", "ext", "perm", "cut", "mx"):
            np.testing.assert_array_equal(got[k], want[k], err_msg=k)
        for k in ("s0", "s1", "outer"):
            if np_dtype == np.int32:
                np.testing.assert_array_equal(got[k], want[k], err_msg=k)
            else:
                tol = (1e-5 if np_dtype == np.float32 else 1e-13) * np.abs(want[k]).max()
                assert np.abs(got[k] - want[k]).max() <= tol, k
        # the in-place update is applied once per launch
        np.testing.assert_array_equal(targets[1].get(), updated)
    ctx.graph_destroy(graph)


def test_small_recording_refuses_what_one_workgroup_should_not_do(ctx):
    from tenncor_amd import capi
    n = 1 << 20
    x, y = ctx.upload(np.ones(n, np.float32)), ctx.empty(n, np.float32)
    ctx.capture_begin(small=True)
    with pytest.raises(capi.TcgError) as err:
        for _ in range(8):
            ctx.ew_unary("EXP", capi.FLOAT, n, x.ptr, y.ptr)
    assert err.value.status == 3 and "single-launch pass" in str(err.value)
    ctx.capture_abort()
    # a launch that cannot be a step is caught when the recording ends
    img, ker = ctx.upload(np.ones(64, np.float32)), ctx.upload(np.ones(4, np.float32))
    out = ctx.empty(49, np.float32)
    ctx.capture_begin(small=True)
    ctx.conv(capi.FLOAT, [8, 8], [2, 2], [0, 1], img.ptr, ker.ptr, out.ptr)
    with pytest.raises(capi.TcgError) as err:
        ctx.capture_end()
    assert err.value.status == 3
    # the context is usable afterwards
    ctx.ew_unary("EXP", capi.FLOAT, 64, img.ptr, out.ptr)
    np.testing.assert_allclose(ctx.d2h(out.ptr, 49, np.float32), np.e, rtol=1e-6)


# ---- graphs of small tensors: the pass as one kernel -----------------------------

def close_to(got, ref, rtol):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    scale = max(np.abs(ref).max(), 1e-300)
    assert np.abs(got - ref).max() <= rtol * scale


def test_small_graph_pass_is_one_launch_and_matches_golden_and_walk():
    """tenncor/test/test_equation.cpp:482-706 (the shapes of configs[0]) under
    the default replaying evaluator: one launch per evaluation, the reference's
    gradients at 1e-12 (double), new inputs against the walk at 1e-12."""
    from tenncor_amd import graph
    fx = EQV["sigmoid_mlp_fast"]
    rng = np.random.default_rng(3)
    x0 = np.array(fx["in_data"], np.float64)
    inputs = [x0, rng.uniform(-1, 1, 30), rng.uniform(-1, 1, 30), x0]
    rows = {}
    for kind in ("plain", "replay"):
        graph.set_evaluator(kind)
        g = graph.Graph()
        try:
            x, leaves, err, grads = mlp(g, graph.Api(g), fx, np.float64)
            rows[kind] = []
            for xv in inputs:
                g.assign(x, xv)
                g.evaluate([err] + grads)
                rows[kind].append([t.get().copy() for t in [err] + grads])
            if kind == "replay":
                st = graph.evaluator_stats()
                assert st["plain"] == 1 and st["recorded"] == 1 and st["replayed"] == 3 and st["launches"] == 1
        finally:
            g.close()
            graph.set_evaluator("default")
    for key, val in zip(("expect_gw0", "expect_gb0", "expect_gw1", "expect_gb1"), rows["replay"][3][1:]):
        np.testing.assert_allclose(val, np.array(fx[key]), rtol=1e-12)
    for got, ref in zip(rows["replay"], rows["plain"]):
        for a, b in zip(got, ref):
            close_to(a, b, 1e-12)


@pytest.mark.parametrize("config", ["mlp", "lstm", "training"])
def test_small_graph_passes_follow_the_walk(config):
    """fp32 graphs whose tensors are small (configs[0]; configs[3] at reduced
    size; an sgd step through ASSIGN_SUB) as one launch per evaluation, against
    the walk at 1e-5 of the largest value (sums run in another order)."""
    from tenncor_amd import graph, configs
    rng = np.random.default_rng(23)
    rows = {}
    for kind in ("plain", "replay"):
        graph.set_evaluator(kind)
        g = graph.Graph()
        try:
            if config == "mlp":
                targets, x, _ = configs.config1_mlp(g)
                feeds = [rng.uniform(-1, 1, 30).astype(np.float32) for _ in range(4)] if kind == "plain" else feeds
            elif config == "lstm":
                targets, x, _, _ = configs.config4_lstm(g, seq=4, batch=3, nin=5, hid=6)
                feeds = [rng.uniform(-1, 1, 3 * 4 * 5).astype(np.float32) for _ in range(4)] if kind == "plain" else feeds
            else:
                api = graph.Api(g)
                w = g.variable(np.linspace(-1, 1, 12).astype(np.float32), [3, 4], "w")
                x = g.variable(np.zeros(8, np.float32), [4, 2], "x")
                loss = api.reduce_sum(api.square(api.tanh(api.matmul(x, w))))
                (dw,) = g.derive(loss, [w])
                targets = [g.functor("ASSIGN_SUB", [w, api.mul(0.05, dw)]), loss]
                feeds = [rng.uniform(-1, 1, 8).astype(np.float32) for _ in range(5)] if kind == "plain" else feeds
            rows[kind] = []
            for feed in feeds:
                g.assign(x, feed)
                g.evaluate(targets)
                rows[kind].append([t.get().copy() for t in targets])
            if kind == "replay":
                st = graph.evaluator_stats()
                assert st["recorded"] == 1 and st["replayed"] == len(feeds) - 1 and st["launches"] == 1
        finally:
            g.close()
            graph.set_evaluator("default")
    for got, ref in zip(rows["replay"], rows["plain"]):
        for a, b in zip(got, ref):
            close_to(a, b, 1e-5)


def test_graphs_with_steps_one_kernel_cannot_take_are_recorded_launch_by_launch():
    """A convolution among small tensors: the single-kernel recording is
    refused, the pass is recorded launch by launch and equals the walk bit for bit."""
    from tenncor_amd import graph
    rng = np.random.default_rng(2)
    xv = rng.integers(1, 9, 2 * 6 * 5 * 2).astype(np.float32)
    kv = rng.integers(-4, 5, 3 * 2 * 3 * 2).astype(np.float32)
    rows = {}
    for kind in ("plain", "replay"):
        graph.set_evaluator(kind)
        g = graph.Graph()
        try:
            api = graph.Api(g)
            x = g.variable(xv, [2, 6, 5, 2], "x")
            k = g.variable(kv, [3, 2, 3, 2], "k")
            total = api.reduce_sum(api.relu(api.conv2d(x, k)))
            rows[kind] = []
            for i in range(4):
                g.assign(x, xv + i)
                g.evaluate([total])
                rows[kind].append(total.get().copy())
            if kind == "replay":
                st = graph.evaluator_stats()
                assert st["recorded"] == 1 and st["replayed"] == 3 and st["launches"] > 1
        finally:
            g.close()
            graph.set_evaluator("default")
    for a, b in zip(rows["replay"], rows["plain"]):
        np.testing.assert_array_equal(a, b)


def test_inputs_that_travel_with_the_launch(ctx):
    """tcg_capture_feed / tcg_graph_feed: the recorded kernel reads a fed input
    from its launch arguments; the device memory behind the address is neither
    read nor written, and feeding a buffer that a step writes is refused."""
    from tenncor_amd import capi
    n = 24
    xs = [np.arange(n, dtype=np.float32) * (k + 1) for k in range(3)]
    x = ctx.upload(np.full(n, -1, np.float32))   # what the device copy holds is never looked at
    w = ctx.upload(np.full(n, 2, np.float32))
    ctx.capture_begin(small=True)
    prod, total = ctx.alloc(n * 4), ctx.alloc(4)
    ctx.ew_binary("MUL", capi.FLOAT, n, x.ptr, w.ptr, prod)
    ctx.reduce("REDUCE_SUM", capi.FLOAT, [n], [0], prod, total)
    ctx.capture_feed(x.ptr, xs[0])
    graph = ctx.capture_end()
    for k, xv in enumerate(xs):
        if k > 0:
            ctx.graph_feed(graph, x.ptr, xv)
        ctx.graph_launch(graph)
        ctx.graph_launch(graph)
        np.testing.assert_array_equal(ctx.d2h(total, 1, np.float32), [2 * xv.sum()])
    np.testing.assert_array_equal(x.get(), np.full(n, -1, np.float32))
    with pytest.raises(capi.TcgError):
        ctx.graph_feed(graph, w.ptr, xs[0])      # never declared
    ctx.graph_destroy(graph)
    ctx.capture_begin(small=True)
    ctx.ew_unary("NEG", capi.FLOAT, n, w.ptr, x.ptr)
    ctx.capture_feed(x.ptr, xs[0])
    with pytest.raises(capi.TcgError, match="written by a step"):
        ctx.capture_end()


def test_timing_evaluator_runs_the_planned_launches_between_events():
    """eigen::TimingEvaluator in the evaluator slot (the place of the reference's
    dbg::PlugableEvaluator, dbg/peval/plugin_eval.hpp:21-42): the launches a
    recording would hold, run one by one with an event on either side.  The
    values are those of the recording's launches (held to the walk like them);
    the report names every kind of launch with its count and device time."""
    from tenncor_amd import graph, configs
    results = {}
    try:
        for kind in ("plain", "timing"):
            graph.set_evaluator(kind)
            g = graph.Graph()
            try:
                targets, x, _, _ = configs.config4_lstm(g, seq=5, batch=64, nin=32, hid=64)
                for _ in range(3):
                    g.assign(x, g.data(x))
                    g.evaluate(targets)
                results[kind] = [t.get().copy() for t in targets]
                if kind == "timing":
                    report = graph.evaluator_timing()
                    # "batch N": the N steps behind that line go out as one launch
                    planned, skip = [], 0
                    for l in g.launch_plan(targets):
                        if l.startswith("folded"):
                            continue
                        if skip:
                            skip -= 1
                        elif l.startswith("batch "):
                            skip = int(l.split(" ")[1])
                            planned.append("batch of %d:" % skip)
                        else:
                            planned.append(l)
            finally:
                g.close()
    finally:
        graph.set_evaluator("default")
    for a, b in zip(results["plain"], results["timing"]):
        assert np.abs(a - b).max() <= 1e-5 * np.abs(a).max()
    lines = report.splitlines()
    assert lines[0].startswith("3 passes timed launch by launch (%d launches in the latest), 0 walked" % len(planned)), lines[0]
    rows = {}
    for line in lines[1:]:
        head, _, what = line.partition(" us  ")
        count, _, rest = head.strip().partition(" x ")
        rows[what] = (int(count), float(rest.split("=")[1]))
    # every planned launch is in the table, three times (one per pass), with a positive time
    for what in set(planned):
        if what.startswith("batch of "):
            found = [v for k, v in rows.items() if k.startswith(what)]
            assert sum(v[0] for v in found) == 3 * planned.count(what) and all(v[1] > 0 for v in found), (what, found)
        else:
            assert rows[what][0] == 3 * planned.count(what) and rows[what][1] > 0, (what, rows.get(what))
    assert any(" with epilogue group " in what for what in rows)
