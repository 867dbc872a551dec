"""tcg_fork / tcg_fork_end / tcg_join: launches that nothing waits for yet run on
a second stream of the context, beside the launches that follow them.

No counterpart in the reference (its device runs one Eigen expression at a
time, internal/eigen/device.hpp:555-570).  What is checked: the values are the
ones the same calls give in a row, bit for bit (the same kernels with the same
arguments); memory given back while forked stays out of the pool until the
join; a recording holds both branches and replays them with new inputs; and
the evaluator's use of it on a graph with two independent convolutions.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture()
def ctx():
    from tenncor_amd import capi
    c = capi.Context(0)
    yield c
    c.close()


def two_branches(ctx, capi, n, a, b, x, forked):
    """product of two n x n matrices (through a temporary that is given back at once)
    beside an elementwise chain over x; then a launch that reads both."""
    prod, act, both = ctx.alloc(n * n * 4), ctx.alloc(n * n * 4), ctx.alloc(n * n * 4)
    if forked:
        ctx.fork()
    tmp = ctx.alloc(n * n * 4)
    ctx.matmul(capi.FLOAT, [n, n], [n, n], a, b, tmp)
    ctx.ew_unary("NEG", capi.FLOAT, n * n, tmp, prod)
    ctx.free(tmp, n * n * 4)
    if forked:
        ctx.fork_end()
    other = ctx.alloc(n * n * 4)  # must not be the block given back above while that may still be in use
    ctx.ew_unary("TANH", capi.FLOAT, n * n, x, other)
    ctx.ew_binary("MUL", capi.FLOAT, n * n, other, x, act)
    if forked:
        assert other != tmp
        ctx.join()
    ctx.ew_binary("ADD", capi.FLOAT, n * n, prod, act, both)
    ctx.free(other, n * n * 4)
    return prod, act, both, tmp


def test_forked_launches_give_the_same_values_and_keep_their_memory_until_the_join(ctx):
    from tenncor_amd import capi
    rng = np.random.default_rng(21)
    n = 512
    a, b, x = (ctx.upload(rng.uniform(-1, 1, n * n).astype(np.float32)) for _ in range(3))
    want = [ctx.d2h(p, n * n, np.float32) for p in two_branches(ctx, capi, n, a.ptr, b.ptr, x.ptr, False)[:3]]
    prod, act, both, tmp = two_branches(ctx, capi, n, a.ptr, b.ptr, x.ptr, True)
    for got, ref in zip((prod, act, both), want):
        np.testing.assert_array_equal(ctx.d2h(got, n * n, np.float32), ref)
    # after the join the temporary is back in the pool
    again = [ctx.alloc(n * n * 4) for _ in range(2)]
    assert tmp in again
    av, bv = a.get().reshape(n, n).astype(np.float64), b.get().reshape(n, n).astype(np.float64)
    assert np.abs(want[0].reshape(n, n) + av @ bv).max() <= 1e-4


def test_a_recording_holds_both_branches(ctx):
    from tenncor_amd import capi
    rng = np.random.default_rng(22)
    n = 256
    hosts = [rng.uniform(-1, 1, n * n).astype(np.float32) for _ in range(3)]
    a, b, x = (ctx.upload(h) for h in hosts)
    ctx.capture_begin()
    prod, act, both, _ = two_branches(ctx, capi, n, a.ptr, b.ptr, x.ptr, True)
    graph = ctx.capture_end()
    ctx.capture_begin()
    serial = two_branches(ctx, capi, n, a.ptr, b.ptr, x.ptr, False)[:3]
    graph_serial = ctx.capture_end()
    assert ctx.graph_stats(graph)[0] == ctx.graph_stats(graph_serial)[0]
    for launch in range(3):
        if launch:
            ctx.h2d(x.ptr, rng.uniform(-1, 1, n * n).astype(np.float32))
            ctx.h2d(a.ptr, rng.uniform(-1, 1, n * n).astype(np.float32))
        ctx.graph_launch(graph_serial)
        want = [ctx.d2h(p, n * n, np.float32) for p in serial]
        ctx.graph_launch(graph)
        for got, ref in zip((prod, act, both), want):
            np.testing.assert_array_equal(ctx.d2h(got, n * n, np.float32), ref)
    ctx.graph_destroy(graph)
    ctx.graph_destroy(graph_serial)


def test_joins_happen_by_themselves_where_the_stream_is_waited_for(ctx):
    from tenncor_amd import capi
    n = 1 << 16
    v = np.arange(n, dtype=np.float32)
    src, dst = ctx.upload(v), ctx.empty(n, np.float32)
    ctx.fork()
    ctx.ew_unary("NEG", capi.FLOAT, n, src.ptr, dst.ptr)
    np.testing.assert_array_equal(dst.get(), -v)  # the download joins first
    ctx.join()                                      # nothing left to wait for
    ctx.fork()
    with pytest.raises(capi.TcgError):
        ctx.fork()                                  # one fork at a time
    ctx.join()
    ctx.ew_unary("SQUARE", capi.FLOAT, n, src.ptr, dst.ptr)
    np.testing.assert_array_equal(dst.get(), v * v)


def test_two_gradients_of_a_convolution_run_side_by_side_and_match_the_walk():
    """configs[4] at reduced size: the kernel gradient of the second layer is read by
    nothing in the pass and goes to the second stream while the image gradient and the
    first layer's kernel gradient run (TCR_FORKS=1; off by default).  Same kernels, same arguments: the values with
    and without the second stream are equal bit for bit, and both follow the walk at
    the tolerance of the products."""
    import os
    import subprocess
    import sys
    import json
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import sys, json, numpy as np\n"
        "sys.path.insert(0, %r)\n"
        "from tenncor_amd import graph, configs\n"
        "out = {}\n"
        "for kind in ('plain', 'replay'):\n"
        "    graph.set_evaluator(kind)\n"
        "    g = graph.Graph()\n"
        "    targets, x, _, _ = configs.config5_cnn(g, batch=16, hw=20, c1=8, c2=16, ncls=10)\n"
        "    for _ in range(3):\n"
        "        g.assign(x, g.data(x))\n"
        "        g.evaluate(targets)\n"
        "    out[kind] = [t.get().astype(np.float64).tolist() for t in targets]\n"
        "    out[kind + '_stats'] = graph.evaluator_stats()\n"
        "    g.close()\n"
        "print(json.dumps(out))\n" % root)
    runs = {}
    for forks in ("1", "0"):
        env = dict(os.environ, TCR_FORKS=forks)
        done = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
        assert done.returncode == 0, done.stderr[-2000:]
        runs[forks] = json.loads(done.stdout.strip().splitlines()[-1])
    assert runs["1"]["replay_stats"]["replayed"] >= 1 and runs["1"]["replay_stats"]["record_failures"] == 0
    for a, b in zip(runs["1"]["replay"], runs["0"]["replay"]):
        np.testing.assert_array_equal(np.array(a), np.array(b))
    for a, b in zip(runs["1"]["replay"], runs["1"]["plain"]):
        a, b = np.array(a), np.array(b)
        assert np.abs(a - b).max() <= 1e-4 * max(1e-30, np.abs(b).max())
