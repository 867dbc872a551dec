"""Batches (tcg_batch_begin / tcg_batch_end): the small launches of a longer
sequence held back and sent out as ONE kernel, big launches in between sent
out as themselves in their place.

The reference has no counterpart (its evaluator calls one Eigen expression per
node, internal/teq/evaluator.hpp:35-62); what is checked is that a sequence
gives the same values with and without batches: at 1e-5 (fp32) / 1e-13 (fp64)
relative to the largest value (a batch sums in another order than the kernels
that run by themselves, and what is computed from a sum inherits the
difference) and exactly in int32, and that a recording of the stream holds a
batch as one launch.
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


def draw_for(rng, np_dtype):
    if np_dtype == np.int32:
        return lambda n: rng.integers(-50, 50, n).astype(np.int32)
    return lambda n: rng.uniform(-1, 1, n).astype(np_dtype)


def close(got, want, np_dtype, name):
    if np_dtype == np.int32:
        np.testing.assert_array_equal(got, want, err_msg=name)
    else:
        tol = (1e-5 if np_dtype == np.float32 else 1e-13) * max(1e-30, np.abs(want).max())
        assert np.abs(got - want).max() <= tol, name


def softmax_like(ctx, dt, rows, cols, hid, x, w, alloc, big=None, floating=True, free=None):
    """dense layer -> row max -> exp(x - max) -> row sum -> divide -> weight gradient:
    the launches behind a classifier, all over rows x cols and rows x hid elements.
    big: (n, src, dst) of an elementwise launch too large for a step, issued in the middle.
    free: gives a temporary back behind its last reader (what a batch keeps in LDS)."""
    logits, mx, mxe, shifted, ex, sm, sme, prob, dw = (alloc(rows * cols), alloc(rows), alloc(rows * cols),
        alloc(rows * cols), alloc(rows * cols), alloc(rows), alloc(rows * cols), alloc(rows * cols), alloc(hid * cols))
    ctx.matmul(dt, [hid, rows], [cols, hid], x, w, logits)
    ctx.reduce("REDUCE_MAX", dt, [cols, rows], [0], logits, mx)
    ctx.extend(dt, [1, rows], [cols, 1], mx, mxe)
    ctx.ew_binary("SUB", dt, rows * cols, logits, mxe, shifted)
    if free:
        free(mxe, rows * cols)
    if big is not None:
        ctx.ew_unary("NEG", dt, big[0], big[1], big[2])
    ctx.ew_unary("EXP" if floating else "ABS", dt, rows * cols, shifted, ex)
    ctx.reduce("REDUCE_SUM", dt, [cols, rows], [0], ex, sm)
    ctx.extend(dt, [1, rows], [cols, 1], sm, sme)
    ctx.ew_binary("DIV" if floating else "ADD", dt, rows * cols, ex, sme, prob)
    if free:
        free(sme, rows * cols)
    ctx.contract(dt, [hid, rows], [cols, rows], [[1, 1]], x, prob, dw)  # x^T . prob -> {cols, hid}
    return {"logits": (logits, rows * cols), "mx": (mx, rows), "shifted": (shifted, rows * cols), "ex": (ex, rows * cols),
            "sm": (sm, rows), "prob": (prob, rows * cols), "dw": (dw, hid * cols)}


@pytest.mark.parametrize("np_dtype", [np.float32, np.float64, np.int32])
def test_batched_sequence_gives_what_the_launches_give(ctx, np_dtype):
    from tenncor_amd import capi
    rng = np.random.default_rng(11)
    dt = capi.dtype_code(np_dtype)
    floating = np_dtype != np.int32
    rows, cols, hid = 128, 10, 64
    draw = draw_for(rng, np_dtype)
    x, w = ctx.upload(draw(rows * hid)), ctx.upload(draw(hid * cols))
    esz = np.dtype(np_dtype).itemsize
    alloc = lambda n: ctx.alloc(n * esz)
    eager = softmax_like(ctx, dt, rows, cols, hid, x.ptr, w.ptr, alloc, floating=floating)
    want = {k: ctx.d2h(p, n, np_dtype) for k, (p, n) in eager.items()}
    ctx.batch_begin()
    held = softmax_like(ctx, dt, rows, cols, hid, x.ptr, w.ptr, alloc, floating=floating)
    ctx.batch_end()
    got = {k: ctx.d2h(p, n, np_dtype) for k, (p, n) in held.items()}
    for k in want:
        close(got[k], want[k], np_dtype, k)
    # temporaries given back inside the batch never reach memory: same values
    ctx.batch_begin()
    lean = softmax_like(ctx, dt, rows, cols, hid, x.ptr, w.ptr, alloc, floating=floating,
                        free=lambda ptr, n: ctx.free(ptr, n * esz))
    ctx.batch_end()
    for k in want:
        np.testing.assert_array_equal(ctx.d2h(lean[k][0], lean[k][1], np_dtype), got[k], err_msg=k)
    # against numpy as well, so that both paths being wrong the same way shows
    xv, wv = x.get().reshape(rows, hid).astype(np.float64), w.get().reshape(hid, cols).astype(np.float64)
    logits = xv @ wv
    close(got["logits"].reshape(rows, cols), logits.astype(np_dtype), np_dtype, "logits vs numpy")
    if np_dtype != np.int32:
        ex = np.exp(logits - logits.max(axis=1, keepdims=True))
        prob = ex / ex.sum(axis=1, keepdims=True)
        tol = 1e-5 if np_dtype == np.float32 else 1e-12
        assert np.abs(got["prob"].reshape(rows, cols) - prob).max() <= tol
        assert np.abs(got["dw"].reshape(hid, cols) - xv.T @ prob).max() <= tol * rows


def test_a_batch_is_one_launch_of_a_recording_and_replays(ctx):
    from tenncor_amd import capi
    rng = np.random.default_rng(12)
    rows, cols, hid = 128, 10, 64
    xv, wv = rng.uniform(-1, 1, rows * hid).astype(np.float32), rng.uniform(-1, 1, hid * cols).astype(np.float32)
    x, w = ctx.upload(xv), ctx.upload(wv)
    alloc = lambda n: ctx.alloc(n * 4)
    want = {k: ctx.d2h(p, n, np.float32) for k, (p, n) in
            softmax_like(ctx, capi.FLOAT, rows, cols, hid, x.ptr, w.ptr, alloc).items()}
    ctx.capture_begin()
    plain = softmax_like(ctx, capi.FLOAT, rows, cols, hid, x.ptr, w.ptr, alloc)
    graph_plain = ctx.capture_end()
    ctx.capture_begin()
    ctx.batch_begin()
    held = softmax_like(ctx, capi.FLOAT, rows, cols, hid, x.ptr, w.ptr, alloc)
    graph = ctx.capture_end()  # ends the batch
    assert ctx.graph_stats(graph_plain)[0] >= 9
    assert ctx.graph_stats(graph)[0] == 1
    for launch in range(3):
        # other work of the context between the replays, and new inputs for the second
        if launch == 1:
            xv = rng.uniform(-1, 1, rows * hid).astype(np.float32)
            ctx.h2d(x.ptr, xv)
            ctx.graph_launch(graph_plain)
            want = {k: ctx.d2h(p, n, np.float32) for k, (p, n) in plain.items()}
        ctx.graph_launch(graph)
        got = {k: ctx.d2h(p, n, np.float32) for k, (p, n) in held.items()}
        for k in want:
            close(got[k], want[k], np.float32, "%s, launch %d" % (k, launch))
    ctx.graph_destroy(graph)
    ctx.graph_destroy(graph_plain)


def test_a_launch_too_large_for_a_step_goes_out_in_its_place(ctx):
    """A launch that cannot be a step sends the steps held so far out in front of itself
    and ends the batch: the launches behind it go out one by one."""
    from tenncor_amd import capi
    rng = np.random.default_rng(13)
    rows, cols, hid = 128, 10, 64
    x, w = ctx.upload(rng.uniform(-1, 1, rows * hid).astype(np.float32)), ctx.upload(rng.uniform(-1, 1, hid * cols).astype(np.float32))
    n = 1 << 20
    src = ctx.upload(rng.uniform(-1, 1, n).astype(np.float32))
    dst = ctx.empty(n, np.float32)
    alloc = lambda k: ctx.alloc(k * 4)
    want = {k: ctx.d2h(p, m, np.float32) for k, (p, m) in
            softmax_like(ctx, capi.FLOAT, rows, cols, hid, x.ptr, w.ptr, alloc).items()}
    ctx.capture_begin()
    ctx.batch_begin()
    held = softmax_like(ctx, capi.FLOAT, rows, cols, hid, x.ptr, w.ptr, alloc, big=(n, src.ptr, dst.ptr))
    graph = ctx.capture_end()
    # the steps before the big launch as one kernel, the big launch, and every launch behind it as itself
    launches = ctx.graph_stats(graph)[0]
    assert 2 < launches < 10
    ctx.graph_launch(graph)
    np.testing.assert_array_equal(dst.get(), -src.get())
    for k in want:
        close(ctx.d2h(held[k][0], held[k][1], np.float32), want[k], np.float32, k)
    ctx.graph_destroy(graph)


def test_a_reduction_in_the_middle_reads_what_the_step_before_wrote(ctx):
    """In-place chains: every step reads the buffer the one before wrote."""
    from tenncor_amd import capi
    rng = np.random.default_rng(14)
    n = 4096
    v = rng.uniform(0.5, 1.5, n).astype(np.float32)
    buf, total, spread = ctx.upload(v), ctx.empty(64, np.float32), ctx.empty(n, np.float32)
    ctx.batch_begin()
    ctx.ew_unary("SQRT", capi.FLOAT, n, buf.ptr, buf.ptr)
    ctx.ew_binary("MUL", capi.FLOAT, n, buf.ptr, buf.ptr, buf.ptr)
    ctx.reduce("REDUCE_SUM", capi.FLOAT, [64, 64], [0], buf.ptr, total.ptr)
    ctx.extend(capi.FLOAT, [1, 64], [64, 1], total.ptr, spread.ptr)
    ctx.ew_binary("DIV", capi.FLOAT, n, buf.ptr, spread.ptr, buf.ptr)
    ctx.batch_end()
    sq = np.sqrt(v) * np.sqrt(v)
    rows = sq.reshape(64, 64)
    np.testing.assert_allclose(total.get(), rows.sum(axis=1), rtol=1e-5)
    np.testing.assert_allclose(buf.get().reshape(64, 64), rows / rows.sum(axis=1, keepdims=True), rtol=1e-5)


def test_sync_and_downloads_end_a_batch(ctx):
    from tenncor_amd import capi
    v = np.arange(256, dtype=np.float32)
    src, dst = ctx.upload(v), ctx.empty(256, np.float32)
    ctx.batch_begin()
    ctx.ew_unary("NEG", capi.FLOAT, 256, src.ptr, dst.ptr)
    np.testing.assert_array_equal(dst.get(), -v)  # the download sends the step out first
    ctx.batch_begin()
    ctx.ew_unary("SQUARE", capi.FLOAT, 256, src.ptr, dst.ptr)
    ctx.sync()
    ctx.batch_end()  # nothing left: does nothing
    np.testing.assert_array_equal(dst.get(), v * v)


def test_a_block_taken_again_inside_a_batch_keeps_what_its_last_owner_left(ctx):
    """A buffer filled before the batch, read by a step and given back; the next
    buffer of that size is the same block, written and read by later steps and given
    back as well.  The first step must still read the old content from memory (a
    block with an earlier owner is not moved into LDS)."""
    from tenncor_amd import capi
    n = 2048
    v = np.arange(n, dtype=np.float32) + 1
    first = ctx.alloc(n * 4)
    ctx.h2d(first, v)
    out = ctx.empty(n, np.float32)
    ctx.batch_begin()
    kept = ctx.alloc(n * 4)
    ctx.ew_unary("NEG", capi.FLOAT, n, first, kept)        # reads what was there before the batch
    ctx.free(first, n * 4)
    again = ctx.alloc(n * 4)                               # the pool hands the same block out again
    ctx.ew_unary("SQUARE", capi.FLOAT, n, kept, again)
    ctx.ew_binary("ADD", capi.FLOAT, n, again, kept, out.ptr)
    ctx.free(again, n * 4)
    ctx.free(kept, n * 4)
    ctx.batch_end()
    assert again == first
    np.testing.assert_array_equal(out.get(), v * v - v)
