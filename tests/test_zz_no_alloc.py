"""tcg_reduce_noalloc: the reduction entry point that allocates nothing.

Its temporaries (partial results of a split reduced dim, what is left of the
tensor between the steps of a reduction over separated dims) live in a fixed
array of device memory instead of blocks of the context's pool.  It shares the
kernels and launch shapes of tcg_reduce, so the two must agree bit for bit --
fp32 included -- and the pool must not move while it runs.  The array keeps
what the last call left in it: the second call of every pair below is smaller
than the first and must not see the first one's partial results.
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


def both(ctx, op, np_dtype, shape, rank_set, data):
    """(tcg_reduce result, tcg_reduce_noalloc result, pool statistics around the second)"""
    from tenncor_amd import capi
    dtype = capi.dtype_code(np_dtype)
    out_shape = [1 if d in rank_set else v for d, v in enumerate(shape)]
    n_out = int(np.prod(out_shape))
    src = ctx.upload(data)
    want = ctx.empty(n_out, np_dtype)
    got = ctx.empty(n_out, np_dtype)
    ctx.reduce(op, dtype, shape, rank_set, src.ptr, want.ptr)
    ctx.sync()
    before = ctx.mem_stats()
    ctx.reduce_noalloc(op, dtype, shape, rank_set, src.ptr, got.ptr)
    after = ctx.mem_stats()
    ctx.sync()
    res = want.get()[:n_out].copy(), got.get()[:n_out].copy(), before, after
    for b in (src, want, got):
        b.release()
    return res


# (first shape, rank set), (second, smaller shape, rank set): each pair runs back to back
PAIRS = [
    # column reduction split over workgroups: partial results [A, S, B] in the array
    (([4096, 2048], [1]), ([1024, 512], [1])),
    # one long row: partial results of the row kernel
    (([1 << 22], [0]), ([1 << 18], [0])),
    # separated dims: a step result and partial results live together
    (([64, 512, 48, 8], [1, 3]), ([32, 96, 16, 4], [1, 3])),
    # everything, odd extents (scalar paths)
    (([1023, 517, 3], [0, 1, 2]), ([129, 65, 3], [0, 2])),
]


@pytest.mark.parametrize("np_dtype", [np.float32, np.int32, np.float64])
@pytest.mark.parametrize("op", ["REDUCE_SUM", "REDUCE_MAX", "REDUCE_MIN", "REDUCE_PROD"])
@pytest.mark.parametrize("pair", PAIRS)
def test_two_calls_in_a_row_match_tcg_reduce(ctx, oracle, np_dtype, op, pair):
    rng = np.random.default_rng(seed=len(repr((np_dtype, op, pair))) * 7919 + 5)
    for shape, rank_set in pair:
        n = int(np.prod(shape))
        if np_dtype == np.int32:
            data = rng.integers(-1000, 1001, n).astype(np.int32)
        elif op == "REDUCE_PROD":
            # ones, with a thousand factors that matter: the product stays in range whatever n is
            data = np.ones(n, dtype=np_dtype)
            where = rng.choice(n, size=min(n, 1024), replace=False)
            data[where] = rng.uniform(0.7, 1.4, where.size).astype(np_dtype)
        else:
            data = rng.uniform(-1, 1, n).astype(np_dtype)
        print("case", np_dtype.__name__, op, shape, rank_set, flush=True)
        want, got, before, after = both(ctx, op, np_dtype, shape, rank_set, data)
        # same kernels, same launch shapes: identical bits in every dtype
        np.testing.assert_array_equal(got, want)
        assert before == after, "the pool moved during tcg_reduce_noalloc: %r -> %r" % (before, after)
        # and against the CPU oracle (int32 exact; floating point at 1e-4 of max(|ref|, mean|ref|))
        ref = oracle.reduce(op, data, shape, rank_set, wide_acc=np_dtype != np.int32)[0]
        if np_dtype == np.int32:
            np.testing.assert_array_equal(got, ref)
        else:
            ref = np.asarray(ref, dtype=np.float64)
            denom = np.maximum(np.abs(ref), np.mean(np.abs(ref)))
            assert (np.abs(got - ref) / denom).max() <= 1e-4


def test_config2_sized_column_reduction_fits(ctx):
    """REDUCE_SUM / REDUCE_MAX over each dim of np[4096, 16384] (BASELINE
    configs[1]) need 512 KiB of partial results at most."""
    from tenncor_amd import capi
    rng = np.random.default_rng(seed=77)
    shape = [16384, 4096]
    data = rng.integers(-1000, 1001, 16384 * 4096).astype(np.int32)
    for rank_set in ([0], [1]):
        for op in ("REDUCE_SUM", "REDUCE_MAX"):
            print("config-2 case", op, rank_set, flush=True)
            want, got, before, after = both(ctx, op, np.int32, shape, rank_set, data)
            np.testing.assert_array_equal(got, want)
            assert before == after
    mat = data.reshape(4096, 16384)
    want, got, _, _ = both(ctx, "REDUCE_SUM", np.int32, shape, [1], data)
    np.testing.assert_array_equal(got, mat.sum(axis=0, dtype=np.int64).astype(np.int32))


def test_sizes_beyond_the_fixed_memory_are_refused(ctx):
    """A reduction over separated dims whose intermediate does not fit 8 MiB:
    a clear error, no allocation, and the next call works."""
    from tenncor_amd import capi
    assert capi.REDUCE_NOALLOC_SCRATCH_BYTES == 8 << 20
    shape = [2048, 4, 2048, 4]                      # reducing dims 1 and 3 leaves 2048*2048*4 B = 16 MiB in between
    src = ctx.empty(int(np.prod(shape)), np.float32)
    dst = ctx.empty(2048 * 2048, np.float32)
    before = ctx.mem_stats()
    with pytest.raises(capi.TcgError) as err:
        ctx.reduce_noalloc("REDUCE_SUM", capi.FLOAT, shape, [1, 3], src.ptr, dst.ptr)
    assert err.value.status == 1 and "do not fit" in str(err.value) and "tcg_reduce" in str(err.value)
    assert ctx.mem_stats() == before
    ctx.sync()
    small = np.arange(24, dtype=np.float32)
    want, got, _, _ = both(ctx, "REDUCE_SUM", np.float32, [4, 3, 2], [0, 2], small)
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(got, small.reshape(2, 3, 4).sum(axis=(0, 2)))
    src.release()
    dst.release()


@pytest.mark.parametrize("np_dtype", [np.int8, np.int64])
def test_the_narrowest_and_the_widest_integers(ctx, np_dtype):
    """The integer widths of the full type configuration share the kernels:
    two calls in a row, the second smaller, bit for bit with tcg_reduce."""
    rng = np.random.default_rng(seed=31 + np.dtype(np_dtype).itemsize)
    info = np.iinfo(np_dtype)
    for shape, rank_set in (([4096, 2048], [1]), ([1024, 512], [1]), ([64, 512, 48, 8], [1, 3]), ([129, 65, 3], [0, 2])):
        n = int(np.prod(shape))
        data = rng.integers(max(info.min, -1000), min(info.max, 1000) + 1, n).astype(np_dtype)
        for op in ("REDUCE_SUM", "REDUCE_MAX"):
            print("case", np_dtype.__name__, op, shape, rank_set, flush=True)
            want, got, before, after = both(ctx, op, np_dtype, shape, rank_set, data)
            np.testing.assert_array_equal(got, want)
            assert before == after


def test_a_recorded_reduction_replayed_after_the_array_was_used_again(ctx):
    """The use the entry point names first: under tcg_capture_begin the launches
    of tcg_reduce_noalloc are recorded with the array's address in them.  An
    eager reduction in between leaves its own partial results there; the
    replay, over new input, must still equal tcg_reduce bit for bit (every
    replay writes its partial results before it reads them)."""
    from tenncor_amd import capi
    rng = np.random.default_rng(seed=91)
    shape, rank_set = [4096, 2048], [1]
    n = 4096 * 2048
    src = ctx.upload(rng.uniform(-1, 1, n).astype(np.float32))
    got = ctx.empty(4096, np.float32)
    want = ctx.empty(4096, np.float32)
    ctx.capture_begin()
    ctx.reduce_noalloc("REDUCE_SUM", capi.FLOAT, shape, rank_set, src.ptr, got.ptr)
    graph = ctx.capture_end()
    try:
        for round_ in range(3):
            fresh = rng.uniform(-1, 1, n).astype(np.float32)
            ctx.h2d(src.ptr, fresh)
            # another reduction through the same array, of another shape, eagerly
            other = ctx.upload(rng.integers(-1000, 1001, 1 << 20).astype(np.int32))
            other_out = ctx.empty(1, np.int32)
            ctx.reduce_noalloc("REDUCE_SUM", capi.INT32, [1 << 20], [0], other.ptr, other_out.ptr)
            ctx.graph_launch(graph)
            ctx.reduce("REDUCE_SUM", capi.FLOAT, shape, rank_set, src.ptr, want.ptr)
            ctx.sync()
            print("replay", round_, flush=True)
            np.testing.assert_array_equal(got.get(), want.get())
            other.release()
            other_out.release()
    finally:
        ctx.graph_destroy(graph)


def test_another_context_waits_for_the_owner_of_the_array(ctx):
    """Two contexts on one GPU share the array.  While the launches of the one
    that used it last may still be running, the other is refused (TCG_ERR_ARG,
    nothing launched); once the first has been synchronised it is let in, and
    both compute what tcg_reduce computes."""
    from tenncor_amd import capi
    other = capi.Context(0)
    try:
        rng = np.random.default_rng(seed=17)
        shape, rank_set = [4096, 8192], [1]
        data = rng.integers(-1000, 1001, 4096 * 8192).astype(np.int32)
        src, out = ctx.upload(data), ctx.empty(4096, np.int32)
        src2, out2 = other.upload(data[:1 << 20]), other.empty(1, np.int32)
        ctx.sync()
        other.sync()
        for _ in range(8):
            ctx.reduce_noalloc("REDUCE_SUM", capi.INT32, shape, rank_set, src.ptr, out.ptr)
        refused = False
        try:
            other.reduce_noalloc("REDUCE_SUM", capi.INT32, [1 << 20], [0], src2.ptr, out2.ptr)
        except capi.TcgError as err:
            refused = True
            assert err.status == 1 and "another context" in str(err)
        print("refused while the owner was busy:", refused, flush=True)
        ctx.sync()
        other.reduce_noalloc("REDUCE_SUM", capi.INT32, [1 << 20], [0], src2.ptr, out2.ptr)
        other.sync()
        np.testing.assert_array_equal(out2.get(), data[:1 << 20].sum(dtype=np.int64).astype(np.int32))
        np.testing.assert_array_equal(out.get(), data.reshape(8192, 4096).sum(axis=0, dtype=np.int64).astype(np.int32))
        # and back: the first context after the second has finished
        ctx.reduce_noalloc("REDUCE_MAX", capi.INT32, shape, rank_set, src.ptr, out.ptr)
        ctx.sync()
        np.testing.assert_array_equal(out.get(), data.reshape(8192, 4096).max(axis=0))
    finally:
        other.close()
