"""Run as a program with TENNCOR_AMD_TYPES=full (tests/test_full_types.py does):
graphs over the element types of cfg/fulltype.yml:1-34 built through the flat
graph API of the full-type host library and evaluated on the GPU, against the
CPU oracle.  Integer results are compared bit for bit.  `python
tests/full_types_graph_case.py build` only builds the graphs (no GPU).
Prints one line per check and exits non-zero on the first mismatch.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from tenncor_amd import capi, graph  # noqa: E402

INTS = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64]
ALL = INTS + [np.float32, np.float64]
# cfg/fulltype.yml `precision`
PRECISION = {np.int8: 1, np.uint8: 2, np.int16: 3, np.uint16: 4, np.int32: 5, np.uint32: 6, np.int64: 7,
             np.uint64: 8, np.float32: 9, np.float64: 10}


def full_range(rng, t, n):
    if np.dtype(t).kind == "f":
        return rng.uniform(-2, 2, n).astype(t)
    info = np.iinfo(t)
    x = rng.integers(info.min, info.max, n, dtype=t, endpoint=True)
    edge = [info.min, info.max, 0, 1][:n]
    x[:len(edge)] = edge
    return x


def build_only():
    assert graph.FULL_TYPES and graph.LIB_PATH.endswith("libtenncor_host_full.so")
    g = graph.Graph()
    api = graph.Api(g)
    rng = np.random.default_rng(0)
    leaves = {}
    for t in ALL:
        v = g.variable(full_range(rng, t, 6), [3, 2], np.dtype(t).name)
        assert capi.NP_OF[v.dtype] == t, (t, v.dtype)
        assert capi.NP_OF[api.unary("SQUARE", v).dtype] == t
        leaves[t] = v
    # the most precise operand decides, the others are cast to it
    for a in ALL:
        for b in ALL:
            out = api.add(leaves[a], leaves[b])
            want = a if PRECISION[a] >= PRECISION[b] else b
            assert capi.NP_OF[out.dtype] == want, (a, b, out.dtype)
            if a != b:
                cast = g.args(out)[0 if want == b else 1]
                assert g.opcode(cast) == "CAST" and capi.NP_OF[cast.dtype] == want
    for t in ALL:
        out = g.functor("CAST", [leaves[np.int64]], dtype=capi.dtype_code(t))
        assert capi.NP_OF[out.dtype] == t
    g.close()
    print("graphs of %d element types built" % len(ALL))


def evaluate_on_gpu():
    from oracle import oracle as orc
    rng = np.random.default_rng(1)
    for evaluator in ("plain", "replay"):
        graph.set_evaluator(evaluator)
        # few elements: under replay the whole pass is one kernel; many: one launch per group
        for t, shape in [(t, shape) for t in ALL for shape in ([37, 11, 3], [300, 41, 3])]:
            g = graph.Graph()
            api = graph.Api(g)
            exact = np.dtype(t).kind != "f"
            n = capi.n_elems(shape)
            a, b = full_range(rng, t, n), full_range(rng, t, n)
            va, vb = g.variable(a, shape, "a"), g.variable(b, shape, "b")
            chain = api.sub(api.mul(api.add(va, vb), va), vb)          # one fused group under replay
            colsum = api.reduce_sum(chain, 1, 1)
            turned = api.permute(chain, [2, 0, 1])
            largest = api.reduce("REDUCE_MAX", va, 0, 1)
            ma, mb = full_range(rng, t, 20 * 9), full_range(rng, t, 14 * 20)
            vma, vmb = g.variable(ma, [20, 9], "ma"), g.variable(mb, [14, 20], "mb")
            prod = api.matmul(vma, vmb)
            ref_chain = orc.binary("SUB", orc.binary("MUL", orc.binary("ADD", a, b), a), b)
            refs = [(chain, ref_chain), (colsum, orc.reduce("REDUCE_SUM", ref_chain, shape, [1])[0]),
                    (turned, orc.permute(ref_chain, shape, [2, 0, 1])[0]),
                    (largest, orc.reduce("REDUCE_MAX", a, shape, [0])[0]),
                    (prod, orc.matmul(ma, [20, 9], mb, [14, 20], wide_acc=not exact)[0])]
            targets = [node for node, _ in refs]
            for _ in range(3):  # under replay: the walk, the recording, a launch of it
                g.evaluate(targets)
                for node, ref in refs:
                    got = node.get()
                    assert got.dtype == t
                    if exact:
                        np.testing.assert_array_equal(got, ref)
                    else:
                        scale = max(float(np.abs(ref).max()), 1.0)
                        np.testing.assert_allclose(got, ref, rtol=0, atol=(1e-4 if t == np.float32 else 1e-12) * scale)
            g.close()
            print("%s %s %d ok" % (evaluator, np.dtype(t).name, n), flush=True)
        # mixed operands and explicit casts
        g = graph.Graph()
        api = graph.Api(g)
        n = 1001
        small, wide = full_range(rng, np.int8, n), full_range(rng, np.uint16, n)
        vs, vw = g.variable(small, [n], "small"), g.variable(wide, [n], "wide")
        mixed = api.mul(vs, vw)
        narrowed = g.functor("CAST", [mixed], dtype=capi.UINT8)
        asfloat = g.functor("CAST", [vs], dtype=capi.FLOAT)
        g.evaluate([mixed, narrowed, asfloat])  # values that are not targets expire with their last reader
        want = orc.binary("MUL", orc.cast(small, capi.UINT16), wide)
        np.testing.assert_array_equal(mixed.get(), want)
        np.testing.assert_array_equal(narrowed.get(), orc.cast(want, capi.UINT8))
        np.testing.assert_array_equal(asfloat.get(), small.astype(np.float32))
        # the host generator: drawn as int64 and narrowed (internal/global/random.hpp:87-91)
        lo, hi = g.variable(np.full(500, -7, np.int16), [500], "lo"), g.variable(np.full(500, 9, np.int16), [500], "hi")
        drawn = g.functor("RAND_UNIF", [lo, hi])
        g.evaluate([drawn])
        got = drawn.get()
        assert got.dtype == np.int16 and got.min() >= -7 and got.max() <= 9 and len(np.unique(got)) == 17
        g.close()
        print("%s mixed ok" % evaluator, flush=True)
    graph.set_evaluator("default")


def random_graphs_on_gpu():
    """The seeded elementwise / view graphs of tests/test_gpu_replay.py in the
    seven integer types beyond INT32: the recordings (launch by launch, and as
    one kernel at the small size) against the walk, bit for bit."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("replay_cases", os.path.join(ROOT, "tests", "test_gpu_replay.py"))
    cases = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(cases)
    for t in INTS:
        if t == np.int32:
            continue
        for shape in ((12, 10), (96, 80)):
            for seed in range(3):
                for with_updates in (False, True):
                    rng = np.random.default_rng(4000 + seed)
                    feeds = [rng.integers(-9, 10, shape[0] * shape[1]).astype(t) for _ in range(3)]

                    def build(g, api):
                        return cases.random_elementwise_graph(g, api, seed, feeds[0], shape, t, with_updates)

                    results, stats = cases.run_both(build, feeds, kinds=("plain", "replay_launches", "replay"))
                    assert stats["replay"]["record_failures"] == 0 and stats["replay"]["replayed"] >= 1, stats
                    cases.assert_same_bits(results)
        print("random %s ok" % np.dtype(t).name, flush=True)


if __name__ == "__main__":
    build_only()
    if sys.argv[1:] != ["build"]:
        evaluate_on_gpu()
        random_graphs_on_gpu()
    print("done")
