"""API-level cases of the reference that fix how assignments, casts and
dependency-only arguments behave (tenncor/test/test_api.cpp:576-735 Assign and
AssignHighToLowPrecision, :746-772 Cast, :774-880 IdentityDependency and
DependsRunOnce), restated with the reference's own 24-element vectors and
printed graphs.  Values are exact (small integers in double/float) except the
cosine chain, compared at 1e-12.
"""
import re

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

DATA = [59, 10, 28, 10, 67, 62, 23, 4, 55, 77, 28, 16, 82, 52, 47, 16, 7, 85, 37, 2, 8, 52, 62, 43]
DATA2 = [22, 15, 74, 38, 61, 95, 62, 81, 99, 76, 7, 22, 56, 50, 19, 13, 12, 10, 31, 40, 60, 54, 6, 83]
SHAPE = [2, 3, 4]
S = "[2\\3\\4\\1\\1\\1\\1\\1]"


@pytest.fixture(params=["plain", "replay_launches", "replay"])
def env(request):
    from tenncor_amd import graph
    graph.set_evaluator(request.param)
    g = graph.Graph()
    try:
        yield g, graph.Api(g), graph
    finally:
        g.close()
        graph.set_evaluator("default")


def lines_of(text, shapes=True):
    out = [line.strip("_ \t") for line in text.split("\n")]
    if not shapes:
        out = [re.sub(r"\[[0-9\\]*\]\)$", ")", line) for line in out]
    return [line for line in out if line]


def test_assign_is_idempotent_and_not_derivable(env):
    g, api, graph = env
    target1 = g.variable(np.array(DATA, np.float64), SHAPE)
    target2 = g.variable(np.array(DATA, np.float64), SHAPE)
    src = g.constant(np.array(DATA2, np.float64), SHAPE)
    ass1 = api.assign(target1, src)
    ass2 = api.assign(target2, api.neg(src))
    for ass, target, sign in ((ass1, target1, 1.0), (ass2, target2, -1.0)):
        g.evaluate([ass])
        g.evaluate([ass])
        assert ass.shape[:3] == SHAPE and target.shape[:3] == SHAPE
        np.testing.assert_array_equal(target.get(), sign * np.array(DATA2, np.float64))
        np.testing.assert_array_equal(ass.get(), sign * np.array(DATA2, np.float64))
        with pytest.raises(graph.GraphError, match="cannot derive ASSIGN"):
            g.derive(ass, [src])


def test_assign_takes_the_type_of_its_target(env):
    from tenncor_amd import capi
    g, api, graph = env
    target1 = g.variable(np.array(DATA, np.float32), SHAPE, "target1")
    target2 = g.variable(np.array(DATA, np.float32), SHAPE, "target2")
    src = g.constant(np.array(DATA2, np.float64), SHAPE)
    ass1 = api.assign(target1, src)
    ass2 = api.assign(target2, api.neg(src))
    assert lines_of(g.to_string(ass1)) == [
        "(ASSIGN<FLOAT>%s)" % S,
        "`--(variable:target1<FLOAT>%s)" % S,
        "`--(CAST<FLOAT>%s)" % S,
        "`--(constant:[22\\15\\74\\38\\61\\...]<DOUBLE>%s)" % S]
    assert lines_of(g.to_string(ass2)) == [
        "(ASSIGN<FLOAT>%s)" % S,
        "`--(variable:target2<FLOAT>%s)" % S,
        "`--(CAST<FLOAT>%s)" % S,
        "`--(NEG<DOUBLE>%s)" % S,
        "`--(constant:[22\\15\\74\\38\\61\\...]<DOUBLE>%s)" % S]
    assert ass1.dtype == capi.FLOAT and ass2.dtype == capi.FLOAT
    for ass, target, sign in ((ass1, target1, 1.0), (ass2, target2, -1.0)):
        g.evaluate([ass])
        g.evaluate([ass])
        assert target.get().dtype == np.float32
        np.testing.assert_array_equal(target.get(), sign * np.array(DATA2, np.float32))
        np.testing.assert_array_equal(ass.get(), sign * np.array(DATA2, np.float32))


def test_cast_chain_is_not_cast_twice(env):
    from tenncor_amd import capi
    g, api, graph = env
    for data, shape in ((DATA, [2, 3, 4]), (DATA[:6], [3, 2])):
        src = g.constant(np.array(data, np.float64), shape)
        as_int = g.functor("CAST", [api.add(api.mul(api.unary("COS", src), 2.1), 4.5)], dtype=capi.INT32)
        out = g.functor("CAST", [api.div(as_int, 2)], dtype=capi.DOUBLE)
        assert lines_of(g.to_string(out), shapes=False) == [
            "(CAST<DOUBLE>)",
            "`--(DIV<INT32>)",
            "`--(CAST<INT32>)",
            "|___`--(ADD<DOUBLE>)",
            "|_______`--(MUL<DOUBLE>)",
            "|_______|___`--(COS<DOUBLE>)",
            "|_______|___|___`--(constant:[59\\10\\28\\10\\67\\...]<DOUBLE>)",
            "|_______|___`--(EXTEND<DOUBLE>)",
            "|_______|_______`--(constant:2.1<DOUBLE>)",
            "|_______`--(EXTEND<DOUBLE>)",
            "|___________`--(constant:4.5<DOUBLE>)",
            "`--(EXTEND<INT32>)",
            "`--(constant:2<INT32>)"]
        d = np.array(data, np.float64)
        g.evaluate([out])
        g.evaluate([out])
        expect = ((np.cos(d) * 2.1 + 4.5).astype(np.int32) // 2).astype(np.float64)
        np.testing.assert_array_equal(out.get(), expect)
        grad = g.functor("CAST", [g.derive(out, [src])[0]], dtype=capi.DOUBLE)
        g.evaluate([grad])
        np.testing.assert_allclose(grad.get(), -np.sin(d) * 2.1 / 2, rtol=1e-12, atol=1e-14)


def test_identity_runs_its_dependencies(env):
    g, api, graph = env
    for start in (np.array(DATA, np.float64), np.zeros(24)):
        target = g.variable(start, SHAPE)
        a = g.constant(np.array(DATA, np.float64), SHAPE)
        b = g.constant(np.array(DATA2, np.float64), SHAPE)
        c = api.add(a, b)
        ass = api.assign(target, api.identity(b, [c]))
        g.evaluate([ass])
        np.testing.assert_array_equal(target.get(), np.array(DATA2, np.float64))
        np.testing.assert_array_equal(ass.get(), np.array(DATA2, np.float64))
        np.testing.assert_array_equal(c.get(), np.array(DATA, np.float64) + np.array(DATA2, np.float64))


def test_ignored_nodes_keep_their_values(env):
    # EVALUATOR.UpdateIgnore (internal/teq/test/test_evaluator.cpp:75-144): the
    # walk does not enter an ignored node; its reader takes the value it holds
    g, api, graph = env
    one = np.ones(6)
    a, b, c, d = (g.variable(one * k, [3, 2], n) for k, n in ((1, "a"), (2, "b"), (3, "c"), (4, "d")))
    x = api.add(a, b)
    y = api.add(x, c)
    target = api.add(y, d)
    g.evaluate([target, y, x])
    np.testing.assert_array_equal(target.get(), one * 10)
    g.assign(a, one * 101)
    g.assign(c, one * 1003)
    y_version = g.version(y)
    g.evaluate_ignoring([target], [y])
    assert g.version(y) == y_version
    np.testing.assert_array_equal(target.get(), one * 10)   # stale y (6) + d
    g.assign(d, one * 10004)
    g.evaluate_ignoring([target], [x])
    np.testing.assert_array_equal(target.get(), one * (3 + 1003 + 10004))  # stale x (3)


def test_ignored_node_with_a_shared_operand(env):
    # EVALUATOR.UpdateIgnoreCommonDesc (test_evaluator.cpp:147-207): u is read by
    # the ignored y and by x; u and x are computed, y is not
    g, api, graph = env
    one = np.ones(6)
    a, b, c = (g.variable(one * k, [3, 2], n) for k, n in ((1, "a"), (20, "b"), (300, "c")))
    u = api.neg(a)
    x = api.add(u, b)
    y = api.add(c, u)
    target = api.add(y, x)
    g.evaluate([target, y, x, u])
    np.testing.assert_array_equal(target.get(), one * (299 + 19))
    g.assign(a, one * 5)
    g.evaluate_ignoring([target], [y])
    np.testing.assert_array_equal(target.get(), one * (299 + 15))
    np.testing.assert_array_equal(u.get(), one * -5)
