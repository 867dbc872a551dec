"""Graph clean-up on the host (no GPU): the rule reader, pattern matching with
symbols and commutative operands, rewriting in place, and the merging of equal
subgraphs.  The semantics follow tenncor/hone/optimize.hpp:19-38,
tenncor/hone/duplicates.hpp:13-101, internal/opt/src/parse.cpp:9-76 and the
matcher of internal/query/querier.hpp:27-53,186-303; the reference's own rule
file (cfg/optimizations.json) is a git-lfs pointer without content, so the
expected graphs below are worked out from those semantics by hand.
"""
import json

import numpy as np
import pytest


@pytest.fixture()
def g():
    from tenncor_amd import graph
    gr = graph.Graph()
    yield gr
    gr.close()


def var(g, label, shape=(3, 2), dtype=np.float32):
    n = int(np.prod(shape))
    return g.variable(np.arange(n, dtype=dtype), list(shape), label)


def full(g, value, shape=(3, 2), dtype=np.float32):
    return g.constant(np.full(int(np.prod(shape)), value, dtype=dtype), list(shape))


def rule(srcs, dest):
    return json.dumps({"conversions": [{"srcs": srcs, "dest": dest}]})


def op(name, *args, **extra):
    body = {"opname": name, "args": list(args)}
    body.update(extra)
    return {"op": body}


X, Y = {"symb": "X"}, {"symb": "Y"}
SHAPE = "[3\\2\\1\\1\\1\\1\\1\\1]"


def test_shipped_rules_parse_and_simplify_a_chain(g):
    x, y = var(g, "x"), var(g, "y")
    a = g.functor("MUL", [x, full(g, 1)])
    b = g.functor("ADD", [full(g, 0), a])
    c = g.functor("NEG", [g.functor("NEG", [b])])
    d = g.functor("ADD", [c, g.functor("NEG", [y])])
    (out,), stats = g.optimize([d], fold=False)
    assert g.to_string(out) == (
        "(SUB<FLOAT>%s)\n_`--(variable:x<FLOAT>%s)\n_`--(variable:y<FLOAT>%s)" % (SHAPE, SHAPE, SHAPE))
    assert stats["converted"] == 4 and stats["folded"] == 0


def test_scalar_patterns_match_constants_of_equal_elements_only(g):
    x = var(g, "x")
    ramp = g.constant(np.array([1, 1, 1, 1, 1, 2], np.float32), [3, 2])
    kept = g.functor("MUL", [x, ramp])
    gone = g.functor("MUL", [full(g, 1), x])  # commutative: the constant may come first
    rules = rule([op("MUL", X, {"cst": 1})], X)
    (a, b), stats = g.optimize([kept, gone], rules, fold=False)
    assert a.id == kept.id and g.opcode(a) == "MUL"
    assert b.id == x.id
    assert stats["converted"] == 1


def test_operands_of_other_opcodes_match_in_order(g):
    x = var(g, "x")
    zero = full(g, 0)
    rules = rule([op("SUB", {"cst": 0}, X)], op("NEG", X))
    (a, b), _ = g.optimize([g.functor("SUB", [zero, x]), g.functor("SUB", [x, zero])], rules, fold=False)
    assert g.opcode(a) == "NEG" and g.args(a)[0].id == x.id
    assert g.opcode(b) == "SUB"


def test_a_symbol_binds_one_node(g):
    x, y = var(g, "x"), var(g, "y")
    rules = rule([op("MUL", X, X)], op("SQUARE", X))
    (a, b), _ = g.optimize([g.functor("MUL", [x, x]), g.functor("MUL", [x, y])], rules, fold=False)
    assert g.opcode(a) == "SQUARE"
    assert g.opcode(b) == "MUL"


def test_operand_counts_must_agree(g):
    # the reference's matcher accepts functors with more operands than the pattern
    # lists (internal/query/querier.hpp:195-196), so ADD(X, 0) -> X would drop y
    x, y = var(g, "x"), var(g, "y")
    three = g.functor("ADD", [x, y, full(g, 0)])
    (out,), stats = g.optimize([three], rule([op("ADD", X, {"cst": 0})], X), fold=False)
    assert out.id == three.id and stats["converted"] == 0


def test_scalar_targets_take_shape_and_dtype_of_their_symbol(g):
    x = var(g, "x", dtype=np.int32)
    prod = g.functor("MUL", [x, full(g, 0, dtype=np.int32)])
    (out,), _ = g.optimize([g.functor("ADD", [prod, x]), ][:1], rule([op("MUL", X, {"cst": 0})], {"cst": {"value": 0, "shape": "X"}}), fold=False)
    zero = g.args(out)[0]
    assert g.to_string(zero) == "(constant:0<INT32>%s)" % SHAPE


def test_attributes_and_captures(g):
    x = var(g, "x")
    inner = g.functor("REDUCE_SUM", [x], rank_set=[0])
    other = g.functor("REDUCE_SUM", [x], rank_set=[1])
    srcs = [op("NEG", op("REDUCE_SUM", X, attrs={"rank_set": {"iarr": {"values": [0]}}}, capture="R"))]
    (a, b), _ = g.optimize([g.functor("NEG", [inner]), g.functor("NEG", [other])], rule(srcs, {"symb": "R"}), fold=False)
    assert a.id == inner.id
    assert g.opcode(b) == "NEG"


def test_functor_targets_carry_attributes(g):
    x = var(g, "x")
    rules = rule([op("ABS", X)], op("EXTEND", op("REDUCE_SUM", X, attrs={"rank_set": {"iarr": {"values": [1]}}}),
                                    attrs={"dimensions": {"iarr": {"values": [1, 2]}}}))
    (out,), _ = g.optimize([g.functor("NEG", [g.functor("ABS", [x])])], rules, fold=False)
    ext = g.args(out)[0]
    red = g.args(ext)[0]
    assert g.opcode(ext) == "EXTEND" and ext.shape[:2] == [3, 2]
    assert g.opcode(red) == "REDUCE_SUM" and red.shape[:2] == [3, 1]


def test_leaf_patterns(g):
    x, y = var(g, "x"), var(g, "y", dtype=np.float32)
    rules = rule([op("NEG", {"leaf": {"label": "x", "usage": "variable", "dtype": "FLOAT", "shape": [3, 2]}}, capture="R")],
                 op("ABS", {"symb": "R"}))
    (a, b), _ = g.optimize([g.functor("SIN", [g.functor("NEG", [x])]), g.functor("SIN", [g.functor("NEG", [y])])], rules, fold=False)
    assert g.opcode(g.args(a)[0]) == "ABS"
    assert g.opcode(g.args(b)[0]) == "NEG"


def test_equal_subgraphs_become_one_node(g):
    x, y = var(g, "x"), var(g, "y")
    left = g.functor("MUL", [g.functor("SIN", [x]), y])
    right = g.functor("MUL", [y, g.functor("SIN", [x])])  # commutative: operand order is ignored
    sub1, sub2 = g.functor("SUB", [x, y]), g.functor("SUB", [y, x])
    root = g.functor("ADD", [left, right, sub1, sub2])
    assert g.count_functors([root]) == 7
    (out,), stats = g.optimize([root], None, fold=False)
    assert g.count_functors([out]) == 5 and stats["merged"] == 2
    args = g.args(out)
    assert args[0].id == args[1].id and args[2].id != args[3].id


def test_equal_constants_merge_but_variables_and_attributes_keep_nodes_apart(g):
    x = var(g, "x")
    twin = var(g, "x")
    a = g.functor("ADD", [x, full(g, 2)])
    b = g.functor("ADD", [x, full(g, 2)])
    c = g.functor("ADD", [twin, full(g, 2)])
    r0 = g.functor("REDUCE_SUM", [x], rank_set=[0])
    r1 = g.functor("REDUCE_SUM", [x], rank_set=[1])
    (oa, ob, oc, o0, o1), stats = g.optimize([a, b, c, r0, r1], None, fold=False)
    assert oa.id == ob.id and oa.id != oc.id and o0.id != o1.id
    assert g.args(oa)[1].id == g.args(oc)[1].id
    assert stats["merged"] == 3  # two constants and one ADD


MALFORMED = [
    ("{", "malformed json"),
    ("[1, 2]", "failed to parse json optimization"),
    ('{"conversions": [{"srcs": [{"op": {"opname": "NOPE", "args": []}}], "dest": {"symb": "X"}}]}', "NOPE"),
    ('{"conversions": [{"srcs": [{"symb": "X"}], "dest": {"symb": "Y"}}]}', "does not bind"),
    ('{"conversions": [{"srcs": [{"what": 1}], "dest": {"symb": "X"}}]}', "unknown node"),
    ('{"conversions": [{"srcs": [{"symb": "X"}]}]}', "dest"),
]


@pytest.mark.parametrize("text,message", MALFORMED, ids=[m[1] for m in MALFORMED])
def test_malformed_rules_are_rejected(g, text, message):
    from tenncor_amd import graph
    x = var(g, "x")
    with pytest.raises(graph.GraphError, match=message):
        g.optimize([g.functor("NEG", [x])], text, fold=False)


def test_mismatched_replacement_is_refused(g):
    from tenncor_amd import graph
    x = var(g, "x")
    root = g.functor("NEG", [g.functor("ABS", [x])])
    bad = rule([op("ABS", X)], op("REDUCE_SUM", X, attrs={"rank_set": {"iarr": {"values": [0]}}}))
    with pytest.raises(graph.GraphError, match="incompatible shape"):
        g.optimize([root], bad, fold=False)
