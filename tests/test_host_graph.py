"""Host graph layer without a GPU: node construction, shape / type / elision
rules (cfg/ops.yml), automatic casts, the gradient builder's output graphs and
the reference's error messages.  Nothing here evaluates a node."""
import numpy as np
import pytest


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


def var(g, shape, dtype=np.float32, label="x"):
    n = int(np.prod(shape))
    return g.variable(np.arange(n, dtype=dtype), shape, label)


def test_library_exports_every_declared_symbol():
    import ctypes
    import os
    import re
    from tenncor_amd import graph
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(root, "include", "tcgraph.h")).read(), flags=re.S)
    declared = sorted(set(re.findall(r"\b(tcr_[a-z0-9_]+)\s*\(", text)))
    assert declared == sorted(graph.EXPORTS)
    lib = ctypes.CDLL(graph.LIB_PATH)
    assert not [s for s in declared if not hasattr(lib, s)]


# internal/eigen/test/test_shaper.cpp:21-437 -- (op, arg shapes, attrs, expected shape)
SHAPE_CASES = [
    ("ADD", [[3, 2], [3, 2]], {}, [3, 2]),
    ("REDUCE_SUM", [[3, 2, 4]], {"rank_set": [1]}, [3, 1, 4]),
    ("REDUCE_MAX", [[3, 2, 4]], {"rank_set": [0, 2]}, [1, 2, 1]),
    ("ARGMAX", [[3, 2, 4]], {"rank": 1}, [3, 1, 4]),
    ("ARGMAX", [[3, 2, 4]], {"rank": 8}, [1]),
    ("PERMUTE", [[3, 2, 4]], {"ranks": [2, 0, 1]}, [4, 3, 2]),
    ("PERMUTE", [[3, 2, 4]], {"ranks": [1, 0]}, [2, 3, 4]),
    ("EXTEND", [[3, 1, 2]], {"dimensions": [1, 4]}, [3, 4, 2]),
    ("RESHAPE", [[3, 2, 4]], {"shape": [6, 4]}, [6, 4]),
    ("SLICE", [[3, 2]], {"dimension_pairs": [1, 2, 1, 1]}, [2, 1]),
    ("SLICE", [[3, 2]], {"dimension_pairs": [1, 200]}, [2, 2]),
    ("PAD", [[2, 3]], {"dimension_pairs": [1, 1]}, [4, 3]),
    ("STRIDE", [[2, 3]], {"dimensions": [1, 2]}, [2, 2]),
    ("SCATTER", [[2, 2]], {"dimensions": [2, 2], "shape": [3, 3, 1, 1, 1, 1, 1, 1]}, [3, 3]),
    ("MATMUL", [[4, 3], [2, 4]], {}, [2, 3]),
    ("MATMUL", [[4, 3, 5], [2, 4, 5]], {}, [2, 3, 5]),
    ("CONTRACT", [[4, 3], [2, 4]], {"rank_pairs": [0, 1]}, [2, 3]),
    ("CONTRACT", [[4, 2, 3], [2, 4, 2]], {"rank_pairs": [0, 1, 1, 2]}, [2, 3]),
    ("CONTRACT", [[768, 1, 256], [2048, 768]], {"rank_pairs": [0, 1]}, [2048, 1, 256]),
    ("CONV", [[3, 3], [2]], {"ranks": [1]}, [3, 2]),
    ("CONV", [[4, 10, 9, 2, 5], [3, 4, 5, 6]], {"ranks": [4, 0, 1, 2]}, [1, 6, 4, 2, 3]),
    ("CONCAT", [[2, 3], [1, 3]], {"rank": 0}, [3, 3]),
    ("CONCAT", [[1, 4], [1, 4], [1, 4]], {"rank": 0}, [3, 4]),
    ("SELECT", [[2, 3], [2, 3], [2, 3]], {}, [2, 3]),
]


@pytest.mark.parametrize("op,shapes,attrs,expect", SHAPE_CASES, ids=[c[0] + str(c[1]) for c in SHAPE_CASES])
def test_shape_rules(g, op, shapes, attrs, expect):
    from tenncor_amd import capi
    args = [var(g, s) for s in shapes]
    out = g.functor(op, args, **attrs)
    assert out.shape == capi.shape8(expect)


ERROR_CASES = [
    ("ADD", [[3, 2], [2, 3]], {}, "cannot ADD with incompatible shapes"),
    ("PERMUTE", [[3, 2]], {"ranks": [1, 1]}, "permute does not support repeated orders"),
    ("EXTEND", [[3, 2]], {"dimensions": [2]}, "cannot extend non-singular dimension 0"),
    ("EXTEND", [[1, 2]], {"dimensions": [0]}, "cannot extend using zero dimensions"),
    ("RESHAPE", [[3, 2]], {"shape": [5]}, "cannot RESHAPE with shapes of different sizes"),
    ("SLICE", [[3, 2]], {"dimension_pairs": [0, 0]}, "cannot create slice with 0 dimensions"),
    ("MATMUL", [[4, 3], [2, 5]], {}, "have mismatch common dimension 0,1"),
    ("MATMUL", [[4, 3, 2], [2, 4, 3]], {}, "do not match for dimensions 2+"),
    ("CONTRACT", [[4, 3], [2, 5]], {"rank_pairs": [0, 1]}, "do not match common dimensions"),
    ("CONTRACT", [[4, 4], [4, 4]], {"rank_pairs": [0, 1, 0, 0]}, "must be unique for each side"),
    ("CONV", [[3, 3], [2, 2]], {"ranks": [1]}, "cannot have ambiguous ranks not specified in kernelshape"),
    ("CONV", [[3, 3], [5]], {"ranks": [1]}, "cannot convolve a kernel of shape"),
    ("CONCAT", [[2, 3], [2, 4]], {"rank": 0}, "cannot group concat incompatible shapes"),
    ("CONCAT", [[2, 3], [2, 3], [2, 3]], {"rank": 0}, "cannot group concat shapes with dimension that is not one"),
    ("REDUCE_SUM", [[3, 2]], {}, "cannot find `rank_set` attribute"),
]


@pytest.mark.parametrize("op,shapes,attrs,message", ERROR_CASES, ids=[c[0] + ":" + c[3][:24] for c in ERROR_CASES])
def test_construction_errors_carry_the_reference_messages(g, op, shapes, attrs, message):
    from tenncor_amd import graph
    args = [var(g, s) for s in shapes]
    with pytest.raises(graph.GraphError) as info:
        g.functor(op, args, **attrs)
    assert message in str(info.value)


def test_redundant_nodes_are_elided(g):
    """cfg/ops.yml FuncOpt: the first child stands in for the node."""
    x = var(g, [3, 2, 4])
    assert g.functor("REDUCE_SUM", [x], rank_set=[]).id == x.id
    assert g.functor("PERMUTE", [x], ranks=[0, 1, 2]).id == x.id
    assert g.functor("PERMUTE", [x], ranks=[]).id == x.id
    assert g.functor("EXTEND", [x], dimensions=[1, 1]).id == x.id
    assert g.functor("RESHAPE", [x], shape=[3, 2, 4, 1, 1, 1, 1, 1]).id == x.id
    assert g.functor("SLICE", [x], dimension_pairs=[0, 65535, 0, 65535]).id == x.id
    assert g.functor("SLICE", [x], dimension_pairs=[0, 3]).id != x.id  # extent must exceed the dim
    assert g.functor("PAD", [x], dimension_pairs=[0, 0, 0, 0]).id == x.id
    assert g.functor("ADD", [x]).id == x.id
    assert g.functor("ARGMAX", [var(g, [3, 1])], rank=1).id != x.id
    y = var(g, [3, 1])
    assert g.functor("ARGMAX", [y], rank=1).id == y.id
    from tenncor_amd import capi
    assert g.functor("CAST", [x], dtype=capi.FLOAT).id == x.id


def test_type_rule_and_automatic_casts(g):
    """cfg/ops.yml:44-62 + tenncor/eteq/caster.hpp: the node takes the most
    precise child dtype; other children get a CAST in front."""
    from tenncor_amd import capi
    f = var(g, [2, 2], np.float32, "f")
    i = var(g, [2, 2], np.int32, "i")
    d = var(g, [2, 2], np.float64, "d")
    out = g.functor("ADD", [i, f])
    assert out.dtype == capi.FLOAT
    a0, a1 = g.args(out)
    assert g.opcode(a0) == "CAST" and a0.dtype == capi.FLOAT and g.args(a0)[0].id == i.id
    assert a1.id == f.id
    out = g.functor("MUL", [f, d, i])
    assert out.dtype == capi.DOUBLE
    assert [g.opcode(a) for a in g.args(out)] == ["CAST", "BAD_OP", "CAST"]
    # ASSIGN takes the target's dtype (cfg/ops.yml:656-664)
    out = g.functor("ASSIGN_SUB", [f, d])
    assert out.dtype == capi.FLOAT and g.opcode(g.args(out)[1]) == "CAST"
    c = g.functor("CAST", [f], dtype=capi.INT32)
    assert c.dtype == capi.INT32


def test_dense_and_conv2d_lower_like_the_reference(g, api):
    """Graph dumps of tenncor/test/test_api.cpp:2433-2446 and :2519-2529."""
    x = g.variable(np.zeros(12, np.float32), [6, 2], "x")
    weight = g.variable(np.zeros(30, np.float32), [5, 6], "weight")
    bias = g.variable(np.zeros(5, np.float32), [5], "bias")
    y = api.dense(x, weight, bias)
    assert g.to_string(y) == (
        "(IDENTITY<FLOAT>[5\\2\\1\\1\\1\\1\\1\\1])\n"
        "_`--(ADD<FLOAT>[5\\2\\1\\1\\1\\1\\1\\1])\n"
        "_____`--(CONTRACT<FLOAT>[5\\2\\1\\1\\1\\1\\1\\1])\n"
        "_____|___`--(variable:x<FLOAT>[6\\2\\1\\1\\1\\1\\1\\1])\n"
        "_____|___`--(variable:weight<FLOAT>[5\\6\\1\\1\\1\\1\\1\\1])\n"
        "_____`--(EXTEND<FLOAT>[5\\2\\1\\1\\1\\1\\1\\1])\n"
        "_________`--(variable:bias<FLOAT>[5\\1\\1\\1\\1\\1\\1\\1])")
    x = g.variable(np.zeros(4 * 10 * 9 * 2, np.float32), [4, 10, 9, 2], "x")
    weight = g.variable(np.zeros(3 * 4 * 5 * 6, np.float32), [3, 4, 5, 6], "weight")
    bias = g.variable(np.zeros(3, np.float32), [3], "bias")
    y = api.identity(api.conv2d(x, weight, bias))
    assert g.to_string(y) == (
        "(IDENTITY<FLOAT>[3\\6\\4\\2\\1\\1\\1\\1])\n"
        "_`--(ADD<FLOAT>[3\\6\\4\\2\\1\\1\\1\\1])\n"
        "_____`--(PERMUTE<FLOAT>[3\\6\\4\\2\\1\\1\\1\\1])\n"
        "_____|___`--(CONV<FLOAT>[1\\6\\4\\2\\3\\1\\1\\1])\n"
        "_____|_______`--(PAD<FLOAT>[4\\10\\9\\2\\5\\1\\1\\1])\n"
        "_____|_______|___`--(variable:x<FLOAT>[4\\10\\9\\2\\1\\1\\1\\1])\n"
        "_____|_______`--(REVERSE<FLOAT>[3\\4\\5\\6\\1\\1\\1\\1])\n"
        "_____|___________`--(variable:weight<FLOAT>[3\\4\\5\\6\\1\\1\\1\\1])\n"
        "_____`--(EXTEND<FLOAT>[3\\6\\4\\2\\1\\1\\1\\1])\n"
        "_________`--(variable:bias<FLOAT>[3\\1\\1\\1\\1\\1\\1\\1])")


S32 = "[3\\2\\1\\1\\1\\1\\1\\1]"


def test_gradient_graphs_match_the_reference_structure(g, api):
    """tenncor/eteq/test/test_backprop.cpp:201-228 (Sigmoid, Tanh), :435-459
    (Contract) and :462-485 (Conv): the same trees with the upstream gradient
    being the all-ones seed of teq::derive."""
    arg = g.variable(np.arange(6, dtype=np.float64) + 1, [3, 2], "arg1")
    op = api.sigmoid(arg)
    (grad,) = g.derive(op, [arg])
    assert g.to_string(grad) == (
        "(MUL<DOUBLE>%s)\n"
        "_`--(MUL<DOUBLE>%s)\n"
        "_|___`--(SIGMOID<DOUBLE>%s)\n"
        "_|___|___`--(variable:arg1<DOUBLE>%s)\n"
        "_|___`--(SUB<DOUBLE>%s)\n"
        "_|_______`--(EXTEND<DOUBLE>%s)\n"
        "_|_______|___`--(constant:1<DOUBLE>[1\\1\\1\\1\\1\\1\\1\\1])\n"
        "_|_______`--(SIGMOID<DOUBLE>%s)\n"
        "_|___________`--(variable:arg1<DOUBLE>%s)\n"
        "_`--(constant:1<DOUBLE>%s)") % ((S32,) * 9)
    op = api.tanh(arg)
    (grad,) = g.derive(op, [arg])
    assert g.to_string(grad) == (
        "(MUL<DOUBLE>%s)\n"
        "_`--(SUB<DOUBLE>%s)\n"
        "_|___`--(EXTEND<DOUBLE>%s)\n"
        "_|___|___`--(constant:1<DOUBLE>[1\\1\\1\\1\\1\\1\\1\\1])\n"
        "_|___`--(SQUARE<DOUBLE>%s)\n"
        "_|_______`--(TANH<DOUBLE>%s)\n"
        "_|___________`--(variable:arg1<DOUBLE>%s)\n"
        "_`--(constant:1<DOUBLE>%s)") % ((S32,) * 7)
    a1 = g.variable(np.arange(6, dtype=np.float64), [3, 2], "arg1")
    a2 = g.variable(np.arange(6, dtype=np.float64), [2, 3], "arg2")
    op = api.contract(a1, a2)
    (grad,) = g.derive(op, [a2])
    assert g.to_string(grad) == (
        "(PERMUTE<DOUBLE>[2\\3\\1\\1\\1\\1\\1\\1])\n"
        "_`--(CONTRACT<DOUBLE>[3\\2\\1\\1\\1\\1\\1\\1])\n"
        "_____`--(constant:1<DOUBLE>[2\\2\\1\\1\\1\\1\\1\\1])\n"
        "_____`--(variable:arg1<DOUBLE>[3\\2\\1\\1\\1\\1\\1\\1])")
    img = g.variable(np.arange(6, dtype=np.float64), [3, 2], "arg1")
    ker = g.variable(np.arange(4, dtype=np.float64), [2, 2], "arg2")
    op = api.convolution(img, ker, [0, 1])
    (grad,) = g.derive(op, [ker])
    assert g.to_string(grad) == (
        "(CONV<DOUBLE>[2\\2\\1\\1\\1\\1\\1\\1])\n"
        "_`--(variable:arg1<DOUBLE>[3\\2\\1\\1\\1\\1\\1\\1])\n"
        "_`--(constant:1<DOUBLE>[2\\1\\1\\1\\1\\1\\1\\1])")


def test_derive_of_unrelated_and_self(g, api):
    x = var(g, [3, 2], np.float64, "x")
    y = var(g, [3, 2], np.float64, "y")
    op = api.exp(x)
    gx, gy, gself = g.derive(op, [x, y, op])
    assert g.opcode(gx) == "MUL"
    assert g.opcode(gy) == "BAD_OP" and g.to_string(gy).startswith("(constant:0<DOUBLE>")
    assert g.to_string(gself).startswith("(constant:1<DOUBLE>")
    from tenncor_amd import graph
    with pytest.raises(graph.GraphError) as info:
        g.derive(g.functor("ARGMAX", [x], rank=0), [x])
    assert "cannot derive ARGMAX" in str(info.value)


def test_mlp_gradient_graph_only_uses_table_opcodes(g, api):
    """config 1: the GradBuilder's output is an ordinary graph over ops.yml opcodes."""
    rng = np.random.default_rng(1)
    x = g.variable(rng.uniform(-1, 1, 30), [10, 3], "x")
    w0 = g.variable(rng.uniform(-1, 1, 90), [9, 10], "w0")
    b0 = g.variable(np.zeros(9), [9], "b0")
    sig0 = api.sigmoid(api.add(api.matmul(x, w0), api.extend(b0, 1, [3])))
    err = api.square(sig0)
    grads = g.derive(err, [w0, b0])
    seen, stack, ops = set(), list(grads), set()
    while stack:
        n = stack.pop()
        if n.id in seen:
            continue
        seen.add(n.id)
        ops.add(g.opcode(n))
        stack.extend(g.args(n))
    assert ops <= {"BAD_OP", "MUL", "SUB", "EXTEND", "SIGMOID", "ADD", "MATMUL", "PERMUTE", "REDUCE_SUM", "SQUARE"}
    assert grads[0].shape[:2] == [9, 10] and grads[1].shape[:2] == [9, 1]


# ---- launch planning of the replaying evaluator (host logic only) -------------

def parse_plan(lines, batches=None):
    """batches: a list that receives (index of the first step, number of steps) for every run
    of small steps that goes out as one launch"""
    steps = []
    for line in lines:
        if line.startswith("batch "):
            if batches is not None:
                batches.append((len(steps), int(line.split(" ")[1])))
            continue
        if line.startswith("padded "):
            continue
        product, marker, epilogue = line.partition(" with epilogue ")
        if marker:
            # a product and the group that reads it as one launch: both steps, the first one flagged
            kind, _, rest = product.partition(" ")
            steps.append((kind, rest.split(" ")[0].split("+"), {"epilogue": 1}))
            line = epilogue
        kind, _, rest = line.partition(" ")
        if kind == "node":
            steps.append(("node", [rest], {}))
        elif kind == "group":
            ops, *fields = rest.split(" ")
            steps.append(("group", ops.split("+"), {k: int(v) for k, v in (f.split("=") for f in fields)}))
        elif kind in ("swapped", "viewed", "summed", "parts", "blocks"):
            steps.append((kind, rest.split(" ")[0].split("+"), {}))
        else:
            steps.append(("folded", [], {"n": int(rest)}))
    return steps


def test_launch_plan_groups_the_elementwise_nodes_of_an_mlp(g):
    from tenncor_amd import configs
    targets, _, _ = configs.config1_mlp(g)
    steps = parse_plan(g.launch_plan(targets))
    launches = [s for s in steps if s[0] != "folded"]
    folded = steps[-1][2]["n"]
    nfunc = g.count_functors(targets)
    # every functor is launched on its own, computed inside a group, or folded into operand views
    in_groups = sum(len(s[1]) for s in launches if s[0] == "group")
    stores = sum(s[2]["stores"] for s in launches if s[0] == "group")
    alone = sum(1 for s in launches if s[0] in ("node", "swapped"))
    assert alone + stores + folded == nfunc
    assert len(launches) < nfunc // 2
    assert any(s[0] == "group" and "SIGMOID" in s[1] and len(s[1]) >= 3 for s in launches)
    # the matrix products and reductions keep their own kernels
    # ... except that the transposed products of the weight gradients are launched as one product
    assert sum(1 for s in launches if s[0] == "node" and s[1][0] in ("CONTRACT", "MATMUL")) == 3
    assert sum(1 for s in launches if s[0] == "swapped") == 2 and "node PERMUTE" not in g.launch_plan(targets)
    for s in launches:
        if s[0] == "group":
            assert s[2]["leaves"] <= 8 and s[2]["stores"] <= 8 and s[2]["instrs"] <= 64


def test_launch_plan_keeps_a_launch_between_two_groups_in_order(g, api):
    """t feeds a matmul whose result comes back into elementwise nodes that also
    read t: the two elementwise parts cannot share a launch."""
    x = var(g, [6, 4], np.float32, "x")
    w = var(g, [6, 6], np.float32, "w")
    s = api.add(x, 1.0)
    t = api.mul(api.square(s), api.neg(s))
    m = api.matmul(t, w)
    u = api.sub(api.add(t, m), api.mul(s, 2.0))
    steps = [st for st in parse_plan(g.launch_plan([u])) if st[0] != "folded"]
    kinds = [(k, ops) for k, ops, _ in steps]
    mm = next(i for i, (k, ops) in enumerate(kinds) if k == "node" and ops == ["MATMUL"])
    before = [ops for k, ops in kinds[:mm] if k == "group"]
    after = [ops for k, ops in kinds[mm + 1:] if k == "group"]
    assert any("SQUARE" in ops and "NEG" in ops for ops in before)
    assert any("SUB" in ops for ops in after)
    assert all("SUB" not in ops for ops in before)
    # s and t are read on both sides of the product: both are stored by the first group
    first = next(st for st in steps if st[0] == "group")
    assert first[2]["stores"] == 2


def test_launch_plan_folds_views_and_splits_oversized_groups(g, api):
    x = var(g, [8, 4], np.float32, "x")
    b = var(g, [8], np.float32, "b")
    wide = var(g, [16, 4], np.float32, "wide")
    # EXTEND, SLICE and PAD in front of elementwise nodes never get a launch
    y = api.add(api.mul(x, api.extend(b, 1, [4])), api.slice(wide, 4, 8, 0))
    z = api.add(api.pad(api.slice(y, 1, 6, 0), [[1, 1]]), x)
    lines = g.launch_plan([z])
    assert all(not l.startswith("node") for l in lines[:-1]), lines
    assert parse_plan(lines)[-1][2]["n"] >= 4
    # ... but a view read by a matrix product is materialised
    m = api.matmul(api.slice(wide, 4, 8, 0), var(g, [3, 8], np.float32, "w"))
    assert "node SLICE" in g.launch_plan([m])
    # a chain longer than one launch's program is cut into several launches
    deep = x
    for k in range(150):
        deep = api.add(api.mul(deep, x), float(k + 1))
    steps = [s for s in parse_plan(g.launch_plan([deep])) if s[0] == "group"]
    assert len(steps) >= 5 and sum(len(s[1]) for s in steps) == 300
    assert all(s[2]["instrs"] <= 64 for s in steps)
    # twenty results of one group: more than one launch stores
    outs = [api.mul(z, float(k + 2)) for k in range(20)]
    steps = [s for s in parse_plan(g.launch_plan(outs)) if s[0] == "group"]
    assert sum(s[2]["stores"] for s in steps) >= 20 and all(s[2]["stores"] <= 16 for s in steps) and len(steps) >= 2


def test_launch_plan_reads_the_operand_of_a_pad_that_only_convolutions_read(g, api):
    x = var(g, [2, 6, 5, 3], np.float32, "x")        # {C, W, H, B}
    k = var(g, [4, 2, 3, 2], np.float32, "k")        # {O, C, KW, KH}
    y = api.conv2d(x, k)
    loss = api.reduce_sum(api.square(y))
    dx, dk = g.derive(loss, [x, k])
    lines = g.launch_plan([loss, dx, dk])
    # forward (reads x where PAD would put it and the kernel through its REVERSE, writes what
    # PERMUTE would make of the result), kernel gradient (reads PAD(x) too, and the upstream
    # gradient through its PERMUTE; the PERMUTE and REVERSE behind it are where it writes) and
    # image gradient (reads the upstream gradient through PERMUTE and PAD, the kernel through
    # both REVERSEs; only one index of its result is sliced back out)
    assert lines.count("viewed PAD+REVERSE+CONV+PERMUTE") == 1
    assert lines.count("viewed PAD+PERMUTE+CONV+PERMUTE+REVERSE") == 1
    assert lines.count("viewed PERMUTE+PAD+REVERSE+REVERSE+CONV+SLICE") == 1
    for op in ("PAD", "CONV", "PERMUTE", "REVERSE"):
        assert "node " + op not in lines
    steps = parse_plan(lines)
    alone = sum(1 for s in steps if s[0] in ("node", "swapped", "viewed"))
    stores = sum(s[2]["stores"] for s in steps if s[0] == "group")
    assert alone + stores + steps[-1][2]["n"] == g.count_functors([loss, dx, dk])
    # a padded image somebody else reads, or asks for, is laid out as before
    padded = g.args(g.args(y)[0])[0]
    assert g.opcode(padded) == "PAD"
    lines = g.launch_plan([y, padded])
    # (the kernel is still read through its REVERSE and the result written as the PERMUTE wants it)
    assert "node PAD" in lines and "viewed REVERSE+CONV+PERMUTE" in lines and "node CONV" not in lines


def test_launch_plan_keeps_reads_of_a_variable_on_their_side_of_an_assignment(g, api):
    """ASSIGN* rewrites its target's buffer in place (internal/eigen/device.hpp:508-544).
    In the walk's children-first order NEG(v) runs before the ASSIGN and MUL(NEG, v)
    after it, so the two cannot share a launch, although MUL reads NEG and both are
    elementwise nodes of one shape."""
    v = var(g, [6, 4], np.float32, "v")
    c = var(g, [6, 4], np.float32, "c")
    x = api.neg(v)
    a = api.assign(v, c)
    y = api.mul(x, v)
    t = api.add(api.add(x, a), y)
    lines = [l for l in g.launch_plan([t]) if not l.startswith("folded")]
    steps = parse_plan(lines)
    at = next(i for i, s in enumerate(steps) if s[1] == ["ASSIGN"])
    before = [op for s in steps[:at] for op in s[1]]
    after = [op for s in steps[at + 1:] for op in s[1]]
    assert before == ["NEG"], lines
    assert sorted(after) == ["ADD", "ADD", "MUL"], lines

    # a view of the variable that is laid out before the assignment and read after it
    # keeps the old value: it is not folded into the launch that reads it
    w = var(g, [6], np.float32, "w")
    d = var(g, [6], np.float32, "d")
    wide = api.extend(w, 1, [4])
    upd = api.assign_add(w, api.mul(api.reduce_sum(api.neg(wide), 1, 1), d))
    late = api.add(api.extend(upd, 1, [4]), api.mul(wide, c))
    lines = g.launch_plan([late])
    assert "node EXTEND" in lines, lines
    steps = parse_plan([l for l in lines if not l.startswith("folded")])
    assert steps[0][1] == ["EXTEND"], lines
    names = [s[1] for s in steps]
    assert names.index(["ASSIGN_ADD"]) < next(i for i, n in enumerate(names) if "MUL" in n and "ADD" in n), lines
    # when every reader of the view comes before the assignment, it is folded as usual
    early = api.add(api.mul(api.extend(w, 1, [4]), c), api.extend(api.assign_add(w, d), 1, [4]))
    lines = g.launch_plan([early])
    assert "node EXTEND" not in lines and lines.index("node ASSIGN_ADD") == 1, lines
    # ... and without an assignment in between the same view is folded
    plain = api.add(api.mul(api.extend(w, 1, [4]), c), c)
    assert "node EXTEND" not in g.launch_plan([plain])

    # two assignments to one variable keep their order, readers in between stay in between
    first = api.assign(v, c)
    mid = api.square(api.identity(first))
    second = api.assign_sub(v, mid)
    tail = api.add(api.neg(second), mid)
    steps = parse_plan([l for l in g.launch_plan([tail]) if not l.startswith("folded")])
    names = [s[1] for s in steps]
    i1, i2 = names.index(["ASSIGN"]), names.index(["ASSIGN_SUB"])
    assert i1 < i2
    assert any("SQUARE" in n for n in names[i1 + 1:i2]) and any("NEG" in n for n in names[i2 + 1:])


def test_launch_plan_multiplies_the_parts_of_concatenations(g, api):
    """The products of an unrolled recurrent layer (cfg/tenncor/layer.yml:716-768 and
    its gradient, tenncor/eteq/backprop.hpp:269-359) read concatenations: [x_t, h] in
    the step itself, the ADD of the four PADded gate gradients on the way back, both
    again in the weight gradient.  A concatenation only products read is never laid
    out: a product over the joined dim runs as a sum of products over the parts, one
    over the other dim as a product per block of the result."""
    from tenncor_amd import configs
    targets = configs.config4_lstm(g, seq=5, batch=64, nin=32, hid=64)[0]
    lines = g.launch_plan(targets)
    # 32 + 64 joined columns in chunks of 32; the gate group of a step is all that reads the product,
    # so the two are one launch and the product's result is never laid out
    assert sum(l.startswith("parts CONCAT+CONTRACT x3 ranges=1 with epilogue group ") and "TANH" in l for l in lines) == 5, lines
    # only the columns of h are read back; the group that reads them is the product's epilogue (on its own
    # it would add the product's two K ranges up)
    assert sum(l.startswith("parts ADD+CONTRACT x4+SLICE ranges=2 with epilogue group ") for l in lines) == 4, lines
    assert lines.count("blocks CONTRACT x5 2x4") == 1, lines
    # TCR_EPILOGUES=0 (read once per process) keeps the two launches apart: not exercised here
    assert not any(l.startswith(("summed", "swapped", "node CONTRACT", "node CONCAT", "group CONCAT ")) for l in lines), lines
    steps = parse_plan(lines)
    alone = sum(1 for s in steps if s[0] in ("node", "swapped", "viewed", "summed", "parts", "blocks"))
    stores = sum(s[2]["stores"] for s in steps if s[0] == "group")
    # (a product that leaves its K ranges to its readers is a launch and never holds a value: counted twice)
    ranged = sum(" ranges=" in l for l in lines)
    assert alone + stores + steps[-1][2]["n"] - ranged == g.count_functors(targets)
    # below the sizes the matrix cores take, everything stays as it was
    small = configs.config4_lstm(g, seq=5, batch=6, nin=8, hid=12)[0]
    assert not any(l.startswith(("parts", "blocks")) for l in g.launch_plan(small))

    x = var(g, [32, 64], np.float32, "x")
    h = var(g, [48, 64], np.float32, "h")
    w1 = var(g, [96, 80], np.float32, "w1")
    w2 = var(g, [96, 80], np.float32, "w2")
    c = var(g, [32, 64], np.float32, "c")
    z = api.concat([x, h], 0)
    p1, p2 = api.matmul(z, w1), api.matmul(z, w2)
    lines = g.launch_plan([api.add(p1, p2)])
    assert lines.count("parts CONCAT+MATMUL x5") == 2 and not any("CONCAT" in l and l.startswith(("group", "node")) for l in lines), lines
    # a concatenation that an elementwise node reads as well is laid out once, for everybody
    lines = g.launch_plan([api.add(p1, p2), api.neg(z)])
    assert not any(l.startswith("parts") for l in lines) and lines.count("node MATMUL") == 2, lines
    # K ranges are left to the readers only where elementwise groups reading through SLICEs are all there is:
    # a transposed operand, few results, a long K
    g0, g1 = var(g, [128, 64], np.float32, "g0"), var(g, [128, 64], np.float32, "g1")
    wt = var(g, [256, 192], np.float32, "wt")
    scale = var(g, [128, 64], np.float32, "scale")
    back = api.contract(api.concat([g0, g1], 0), wt, ((0, 0),))      # [192, 64], K = 256 along the memory of both
    lines = g.launch_plan([api.mul(api.slice(back, 64, 128, 0), scale)])
    # ... one launch reads them: it becomes the product's epilogue
    assert lines[0] == "parts CONCAT+CONTRACT x2+SLICE ranges=2 with epilogue group MUL leaves=2 stores=1 instrs=2", lines
    # ... two launches of different shapes read them: the ranges wait in memory for both
    back3 = api.contract(api.concat([g0, g1], 0), wt, ((0, 0),))
    half = var(g, [64, 64], np.float32, "half")
    lines = g.launch_plan([api.mul(api.slice(back3, 64, 128, 0), scale), api.mul(api.slice(back3, 0, 64, 0), half)])
    assert lines[0] == "parts CONCAT+CONTRACT x2 ranges=2" and sum(l.startswith("group MUL leaves=2") for l in lines) == 2, lines
    # ... a reduction reads the slice as a tensor: the product adds its ranges up itself, into the window
    back2 = api.contract(api.concat([g0, g1], 0), wt, ((0, 0),))
    lines = g.launch_plan([api.reduce_sum(api.slice(back2, 64, 128, 0), 0, 1)])
    assert lines[0] == "parts CONCAT+CONTRACT x2+SLICE", lines
    # an assignment to a part between the concatenation and a product that reads it:
    # the concatenation holds the old value, the part's buffer the new one
    upd = api.assign(x, c)
    q1, q2 = api.matmul(z, w1), api.matmul(z, w2)
    t = api.add(api.add(q1, api.matmul(api.concat([upd, h], 0), w1)), q2)
    lines = g.launch_plan([t])
    assert any(l.startswith(("group CONCAT", "node CONCAT")) for l in lines) and lines.count("node MATMUL") >= 2, lines


def test_launch_plan_lays_out_a_view_that_only_a_swapped_product_reads(g, api):
    """The gradient of a weight behind a SLICE of its product is
    PERMUTE{1,0}(CONTRACT(PAD(gradient), x)) (tenncor/eteq/backprop.hpp:269-359,
    402-421).  The PERMUTE is launched as the product with its operands
    exchanged, the CONTRACT beneath it is looked through -- but that product
    reads its operands from memory, so a PAD that nothing else reads is still
    laid out in front of it (it used to be folded away like a view under an
    elementwise node, and the recording failed for want of its data)."""
    x = var(g, [15, 1, 5], np.float32, "x")
    w = var(g, [32, 15], np.float32, "w")
    gate = api.slice(api.contract(x, w), 8, 8, 0)
    loss = api.reduce_sum(api.square(api.tanh(gate)))
    (dw,) = g.derive(loss, [w])
    lines = g.launch_plan([loss, dw])
    assert "node PAD" in lines and "swapped CONTRACT+PERMUTE" in lines, lines
    assert lines.index("node PAD") < lines.index("swapped CONTRACT+PERMUTE"), lines


def test_launch_plan_reads_a_view_of_a_group_result_in_a_later_launch(g, api):
    """A node that reads another elementwise node through a folded view reads it
    from memory, at other coordinates than its own: the two cannot share a
    launch (whose loads all come before its stores), even when the reader also
    reads the same node directly.  The gradient of a SLICE that was added back
    onto its own operand has this shape."""
    a = var(g, [64, 16], np.float32, "a")
    b = var(g, [64, 16], np.float32, "b")
    h = api.mul(api.sigmoid(a), api.tanh(b))
    y = api.add(h, api.pad(api.slice(h, 8, 40, 0), [[8, 16]]))
    lines = g.launch_plan([api.square(y)])
    steps = [s for s in parse_plan(lines) if s[0] == "group"]
    assert len(steps) == 2 and "MUL" in steps[0][1] and steps[0][2]["stores"] == 1, lines
    assert steps[1][1] == ["ADD", "SQUARE"] and steps[1][2]["leaves"] == 2, lines
    # through an IDENTITY (the same coordinates) the value stays in a register
    lines = g.launch_plan([api.add(h, api.identity(h))])
    assert len([l for l in lines if l.startswith("group")]) == 1, lines


def test_launch_plan_pads_a_weight_that_many_backward_steps_read():
    """The transposed weight of the backward steps of an unrolled LSTM (cfg/tenncor/layer.yml:716-768
    through tenncor/eteq/backprop.hpp:269-359) is read by every step's product as a K-contiguous
    operand with rows of 4 * hid elements: with nine and more steps and rows of 256 and more the
    plan lists it as copied once per pass with a longer leading dim; a short sequence, or a leaf the
    pass assigns to, is left where it lies."""
    from tenncor_amd import graph, configs
    for seq, want in ((12, 1), (4, 0)):
        g = graph.Graph()
        try:
            targets, x, w, _ = configs.config4_lstm(g, seq=seq, batch=64, nin=32, hid=64)
            lines = g.launch_plan(targets)
            assert sum(int(l.split(" ")[1]) for l in lines if l.startswith("padded ")) == want, lines
            if want:
                # a training step in the same pass rewrites the weight: no copy may stand in for it
                loss, dw = targets
                lines = g.launch_plan([loss, graph.Api(g).assign_sub(w, dw)])
                assert not any(l.startswith("padded ") for l in lines), lines
        finally:
            g.close()
