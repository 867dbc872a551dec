"""Writes the JSON fixtures in this folder from the numeric literals that the
reference's own C++ tests hold.

Run once in the authoring container (the reference tree is not available where
the GPU tests run): ``python tests/golden/extract_reference_vectors.py``.
It only reads the test sources as text: every ``std::vector<T> name = {...};``
(or ``name{...}``) inside a given line range becomes ``name -> list``, every
``double name = literal;`` becomes ``name -> number``, every printed graph a
test expects (the adjacent string literals of an ``EXPECT_GRAPHEQ``) becomes
one string, and the result is committed as data.  The printed graphs that the
reference keeps as files of their own (models/test/opt*.txt, cnn_opt.txt:
expected outputs of its optimisation tests) are copied to optimized/.  Nothing of the reference is executed and no
source text is kept.
"""
import ast
import json
import os
import re
import sys

REF = os.environ.get("TENNCOR_REFERENCE", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))

VEC_RE = re.compile(
    r"std::vector<\s*(double|float|int32_t)\s*>\s*(\w+)\s*(?:=\s*)?\{(.*?)\}\s*;", re.S)
DIMS_RE = re.compile(r"teq::DimsT\s+(\w+)\s*=\s*\{(.*?)\}\s*;", re.S)
SHAPE_RE = re.compile(r"teq::Shape\s+(\w+)\s*\(\s*\{(.*?)\}\s*\)\s*;", re.S)
NESTED_RE = re.compile(
    r"std::vector<\s*std::vector<\s*double\s*>\s*>\s*(\w+)\s*(?:=\s*)?\{((?:\s*\{[^{}]*\}\s*,?)*)\s*\}\s*;", re.S)
DIM_RE = re.compile(r"teq::(?:DimT|RankT)\s+(\w+)\s*=\s*(\d+)\s*;")
SCALAR_RE = re.compile(r"\b(?:double|float)\s+(\w+)\s*=\s*([0-9eE+\-.]+)f?\s*;")
LITERAL_LINE_RE = re.compile(r'^\s*"((?:[^"\\]|\\.)*)"[^"]*$')


def _strip_comments(text):
    text = re.sub(r"//[^\n]*", "", text)
    return re.sub(r"/\*.*?\*/", "", text, flags=re.S)


def _eval_number(expr):
    """Evaluate a C numeric literal expression such as ``4./3`` or ``62+31``."""
    expr = expr.strip()
    if not expr:
        return None
    if not re.fullmatch(r"[0-9eE+\-*/. ()]+", expr):
        raise ValueError("not a numeric literal: %r" % expr)
    node = ast.parse(expr, mode="eval")
    for sub in ast.walk(node):
        if not isinstance(sub, (ast.Expression, ast.BinOp, ast.UnaryOp, ast.Constant,
                                ast.Add, ast.Sub, ast.Mult, ast.Div, ast.USub, ast.UAdd)):
            raise ValueError("unexpected syntax in %r" % expr)
    return eval(compile(node, "<literal>", "eval"), {"__builtins__": {}})


def _numbers(body):
    vals = []
    for piece in body.replace("\n", " ").split(","):
        v = _eval_number(piece)
        if v is not None:
            vals.append(v)
    return vals


def read_block(relpath, first, last):
    with open(os.path.join(REF, relpath)) as f:
        lines = f.readlines()
    text = _strip_comments("".join(lines[first - 1:last]))
    out = {"_source": "%s:%d-%d" % (relpath, first, last)}
    for ctype, name, body in VEC_RE.findall(text):
        vals = _numbers(body)
        if ctype == "int32_t":
            vals = [int(v) for v in vals]
        else:
            vals = [float(v) for v in vals]
        out[name] = vals
    for name, body in NESTED_RE.findall(text):
        out[name] = [[float(v) for v in _numbers(inner)] for inner in re.findall(r"\{([^{}]*)\}", body)]
    for name, literal in DIM_RE.findall(text):
        out[name] = int(literal)
    for regex in (DIMS_RE, SHAPE_RE):
        for name, body in regex.findall(text):
            try:
                out[name] = [int(v) for v in _numbers(body)]
            except ValueError:
                pass  # spelled with named dims: the test restates it from those
    for name, literal in SCALAR_RE.findall(text):
        out[name] = float(literal)
    return out


def _unescape(body):
    return re.sub(r"\\(.)", lambda m: {"n": "\n", "t": "\t"}.get(m.group(1), m.group(1)), body)


def read_expected_graphs(relpath, first, last):
    """The printed graphs of the EXPECT_GRAPHEQ calls in a line range, in order:
    runs of lines that hold nothing but a string literal."""
    with open(os.path.join(REF, relpath)) as f:
        lines = f.readlines()[first - 1:last]
    graphs, run = [], []
    for line in lines + [""]:
        m = LITERAL_LINE_RE.match(line)
        if m and ("`--" in m.group(1) or m.group(1).startswith("(")):
            run.append(_unescape(m.group(1)))
        elif run:
            graphs.append("".join(run))
            run = []
    return graphs


BLOCKS = {
    # whole-graph goldens
    "matmul_complex": ("tenncor/test/test_equation.cpp", 26, 136),
    "contract_equivalent": ("tenncor/test/test_equation.cpp", 139, 249),
    "sigmoid_mlp_slow": ("tenncor/test/test_equation.cpp", 252, 479),
    "sigmoid_mlp_fast": ("tenncor/test/test_equation.cpp", 482, 706),
    "tanh_rnn": ("tenncor/test/test_equation.cpp", 709, 839),
    # operator-with-gradient goldens
    "api_matmul": ("tenncor/test/test_api.cpp", 1986, 2085),
    "api_contract": ("tenncor/test/test_api.cpp", 2089, 2190),
    "api_convolution": ("tenncor/test/test_api.cpp", 2265, 2373),
    "api_group_sum": ("tenncor/test/test_api.cpp", 2376, 2414),
}


LAYER_BLOCKS = {
    # recurrent layers built through the layer API: gradients, and three groups
    # of assignments of a hand-written rms-momentum training step
    "equation_tanh_rnn_layer": ("tenncor/test/test_equation.cpp", 842, 969),
    "equation_tanh_rnn_layer_connect": ("tenncor/test/test_equation.cpp", 972, 1101),
    "connect_tanh_rnn": ("tenncor/test/test_layer.cpp", 264, 387),
    "connect_dense_tanh_rnn": ("tenncor/test/test_layer.cpp", 390, 571),
    "connect_tanh_rnn_full": ("tenncor/test/test_layer.cpp", 574, 813),
    "connect_tanh_rnn_cross_entropy": ("tenncor/test/test_layer.cpp", 816, 1058),
    "connect_tanh_rnn_training": ("tenncor/test/test_layer.cpp", 1061, 1593),
    "bind_softmax": ("tenncor/test/test_layer.cpp", 199, 261),
    "dense_connection": ("tenncor/test/test_layer.cpp", 36, 96),
    "conv_connection": ("tenncor/test/test_layer.cpp", 99, 120),
}


def write_layer_fixtures():
    fixtures = {}
    for key, (path, first, last) in LAYER_BLOCKS.items():
        fixtures[key] = read_block(path, first, last)
        if key in ("bind_softmax", "dense_connection", "conv_connection"):
            fixtures[key]["expected_graphs"] = read_expected_graphs(path, first, last)
        names = [k for k in fixtures[key] if not k.startswith("_")]
        print("%-32s %s" % (key, ", ".join(names)))
    with open(os.path.join(HERE, "layer_goldens.json"), "w") as f:
        json.dump(fixtures, f, indent=0, separators=(",", ":"))


def write_backprop_fixtures():
    """tenncor/eteq/test/test_backprop.cpp: per TEST, the opcodes handed to the
    unary/binary helpers (if any) and the printed gradient graphs it expects."""
    path = "tenncor/eteq/test/test_backprop.cpp"
    with open(os.path.join(REF, path)) as f:
        lines = f.readlines()
    starts = [(i + 1, re.match(r"TEST\(BACKPROP,\s*(\w+)\)", line).group(1))
              for i, line in enumerate(lines) if line.startswith("TEST(BACKPROP")]
    fixtures = {"_source": path}
    for idx, (first, name) in enumerate(starts):
        last = starts[idx + 1][0] - 1 if idx + 1 < len(starts) else len(lines)
        text = "".join(lines[first - 1:last])
        fixtures[name] = {
            "lines": "%d-%d" % (first, last),
            "helper_opcodes": re.findall(r"(unary|binary)_derivative\(egen::(\w+)", text),
            "expected_graphs": read_expected_graphs(path, first, last),
        }
        print("%-14s %s %d graph(s)" % (name, fixtures[name]["helper_opcodes"], len(fixtures[name]["expected_graphs"])))
    with open(os.path.join(HERE, "backprop_goldens.json"), "w") as f:
        json.dump(fixtures, f, indent=0, separators=(",", ":"))


# printed graphs the reference's optimisation tests compare against
# (tenncor/test/test_opt.cpp:211-255,381-386): data files of its test folder
EXPECTED_GRAPH_FILES = {
    "models/test/opt0.txt": "rnn_layer_root0.txt",
    "models/test/opt1.txt": "rnn_layer_root1.txt",
    "models/test/opt2.txt": "rnn_layer_root2.txt",
    "models/test/opt3.txt": "rnn_layer_root3.txt",
    "models/test/cnn_opt.txt": "cnn_layer.txt",
}


def copy_expected_graph_files():
    outdir = os.path.join(HERE, "optimized")
    os.makedirs(outdir, exist_ok=True)
    for src, dst in EXPECTED_GRAPH_FILES.items():
        with open(os.path.join(REF, src)) as f:
            text = f.read()
        with open(os.path.join(outdir, dst), "w") as f:
            f.write(text)
        print("%-26s %d lines" % (dst, text.count("\n")))


GRAPH_BLOCKS = {
    # optimiser update rules: the graph each builds and the values one step leaves
    "approx_sgd": ("tenncor/test/test_approx.cpp", 21, 45),
    "approx_adagrad": ("tenncor/test/test_approx.cpp", 48, 86),
    "approx_adadelta": ("tenncor/test/test_approx.cpp", 89, 286),
    "approx_rms_momentum": ("tenncor/test/test_approx.cpp", 289, 385),
    "approx_adam": ("tenncor/test/test_approx.cpp", 388, 512),
    # a convolution layer trained one adadelta step: inputs and the error after the step
    "opt_cnn_layer": ("tenncor/test/test_opt.cpp", 261, 408),
}


def write_graph_fixtures():
    fixtures = {}
    for key, (path, first, last) in GRAPH_BLOCKS.items():
        fixtures[key] = read_block(path, first, last)
        if key.startswith("approx_"):
            fixtures[key]["expected_graphs"] = read_expected_graphs(path, first, last)
        names = [k for k in fixtures[key] if not k.startswith("_")]
        print("%-22s %s" % (key, ", ".join(names)))
    with open(os.path.join(HERE, "approx_goldens.json"), "w") as f:
        json.dump(fixtures, f, indent=0, separators=(",", ":"))


def main():
    write_graph_fixtures()
    write_layer_fixtures()
    write_backprop_fixtures()
    copy_expected_graph_files()
    fixtures = {}
    for key, (path, first, last) in BLOCKS.items():
        fixtures[key] = read_block(path, first, last)
        names = [k for k in fixtures[key] if not k.startswith("_")]
        print("%-22s %s" % (key, ", ".join(names)))
    with open(os.path.join(HERE, "equation_vectors.json"), "w") as f:
        json.dump(fixtures, f, indent=0, separators=(",", ":"))
    return 0


if __name__ == "__main__":
    sys.exit(main())
