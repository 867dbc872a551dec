"""Writes the JSON fixtures in this folder from the numeric literals that the
reference's own C++ tests hold.

Run once in the authoring container (the reference tree is not available where
the GPU tests run): ``python tests/golden/extract_reference_vectors.py``.
It only reads the test sources as text: every ``std::vector<T> name = {...};``
(or ``name{...}``) inside a given line range becomes ``name -> list`` and the
result is committed as data.  Nothing of the reference is executed and no
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
    for name, body in DIMS_RE.findall(text):
        out[name] = [int(v) for v in _numbers(body)]
    for name, body in SHAPE_RE.findall(text):
        out[name] = [int(v) for v in _numbers(body)]
    return out


BLOCKS = {
    # whole-graph goldens
    "matmul_complex": ("tenncor/test/test_equation.cpp", 26, 136),
    "contract_equivalent": ("tenncor/test/test_equation.cpp", 139, 249),
    "sigmoid_mlp_slow": ("tenncor/test/test_equation.cpp", 252, 479),
    "sigmoid_mlp_fast": ("tenncor/test/test_equation.cpp", 482, 706),
    "tanh_rnn": ("tenncor/test/test_equation.cpp", 709, 839),
    # operator-with-gradient goldens
    "api_matmul": ("tenncor/test/test_api.cpp", 1986, 2085),
    "api_convolution": ("tenncor/test/test_api.cpp", 2265, 2373),
    "api_group_sum": ("tenncor/test/test_api.cpp", 2376, 2414),
}


def main():
    fixtures = {}
    for key, (path, first, last) in BLOCKS.items():
        fixtures[key] = read_block(path, first, last)
        names = [k for k in fixtures[key] if not k.startswith("_")]
        print("%-22s %s" % (key, ", ".join("%s[%d]" % (n, len(fixtures[key][n])) for n in names)))
    with open(os.path.join(HERE, "equation_vectors.json"), "w") as f:
        json.dump(fixtures, f, indent=0, separators=(",", ":"))
    return 0


if __name__ == "__main__":
    sys.exit(main())
