"""ctypes binding of ``include/tcgraph.h`` (``libtenncor_host.so``): the C++
host graph layer -- Variable / Constant / Functor nodes, the gradient builder,
the evaluator and the GPU device -- driven from Python the way the reference's
pybind11 module drives tenncor (tenncor/python/*.cpp).

``Graph`` owns nodes; ``Node`` is a handle with numpy-side shape bookkeeping.
The composite helpers at the bottom restate the generated ``TenncorAPI`` methods
the benchmark configurations are built from (cfg/tenncor/*.yml); they only
compose primitive opcodes.
"""
import ctypes
import os

import numpy as np

from . import capi

_PKG = os.path.dirname(os.path.abspath(__file__))
# One type configuration per process, as in the reference (its ETEQ_CFG picks
# cfg/mintype.yml or cfg/fulltype.yml when the sources are generated): set
# TENNCOR_AMD_TYPES=full before the first use for the build that also knows
# INT8, UINT8, INT16, UINT16, UINT32, INT64 and UINT64.
FULL_TYPES = os.environ.get("TENNCOR_AMD_TYPES", "min") == "full"
LIB_PATH = os.path.join(_PKG, "libtenncor_host_full.so" if FULL_TYPES else "libtenncor_host.so")

OP = capi.OP
DOUBLE, FLOAT, INT32 = capi.DOUBLE, capi.FLOAT, capi.INT32
RANK_CAP = 8
DIM_MAX = 65535  # std::numeric_limits<teq::DimT>::max()

EXPORTS = [
    "tcr_last_error", "tcr_graph_create", "tcr_graph_destroy", "tcr_variable", "tcr_constant", "tcr_assign", "tcr_prefetch",
    "tcr_functor", "tcr_derive", "tcr_local_derivative", "tcr_evaluate", "tcr_evaluate_ignoring", "tcr_sync", "tcr_shape", "tcr_dtype", "tcr_data",
    "tcr_version", "tcr_opcode", "tcr_nargs", "tcr_args", "tcr_to_string", "tcr_count_functors",
    "tcr_set_evaluator", "tcr_evaluator_stats", "tcr_evaluator_record_error", "tcr_evaluator_record_cost", "tcr_evaluator_timing", "tcr_attr", "tcr_launch_plan", "tcr_optimize",
    "tcr_set_random", "tcr_seed",
]

EVAL_PLAIN, EVAL_REPLAY, EVAL_REPLAY_UNFUSED, EVAL_REPLAY_LAUNCHES, EVAL_DEFAULT, EVAL_TIMING = 0, 1, 2, 3, 4, 5

# conversions shipped with the package (the reference's cfg/optimizations.json
# is a git-lfs pointer without content)
DEFAULT_RULES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host", "cfg", "optimizations.json")

_lib = None


class GraphError(RuntimeError):
    pass


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("%s is missing: build it with `python -m tenncor_amd.build`" % LIB_PATH)
    capi.load()  # libtcg.so first, so that the dependency resolves in-tree
    lib = ctypes.CDLL(LIB_PATH)
    vp, i32 = ctypes.c_void_p, ctypes.c_int
    i32p, u64p = ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_uint64)
    sig = {
        "tcr_graph_create": [ctypes.POINTER(vp)],
        "tcr_graph_destroy": [vp],
        "tcr_variable": [vp, i32, u64p, vp, ctypes.c_char_p, i32p],
        "tcr_constant": [vp, i32, u64p, vp, i32p],
        "tcr_assign": [vp, i32, vp],
        "tcr_prefetch": [vp, i32],
        "tcr_functor": [vp, i32, i32, i32p, i32, ctypes.POINTER(ctypes.c_char_p),
                        ctypes.POINTER(ctypes.POINTER(ctypes.c_int64)), i32p, i32p],
        "tcr_derive": [vp, i32, i32, i32p, i32p],
        "tcr_local_derivative": [vp, i32, i32, i32, i32p],
        "tcr_evaluate_ignoring": [vp, i32, i32p, i32, i32p],
        "tcr_evaluate": [vp, i32, i32p],
        "tcr_sync": [vp],
        "tcr_shape": [vp, i32, u64p],
        "tcr_dtype": [vp, i32, i32p],
        "tcr_data": [vp, i32, vp, ctypes.c_size_t],
        "tcr_version": [vp, i32, u64p],
        "tcr_opcode": [vp, i32, i32p],
        "tcr_nargs": [vp, i32, i32p],
        "tcr_args": [vp, i32, i32p, i32],
        "tcr_to_string": [vp, i32, ctypes.c_char_p, ctypes.c_size_t],
        "tcr_attr": [vp, i32, ctypes.c_char_p, ctypes.POINTER(ctypes.c_int64), i32, i32p],
        "tcr_count_functors": [vp, i32, i32p, i32p],
        "tcr_set_evaluator": [i32],
        "tcr_evaluator_stats": [u64p],
        "tcr_evaluator_record_error": [ctypes.c_char_p, ctypes.c_size_t, u64p],
        "tcr_evaluator_timing": [ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_size_t)],
        "tcr_evaluator_record_cost": [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double), u64p, u64p],
        "tcr_launch_plan": [vp, i32, i32p, ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_size_t)],
        "tcr_optimize": [vp, i32, i32p, ctypes.c_char_p, i32, i32p, u64p],
        "tcr_set_random": [i32],
        "tcr_seed": [ctypes.c_uint64],
    }
    for name, argtypes in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
    lib.tcr_last_error.argtypes = []
    lib.tcr_last_error.restype = ctypes.c_char_p
    _lib = lib
    return lib


def set_evaluator(kind):
    """teq::set_eval: "default" (no evaluator registered: teq::get_eval then
    makes "replay", or "plain" under TCR_EVAL_PLAIN=1), "plain" (node-by-node walk), "replay"
    (record a target set's launches on its second evaluation, with elementwise
    functors sharing launches and the pass of a graph of small tensors as one
    kernel, and enqueue the recording afterwards), "replay_launches" (the same
    without single-kernel passes: bit-identical to the walk) or
    "replay_unfused" (one launch per functor).  Process-wide, like the
    reference's evaluator slot."""
    lib = load()
    code = {"plain": EVAL_PLAIN, "replay": EVAL_REPLAY, "replay_unfused": EVAL_REPLAY_UNFUSED,
            "replay_launches": EVAL_REPLAY_LAUNCHES, "default": EVAL_DEFAULT, "timing": EVAL_TIMING}[kind]
    if lib.tcr_set_evaluator(code) != 0:
        raise GraphError(lib.tcr_last_error().decode())


def set_random(where):
    """Where RAND_UNIF nodes built from now on draw: "host" (the reference's
    std::default_random_engine, the default) or "device" (counter-based
    generator on the GPU; another stream, the same distributions)."""
    lib = load()
    if lib.tcr_set_random({"host": 0, "device": 1}[where]) != 0:
        raise GraphError(lib.tcr_last_error().decode())


def seed(value):
    """global::seed: seeds the host generator and restarts the device stream."""
    lib = load()
    if lib.tcr_seed(int(value)) != 0:
        raise GraphError(lib.tcr_last_error().decode())


def evaluator_timing():
    """Under set_evaluator("timing"): device microseconds per kind of launch, as text
    (the launches the replaying evaluator would record, run and timed one by one)."""
    lib = load()
    need = ctypes.c_size_t()
    if lib.tcr_evaluator_timing(None, 0, ctypes.byref(need)) != 0:
        raise GraphError(lib.tcr_last_error().decode())
    buf = ctypes.create_string_buffer(need.value + 1)
    if lib.tcr_evaluator_timing(buf, len(buf), None) != 0:
        raise GraphError(lib.tcr_last_error().decode())
    return buf.value.decode()


def evaluator_stats():
    """Counters of the replaying evaluator as a dict (zeros under "plain")."""
    lib = load()
    out = (ctypes.c_uint64 * 6)()
    if lib.tcr_evaluator_stats(out) != 0:
        raise GraphError(lib.tcr_last_error().decode())
    keys = ("plain", "recorded", "replayed", "skipped", "launches", "reserved_bytes")
    stats = dict(zip(keys, [int(v) for v in out]))
    buf = ctypes.create_string_buffer(2048)
    failures = ctypes.c_uint64()
    if lib.tcr_evaluator_record_error(buf, len(buf), ctypes.byref(failures)) != 0:
        raise GraphError(lib.tcr_last_error().decode())
    record_ms, jit_ms = ctypes.c_double(), ctypes.c_double()
    compiled, from_disk = ctypes.c_uint64(), ctypes.c_uint64()
    if lib.tcr_evaluator_record_cost(ctypes.byref(record_ms), ctypes.byref(jit_ms), ctypes.byref(compiled), ctypes.byref(from_disk)) != 0:
        raise GraphError(lib.tcr_last_error().decode())
    stats.update(record_ms=round(record_ms.value, 3), jit_ms=round(jit_ms.value, 3), jit_compiled=int(compiled.value),
                 jit_from_disk=int(from_disk.value))
    stats["record_failures"] = int(failures.value)
    stats["record_error"] = buf.value.decode()
    return stats


def _ints(vals):
    return (ctypes.c_int * len(vals))(*[int(v) for v in vals])


class Node:
    def __init__(self, graph, nid):
        self.graph = graph
        self.id = nid

    @property
    def shape(self):
        return self.graph.shape(self)

    @property
    def dtype(self):
        return self.graph.dtype(self)

    def get(self):
        return self.graph.data(self)

    def __repr__(self):
        return "Node(%d)" % self.id


class Graph:
    def __init__(self):
        self.lib = load()
        h = ctypes.c_void_p()
        self._check(self.lib.tcr_graph_create(ctypes.byref(h)))
        self.h = h

    def close(self):
        if self.h:
            self.lib.tcr_graph_destroy(self.h)
            self.h = None

    def _check(self, rc):
        if rc != 0:
            raise GraphError(self.lib.tcr_last_error().decode())

    # ---- leaves ----
    def variable(self, data, shape, label=""):
        data = np.ascontiguousarray(data).reshape(-1)
        assert data.size == capi.n_elems(shape)
        out = ctypes.c_int()
        s = (ctypes.c_uint64 * 8)(*capi.shape8(shape))
        self._check(self.lib.tcr_variable(self.h, capi.dtype_code(data.dtype), s, data.ctypes.data,
                                          label.encode(), ctypes.byref(out)))
        return Node(self, out.value)

    def constant(self, data, shape):
        data = np.ascontiguousarray(data).reshape(-1)
        assert data.size == capi.n_elems(shape)
        out = ctypes.c_int()
        s = (ctypes.c_uint64 * 8)(*capi.shape8(shape))
        self._check(self.lib.tcr_constant(self.h, capi.dtype_code(data.dtype), s, data.ctypes.data, ctypes.byref(out)))
        return Node(self, out.value)

    def scalar(self, value, np_dtype, shape=()):
        return self.constant(np.full(capi.n_elems(shape), value, dtype=np_dtype), list(shape))

    def assign(self, var, data):
        data = np.ascontiguousarray(data, dtype=capi.NP_OF[var.dtype]).reshape(-1)
        assert data.size == capi.n_elems(var.shape)
        self._check(self.lib.tcr_assign(self.h, var.id, data.ctypes.data))

    def prefetch(self, leaf):
        """Copy the leaf's value to the device now rather than inside the next evaluation."""
        self._check(self.lib.tcr_prefetch(self.h, leaf.id))

    # ---- functors ----
    def functor(self, op, args, **attrs):
        """attrs: key -> list of ints (pairs flattened), a Node for `tensor`."""
        opcode = OP[op] if isinstance(op, str) else int(op)
        keys, arrays = [], []
        for key, val in attrs.items():
            if isinstance(val, Node):
                val = [val.id]
            elif np.isscalar(val):
                val = [int(val)]
            keys.append(key.encode())
            arrays.append((ctypes.c_int64 * len(val))(*[int(v) for v in val]))
        ckeys = (ctypes.c_char_p * len(keys))(*keys)
        cvals = (ctypes.POINTER(ctypes.c_int64) * len(keys))(
            *[ctypes.cast(a, ctypes.POINTER(ctypes.c_int64)) for a in arrays])
        clens = _ints([len(a) for a in arrays])
        out = ctypes.c_int()
        self._check(self.lib.tcr_functor(self.h, opcode, len(args), _ints([a.id for a in args]), len(keys),
                                         ckeys, cvals, clens, ctypes.byref(out)))
        return Node(self, out.value)

    def derive(self, root, targets):
        out = (ctypes.c_int * len(targets))()
        self._check(self.lib.tcr_derive(self.h, root.id, len(targets), _ints([t.id for t in targets]), out))
        return [Node(self, out[i]) for i in range(len(targets))]

    def local_derivative(self, op, supgrad, arg_idx):
        """eteq::DerivativeFuncs::lderive: what functor `op` passes to its
        argument arg_idx when the gradient `supgrad` arrives at it."""
        out = ctypes.c_int()
        self._check(self.lib.tcr_local_derivative(self.h, op.id, supgrad.id, int(arg_idx), ctypes.byref(out)))
        return Node(self, out.value)

    def evaluate(self, targets):
        self._check(self.lib.tcr_evaluate(self.h, len(targets), _ints([t.id for t in targets])))

    def evaluate_ignoring(self, targets, ignored):
        """iEvaluator::evaluate(device, targets, ignored): the walk stops at the
        ignored nodes, whose readers use the values they already hold."""
        self._check(self.lib.tcr_evaluate_ignoring(self.h, len(targets), _ints([t.id for t in targets]),
                                                   len(ignored), _ints([t.id for t in ignored])))

    def sync(self):
        self._check(self.lib.tcr_sync(self.h))

    # ---- inspection ----
    def shape(self, node):
        s = (ctypes.c_uint64 * 8)()
        self._check(self.lib.tcr_shape(self.h, node.id, s))
        return list(s)

    def dtype(self, node):
        d = ctypes.c_int()
        self._check(self.lib.tcr_dtype(self.h, node.id, ctypes.byref(d)))
        return d.value

    def data(self, node):
        out = np.empty(capi.n_elems(self.shape(node)), dtype=capi.NP_OF[self.dtype(node)])
        self._check(self.lib.tcr_data(self.h, node.id, out.ctypes.data, out.nbytes))
        return out

    def version(self, node):
        v = ctypes.c_uint64()
        self._check(self.lib.tcr_version(self.h, node.id, ctypes.byref(v)))
        return v.value

    def opcode(self, node):
        o = ctypes.c_int()
        self._check(self.lib.tcr_opcode(self.h, node.id, ctypes.byref(o)))
        return capi.OPCODES[o.value]

    def args(self, node):
        n = ctypes.c_int()
        self._check(self.lib.tcr_nargs(self.h, node.id, ctypes.byref(n)))
        buf = (ctypes.c_int * max(n.value, 1))()
        self._check(self.lib.tcr_args(self.h, node.id, buf, n.value))
        return [Node(self, buf[i]) for i in range(n.value)]

    def attr(self, node, key):
        """The integer list a functor holds under an attribute key (None when
        it has none): "tensor" gives the node, "dtype" the type code."""
        n = ctypes.c_int()
        self._check(self.lib.tcr_attr(self.h, node.id, key.encode(), None, 0, ctypes.byref(n)))
        if n.value < 0:
            return None
        buf = (ctypes.c_int64 * max(n.value, 1))()
        self._check(self.lib.tcr_attr(self.h, node.id, key.encode(), buf, n.value, ctypes.byref(n)))
        if key == "tensor":
            return Node(self, int(buf[0]))
        return [int(buf[i]) for i in range(n.value)]

    def to_string(self, node):
        buf = ctypes.create_string_buffer(1 << 20)
        self._check(self.lib.tcr_to_string(self.h, node.id, buf, len(buf)))
        return buf.value.decode()

    def launch_plan(self, targets):
        """The launches one recorded pass over `targets` would consist of: a list
        of lines, "node OP" or "group OP+OP... leaves=L stores=S instrs=I", and a
        final "folded N".  Pure host logic: works without a GPU."""
        ids = _ints([t.id for t in targets])
        need = ctypes.c_size_t()
        self._check(self.lib.tcr_launch_plan(self.h, len(targets), ids, None, 0, ctypes.byref(need)))
        buf = ctypes.create_string_buffer(need.value + 1)
        self._check(self.lib.tcr_launch_plan(self.h, len(targets), ids, buf, need.value + 1, ctypes.byref(need)))
        return buf.value.decode().splitlines()

    def optimize(self, roots, rules=DEFAULT_RULES, fold=True):
        """hone::optimize (tenncor/hone/optimize.hpp:19-38): merge equal
        subgraphs, fold functors of constants into constants (evaluated on the
        GPU unless fold=False) and apply the conversions of `rules`: JSON text,
        a path to a JSON file, or None for no conversions.  Readers of replaced
        nodes are rewired in place.  Returns (new roots, stats)."""
        text = None
        if rules is not None:
            text = rules
            if os.path.exists(rules):
                with open(rules) as f:
                    text = f.read()
            text = text.encode()
        ids = _ints([r.id for r in roots])
        out = (ctypes.c_int * len(roots))()
        stats = (ctypes.c_uint64 * 4)()
        self._check(self.lib.tcr_optimize(self.h, len(roots), ids, text, int(bool(fold)), out, stats))
        keys = ("merged", "folded", "converted", "rounds")
        return [Node(self, out[i]) for i in range(len(roots))], dict(zip(keys, [int(v) for v in stats]))

    def count_functors(self, nodes):
        c = ctypes.c_int()
        self._check(self.lib.tcr_count_functors(self.h, len(nodes), _ints([n.id for n in nodes]), ctypes.byref(c)))
        return c.value


class Api:
    """The TenncorAPI methods the configurations use (cfg/tenncor/core.yml,
    nn.yml, layer.yml, loss.yml), restated over Graph.functor."""

    def __init__(self, graph):
        self.g = graph

    def _like(self, scalar, like):
        """eteq::make_constant_like: scalar Constant + EXTEND to `like`
        (tenncor/eteq/make.hpp:168-183)."""
        cst = self.g.scalar(scalar, capi.NP_OF[like.dtype])
        return self.g.functor("EXTEND", [cst], tensor=like)

    def _operand(self, x, like):
        return x if isinstance(x, Node) else self._like(x, like)

    def unary(self, op, x):
        return self.g.functor(op, [x])

    def binary(self, op, a, b):
        if not isinstance(a, Node):
            a = self._like(a, b)
        b = self._operand(b, a)
        return self.g.functor(op, [a, b])

    def add(self, a, b):
        return self.binary("ADD", a, b)

    def sub(self, a, b):
        return self.binary("SUB", a, b)

    def mul(self, a, b):
        return self.binary("MUL", a, b)

    def div(self, a, b):
        return self.binary("DIV", a, b)

    def pow(self, a, b):
        return self.binary("POW", a, b)

    def sigmoid(self, x):
        return self.unary("SIGMOID", x)

    def tanh(self, x):
        return self.unary("TANH", x)

    def exp(self, x):
        return self.unary("EXP", x)

    def log(self, x):
        return self.unary("LOG", x)

    def neg(self, x):
        return self.unary("NEG", x)

    def square(self, x):
        return self.unary("SQUARE", x)

    def identity(self, x, execute_in_parallel=()):
        """core.yml:171-187: the value of `x`; further arguments are only
        dependencies, evaluated along with it."""
        return self.g.functor("IDENTITY", [x] + list(execute_in_parallel))

    def sqrt(self, x):
        return self.unary("SQRT", x)

    def assign(self, target, source):
        return self.g.functor("ASSIGN", [target, source])

    def assign_add(self, target, source):
        return self.g.functor("ASSIGN_ADD", [target, source])

    def assign_sub(self, target, source):
        return self.g.functor("ASSIGN_SUB", [target, source])

    def if_then_else(self, condition, then, otherwise):
        """core.yml:634-651: choosing between a tensor and itself is that tensor."""
        if then.id == otherwise.id:
            return then
        return self.g.functor("SELECT", [condition, then, otherwise])

    def relu(self, x):
        """core.yml:1261-1267: max(arg, 0)."""
        return self.binary("MAX", x, 0.0)

    def matmul(self, a, b):
        return self.g.functor("MATMUL", [a, b])

    def contract(self, a, b, dims=((0, 1),)):
        return self.g.functor("CONTRACT", [a, b], rank_pairs=[v for p in dims for v in p])

    def transpose(self, x):
        return self.permute(x, [1, 0])

    def permute(self, x, order):
        return self.g.functor("PERMUTE", [x], ranks=list(order))

    def extend(self, x, offset, xlist):
        """core.yml:679-693."""
        return self.g.functor("EXTEND", [x], dimensions=[1] * offset + list(xlist))

    def extend_like(self, x, like):
        return self.g.functor("EXTEND", [x], tensor=like)

    def reduce(self, op, x, offset=0, ndims=RANK_CAP):
        """core.yml:773-800: dims offset .. offset+ndims-1."""
        dims = list(range(offset, min(offset + ndims, RANK_CAP)))
        return self.g.functor(op, [x], rank_set=dims)

    def reduce_sum(self, x, offset=0, ndims=RANK_CAP):
        return self.reduce("REDUCE_SUM", x, offset, ndims)

    def reduce_max(self, x, offset=0, ndims=RANK_CAP):
        return self.reduce("REDUCE_MAX", x, offset, ndims)

    def slice(self, x, offset, extent, dimension):
        """core.yml:909-927."""
        ext = [0, DIM_MAX] * max(RANK_CAP, dimension)
        ext[2 * dimension:2 * dimension + 2] = [offset, extent]
        return self.g.functor("SLICE", [x], dimension_pairs=ext)

    def pad(self, x, pairs):
        return self.g.functor("PAD", [x], dimension_pairs=[v for p in pairs for v in p])

    def reverse(self, x, dims):
        return self.g.functor("REVERSE", [x], rank_set=list(dims))

    def concat(self, args, axis):
        return self.g.functor("CONCAT", list(args), rank=axis)

    def convolution(self, img, kernel, dims):
        return self.g.functor("CONV", [img, kernel], ranks=list(dims))

    def dense(self, x, weight, bias=None, dims=((0, 1),)):
        """nn.yml:14-47 fully_connect with one pair, wrapped in the IDENTITY the
        layer tagging adds (tenncor/test/test_api.cpp:2433-2440)."""
        out = self.contract(x, weight, dims)
        if bias is not None:
            out = self.add(out, self.extend_like(bias, out))
        return self.identity(out)

    def conv2d(self, image, kernel, bias=None, zero_padding=((0, 0), (0, 0))):
        """nn.yml:48-98: image {in,w,h,batch}, kernel {out,in,kw,kh} ->
        {out,w',h',batch}; zero_padding = ((before, after) along the width,
        (before, after) along the height)."""
        cimage = image
        if any(p > 0 for pair in zero_padding for p in pair):
            cimage = self.pad(cimage, [(0, 0), tuple(zero_padding[0]), tuple(zero_padding[1])])
        img_pad = kernel.shape[0] - 1
        cimage = self.pad(cimage, [(0, 0)] * 4 + [(img_pad, img_pad)])
        out = self.permute(self.convolution(cimage, self.reverse(kernel, [0]), [4, 0, 1, 2]), [4, 1, 2, 3])
        if bias is not None:
            out = self.add(out, self.extend_like(bias, out))
        return out

    def softmax(self, x, offset=0, ndims=RANK_CAP):
        """core.yml:1232-1260."""
        eps = float(np.finfo(np.float32).eps)
        shifted = self.sub(x, self.extend_like(self.reduce_max(x, offset, ndims), x))
        exarg = self.exp(shifted)
        return self.div(exarg, self.extend_like(self.add(self.reduce_sum(exarg, offset, ndims), eps), exarg))

    def cross_entropy(self, target, x):
        """loss.yml:40-59."""
        eps = float(np.finfo(np.float32).eps)
        inp = self.add(x, eps)
        not_in = self.sub(1.0, inp)
        not_targ = self.sub(1.0, target)
        return self.neg(self.add(self.mul(target, self.log(inp)), self.mul(not_targ, self.log(not_in))))

    def reduce_mean(self, x):
        """core.yml:1096: the sum over every dim divided by the element count."""
        return self.div(self.reduce_sum(x), float(capi.n_elems(x.shape)))

    def rnn(self, x, init_state, cell, activation, seq_dim=1):
        """layer.yml:694-715.  cell = callable(concat(x_t, state)) (a dense layer
        over both); init_state has the shape of one slice with the hidden size
        in dim 0 (layer.yml:291-292 extends a {hidden} variable like a slice)."""
        state, states = init_state, []
        for i in range(x.shape[seq_dim]):
            inslice = self.slice(x, i, 1, seq_dim)
            state = activation(cell(self.concat([inslice, state], 0)))
            states.append(state)
        return self.identity(self.concat(states, seq_dim))

    def lstm(self, x, init_state, init_hidden, gates, seq_dim=1):
        """layer.yml:716-768.  gates = dict name -> callable(xc) for the g, i, f
        and o gate layers (each a dense layer over concat(x_t, hidden))."""
        nseq = x.shape[seq_dim]
        state, hidden, states = init_state, init_hidden, []
        for i in range(nseq):
            inslice = self.slice(x, i, 1, seq_dim)
            xc = self.concat([inslice, hidden], 0)
            gate = self.tanh(gates["g"](xc))
            inp = self.sigmoid(gates["i"](xc))
            forget = self.sigmoid(gates["f"](xc))
            output = self.sigmoid(gates["o"](xc))
            state = self.add(self.mul(gate, inp), self.mul(state, forget))
            hidden = self.mul(state, output)
            states.append(hidden)
        return self.identity(self.concat(states, seq_dim))


class Approx:
    """The update rules of cfg/tenncor/approx.yml (ApproxAPI): for every
    variable an assignment node that applies one optimisation step in place on
    the device copy of the variable.  Each method returns [(variable, assign
    node)], the reference's layr::VarErrsT."""

    def __init__(self, api):
        self.api = api
        self.g = api.g
        self.slots = {}  # label -> the state variables created under it, in order

    def _typed(self, like, *values):
        """Scalars in the dtype of the variables, as the reference's templates
        hold them (``T nodecay = 1. - decay``): 1 - 0.999f is 0.000999987."""
        np_dtype = capi.NP_OF[like.dtype]
        return [np_dtype(v) for v in values]

    def _epsilon(self, like, epsilon):
        """std::numeric_limits<T>::epsilon(), the default of every rule's epsilon."""
        if epsilon is not None:
            return epsilon
        np_dtype = capi.NP_OF[like.dtype]
        return float(np.finfo(np_dtype).eps) if np.issubdtype(np_dtype, np.floating) else 0

    def _variable_like(self, scalar, like, label):
        """eteq::make_variable_like (tenncor/eteq/make.hpp:185-200)."""
        np_dtype = capi.NP_OF[like.dtype]
        var = self.g.variable(np.full(capi.n_elems(like.shape), scalar, np_dtype), like.shape, label)
        self.slots.setdefault(label, []).append(var)
        return var

    def sgd(self, error, variables, learning_rate=0.5):
        """approx.yml:12-52: x -= learning_rate * f'(x)."""
        a = self.api
        ders = self.g.derive(error, variables)
        return [(x, a.assign_sub(x, a.mul(der, learning_rate))) for x, der in zip(variables, ders)]

    def adagrad(self, error, variables, learning_rate=0.5, epsilon=None):
        """approx.yml:53-94: momentum += f'(x)^2; x -= lr f'(x) / (sqrt(momentum) + eps)."""
        a = self.api
        out = []
        for x, der in zip(variables, self.g.derive(error, variables)):
            momentum = self._variable_like(1, der, "momentum")
            update = a.assign_add(momentum, a.square(der))
            out.append((x, a.assign_sub(x, a.div(a.mul(der, learning_rate), a.add(a.sqrt(update), self._epsilon(der, epsilon))))))
        return out

    def adam(self, error, variables, step_rate=0.001, decay1=0.9, decay2=0.999,
             epsilon=None):
        """approx.yml:95-176."""
        a = self.api
        out = []
        for x, der in zip(variables, self.g.derive(error, variables)):
            decay1, decay2 = self._typed(der, decay1, decay2)
            nodecay1, nodecay2 = float(1 - decay1), float(1 - decay2)
            decay1, decay2 = float(decay1), float(decay2)
            m = self._variable_like(0, der, "moment1")
            v = self._variable_like(0, der, "moment2")
            t = self._variable_like(0, der, "t")
            one_t = a._like(1, der)
            next_m = a.assign(m, a.add(a.mul(decay1, m), a.mul(nodecay1, der)))
            next_v = a.assign(v, a.add(a.mul(decay2, v), a.mul(nodecay2, a.square(der))))
            incr = a.assign_add(t, one_t)
            m_corr = a.div(next_m, a.sub(one_t, a.pow(decay1, incr)))
            v_corr = a.div(next_v, a.sub(one_t, a.pow(decay2, incr)))
            delta = a.mul(step_rate, a.div(m_corr, a.add(a.sqrt(v_corr), self._epsilon(der, epsilon))))
            out.append((x, a.assign_sub(x, delta)))
        return out

    def adadelta(self, error, variables, step_rate=1.0, decay=0.9, offset=0.0001,
                 epsilon=None):
        """approx.yml:177-247."""
        a = self.api
        out = []
        for x, der in zip(variables, self.g.derive(error, variables)):
            (decay,) = self._typed(der, decay)
            nodecay, decay = float(1 - decay), float(decay)
            msg = self._variable_like(0, der, "ex_sqr_grad")
            msd = self._variable_like(0, der, "ex_sqr_delx")
            msg_next = a.assign(msg, a.add(a.mul(decay, msg), a.mul(nodecay, a.square(der))))
            delta = a.mul(a.mul(step_rate, a.div(a.sqrt(a.add(msd, offset)),
                                                 a.add(a.sqrt(a.add(msg_next, offset)), self._epsilon(der, epsilon)))), der)
            msd_next = a.assign(msd, a.add(a.mul(decay, msd), a.mul(nodecay, a.square(delta))))
            out.append((x, a.assign_sub(x, a.identity(delta, [msd_next]))))
        return out

    def rms_momentum(self, error, variables, learning_rate=0.5, discount_factor=0.99,
                     epsilon=None):
        """approx.yml:248-304."""
        a = self.api
        out = []
        for x, der in zip(variables, self.g.derive(error, variables)):
            (discount_factor,) = self._typed(der, discount_factor)
            nodiscount, discount_factor = float(1 - discount_factor), float(discount_factor)
            momentum = self._variable_like(1, der, "momentum")
            update = a.assign(momentum, a.add(a.mul(discount_factor, momentum),
                                              a.mul(nodiscount, a.square(der))))
            out.append((x, a.assign_sub(x, a.div(a.mul(der, learning_rate), a.add(a.sqrt(update), self._epsilon(der, epsilon))))))
        return out

    def apply_update(self, error, updates):
        """tenncor/trainer/apply_update.hpp:13-41 without the re-trailing of the
        error through the assignments: one node that yields the error (at the
        weights the step started from) and depends on every assignment."""
        return self.api.identity(error, [assign for _, assign in updates])
