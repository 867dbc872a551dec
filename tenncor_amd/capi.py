"""ctypes binding of the C ABI in ``include/tcg.h`` (``libtcg.so``).

Thin by design: one Python method per exported function, device buffers are
plain integers (device addresses), shapes are tenncor shapes (dim 0 fastest).
The library is loaded from the package folder; if it is missing this module
raises -- there is no fallback path.
"""
import ctypes
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libtcg.so")

RANK_CAP = 8
# enum tcg_dtype (include/tcg.h); the codes after INT32 are the integer widths
# of the reference's full type configuration (cfg/fulltype.yml:11-34)
DOUBLE, FLOAT, INT32 = 1, 2, 3
INT8, UINT8, INT16, UINT16, UINT32, INT64, UINT64 = 4, 5, 6, 7, 8, 9, 10
NP_OF = {DOUBLE: np.float64, FLOAT: np.float32, INT32: np.int32,
         INT8: np.int8, UINT8: np.uint8, INT16: np.int16, UINT16: np.uint16,
         UINT32: np.uint32, INT64: np.int64, UINT64: np.uint64}
# include/tcg.h: the fixed device memory tcg_reduce_noalloc keeps its temporaries in
REDUCE_NOALLOC_SCRATCH_BYTES = 8 << 20

OPCODES = [
    "BAD_OP", "IDENTITY", "ABS", "NEG", "SIN", "COS", "TAN", "EXP", "LOG", "SQRT", "ROUND",
    "SIGMOID", "TANH", "SQUARE", "CUBE", "RAND_UNIF", "REVERSE", "REDUCE_SUM", "REDUCE_PROD",
    "REDUCE_MIN", "REDUCE_MAX", "ARGMAX", "PERMUTE", "EXTEND", "RESHAPE", "SLICE", "PAD",
    "STRIDE", "SCATTER", "POW", "ADD", "SUB", "MUL", "DIV", "MIN", "MAX", "EQ", "NEQ", "LT",
    "GT", "MATMUL", "CONTRACT", "CONV", "SELECT", "CONCAT", "ASSIGN", "ASSIGN_ADD",
    "ASSIGN_SUB", "ASSIGN_MUL", "ASSIGN_DIV", "CAST",
]
OP = {name: i for i, name in enumerate(OPCODES)}

OPD_NONE, OPD_ACC, OPD_T0, OPD_T1, OPD_IMM, OPD_LEAF0 = 0, 1, 2, 3, 4, 8

# every symbol include/tcg.h declares
EXPORTS = [
    "tcg_ctx_create", "tcg_ctx_destroy", "tcg_last_error", "tcg_device_arch", "tcg_alloc", "tcg_free",
    "tcg_mem_stats", "tcg_mem_stats_kept", "tcg_hold", "tcg_release", "tcg_h2d", "tcg_d2h", "tcg_d2d", "tcg_fill_zero", "tcg_sync", "tcg_timer_begin",
    "tcg_timer_end", "tcg_event_create", "tcg_event_destroy", "tcg_event_record", "tcg_event_elapsed",
    "tcg_ew_unary", "tcg_ew_binary", "tcg_ew_nary", "tcg_ew_select", "tcg_cast",
    "tcg_assign", "tcg_ew_fused", "tcg_ew_fusedx", "tcg_reduce", "tcg_reduce_noalloc", "tcg_argmax", "tcg_extend", "tcg_permute", "tcg_slice",
    "tcg_pad", "tcg_pad_interior", "tcg_reverse", "tcg_stride", "tcg_scatter", "tcg_concat", "tcg_matmul", "tcg_contract", "tcg_contract_sum",
    "tcg_gemm", "tcg_gemm_terms", "tcg_gemm_terms_ranges", "tcg_gemm_terms_grid", "tcg_gemm_terms_fx", "tcg_jit_stats", "tcg_conv", "tcg_conv_boxed", "tcg_conv_dense_box", "tcg_conv_views", "tcg_conv_route_counts", "tcg_capture_begin", "tcg_capture_begin_small", "tcg_capture_feed", "tcg_graph_feed", "tcg_capture_end", "tcg_capture_abort", "tcg_batch_begin", "tcg_batch_end", "tcg_fork", "tcg_fork_end", "tcg_join",
    "tcg_graph_launch", "tcg_graph_claim", "tcg_graph_stats", "tcg_graph_destroy",
    "tcg_rand_seed", "tcg_rand_state", "tcg_rand_uniform",
]


class TcgError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("tcg status %d: %s" % (status, message))
        self.status = status


class EwInstr(ctypes.Structure):
    _fields_ = [("opcode", ctypes.c_uint8), ("a", ctypes.c_uint8), ("b", ctypes.c_uint8),
                ("dst", ctypes.c_uint8), ("pad_", ctypes.c_uint32), ("imm", ctypes.c_double)]


class FxLeaf(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("offset", ctypes.c_int64), ("stride", ctypes.c_int64 * 8),
                ("lo", ctypes.c_uint64 * 8), ("hi", ctypes.c_uint64 * 8),
                ("sum_stride", ctypes.c_int64), ("nsum", ctypes.c_uint32), ("from_product", ctypes.c_uint32)]


class FxInstr(ctypes.Structure):
    _fields_ = [("opcode", ctypes.c_uint8), ("a", ctypes.c_uint8), ("b", ctypes.c_uint8), ("c", ctypes.c_uint8),
                ("dst", ctypes.c_uint8), ("pad_", ctypes.c_uint8 * 3), ("imm", ctypes.c_double)]


FX_NONE, FX_IMM, FX_LEAF0, FX_REG0, FX_STORE, FX_BITOR = 0, 1, 8, 32, 255, 254

_lib = None


def load():
    """Load libtcg.so and declare the argument types of every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("%s is missing: build it with `python -m tenncor_amd.build` "
                          "(there is no CPU fallback)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    vp, u64, i32, sz = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int, ctypes.c_size_t
    u64p, vpp = ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_void_p)
    i64p = ctypes.POINTER(ctypes.c_int64)
    sig = {
        "tcg_ctx_create": [i32, ctypes.POINTER(vp)],
        "tcg_ctx_destroy": [vp],
        "tcg_alloc": [vp, sz, ctypes.POINTER(vp)],
        "tcg_free": [vp, vp, sz],
        "tcg_mem_stats": [vp, u64p, u64p],
        "tcg_mem_stats_kept": [vp, u64p],
        "tcg_hold": [vp],
        "tcg_batch_begin": [vp],
        "tcg_fork": [vp],
        "tcg_fork_end": [vp],
        "tcg_join": [vp],
        "tcg_batch_end": [vp],
        "tcg_release": [vp],
        "tcg_h2d": [vp, vp, vp, sz],
        "tcg_d2h": [vp, vp, vp, sz],
        "tcg_d2d": [vp, vp, vp, sz],
        "tcg_fill_zero": [vp, vp, sz],
        "tcg_sync": [vp],
        "tcg_timer_begin": [vp],
        "tcg_timer_end": [vp, ctypes.POINTER(ctypes.c_float)],
        "tcg_event_create": [vp, ctypes.POINTER(vp)],
        "tcg_event_destroy": [vp, vp],
        "tcg_event_record": [vp, vp],
        "tcg_event_elapsed": [vp, vp, vp, ctypes.POINTER(ctypes.c_float)],
        "tcg_ew_unary": [vp, i32, i32, u64, vp, vp],
        "tcg_ew_binary": [vp, i32, i32, u64, vp, vp, vp],
        "tcg_ew_nary": [vp, i32, i32, u64, i32, vpp, vp],
        "tcg_ew_select": [vp, i32, u64, vp, vp, vp, vp],
        "tcg_cast": [vp, i32, i32, u64, vp, vp],
        "tcg_assign": [vp, i32, i32, u64, vp, vp],
        "tcg_rand_seed": [vp, u64],
        "tcg_rand_state": [vp, ctypes.POINTER(ctypes.c_uint64)],
        "tcg_rand_uniform": [vp, i32, u64, vp, vp, vp],
        "tcg_ew_fused": [vp, i32, u64, i32, vpp, i32, ctypes.POINTER(EwInstr), vp],
        "tcg_ew_fusedx": [vp, i32, u64p, i32, ctypes.POINTER(FxLeaf), i32, ctypes.POINTER(FxInstr), i32, vpp],
        "tcg_reduce": [vp, i32, i32, u64p, ctypes.c_uint, vp, vp],
        "tcg_reduce_noalloc": [vp, i32, i32, u64p, ctypes.c_uint, vp, vp],
        "tcg_argmax": [vp, i32, u64p, i32, vp, vp],
        "tcg_extend": [vp, i32, u64p, u64p, vp, vp],
        "tcg_permute": [vp, i32, u64p, u64p, vp, vp],
        "tcg_slice": [vp, i32, u64p, u64p, u64p, vp, vp],
        "tcg_pad": [vp, i32, u64p, u64p, u64p, vp, vp],
        "tcg_pad_interior": [vp, i32, u64p, u64p, u64p, vp, vp],
        "tcg_reverse": [vp, i32, u64p, ctypes.c_uint, vp, vp],
        "tcg_stride": [vp, i32, u64p, u64p, u64p, vp, vp],
        "tcg_scatter": [vp, i32, u64p, u64p, u64p, vp, vp],
        "tcg_concat": [vp, i32, i32, i32, u64p, vpp, vp],
        "tcg_matmul": [vp, i32, u64p, u64p, vp, vp, vp],
        "tcg_contract": [vp, i32, u64p, u64p, i32, u64p, vp, vp, vp],
        "tcg_contract_sum": [vp, i32, u64p, u64p, i32, u64p, i32, vpp, vpp, vp],
        "tcg_gemm": [vp, i32, u64, u64, u64, u64, vp, u64, u64, i32, vp, u64, u64, i32, vp, u64, u64],
        "tcg_gemm_terms": [vp, i32, u64, u64, u64, i32, vpp, u64p, i32, vpp, u64p, i32, vp, u64],
        "tcg_gemm_terms_ranges": [vp, i32, u64, u64, u64, i32, vpp, u64p, i32, vpp, u64p, i32, i32, vp],
        "tcg_gemm_terms_grid": [vp, i32, i32, u64p, i32, u64p, u64, i32, vpp, u64p, i32, vpp, u64p, i32, vp, u64],
        "tcg_gemm_terms_fx": [vp, i32, u64, u64, u64, i32, vpp, u64p, i32, vpp, u64p, i32,
                              u64p, i32, ctypes.POINTER(FxLeaf), i32, ctypes.POINTER(FxInstr), i32, vpp],
        "tcg_jit_stats": [vp, u64p, u64p, ctypes.POINTER(ctypes.c_double)],
        "tcg_conv": [vp, i32, u64p, u64p, i32, u64p, vp, vp, vp],
        "tcg_conv_boxed": [vp, i32, u64p, u64p, i32, u64p, u64p, u64p, u64p, u64p, vp, vp, vp],
        "tcg_conv_dense_box": [vp, i32, u64p, u64p, i32, u64p, u64p, u64p, u64p, u64p, vp, vp, vp],
        "tcg_conv_views": [vp, i32, u64p, u64p, i32, u64p, u64p, u64p, u64p, u64p, vp, i64p, vp, i64p, vp, i64p],
        "tcg_conv_route_counts": [vp, u64p, u64p, u64p],
        "tcg_capture_begin": [vp],
        "tcg_capture_end": [vp, ctypes.POINTER(vp)],
        "tcg_capture_abort": [vp],
        "tcg_capture_begin_small": [vp],
        "tcg_capture_feed": [vp, vp, sz, vp],
        "tcg_graph_feed": [vp, vp, vp, vp, sz],
        "tcg_graph_launch": [vp, vp],
        "tcg_graph_claim": [vp, vp, vp],
        "tcg_graph_stats": [vp, u64p, u64p],
        "tcg_graph_destroy": [vp, vp],
    }
    for name, argtypes in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
    lib.tcg_last_error.argtypes = [vp]
    lib.tcg_last_error.restype = ctypes.c_char_p
    lib.tcg_device_arch.argtypes = [vp]
    lib.tcg_device_arch.restype = ctypes.c_char_p
    _lib = lib
    return lib


def shape8(shape, fill=1):
    s = [int(d) for d in shape] + [fill] * (RANK_CAP - len(shape))
    return s[:RANK_CAP]


def n_elems(shape):
    n = 1
    for d in shape8(shape):
        n *= d
    return n


def _u64(vals):
    return (ctypes.c_uint64 * len(vals))(*[int(v) for v in vals])


def _mask(ranks):
    m = 0
    for r in ranks:
        m |= 1 << int(r)
    return m


def dtype_code(np_dtype):
    t = np.dtype(np_dtype)
    for code, npt in NP_OF.items():
        if t == npt:
            return code
    raise TypeError("unsupported dtype %s" % t)


def _opcode(op):
    return OP[op] if isinstance(op, str) else int(op)


class Context:
    """One device context (tcg_ctx): a stream, a memory pool, the launches."""

    def __init__(self, device=0):
        self.lib = load()
        handle = ctypes.c_void_p()
        rc = self.lib.tcg_ctx_create(device, ctypes.byref(handle))
        if rc != 0:
            raise TcgError(rc, self.lib.tcg_last_error(None).decode())
        self.handle = handle

    def close(self):
        if self.handle:
            self.lib.tcg_ctx_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _check(self, rc):
        if rc != 0:
            raise TcgError(rc, self.lib.tcg_last_error(self.handle).decode())

    @property
    def arch(self):
        return self.lib.tcg_device_arch(self.handle).decode()

    # ---- memory ----
    def alloc(self, nbytes):
        p = ctypes.c_void_p()
        self._check(self.lib.tcg_alloc(self.handle, nbytes, ctypes.byref(p)))
        return p.value

    def free(self, ptr, nbytes):
        self._check(self.lib.tcg_free(self.handle, ptr, nbytes))

    def mem_stats(self):
        a, b = ctypes.c_uint64(), ctypes.c_uint64()
        self._check(self.lib.tcg_mem_stats(self.handle, ctypes.byref(a), ctypes.byref(b)))
        return a.value, b.value

    def mem_stats_kept(self):
        """Bytes of convolution tables the context keeps outside its pool."""
        a = ctypes.c_uint64()
        self._check(self.lib.tcg_mem_stats_kept(self.handle, ctypes.byref(a)))
        return a.value

    def h2d(self, dst, host):
        host = np.ascontiguousarray(host)
        self._check(self.lib.tcg_h2d(self.handle, dst, host.ctypes.data, host.nbytes))

    def d2h(self, src, n, np_dtype):
        out = np.empty(int(n), dtype=np_dtype)
        self._check(self.lib.tcg_d2h(self.handle, out.ctypes.data, src, out.nbytes))
        return out

    def d2d(self, dst, src, nbytes):
        self._check(self.lib.tcg_d2d(self.handle, dst, src, nbytes))

    def fill_zero(self, dst, nbytes):
        self._check(self.lib.tcg_fill_zero(self.handle, dst, nbytes))

    def upload(self, host):
        """Allocate a device buffer holding ``host`` (flattened); returns a DevBuf."""
        host = np.ascontiguousarray(host).reshape(-1)
        buf = DevBuf(self, host.size, host.dtype)
        self.h2d(buf.ptr, host)
        return buf

    def empty(self, n, np_dtype):
        return DevBuf(self, n, np_dtype)

    def sync(self):
        self._check(self.lib.tcg_sync(self.handle))

    def timer_begin(self):
        self._check(self.lib.tcg_timer_begin(self.handle))

    def timer_end(self):
        ms = ctypes.c_float()
        self._check(self.lib.tcg_timer_end(self.handle, ctypes.byref(ms)))
        return ms.value

    def event(self):
        ev = ctypes.c_void_p()
        self._check(self.lib.tcg_event_create(self.handle, ctypes.byref(ev)))
        return ev.value

    def event_destroy(self, ev):
        self._check(self.lib.tcg_event_destroy(self.handle, ev))

    def record(self, ev):
        self._check(self.lib.tcg_event_record(self.handle, ev))

    def elapsed_ms(self, start, stop):
        ms = ctypes.c_float()
        self._check(self.lib.tcg_event_elapsed(self.handle, start, stop, ctypes.byref(ms)))
        return ms.value

    # ---- elementwise ----
    def ew_unary(self, op, dtype, n, src, dst):
        self._check(self.lib.tcg_ew_unary(self.handle, _opcode(op), dtype, n, src, dst))

    def ew_binary(self, op, dtype, n, a, b, dst):
        self._check(self.lib.tcg_ew_binary(self.handle, _opcode(op), dtype, n, a, b, dst))

    def ew_nary(self, op, dtype, n, srcs, dst):
        ptrs = (ctypes.c_void_p * len(srcs))(*srcs)
        self._check(self.lib.tcg_ew_nary(self.handle, _opcode(op), dtype, n, len(srcs), ptrs, dst))

    def ew_select(self, dtype, n, cond, then, otherwise, dst):
        self._check(self.lib.tcg_ew_select(self.handle, dtype, n, cond, then, otherwise, dst))

    def cast(self, out_dtype, in_dtype, n, src, dst):
        self._check(self.lib.tcg_cast(self.handle, out_dtype, in_dtype, n, src, dst))

    def assign(self, op, dtype, n, target, source):
        self._check(self.lib.tcg_assign(self.handle, _opcode(op), dtype, n, target, source))

    def rand_seed(self, seed):
        self._check(self.lib.tcg_rand_seed(self.handle, int(seed)))

    def rand_state(self):
        """(seed, generator blocks drawn so far)."""
        out = (ctypes.c_uint64 * 2)()
        self._check(self.lib.tcg_rand_state(self.handle, out))
        return int(out[0]), int(out[1])

    def rand_uniform(self, dtype, n, lo, hi, dst):
        self._check(self.lib.tcg_rand_uniform(self.handle, dtype, n, lo, hi, dst))

    def ew_fused(self, dtype, n, leaves, program, dst):
        """program: list of (opcode, a, b, dst[, imm])."""
        instrs = (EwInstr * len(program))()
        for i, ins in enumerate(program):
            instrs[i].opcode = _opcode(ins[0])
            instrs[i].a, instrs[i].b, instrs[i].dst = ins[1], ins[2], ins[3]
            instrs[i].imm = float(ins[4]) if len(ins) > 4 else 0.0
        ptrs = (ctypes.c_void_p * len(leaves))(*leaves)
        self._check(self.lib.tcg_ew_fused(self.handle, dtype, n, len(leaves), ptrs, len(program), instrs, dst))

    @staticmethod
    def _fx_group(shape, leaves, program, outs):
        shp = shape8(shape)
        dense = [1] * RANK_CAP
        for d in range(1, RANK_CAP):
            dense[d] = dense[d - 1] * shp[d - 1]
        lv = (FxLeaf * len(leaves))()
        for k, leaf in enumerate(leaves):
            lv[k].ptr = leaf.get("ptr")
            lv[k].offset = int(leaf.get("offset", 0))
            for d in range(RANK_CAP):
                lv[k].stride[d] = int(leaf.get("stride", dense)[d])
                lv[k].lo[d] = int(leaf.get("lo", [0] * RANK_CAP)[d])
                lv[k].hi[d] = int(leaf.get("hi", shp)[d])
            lv[k].nsum = int(leaf.get("nsum", 0))
            lv[k].sum_stride = int(leaf.get("sum_stride", 0))
            lv[k].from_product = int(leaf.get("from_product", 0))
        instrs = (FxInstr * len(program))()
        for i, ins in enumerate(program):
            instrs[i].opcode = {"STORE": FX_STORE, "BITOR": FX_BITOR}.get(ins[0]) or _opcode(ins[0])
            instrs[i].a, instrs[i].b, instrs[i].c, instrs[i].dst = ins[1], ins[2], ins[3], ins[4]
            instrs[i].imm = float(ins[5]) if len(ins) > 5 else 0.0
        ptrs = (ctypes.c_void_p * len(outs))(*outs)
        return shp, lv, instrs, ptrs

    def ew_fusedx(self, dtype, shape, leaves, program, outs):
        """leaves: dicts with ptr, and optionally offset, stride (8 element
        strides; default: dense over `shape`), lo, hi (default: everything),
        nsum and sum_stride (the value is the sum of nsum elements that far apart).
        program: tuples (opcode | "STORE", a, b, c, dst[, imm])."""
        shp, lv, instrs, ptrs = self._fx_group(shape, leaves, program, outs)
        self._check(self.lib.tcg_ew_fusedx(self.handle, dtype, _u64(shp), len(leaves), lv, len(program), instrs,
                                           len(outs), ptrs))

    def gemm_terms_fx(self, dtype, M, N, K, a_ptrs, lda, trans_a, b_ptrs, ldb, trans_b, shape, leaves, program, outs):
        """gemm_terms with the group that reads its result as the epilogue of
        the same launch.  Leaves with from_product=1 address the M x N result
        (row length N): offset = first column, stride as over a [N, M] tensor."""
        n = len(a_ptrs)
        pa = (ctypes.c_void_p * n)(*a_ptrs)
        pb = (ctypes.c_void_p * n)(*b_ptrs)
        la = (ctypes.c_uint64 * n)(*[int(v) for v in lda])
        lb = (ctypes.c_uint64 * n)(*[int(v) for v in ldb])
        shp, lv, instrs, ptrs = self._fx_group(shape, leaves, program, outs)
        self._check(self.lib.tcg_gemm_terms_fx(self.handle, dtype, M, N, K, n, pa, la, int(trans_a), pb, lb, int(trans_b),
                                               _u64(shp), len(leaves), lv, len(program), instrs, len(outs), ptrs))

    # ---- reductions ----
    def reduce(self, op, dtype, shape, rank_set, src, dst):
        self._check(self.lib.tcg_reduce(self.handle, _opcode(op), dtype, _u64(shape8(shape)), _mask(rank_set), src, dst))

    def reduce_noalloc(self, op, dtype, shape, rank_set, src, dst):
        """tcg_reduce with its temporaries in the library's fixed device array."""
        self._check(self.lib.tcg_reduce_noalloc(self.handle, _opcode(op), dtype, _u64(shape8(shape)), _mask(rank_set),
                                                src, dst))

    def argmax(self, dtype, shape, return_dim, src, dst):
        self._check(self.lib.tcg_argmax(self.handle, dtype, _u64(shape8(shape)), int(return_dim), src, dst))

    # ---- data movement ----
    def extend(self, dtype, inshape, bcast, src, dst):
        self._check(self.lib.tcg_extend(self.handle, dtype, _u64(shape8(inshape)), _u64(shape8(bcast)), src, dst))

    def permute(self, dtype, inshape, order8, src, dst):
        self._check(self.lib.tcg_permute(self.handle, dtype, _u64(shape8(inshape)), _u64(order8), src, dst))

    def slice(self, dtype, inshape, offsets, extents, src, dst):
        self._check(self.lib.tcg_slice(self.handle, dtype, _u64(shape8(inshape)), _u64(shape8(offsets, 0)),
                                       _u64(shape8(extents)), src, dst))

    def pad(self, dtype, inshape, before, after, src, dst):
        self._check(self.lib.tcg_pad(self.handle, dtype, _u64(shape8(inshape)), _u64(shape8(before, 0)),
                                     _u64(shape8(after, 0)), src, dst))

    def pad_interior(self, dtype, inshape, before, after, src, dst):
        self._check(self.lib.tcg_pad_interior(self.handle, dtype, _u64(shape8(inshape)), _u64(shape8(before, 0)),
                                              _u64(shape8(after, 0)), src, dst))

    def reverse(self, dtype, shape, rank_set, src, dst):
        self._check(self.lib.tcg_reverse(self.handle, dtype, _u64(shape8(shape)), _mask(rank_set), src, dst))

    def stride(self, dtype, inshape, incr, outshape, src, dst):
        self._check(self.lib.tcg_stride(self.handle, dtype, _u64(shape8(inshape)), _u64(shape8(incr)),
                                        _u64(shape8(outshape)), src, dst))

    def scatter(self, dtype, inshape, incr, outshape, src, dst):
        self._check(self.lib.tcg_scatter(self.handle, dtype, _u64(shape8(inshape)), _u64(shape8(incr)),
                                         _u64(shape8(outshape)), src, dst))

    def concat(self, dtype, axis, shapes, srcs, dst):
        flat = [d for s in shapes for d in shape8(s)]
        ptrs = (ctypes.c_void_p * len(srcs))(*srcs)
        self._check(self.lib.tcg_concat(self.handle, dtype, int(axis), len(srcs), _u64(flat), ptrs, dst))

    # ---- contractions ----
    def matmul(self, dtype, ashape, bshape, a, b, dst):
        self._check(self.lib.tcg_matmul(self.handle, dtype, _u64(shape8(ashape)), _u64(shape8(bshape)), a, b, dst))

    def contract(self, dtype, ashape, bshape, pairs, a, b, dst):
        flat = [int(v) for p in pairs for v in p]
        self._check(self.lib.tcg_contract(self.handle, dtype, _u64(shape8(ashape)), _u64(shape8(bshape)),
                                          len(pairs), _u64(flat), a, b, dst))

    def contract_sum(self, dtype, ashape, bshape, pairs, a_list, b_list, dst):
        """sum_t CONTRACT(a_list[t], b_list[t]) into dst."""
        flat = [int(v) for p in pairs for v in p]
        pa = (ctypes.c_void_p * len(a_list))(*a_list)
        pb = (ctypes.c_void_p * len(b_list))(*b_list)
        self._check(self.lib.tcg_contract_sum(self.handle, dtype, _u64(shape8(ashape)), _u64(shape8(bshape)),
                                              len(pairs), _u64(flat), len(a_list), pa, pb, dst))

    def gemm(self, dtype, M, N, K, batch, A, lda, stride_a, trans_a, B, ldb, stride_b, trans_b, C, ldc, stride_c):
        self._check(self.lib.tcg_gemm(self.handle, dtype, M, N, K, batch, A, lda, stride_a, int(trans_a),
                                      B, ldb, stride_b, int(trans_b), C, ldc, stride_c))

    def conv(self, dtype, imgshape, kshape, ranks, img, kernel, dst):
        r = [int(v) for v in ranks][:RANK_CAP]
        self._check(self.lib.tcg_conv(self.handle, dtype, _u64(shape8(imgshape)), _u64(shape8(kshape)),
                                      len(r), _u64(r if r else [0]), img, kernel, dst))

    def conv_boxed(self, dtype, imgshape, kshape, ranks, img_box, out_box, img, kernel, dst):
        """img_box / out_box: (lo[8], hi[8]) or None for the whole extent."""
        r = [int(v) for v in ranks][:RANK_CAP]
        ilo, ihi = (_u64(img_box[0]), _u64(img_box[1])) if img_box else (None, None)
        olo, ohi = (_u64(out_box[0]), _u64(out_box[1])) if out_box else (None, None)
        self._check(self.lib.tcg_conv_boxed(self.handle, dtype, _u64(shape8(imgshape)), _u64(shape8(kshape)),
                                            len(r), _u64(r if r else [0]), ilo, ihi, olo, ohi, img, kernel, dst))

    def conv_dense_box(self, dtype, imgshape, kshape, ranks, img_box, out_box, box, kernel, dst):
        """conv_boxed with `box` holding only the elements inside img_box."""
        r = [int(v) for v in ranks][:RANK_CAP]
        olo, ohi = (_u64(out_box[0]), _u64(out_box[1])) if out_box else (None, None)
        self._check(self.lib.tcg_conv_dense_box(self.handle, dtype, _u64(shape8(imgshape)), _u64(shape8(kshape)),
                                                len(r), _u64(r if r else [0]), _u64(img_box[0]), _u64(img_box[1]),
                                                olo, ohi, box, kernel, dst))

    def gemm_terms(self, dtype, M, N, K, a_ptrs, lda, trans_a, b_ptrs, ldb, trans_b, c, ldc):
        """C = sum_t A_t B_t, every term with its own operand addresses and leading dims."""
        n = len(a_ptrs)
        pa = (ctypes.c_void_p * n)(*a_ptrs)
        pb = (ctypes.c_void_p * n)(*b_ptrs)
        la = (ctypes.c_uint64 * n)(*[int(v) for v in lda])
        lb = (ctypes.c_uint64 * n)(*[int(v) for v in ldb])
        self._check(self.lib.tcg_gemm_terms(self.handle, dtype, M, N, K, n, pa, la, int(trans_a), pb, lb, int(trans_b), c, ldc))

    def gemm_terms_grid(self, dtype, Mp, Np, K, a_ptrs, lda, trans_a, b_ptrs, ldb, trans_b, c, ldc):
        """a_ptrs[i][t], b_ptrs[j][t]: block (i, j) of C = sum_t A[i][t] B[j][t]; lda / ldb per part."""
        nterms = len(a_ptrs[0])
        flat_a = [p for row in a_ptrs for p in row]
        flat_b = [p for row in b_ptrs for p in row]
        pa = (ctypes.c_void_p * len(flat_a))(*flat_a)
        pb = (ctypes.c_void_p * len(flat_b))(*flat_b)
        self._check(self.lib.tcg_gemm_terms_grid(self.handle, dtype, len(Mp), _u64(Mp), len(Np), _u64(Np), K, nterms,
                                                 pa, _u64(lda), int(trans_a), pb, _u64(ldb), int(trans_b), c, ldc))

    def gemm_terms_ranges(self, dtype, M, N, K, a_ptrs, lda, trans_a, b_ptrs, ldb, trans_b, nranges, ranges):
        """The same sum with its summed index cut into nranges ranges left side by side."""
        n = len(a_ptrs)
        pa = (ctypes.c_void_p * n)(*a_ptrs)
        pb = (ctypes.c_void_p * n)(*b_ptrs)
        la = (ctypes.c_uint64 * n)(*[int(v) for v in lda])
        lb = (ctypes.c_uint64 * n)(*[int(v) for v in ldb])
        self._check(self.lib.tcg_gemm_terms_ranges(self.handle, dtype, M, N, K, n, pa, la, int(trans_a), pb, lb,
                                                   int(trans_b), int(nranges), ranges))

    def conv_views(self, dtype, imgshape, kshape, ranks, img_box, out_box, box, box_stride, kernel, kernel_stride,
                   dst, out_stride):
        """conv_dense_box over strided operands and a strided result: `box`,
        `kernel` and `dst` are the addresses of image element img_box[0], of
        kernel element 0 and of output element out_box[0]; strides count elements."""
        r = [int(v) for v in ranks][:RANK_CAP]
        olo, ohi = (_u64(out_box[0]), _u64(out_box[1])) if out_box else (None, None)
        i64 = lambda vals: (ctypes.c_int64 * 8)(*[int(v) for v in vals])
        self._check(self.lib.tcg_conv_views(self.handle, dtype, _u64(shape8(imgshape)), _u64(shape8(kshape)),
                                            len(r), _u64(r if r else [0]), _u64(img_box[0]), _u64(img_box[1]),
                                            olo, ohi, box, i64(box_stride), kernel, i64(kernel_stride),
                                            dst, i64(out_stride)))

    def conv_route_counts(self):
        """Convolutions of this context that ran (a) as a product reading the image out of a patch
        in LDS, (b) as one launch for a short summed index, (c) as few rows under a long summed index."""
        a, b, c = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_uint64()
        self._check(self.lib.tcg_conv_route_counts(self.handle, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)))
        return {"patch": a.value, "short_sum": b.value, "few_rows": c.value}

    def jit_stats(self):
        """Kernels compiled at run time by this process, kernels loaded from the
        disk cache instead, and the milliseconds both took."""
        compiled, from_disk, ms = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_double()
        self._check(self.lib.tcg_jit_stats(self.handle, ctypes.byref(compiled), ctypes.byref(from_disk), ctypes.byref(ms)))
        return {"compiled": compiled.value, "from_disk": from_disk.value, "ms": ms.value}

    # ---- recorded launch sequences ----
    def batch_begin(self):
        """Small launches from here on are held back as steps of one kernel."""
        self._check(self.lib.tcg_batch_begin(self.handle))

    def batch_end(self):
        self._check(self.lib.tcg_batch_end(self.handle))

    def fork(self):
        """Calls from here to fork_end() run on a second stream, beside what follows fork_end()."""
        self._check(self.lib.tcg_fork(self.handle))

    def fork_end(self):
        self._check(self.lib.tcg_fork_end(self.handle))

    def join(self):
        self._check(self.lib.tcg_join(self.handle))

    def capture_begin(self, small=False):
        """small: record the sequence as the steps of one kernel."""
        if small:
            self._check(self.lib.tcg_capture_begin_small(self.handle))
        else:
            self._check(self.lib.tcg_capture_begin(self.handle))

    def capture_feed(self, devptr, host):
        """The launch supplies the content of `devptr` (single-launch recordings)."""
        host = np.ascontiguousarray(host)
        self._check(self.lib.tcg_capture_feed(self.handle, devptr, host.nbytes, host.ctypes.data))

    def graph_feed(self, graph, devptr, host):
        host = np.ascontiguousarray(host)
        self._check(self.lib.tcg_graph_feed(self.handle, graph, devptr, host.ctypes.data, host.nbytes))

    def capture_end(self):
        g = ctypes.c_void_p()
        self._check(self.lib.tcg_capture_end(self.handle, ctypes.byref(g)))
        return g

    def capture_abort(self):
        self._check(self.lib.tcg_capture_abort(self.handle))

    def graph_launch(self, graph):
        self._check(self.lib.tcg_graph_launch(self.handle, graph))

    def graph_claim(self, graph, ptr):
        self._check(self.lib.tcg_graph_claim(self.handle, graph, ptr))

    def graph_stats(self, graph):
        nodes, nbytes = ctypes.c_uint64(), ctypes.c_uint64()
        self._check(self.lib.tcg_graph_stats(graph, ctypes.byref(nodes), ctypes.byref(nbytes)))
        return nodes.value, nbytes.value

    def graph_destroy(self, graph):
        self._check(self.lib.tcg_graph_destroy(self.handle, graph))


class DevBuf:
    """A device buffer from the context's pool, returned to it on release."""

    def __init__(self, ctx, n, np_dtype):
        self.ctx = ctx
        self.n = int(n)
        self.np_dtype = np.dtype(np_dtype)
        self.dtype = dtype_code(np_dtype)
        self.nbytes = max(self.n, 1) * self.np_dtype.itemsize
        self.ptr = ctx.alloc(self.nbytes)

    def get(self):
        return self.ctx.d2h(self.ptr, self.n, self.np_dtype)

    def release(self):
        if self.ptr is not None and self.ctx.handle:
            self.ctx.free(self.ptr, self.nbytes)
        self.ptr = None

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass
