"""tcg_gemm_terms_fx: a sum of matrix products with the elementwise group that
reads its result as the epilogue of the same launch -- what a time step of a
recurrent cell is (cfg/tenncor/layer.yml:297-345, 716-768: the gate product
over [x_t, h] followed by the gate activations and the state update;
tenncor/eteq/backprop.hpp:269-359: backwards the gate gradients times the
transposed weight followed by the derivative factors of the step before).

Held against (i) the oracle: the product summed in double by numpy's matmul,
rounded to fp32 where the separate launches would round it, then the group
node by node through the oracle's scalar routines, at the 1e-4 bar of a
contraction; (ii) tcg_gemm_terms followed by tcg_ew_fusedx on the same
operands, which differ from the single launch only in the order of the
additions over K: 1e-5 of the largest entry.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ACC_RTOL = 1e-4


@pytest.fixture(scope="module")
def ctx():
    from tenncor_amd import capi
    c = capi.Context(0)
    yield c
    c.close()


def assert_acc_close(got, ref, rtol=ACC_RTOL):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    floor = np.mean(np.abs(ref)) if ref.size else 0.0
    denom = np.maximum(np.abs(ref), floor)
    denom[denom == 0] = 1.0
    err = np.abs(got - ref) / denom
    assert err.max() <= rtol, "max rel err %.3g at %d (got %r ref %r)" % (
        err.max(), err.argmax(), got.flat[err.argmax()], ref.flat[err.argmax()])


GUARD = 64


class Guarded:
    """A device buffer with a border of sentinels on both sides."""

    def __init__(self, ctx, n):
        self.n = n
        self.buf = ctx.upload(np.full(n + 2 * GUARD, 777, np.float32))
        self.ptr = self.buf.ptr + 4 * GUARD

    def get(self):
        got = self.buf.get()
        assert (got[:GUARD] == 777).all() and (got[-GUARD:] == 777).all(), "a launch wrote outside its result"
        return got[GUARD:-GUARD]


def lstm_gates(capi, J):
    """c' = tanh(g) sigmoid(i) + c sigmoid(f); o' = sigmoid(o); h = c' o': the
    group of a step of cfg/tenncor/layer.yml:716-768 over the four column
    blocks of the gate product (leaves 0..3) and the state before (leaf 4)."""
    L, R, NONE = capi.FX_LEAF0, capi.FX_REG0, capi.FX_NONE
    prog = [("TANH", L, NONE, NONE, R), ("SIGMOID", L + 1, NONE, NONE, R + 1), ("MUL", R, R + 1, NONE, R),
            ("SIGMOID", L + 2, NONE, NONE, R + 1), ("MUL", L + 4, R + 1, NONE, R + 1), ("ADD", R, R + 1, NONE, R),
            ("STORE", R, NONE, NONE, 0), ("SIGMOID", L + 3, NONE, NONE, R + 1), ("STORE", R + 1, NONE, NONE, 1),
            ("MUL", R, R + 1, NONE, R + 2), ("STORE", R + 2, NONE, NONE, 2)]

    def reference(orc, C, extra):
        g, i, f, o = (np.ascontiguousarray(C[:, k * J:(k + 1) * J]).reshape(-1) for k in range(4))
        c_new = orc.binary("ADD", orc.binary("MUL", orc.unary("TANH", g), orc.unary("SIGMOID", i)),
                           orc.binary("MUL", extra[0].reshape(-1), orc.unary("SIGMOID", f)))
        so = orc.unary("SIGMOID", o)
        return [c_new, so, orc.binary("MUL", c_new, so)]
    return prog, 3, 1, reference


def scaled_window(capi, J):
    """out0 = p * e0 + e1, out1 = p * e2 + 0.5: one block of the product
    (leaf 0), three operands of the group's own, an immediate."""
    L, R, NONE, IMM = capi.FX_LEAF0, capi.FX_REG0, capi.FX_NONE, capi.FX_IMM
    prog = [("MUL", L, L + 1, NONE, R), ("ADD", R, L + 2, NONE, R), ("STORE", R, NONE, NONE, 0),
            ("MUL", L, L + 3, NONE, R + 1), ("ADD", R + 1, IMM, NONE, R + 1, 0.5), ("STORE", R + 1, NONE, NONE, 1)]

    def reference(orc, C, extra):
        p = np.ascontiguousarray(C[:, :J]).reshape(-1)
        half = np.full(p.size, 0.5, np.float32)
        return [orc.binary("ADD", orc.binary("MUL", p, extra[0].reshape(-1)), extra[1].reshape(-1)),
                orc.binary("ADD", orc.binary("MUL", p, extra[2].reshape(-1)), half)]
    return prog, 2, 3, reference


CASES = [
    # name, M, J, blocks of the product the group reads, terms, K per term, trans_b, first column read, extra columns of the result
    ("lstm_step_forward", 256, 512, 4, 3, 256, 0, 0, 0),
    ("lstm_step_backward", 256, 512, 1, 4, 512, 1, 0, 0),
    ("one_tile", 32, 16, 4, 1, 64, 0, 0, 0),
    ("two_terms_transposed", 32, 16, 1, 2, 32, 1, 0, 0),
    ("ragged_rows", 40, 32, 4, 3, 48, 0, 0, 0),
    ("rows_below_a_tile", 5, 64, 1, 1, 128, 1, 0, 0),
    ("one_wave_four_per_lane", 48, 64, 1, 3, 16, 1, 0, 0),
    ("window_of_a_wider_result", 64, 128, 1, 2, 128, 1, 64, 192),
    ("window_of_a_wider_result_row_major", 64, 64, 1, 2, 64, 0, 128, 64),
    ("long_k_in_a_loop", 64, 64, 1, 1, 8192, 1, 0, 0),
]


@pytest.mark.parametrize("name,M,J,G,terms,KT,trans_b,first,more", CASES, ids=[c[0] for c in CASES])
def test_product_with_epilogue_equals_product_then_group(ctx, oracle, name, M, J, G, terms, KT, trans_b, first, more):
    from tenncor_amd import capi
    rng = np.random.default_rng(abs(hash((M, J, G, terms, KT))) % (1 << 31))
    N = first + G * J + more
    # operands are parts of wider tensors: leading dims above the extents
    lda, ldb = KT + 8, (KT + 4 if trans_b else N + 12)
    A = [rng.uniform(-1, 1, (M, lda)).astype(np.float32) for _ in range(terms)]
    B = [(rng.standard_normal((N, ldb) if trans_b else (KT, ldb)) / np.sqrt(KT * terms)).astype(np.float32) for _ in range(terms)]
    dA, dB = [ctx.upload(a) for a in A], [ctx.upload(b) for b in B]
    C64 = np.zeros((M, N))
    for a, b in zip(A, B):
        C64 += a[:, :KT].astype(np.float64) @ (b[:, :KT].astype(np.float64).T if trans_b else b[:, :N].astype(np.float64))
    make = lstm_gates if G == 4 else scaled_window
    prog, nout, nextra, reference = make(capi, J)
    extra = [rng.uniform(-1, 1, (M, J)).astype(np.float32) for _ in range(nextra)]
    dE = [ctx.upload(e) for e in extra]
    want = reference(oracle, C64[:, first:first + G * J].astype(np.float32), extra)
    shape = [J, 1, M]
    pstride = [1, N, N, N * M, N * M, N * M, N * M, N * M]
    fused = [Guarded(ctx, M * J) for _ in range(nout)]
    apart = [Guarded(ctx, M * J) for _ in range(nout)]
    a_ptrs, b_ptrs = [a.ptr for a in dA], [b.ptr for b in dB]
    leaves = [{"from_product": 1, "offset": first + g * J, "stride": pstride} for g in range(G)] + [{"ptr": e.ptr} for e in dE]
    ctx.gemm_terms_fx(capi.FLOAT, M, N, KT, a_ptrs, [lda] * terms, 0, b_ptrs, [ldb] * terms, trans_b, shape, leaves, prog,
                      [o.ptr for o in fused])
    Cd = ctx.empty(M * N, np.float32)
    ctx.gemm_terms(capi.FLOAT, M, N, KT, a_ptrs, [lda] * terms, 0, b_ptrs, [ldb] * terms, trans_b, Cd.ptr, N)
    leaves = [{"ptr": Cd.ptr, "offset": first + g * J, "stride": pstride} for g in range(G)] + [{"ptr": e.ptr} for e in dE]
    ctx.ew_fusedx(capi.FLOAT, shape, leaves, prog, [o.ptr for o in apart])
    for k in range(nout):
        got, two = fused[k].get(), apart[k].get()
        assert_acc_close(got, want[k])
        scale = np.abs(want[k]).max()
        assert np.abs(got.astype(np.float64) - two).max() <= 1e-5 * scale
    # the same launch again (its kernel now comes from the cache) gives the same bits
    again = [Guarded(ctx, M * J) for _ in range(nout)]
    leaves = [{"from_product": 1, "offset": first + g * J, "stride": pstride} for g in range(G)] + [{"ptr": e.ptr} for e in dE]
    ctx.gemm_terms_fx(capi.FLOAT, M, N, KT, a_ptrs, [lda] * terms, 0, b_ptrs, [ldb] * terms, trans_b, shape, leaves, prog,
                      [o.ptr for o in again])
    for k in range(nout):
        np.testing.assert_array_equal(again[k].get(), fused[k].get())


def test_group_operands_through_views(ctx, oracle):
    """The group's own operands keep every form tcg_ew_fusedx reads: a row
    broadcast over the rows (EXTEND of a bias), a zero-bordered window (PAD)
    and a strided slice of a wider tensor, beside two blocks of the product."""
    from tenncor_amd import capi
    L, R, NONE = capi.FX_LEAF0, capi.FX_REG0, capi.FX_NONE
    rng = np.random.default_rng(11)
    M, J, KT = 64, 32, 64
    N = 2 * J
    A = rng.uniform(-1, 1, (M, KT)).astype(np.float32)
    B = (rng.standard_normal((KT, N)) / 8).astype(np.float32)
    bias = rng.uniform(-1, 1, J).astype(np.float32)
    inner = rng.uniform(-1, 1, (M - 16, J - 8)).astype(np.float32)     # sits at rows 8.., columns 4.. of the group
    wide = rng.uniform(-1, 1, (M, 3 * J)).astype(np.float32)           # columns J..2J are read
    dA, dB, dbias, dinner, dwide = (ctx.upload(v) for v in (A, B, bias, inner, wide))
    C = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)
    padded = np.zeros((M, J), np.float32)
    padded[8:M - 8, 4:J - 4] = inner
    # out = (p0 + bias) * p1 + padded - slice
    prog = [("ADD", L, L + 2, NONE, R), ("MUL", R, L + 1, NONE, R), ("ADD", R, L + 3, NONE, R), ("SUB", R, L + 4, NONE, R),
            ("STORE", R, NONE, NONE, 0)]
    want = oracle.binary("SUB", oracle.binary("ADD", oracle.binary("MUL", oracle.binary(
        "ADD", np.ascontiguousarray(C[:, :J]).reshape(-1), np.tile(bias, M)), np.ascontiguousarray(C[:, J:]).reshape(-1)),
        padded.reshape(-1)), np.ascontiguousarray(wide[:, J:2 * J]).reshape(-1))
    shape = [J, M]
    pstride = [1, N] + [N * M] * 6
    jin = J - 8
    leaves = [{"from_product": 1, "offset": 0, "stride": pstride}, {"from_product": 1, "offset": J, "stride": pstride},
              {"ptr": dbias.ptr, "stride": [1, 0, 0, 0, 0, 0, 0, 0]},
              {"ptr": dinner.ptr, "offset": -(8 * jin + 4), "stride": [1, jin] + [jin * (M - 16)] * 6,
               "lo": [4, 8, 0, 0, 0, 0, 0, 0], "hi": [J - 4, M - 8, 1, 1, 1, 1, 1, 1]},
              {"ptr": dwide.ptr, "offset": J, "stride": [1, 3 * J] + [3 * J * M] * 6}]
    out = Guarded(ctx, M * J)
    ctx.gemm_terms_fx(capi.FLOAT, M, N, KT, [dA.ptr], [KT], 0, [dB.ptr], [N], 0, shape, leaves, prog, [out.ptr])
    assert_acc_close(out.get(), want)


def test_shapes_the_kernel_does_not_take_are_refused_before_anything_runs(ctx):
    """TCG_ERR_UNSUPPORTED (3) and untouched results: the caller then runs the
    product and the group as two launches."""
    from tenncor_amd import capi
    L, R, NONE = capi.FX_LEAF0, capi.FX_REG0, capi.FX_NONE
    M, J, KT = 32, 64, 32
    N = J
    a = ctx.upload(np.ones(M * KT, np.float32))
    b = ctx.upload(np.ones(KT * N, np.float32))
    prog = [("NEG", L, NONE, NONE, R), ("STORE", R, NONE, NONE, 0)]
    pstride = [1, N] + [N * M] * 6
    good = [{"from_product": 1, "offset": 0, "stride": pstride}]

    def refused(dtype=capi.FLOAT, K=KT, trans_a=0, leaves=good, shape=(J, M)):
        out = Guarded(ctx, M * J)
        with pytest.raises(capi.TcgError) as err:
            ctx.gemm_terms_fx(dtype, M, N, K, [a.ptr], [K], trans_a, [b.ptr], [N], 0, list(shape), leaves, prog, [out.ptr])
        assert err.value.status == 3, err.value
        assert (out.get() == 777).all()

    refused(dtype=capi.INT32)
    refused(trans_a=1)
    refused(K=24)                                                                   # not whole steps of 16
    refused(leaves=[{"from_product": 1, "offset": 0, "stride": [1, 2 * N] + [N * M] * 6}])   # skips rows of the result
    refused(leaves=[{"from_product": 1, "offset": 8, "stride": pstride}])          # runs past the last column
    refused(leaves=[{"ptr": a.ptr}])                                                # nothing reads the product
    refused(shape=(J, M // 2))                                                      # fewer rows than the product
    # the well-formed call goes through
    out = Guarded(ctx, M * J)
    ctx.gemm_terms_fx(capi.FLOAT, M, N, KT, [a.ptr], [KT], 0, [b.ptr], [N], 0, [J, M], good, prog, [out.ptr])
    np.testing.assert_array_equal(out.get(), np.full(M * J, -float(KT), np.float32))
