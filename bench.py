#!/usr/bin/env python3
"""Benchmark of the operator hot path on one MI355X.

Workload (the elementwise+reduce microbenchmark, second of the five configurations): fp32 and
int32 tensors np[4096,16384] (tenncor shape {16384,4096}).  One step evaluates,
node by node as the reference does (every node materialises its output):
  fp32 : t1=ADD(a,b) t2=MUL(t1,c) t3=EXP(t2) t4=TANH(t3) t5=SIGMOID(t4),
         REDUCE_SUM and REDUCE_MAX of t5 over dim 0 and over dim 1
  int32: u1=ADD(x,y) u2=MUL(u1,z), REDUCE_SUM and REDUCE_MAX of u2 over each dim
`value` = algorithmic bytes of one step / time of one step, inputs resident in
HBM before the timed region.  Per-kernel durations are taken with HIP events
recorded on the launch stream inside the timed region.

Prints ONE JSON line.  Everything runs on one GPU; --gpus > 1 is refused.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
MFMA_F32_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix, published
MFMA_F64_PEAK_TFLOPS = 78.6  # MI355X dense fp64 matrix, published

ROWS, COLS = 4096, 16384
N = ROWS * COLS
SHAPE = [COLS, ROWS]  # tenncor order: dim 0 fastest

# Which kernels of the profile make up one launch of each kernel class of the step
CLASS_KERNELS = {
    "ew_binary_f32": ["ew_binary_vec_k<float, 30>", "ew_binary_vec_k<float, 32>"],
    "ew_binary_i32": ["ew_binary_vec_k<int, 30>", "ew_binary_vec_k<int, 32>"],
    "ew_unary_f32": ["ew_unary_vec_k<float, 7>", "ew_unary_vec_k<float, 11>", "ew_unary_vec_k<float, 12>"],
    "reduce_dim0_f32": ["reduce_inner_k<float, 17, true>", "reduce_inner_k<float, 20, true>"],
    "reduce_dim0_i32": ["reduce_inner_k<int, 17, true>", "reduce_inner_k<int, 20, true>"],
    "reduce_dim1_f32": ["reduce_outer_k<float, 17, true, 512, 4>", "reduce_outer_k<float, 20, true, 512, 4>"],
    "reduce_dim1_i32": ["reduce_outer_k<int, 17, true, 512, 4>", "reduce_outer_k<int, 20, true, 512, 4>"],
}
LAUNCHES_PER_STEP = {"ew_binary_f32": 2, "ew_unary_f32": 3, "reduce_dim0_f32": 2, "reduce_dim1_f32": 2,
                     "ew_binary_i32": 2, "reduce_dim0_i32": 2, "reduce_dim1_i32": 2}
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "config2_hbm_traffic_pmc.txt")


def measured_traffic(path=TRAFFIC_SUMMARY):
    """HBM bytes per launch of every kernel class, from the committed summary of
    two `rocprofv3 --pmc` runs of this script (FETCH_SIZE, then WRITE_SIZE, KiB
    per dispatch).  The summary states how many passes over the step the
    profiled command made and the factor each counter is scaled by (what it
    reads for the plain NEG copy of known size); its table gives the calls and
    the raw averages per kernel.  A class whose kernels are not all in the
    table (the kernels changed since the profile was taken) reports None."""
    try:
        text = open(path).read().splitlines()
    except OSError:
        return {}
    passes, scale_f, scale_w, rows = None, None, None, {}
    for line in text:
        parts = line.split()
        if line.startswith("passes:"):
            passes = int(parts[1])
        elif line.startswith("scale:"):
            scale_f, scale_w = float(parts[2]), float(parts[4])
        elif len(parts) >= 4 and parts[-1].replace(".", "").isdigit() and parts[-2].replace(".", "").isdigit() \
                and parts[-3].isdigit():
            rows[" ".join(parts[:-3])] = (int(parts[-3]), float(parts[-2]), float(parts[-1]))
    if not passes or scale_f is None:
        return {}
    out = {}
    for cls, names in CLASS_KERNELS.items():
        if not all(n in rows for n in names):
            out[cls] = None
            continue
        kib = sum(rows[n][0] * (rows[n][1] * scale_f + rows[n][2] * scale_w) for n in names)
        out[cls] = int(round(kib * 1024 / (passes * LAUNCHES_PER_STEP[cls])))
    return out


def algorithmic_bytes():
    """Per-kernel algorithmic bytes of one step (4-byte elements)."""
    e = 4
    return {
        "ew_binary_f32": 2 * 3 * e * N,                 # ADD, MUL
        "ew_unary_f32": 3 * 2 * e * N,                  # EXP, TANH, SIGMOID
        "reduce_dim0_f32": 2 * (e * N + e * ROWS),      # SUM, MAX -> {1,4096}
        "reduce_dim1_f32": 2 * (e * N + e * COLS),      # SUM, MAX -> {16384,1}
        "ew_binary_i32": 2 * 3 * e * N,
        "reduce_dim0_i32": 2 * (e * N + e * ROWS),
        "reduce_dim1_i32": 2 * (e * N + e * COLS),
    }


class Step:
    """Device-resident inputs and outputs of the config-2 graph."""

    def __init__(self, ctx, seed=2):
        from tenncor_amd import capi
        self.ctx, self.capi = ctx, capi
        rng = np.random.default_rng(seed)
        self.f = [ctx.upload(rng.uniform(-1, 1, N).astype(np.float32)) for _ in range(3)]
        self.i = [ctx.upload(rng.integers(-1000, 1001, N, dtype=np.int32)) for _ in range(3)]
        self.t = [ctx.empty(N, np.float32) for _ in range(5)]
        self.u = [ctx.empty(N, np.int32) for _ in range(2)]
        self.rf = [ctx.empty(ROWS, np.float32), ctx.empty(ROWS, np.float32),
                   ctx.empty(COLS, np.float32), ctx.empty(COLS, np.float32)]
        self.ri = [ctx.empty(ROWS, np.int32), ctx.empty(ROWS, np.int32),
                   ctx.empty(COLS, np.int32), ctx.empty(COLS, np.int32)]

    def launches(self):
        """(kernel class, thunk) in evaluation order."""
        c, F, I = self.ctx, self.capi.FLOAT, self.capi.INT32
        f, t, rf, i, u, ri = self.f, self.t, self.rf, self.i, self.u, self.ri
        return [
            ("ew_binary_f32", lambda: c.ew_binary("ADD", F, N, f[0].ptr, f[1].ptr, t[0].ptr)),
            ("ew_binary_f32", lambda: c.ew_binary("MUL", F, N, t[0].ptr, f[2].ptr, t[1].ptr)),
            ("ew_unary_f32", lambda: c.ew_unary("EXP", F, N, t[1].ptr, t[2].ptr)),
            ("ew_unary_f32", lambda: c.ew_unary("TANH", F, N, t[2].ptr, t[3].ptr)),
            ("ew_unary_f32", lambda: c.ew_unary("SIGMOID", F, N, t[3].ptr, t[4].ptr)),
            ("reduce_dim0_f32", lambda: c.reduce("REDUCE_SUM", F, SHAPE, [0], t[4].ptr, rf[0].ptr)),
            ("reduce_dim0_f32", lambda: c.reduce("REDUCE_MAX", F, SHAPE, [0], t[4].ptr, rf[1].ptr)),
            ("reduce_dim1_f32", lambda: c.reduce("REDUCE_SUM", F, SHAPE, [1], t[4].ptr, rf[2].ptr)),
            ("reduce_dim1_f32", lambda: c.reduce("REDUCE_MAX", F, SHAPE, [1], t[4].ptr, rf[3].ptr)),
            ("ew_binary_i32", lambda: c.ew_binary("ADD", I, N, i[0].ptr, i[1].ptr, u[0].ptr)),
            ("ew_binary_i32", lambda: c.ew_binary("MUL", I, N, u[0].ptr, i[2].ptr, u[1].ptr)),
            ("reduce_dim0_i32", lambda: c.reduce("REDUCE_SUM", I, SHAPE, [0], u[1].ptr, ri[0].ptr)),
            ("reduce_dim0_i32", lambda: c.reduce("REDUCE_MAX", I, SHAPE, [0], u[1].ptr, ri[1].ptr)),
            ("reduce_dim1_i32", lambda: c.reduce("REDUCE_SUM", I, SHAPE, [1], u[1].ptr, ri[2].ptr)),
            ("reduce_dim1_i32", lambda: c.reduce("REDUCE_MAX", I, SHAPE, [1], u[1].ptr, ri[3].ptr)),
        ]


def run_gpu(steps, warmup, graphs=True):
    from tenncor_amd import capi
    ctx = capi.Context(0)
    st = Step(ctx)
    launches = st.launches()
    for _ in range(warmup):
        for _, fn in launches:
            fn()
    ctx.sync()
    # one event before and after every launch, all on the launch stream
    events = [[ctx.event() for _ in range(len(launches) + 1)] for _ in range(steps)]
    t0 = time.perf_counter()
    for s in range(steps):
        ctx.record(events[s][0])
        for k, (_, fn) in enumerate(launches):
            fn()
            ctx.record(events[s][k + 1])
    ctx.sync()
    wall = time.perf_counter() - t0
    per_class = {}
    for s in range(steps):
        for k, (name, _) in enumerate(launches):
            per_class.setdefault(name, []).append(ctx.elapsed_ms(events[s][k], events[s][k + 1]))
    for evs in events:
        for ev in evs:
            ctx.event_destroy(ev)
    extra = run_extras(ctx, capi)
    arch = ctx.arch
    ctx.close()
    if graphs:
        extra.update(run_graph_configs())
    return wall, per_class, extra, arch


def run_extras(ctx, capi):
    """The other parts of the metric triple: fused chain, fp32 MATMUL, PERMUTE."""
    extra = {}
    # fused chain: 3 leaf reads + 1 write
    rng = np.random.default_rng(22)
    leaves = [ctx.upload(rng.uniform(-1, 1, N).astype(np.float32)) for _ in range(3)]
    out = ctx.empty(N, np.float32)
    # the chain as one group launch (the kernel is compiled for the program on first use)
    L, R, NONE = capi.FX_LEAF0, capi.FX_REG0, capi.FX_NONE
    group = [("ADD", L, L + 1, NONE, R), ("MUL", R, L + 2, NONE, R), ("EXP", R, NONE, NONE, R),
             ("TANH", R, NONE, NONE, R), ("SIGMOID", R, NONE, NONE, R), ("STORE", R, NONE, NONE, 0)]
    reps = 10
    runs = {
        "fused_chain": lambda: ctx.ew_fusedx(capi.FLOAT, [COLS, ROWS], [{"ptr": b.ptr} for b in leaves], group, [out.ptr]),
    }
    for key, fn in runs.items():
        for _ in range(2):
            fn()
        ctx.timer_begin()
        for _ in range(reps):
            fn()
        ms = ctx.timer_end() / reps
        extra[key + "_GBps"] = round(4 * 4 * N / (ms * 1e-3) / 1e9, 1)
        extra[key + "_ms"] = round(ms, 4)
    # plain streaming copy (NEG: N floats in, N floats out), the known-size kernel
    # that hardware byte counters are scaled by
    for _ in range(2):
        ctx.ew_unary("NEG", capi.FLOAT, N, leaves[0].ptr, out.ptr)
    ctx.timer_begin()
    for _ in range(reps):
        ctx.ew_unary("NEG", capi.FLOAT, N, leaves[0].ptr, out.ptr)
    ms = ctx.timer_end() / reps
    extra["copy_GBps"] = round(2 * 4 * N / (ms * 1e-3) / 1e9, 1)
    for b in leaves + [out]:
        b.release()
    # 4096^3 fp32 MATMUL (configs[2])
    M = 4096
    a = ctx.upload((rng.standard_normal(M * M) / 64).astype(np.float32))
    b = ctx.upload((rng.standard_normal(M * M) / 64).astype(np.float32))
    c = ctx.empty(M * M, np.float32)
    reps = 20
    extra.update(time_matmul_4096(ctx, capi, a, b, c, settle=40, reps=reps))
    # the same product in double (v_mfma_f64_16x16x4_f64)
    M2 = 4096
    a64 = ctx.upload(rng.standard_normal(M2 * M2) / 64)
    b64 = ctx.upload(rng.standard_normal(M2 * M2) / 64)
    c64 = ctx.empty(M2 * M2, np.float64)
    for _ in range(10):
        ctx.matmul(capi.DOUBLE, [M2, M2], [M2, M2], a64.ptr, b64.ptr, c64.ptr)
    ctx.timer_begin()
    for _ in range(reps):
        ctx.matmul(capi.DOUBLE, [M2, M2], [M2, M2], a64.ptr, b64.ptr, c64.ptr)
    ms = ctx.timer_end() / reps
    tf = 2.0 * M2 ** 3 / (ms * 1e-3) / 1e12
    extra["matmul_4096_fp64_TFLOPs"] = round(tf, 2)
    extra["matmul_4096_frac_of_fp64_mfma_peak"] = round(tf / MFMA_F64_PEAK_TFLOPS, 4)
    for buf in (a64, b64, c64):
        buf.release()
    # PERMUTE of the result (HBM-bound)
    d = ctx.empty(M * M, np.float32)
    order = [1, 0, 2, 3, 4, 5, 6, 7]
    for _ in range(2):
        ctx.permute(capi.FLOAT, [M, M], order, c.ptr, d.ptr)
    ctx.timer_begin()
    for _ in range(reps):
        ctx.permute(capi.FLOAT, [M, M], order, c.ptr, d.ptr)
    ms = ctx.timer_end() / reps
    extra["permute_4096_GBps"] = round(2 * 4 * M * M / (ms * 1e-3) / 1e9, 1)
    for buf in (a, b, c, d):
        buf.release()
    # batched CONTRACT np[64,512,512] x np[64,512,512] + PERMUTE {1,0,2} (configs[2])
    nb, m = 64, 512
    a = ctx.upload((rng.standard_normal(nb * m * m) / np.sqrt(m)).astype(np.float32))
    b = ctx.upload((rng.standard_normal(nb * m * m) / np.sqrt(m)).astype(np.float32))
    c = ctx.empty(nb * m * m, np.float32)
    d = ctx.empty(nb * m * m, np.float32)
    # (300 untimed launches: the same 40 ms of matrix work that settle the clock before
    # the 4096^3 product is timed; 40 launches, 6 ms, read 107-110 TFLOP/s on the way up)
    for _ in range(300):
        ctx.matmul(capi.FLOAT, [m, m, nb], [m, m, nb], a.ptr, b.ptr, c.ptr)
    ctx.timer_begin()
    for _ in range(reps):
        ctx.matmul(capi.FLOAT, [m, m, nb], [m, m, nb], a.ptr, b.ptr, c.ptr)
    ms = ctx.timer_end() / reps
    extra["matmul_64x512_fp32_TFLOPs"] = round(nb * 2.0 * m ** 3 / (ms * 1e-3) / 1e12, 2)
    extra["matmul_64x512_untimed_launches_before"] = 300
    order = [1, 0, 2, 3, 4, 5, 6, 7]
    for _ in range(2):
        ctx.permute(capi.FLOAT, [m, m, nb], order, c.ptr, d.ptr)
    ctx.timer_begin()
    for _ in range(reps):
        ctx.permute(capi.FLOAT, [m, m, nb], order, c.ptr, d.ptr)
    ms = ctx.timer_end() / reps
    extra["permute_64x512_GBps"] = round(2 * 4 * nb * m * m / (ms * 1e-3) / 1e9, 1)
    for buf in (a, b, c, d):
        buf.release()
    return extra


def time_matmul_4096(ctx, capi, a, b, c, settle, reps):
    """`reps` 4096^3 fp32 products timed with HIP events on the launch stream,
    after `settle` untimed ones: the matrix clock takes some 30 ms of matrix
    work to settle after streaming kernels."""
    M = 4096
    for _ in range(settle):
        ctx.matmul(capi.FLOAT, [M, M], [M, M], a.ptr, b.ptr, c.ptr)
    ctx.timer_begin()
    for _ in range(reps):
        ctx.matmul(capi.FLOAT, [M, M], [M, M], a.ptr, b.ptr, c.ptr)
    ms = ctx.timer_end() / reps
    flops = 2 * M ** 3
    tf = flops / (ms * 1e-3) / 1e12
    return {
        "matmul_4096_fp32_TFLOPs": round(tf, 2), "matmul_4096_fp32_ms": round(ms, 4),
        "matmul_4096_frac_of_fp32_mfma_peak": round(tf / MFMA_F32_PEAK_TFLOPS, 4),
        "roofline_matmul": {"bound": "mfma", "kernel": "gemm_mfma_direct_k (128 x 128 tiles, slabs from memory straight into LDS) on 4096^3 fp32",
                            "flops": flops, "avg_ms": round(ms, 4), "achieved": round(tf, 2),
                            "peak": MFMA_F32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / MFMA_F32_PEAK_TFLOPS, 4),
                            "launches": reps, "untimed_launches_before": settle},
    }


def run_matmul_only(settle=100, reps=100, f64=False, batched=None):
    """The product third of the metric alone: nothing but 4096^3 fp32 launches in
    the process, so that a kernel trace or a counter run of this command holds
    one kernel at one shape.  f64: the same product in double (not part of the
    metric; its line has no roofline_matmul object).  batched = (count, size):
    the batched CONTRACT of configs[2] alone (the untimed launches settle the
    matrix clock: 300 of 64 x 512^3 are 45 ms of matrix work)."""
    from tenncor_amd import capi
    ctx = capi.Context(0)
    M = 4096
    rng = np.random.default_rng(3)
    if batched:
        nb, m = batched
        a = ctx.upload((rng.standard_normal(nb * m * m) / np.sqrt(m)).astype(np.float32))
        b = ctx.upload((rng.standard_normal(nb * m * m) / np.sqrt(m)).astype(np.float32))
        c = ctx.empty(nb * m * m, np.float32)
        shape = [m, m, nb]
        for _ in range(settle):
            ctx.matmul(capi.FLOAT, shape, shape, a.ptr, b.ptr, c.ptr)
        ctx.timer_begin()
        for _ in range(reps):
            ctx.matmul(capi.FLOAT, shape, shape, a.ptr, b.ptr, c.ptr)
        ms = ctx.timer_end() / reps
        tf = nb * 2.0 * m ** 3 / (ms * 1e-3) / 1e12
        out = {"matmul_batched": "%d x %d^3 fp32" % (nb, m), "TFLOPs": round(tf, 2), "ms": round(ms, 4),
               "frac_of_fp32_mfma_peak": round(tf / MFMA_F32_PEAK_TFLOPS, 4), "launches": reps,
               "untimed_launches_before": settle, "device": ctx.arch}
        ctx.close()
        return out
    if f64:
        a = ctx.upload(rng.standard_normal(M * M) / 64)
        b = ctx.upload(rng.standard_normal(M * M) / 64)
        c = ctx.empty(M * M, np.float64)
        for _ in range(settle):
            ctx.matmul(capi.DOUBLE, [M, M], [M, M], a.ptr, b.ptr, c.ptr)
        ctx.timer_begin()
        for _ in range(reps):
            ctx.matmul(capi.DOUBLE, [M, M], [M, M], a.ptr, b.ptr, c.ptr)
        ms = ctx.timer_end() / reps
        tf = 2 * M ** 3 / (ms * 1e-3) / 1e12
        out = {"matmul_4096_fp64_TFLOPs": round(tf, 2), "matmul_4096_fp64_ms": round(ms, 4),
               "matmul_4096_frac_of_fp64_mfma_peak": round(tf / MFMA_F64_PEAK_TFLOPS, 4),
               "launches": reps, "untimed_launches_before": settle, "device": ctx.arch}
        ctx.close()
        return out
    a = ctx.upload((rng.standard_normal(M * M) / 64).astype(np.float32))
    b = ctx.upload((rng.standard_normal(M * M) / 64).astype(np.float32))
    c = ctx.empty(M * M, np.float32)
    out = time_matmul_4096(ctx, capi, a, b, c, settle, reps)
    out["device"] = ctx.arch
    ctx.close()
    return out


def run_graph_configs(only=None, evaluator=None, reps=20, optimize=False):
    """configs[0], [3], [4] through the host graph layer (Functor nodes, the
    gradient builder, teq::Evaluator + eigen::Device): wall time of
    evaluate(targets) after re-assigning the input, which forces a full
    recompute (the recipe of tenncor/bm/benchmark.cpp:377-391)."""
    from tenncor_amd import graph as tg, configs
    out = {}
    rng = np.random.default_rng(0)

    def timed(g, targets, x, fresh, reps, resident=True, warm=2):
        """resident: the new input is on the device when the clock starts (tcr_prefetch: the
        host-to-device copy that `assign` makes necessary happens before the timed region, as
        for the headline value); False: the evaluation makes the copy, as it does for a caller
        who assigns and evaluates."""
        for _ in range(warm):
            g.assign(x, fresh())
            g.evaluate(targets)
        g.sync()
        ts = []
        for _ in range(reps):
            g.assign(x, fresh())
            if resident:
                g.prefetch(x)
                g.sync()
            t0 = time.perf_counter()
            g.evaluate(targets)
            g.sync()
            ts.append(time.perf_counter() - t0)
        return float(np.median(ts))

    # no suffix: the evaluator a context gets when nothing was registered (teq::get_eval's
    # default: the one that records a target set's launches on its second pass and enqueues
    # the recording afterwards); "_walk": teq::Evaluator, the node-by-node walk
    kinds = (("default", ""), ("plain", "_walk")) if evaluator is None else ((evaluator, ""),)
    for kind, tag in kinds:
        tg.set_evaluator(kind)
        replays = kind != "plain"
        if only is not None:
            # one configuration under one evaluator (the form profiles are taken in)
            g = tg.Graph()
            if only == 1:
                targets, x, _ = configs.config1_mlp(g)
            elif only == 4:
                targets, x, _, flops = configs.config4_lstm(g)
                xs = rng.uniform(-1, 1, 256 * 64 * 256).astype(np.float32)
                fresh = lambda: xs
            else:
                targets, x, _, flops = configs.config5_cnn(g)
                xs = rng.uniform(0, 1, 128 * 28 * 28).astype(np.float32)
                fresh = lambda: xs
            if only == 1:
                fresh, reps = (lambda: rng.uniform(-1, 1, 30).astype(np.float32)), 300
            cleanup = None
            if optimize:
                # hone::optimize first: equal subgraphs merged, constants folded,
                # the shipped conversions applied
                targets, cleanup = g.optimize(targets)
            # (the 120 bytes of config 1's input travel in the launch arguments: nothing to prefetch)
            t = timed(g, targets, x, fresh, reps, resident=only != 1, warm=2 if only == 1 else 10)
            out = {"graph_config": only, "evaluator": kind, "ms_per_eval": round(t * 1e3, 4),
                   "functors": g.count_functors(targets), "evaluator_stats": tg.evaluator_stats()}
            if cleanup is not None:
                out["optimize"] = cleanup
            if kind == "timing":
                out["timing_report"] = tg.evaluator_timing().splitlines()
            tg.set_evaluator("default")
            return out
        g = tg.Graph()
        targets, x, _ = configs.config1_mlp(g)
        t = timed(g, targets, x, lambda: rng.uniform(-1, 1, 30).astype(np.float32), 300, resident=False)
        out["config1_mlp%s_evals_per_sec" % tag] = round(1.0 / t, 1)
        out["config1_mlp%s_us_per_eval" % tag] = round(t * 1e6, 1)
        out["config1_mlp_functors"] = g.count_functors(targets)
        def recording_cost(name):
            # what the first passes cost and no timed pass shows: planning, kernels compiled
            # at run time (or loaded from the files an earlier process left), the capture
            st = tg.evaluator_stats()
            out[name + "_record_ms"] = st["record_ms"]
            out[name + "_record_jit"] = {"ms": st["jit_ms"], "compiled": st["jit_compiled"], "from_disk": st["jit_from_disk"]}

        if replays:
            recording_cost("config1_mlp")
            out["config1_mlp_launches_per_eval"] = tg.evaluator_stats()["launches"]
        g.close()
        if replays:
            # the same recording kept launch by launch (bit-identical to the walk)
            tg.set_evaluator("replay_launches")
            g = tg.Graph()
            targets, x, _ = configs.config1_mlp(g)
            t = timed(g, targets, x, lambda: rng.uniform(-1, 1, 30).astype(np.float32), 300, resident=False)
            out["config1_mlp_launch_by_launch_us_per_eval"] = round(t * 1e6, 1)
            g.close()
            tg.set_evaluator(kind)

        g = tg.Graph()
        targets, x, _, flops = configs.config4_lstm(g)
        xs = rng.uniform(-1, 1, 256 * 64 * 256).astype(np.float32)
        # medians over enough passes for the clocks to settle (a recorded pass takes 4 ms, a walked one 14)
        t = timed(g, targets, x, lambda: xs, 40 if replays else 10, warm=10 if replays else 2)
        out["config4_lstm%s_ms_per_step" % tag] = round(t * 1e3, 3)
        out["config4_lstm%s_gemm_TFLOPs" % tag] = round(flops / t / 1e12, 2)
        # the same with the 16.8 MB input copied to the device inside the timed evaluation
        t = timed(g, targets, x, lambda: xs, 20 if replays else 5, resident=False)
        out["config4_lstm%s_ms_per_step_with_input_upload" % tag] = round(t * 1e3, 3)
        out["config4_lstm_functors"] = g.count_functors(targets)
        if replays:
            recording_cost("config4_lstm")
            out["config4_lstm_launches"] = tg.evaluator_stats()["launches"]
        g.close()

        g = tg.Graph()
        targets, x, _, flops = configs.config5_cnn(g)
        xs = rng.uniform(0, 1, 128 * 28 * 28).astype(np.float32)
        t = timed(g, targets, x, lambda: xs, 60 if replays else 20, warm=20 if replays else 2)
        out["config5_cnn%s_ms_per_step" % tag] = round(t * 1e3, 3)
        out["config5_cnn%s_useful_TFLOPs" % tag] = round(flops / t / 1e12, 3)
        t = timed(g, targets, x, lambda: xs, 30 if replays else 10, resident=False)
        out["config5_cnn%s_ms_per_step_with_input_upload" % tag] = round(t * 1e3, 3)
        out["config5_cnn_functors"] = g.count_functors(targets)
        if replays:
            recording_cost("config5_cnn")
            out["config5_cnn_launches"] = tg.evaluator_stats()["launches"]
        g.close()
    tg.set_evaluator("default")
    out["graph_timing"] = ("evaluate(targets) + sync after the input was re-assigned; the new input is on the device when the "
                           "clock starts (tcr_prefetch), *_with_input_upload leaves the copy to the evaluation")
    out["default_evaluator"] = "replay (teq::get_eval registers eigen::ReplayEvaluator; TCR_EVAL_PLAIN=1 keeps the walk)"
    return out


def run_cpu_baseline():
    """The oracle (a scalar C port of the reference semantics) on one host core,
    on a row slab of the same workload sized for roughly 10-30 s."""
    from oracle import oracle as orc
    orc.build()
    rows = ROWS  # the whole tensor: about 15 s on one core
    n = rows * COLS
    shape = [COLS, rows]
    rng = np.random.default_rng(2)
    f = [rng.uniform(-1, 1, n).astype(np.float32) for _ in range(3)]
    i = [rng.integers(-1000, 1001, n, dtype=np.int32) for _ in range(3)]
    e = 4
    nbytes = (2 * 3 + 3 * 2) * e * n + 2 * (e * n + e * rows) + 2 * (e * n + e * COLS)
    nbytes += 2 * 3 * e * n + 2 * (e * n + e * rows) + 2 * (e * n + e * COLS)
    def one_pass(lo, hi):
        """The whole graph on rows [lo, hi) of every operand."""
        sl = slice(lo * COLS, hi * COLS)
        shp = [COLS, hi - lo]
        t = orc.binary("ADD", f[0][sl], f[1][sl])
        t = orc.binary("MUL", t, f[2][sl])
        t = orc.unary("EXP", t)
        t = orc.unary("TANH", t)
        t = orc.unary("SIGMOID", t)
        for op in ("REDUCE_SUM", "REDUCE_MAX"):
            orc.reduce(op, t, shp, [0])
            orc.reduce(op, t, shp, [1])
        u = orc.binary("ADD", i[0][sl], i[1][sl])
        u = orc.binary("MUL", u, i[2][sl])
        for op in ("REDUCE_SUM", "REDUCE_MAX"):
            orc.reduce(op, u, shp, [0])
            orc.reduce(op, u, shp, [1])

    passes = 0
    t0 = time.perf_counter()
    while passes < 1 or (time.perf_counter() - t0 < 10.0 and passes < 16):
        one_pass(0, rows)
        passes += 1
    dt = time.perf_counter() - t0
    # the same port on every host core this process may use: row slabs evaluated
    # side by side (the C routines release the interpreter lock).  The
    # reference itself has no thread pool; this is only the ceiling of the port.
    from concurrent.futures import ThreadPoolExecutor
    cores = max(1, min(int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1), 64))
    bounds = [rows * k // cores for k in range(cores + 1)]
    mpasses = 0
    t1 = time.perf_counter()
    with ThreadPoolExecutor(max_workers=cores) as pool:
        while mpasses < 1 or (time.perf_counter() - t1 < 5.0 and mpasses < 64):
            list(pool.map(lambda k: one_pass(bounds[k], bounds[k + 1]), range(cores)))
            mpasses += 1
    mdt = time.perf_counter() - t1
    # the product part of the metric: the port's triple loop on one core, and the
    # host's BLAS (numpy) on the same operands as the figure an optimised CPU
    # library reaches (the reference multiplies through Eigen's blocked kernel)
    m = 1024
    a = (rng.standard_normal(m * m) / 32).astype(np.float32)
    b = (rng.standard_normal(m * m) / 32).astype(np.float32)
    t2 = time.perf_counter()
    orc.matmul(a, [m, m], b, [m, m])
    port_dt = time.perf_counter() - t2
    # the host's BLAS at the metric's own size (the port's triple loop would take
    # five minutes there, so it keeps its 1024^3 sample)
    mb = 4096
    a2 = (rng.standard_normal(mb * mb) / 64).astype(np.float32).reshape(mb, mb)
    b2 = (rng.standard_normal(mb * mb) / 64).astype(np.float32).reshape(mb, mb)
    a2 @ b2
    blas_reps = 3
    t3 = time.perf_counter()
    for _ in range(blas_reps):
        a2 @ b2
    blas_dt = (time.perf_counter() - t3) / blas_reps
    matmul = {"port_GFLOPs": round(2.0 * m ** 3 / port_dt / 1e9, 2), "cores": 1,
              "port_sample": "fp32 %d^3, the oracle's triple loop (the metric's product is 4096^3)" % m,
              "host_blas_GFLOPs": round(2.0 * mb ** 3 / blas_dt / 1e9, 1), "host_blas_cores": cores,
              "host_blas_ms": round(blas_dt * 1e3, 1),
              "host_blas_sample": "fp32 %d^3 through numpy's BLAS, mean of %d (the reference multiplies "
                                  "through Eigen's blocked kernel)" % (mb, blas_reps)}
    return {
        "matmul": matmul,
        "graphs": run_cpu_graph_baseline(matmul["port_GFLOPs"], cores),
        "value": round(passes * nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": "the same graph on np[%d,%d] (the whole workload), %d passes, %.1f s single-thread"
                  % (rows, COLS, passes, dt),
        "all_cores": {"value": round(mpasses * nbytes / mdt / 1e9, 3), "unit": "GB/s", "cores": cores,
                      "sample": "row slabs of the same workload on %d threads, %d passes, %.1f s" % (cores, mpasses, mdt)},
    }


def run_cpu_graph_baseline(port_gflops, cores):
    """The graph third of the metric on the host (tenncor/bm/benchmark.cpp:334-393:
    re-assign the input, time evaluate).  configs[0]: the whole graph, node by
    node in the evaluator's order, every node by the oracle's scalar routine,
    inside one C call (oracle/graph_tape.c), one core -- the reference's
    evaluator is single-threaded too.  configs[3] and [4]: their matrix
    products at full size through the host's BLAS (what an optimised CPU
    library reaches; the reference multiplies through Eigen's blocked kernel
    on one core), the port's triple loop extrapolated from its measured rate,
    and the whole graph on the port at reduced size."""
    from tenncor_amd import graph as tg, configs
    from oracle import graph_tape
    out = {}
    rng = np.random.default_rng(0)
    g = tg.Graph()
    targets, x, _ = configs.config1_mlp(g)
    tape = graph_tape.Tape(g, targets)
    tape.run(200)
    secs = []
    for _ in range(10):
        tape.set(x, rng.uniform(-1, 1, 30).astype(np.float32))
        secs += tape.run(200)
    us = float(np.median(secs)) * 1e6
    out["config1_mlp"] = {"us_per_eval": round(us, 2), "evals_per_sec": round(1e6 / us, 1), "cores": 1, "kind": "port",
                          "sample": "the whole graph (%d functors), 2000 evaluations, median" % tape.nops}
    g.close()

    def blas_ms(shapes, reps=2):
        mats = [(rng.standard_normal((m, k)).astype(np.float32), rng.standard_normal((k, n)).astype(np.float32)) for m, k, n, _ in shapes]
        for a, b in mats:
            a @ b
        t0 = time.perf_counter()
        for _ in range(reps):
            for (a, b), (_, _, _, count) in zip(mats, shapes):
                for _ in range(count):
                    a @ b
        return (time.perf_counter() - t0) / reps * 1e3

    # configs[3]: per time step the gate product [x_t, h] W, its transpose-weight product
    # backwards and its weight-gradient term, 64 steps (the walk multiplies all 768 columns back)
    shapes4 = [(256, 768, 2048, 64), (256, 2048, 768, 64), (768, 256, 2048, 64)]
    flops4 = sum(2.0 * m * k * n * c for m, k, n, c in shapes4)
    ms4 = blas_ms(shapes4, reps=1)
    g = tg.Graph()
    small = dict(seq=8, batch=32, nin=32, hid=64)
    targets, x, _, small_flops = configs.config4_lstm(g, **small)
    tape = graph_tape.Tape(g, targets)
    small_ms = float(np.median(tape.run(5))) * 1e3
    out["config4_lstm"] = {
        "products_host_blas_ms": round(ms4, 1), "products_host_blas_GFLOPs": round(flops4 / ms4 / 1e6, 1), "host_blas_cores": cores,
        "products_port_extrapolated_s": round(flops4 / (port_gflops * 1e9), 1), "port_cores": 1,
        "sample": "the 192 products of the configuration at full size (%.1f GFLOP) through numpy's BLAS; the port's time is "
                  "that work at the rate of its 1024^3 product" % (flops4 / 1e9),
        "reduced_graph_on_port": {"ms_per_eval": round(small_ms, 2), "functors": tape.nops, "size": small,
                                  "product_GFLOP": round(small_flops / 1e9, 4)}}
    g.close()
    # configs[4]: the convolutions of both layers as the products they lower to (forward, image
    # gradient of the second layer as executed, both kernel gradients)
    shapes5 = [(73728, 25, 32, 1), (51200, 800, 64, 1), (73728, 1600, 32, 1), (800, 51200, 64, 1), (25, 73728, 32, 1)]
    flops5 = sum(2.0 * m * k * n * c for m, k, n, c in shapes5)
    ms5 = blas_ms(shapes5, reps=2)
    g = tg.Graph()
    small = dict(batch=4, hw=16, c1=8, c2=8, ncls=10)
    targets, x, _, small_flops = configs.config5_cnn(g, **small)
    tape = graph_tape.Tape(g, targets)
    small_ms = float(np.median(tape.run(3))) * 1e3
    out["config5_cnn"] = {
        "products_host_blas_ms": round(ms5, 2), "products_host_blas_GFLOPs": round(flops5 / ms5 / 1e6, 1), "host_blas_cores": cores,
        "products_port_extrapolated_s": round(flops5 / (port_gflops * 1e9), 1), "port_cores": 1,
        "sample": "the five products the convolutions lower to at batch 128 (%.1f GFLOP, operands already gathered) through "
                  "numpy's BLAS" % (flops5 / 1e9),
        "reduced_graph_on_port": {"ms_per_eval": round(small_ms, 2), "functors": tape.nops, "size": small,
                                  "useful_GFLOP": round(small_flops / 1e9, 4),
                                  "note": "the port evaluates the padded convolutions of the conv2d idiom literally"}}
    g.close()
    return out


def run_matmul_ramp(blocks=12, per_block=10):
    """4096^3 fp32 products back to back from a cold start, timed in blocks of
    ten: how long the matrix clock takes to settle (the reason the product
    metric above is taken after 40 untimed launches)."""
    from tenncor_amd import capi
    ctx = capi.Context(0)
    n = 4096
    rng = np.random.default_rng(3)
    a = ctx.upload((rng.standard_normal(n * n) / 64).astype(np.float32))
    b = ctx.upload((rng.standard_normal(n * n) / 64).astype(np.float32))
    c = ctx.empty(n * n, np.float32)
    out = []
    for _ in range(blocks):
        ctx.timer_begin()
        for _ in range(per_block):
            ctx.matmul(capi.FLOAT, [n, n], [n, n], a.ptr, b.ptr, c.ptr)
        ms = ctx.timer_end() / per_block
        out.append(round(2.0 * n ** 3 / (ms * 1e-3) / 1e12, 1))
    return {"matmul_4096_fp32_TFLOPs_per_block_of_%d" % per_block: out}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graphs", action="store_true", help="skip the whole-graph side metrics (configs 1, 4, 5)")
    ap.add_argument("--graph-config", type=int, choices=[1, 4, 5], default=None,
                    help="time only this whole-graph configuration and print its line (for profiling)")
    ap.add_argument("--evaluator", choices=["default", "plain", "replay", "replay_launches", "replay_unfused", "timing"], default="replay",
                    help="with --graph-config; timing: the recording's launches run one by one between HIP events, "
                         "device microseconds per kind of launch in the line's timing_report")
    ap.add_argument("--f64", action="store_true", help="with --matmul-only: the 4096^3 product in double")
    ap.add_argument("--batched", default=None, metavar="COUNTxSIZE",
                    help="with --matmul-only: COUNT products of SIZE^3 in one launch (64x512 is the batched CONTRACT of configs[2])")
    ap.add_argument("--reps", type=int, default=None,
                    help="timed evaluations with --graph-config 4 or 5 (default 20), timed launches with --matmul-only (100)")
    ap.add_argument("--optimize", action="store_true",
                    help="with --graph-config: clean the graph up first (duplicates merged, constants folded, conversions)")
    ap.add_argument("--matmul-only", action="store_true",
                    help="run only 4096^3 fp32 products (--settle untimed, then --reps timed) and print their line")
    ap.add_argument("--settle", type=int, default=100, help="untimed launches before the timed ones with --matmul-only")
    ap.add_argument("--matmul-ramp", action="store_true",
                    help="print the 4096^3 product rate of successive blocks of ten launches from a cold start")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this backend runs on one GPU; --gpus %d is not supported "
                 "(no collectives or sharding are part of this build)" % args.gpus)

    if args.matmul_ramp:
        print(json.dumps(run_matmul_ramp()))
        return
    if args.matmul_only:
        batched = tuple(int(v) for v in args.batched.lower().split("x")) if args.batched else None
        print(json.dumps(run_matmul_only(settle=args.settle, reps=args.reps or 100, f64=args.f64, batched=batched)))
        return
    if args.graph_config is not None:
        print(json.dumps(run_graph_configs(only=args.graph_config, evaluator=args.evaluator, reps=args.reps or 20, optimize=args.optimize)))
        return
    wall, per_class, extra, arch = run_gpu(args.steps, args.warmup, graphs=not args.no_graphs)
    abytes = algorithmic_bytes()
    launches_per_step = LAUNCHES_PER_STEP
    total_bytes = sum(abytes.values())
    ms_per_step = wall * 1e3 / args.steps
    value = total_bytes / (wall / args.steps) / 1e9
    kernels = {}
    for name, times in per_class.items():
        avg_ms = float(np.mean(times))
        per_launch = abytes[name] / launches_per_step[name]
        kernels[name] = {"avg_ms": round(avg_ms, 4), "GBps": round(per_launch / (avg_ms * 1e-3) / 1e9, 1),
                         "frac": round(per_launch / (avg_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    dominant = max(kernels, key=lambda k: kernels[k]["avg_ms"] * launches_per_step[k])
    dom = kernels[dominant]
    result = {
        "metric": "graph evals/sec; elementwise+reduce HBM GB/s; fp32 MATMUL TFLOP/s",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32+i32", "data": "synthetic",
        "config": {"workload": "configs[1]: elementwise+reduce microbench, fp32 and int32 np[4096,16384], "
                               "node-by-node (ADD,MUL,EXP,TANH,SIGMOID + REDUCE_SUM/MAX over each dim; "
                               "int32 ADD,MUL + the same reductions)",
                   "algorithmic_bytes_per_step": total_bytes, "device": arch},
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": dom["GBps"], "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": dom["frac"], "traffic": measured_traffic().get(dominant),
                     "traffic_source": "profiles/config2_hbm_traffic_pmc.txt"},
        "roofline_matmul": extra.pop("roofline_matmul", None),
        "kernels": kernels,
        "extra": extra,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = run_cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
