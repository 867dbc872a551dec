/*
 * tcg.h -- C ABI of the MI355X (gfx950) evaluation backend for tenncor
 * operator graphs.
 *
 * The tenncor reference has no FFI on this path: its seam is the C++ pair
 * `egen::typed_exec<T>(opcode, out, outshape, in, attrib)` (generated from
 * cfg/ops.yml:6 by tools/egen/plugins/opcodes.py:36-46), which builds one
 * Eigen closure per graph node, and `eigen::Device::calc`
 * (internal/eigen/device.hpp:546-576), which runs it into a buffer borrowed
 * from `eigen::iRuntimeMemory` (internal/eigen/memory.hpp:14-22).  Every entry
 * point below is what one `stmt` of cfg/ops.yml binds to once the Eigen
 * closure is replaced by a stream-ordered GPU launch; the comment on each
 * names the statement and the Eigen call site it replaces.
 *
 * Conventions
 *   - all functions return 0 (TCG_OK) or a tcg_status; no C++ exception
 *     crosses this boundary; tcg_last_error() gives the message
 *   - shapes are uint64_t[8] in tenncor order: dim 0 is the fastest-varying
 *     dim, unused dims are 1 (internal/teq/shape.hpp:56-59)
 *   - dtype codes: 1 double, 2 float, 3 int32 (the order of cfg/mintype.yml:4-13,
 *     the default build's types), then the integer widths the full build adds
 *     (cfg/fulltype.yml:11-34): 4 int8, 5 uint8, 6 int16, 7 uint16, 8 uint32,
 *     9 int64, 10 uint64.  These codes are this library's and do not move
 *     with the host layer's build switch (whose own enum follows the yaml it
 *     is built for).  Integer arithmetic wraps modulo 2^width
 *   - opcodes are the values of egen::_GENERATED_OPCODE, i.e. the key order
 *     of cfg/ops.yml with BAD_OP = 0 (tools/egen/plugins/opcodes.py:16-22)
 *   - data pointers are DEVICE pointers (from tcg_alloc, or any HIP device
 *     allocation of the same device); element offsets into them are allowed
 *     (the reference aliases last-dim slices by pointer offset,
 *     internal/eigen/operator.hpp:231-248)
 *   - every launch is ordered on the context's single stream; one host thread
 *     per context (the reference evaluates single-threaded)
 *   - the library never falls back to the CPU: if no gfx950 device is present
 *     tcg_ctx_create fails
 */
#ifndef TCG_H
#define TCG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TCG_RANK_CAP 8

typedef struct tcg_ctx tcg_ctx;

enum tcg_status
{
	TCG_OK = 0,
	TCG_ERR_ARG = 1,         /* argument the reference would reject at node construction */
	TCG_ERR_HIP = 2,         /* a HIP runtime call failed */
	TCG_ERR_UNSUPPORTED = 3, /* opcode/dtype combination not implemented on the device */
	TCG_ERR_OOM = 4
};

/* Element types.  1..3 are the reference's default configuration in its own
 * numbering (cfg/mintype.yml:4-13); 4..10 are the integer widths its full
 * configuration adds (cfg/fulltype.yml:11-34), which the reference numbers in
 * another order (the enum it generates follows the key order of the file): a
 * binding built for that configuration maps its codes onto these.  Integer
 * arithmetic wraps modulo 2^width; integer division by zero, and the lowest
 * value of a 32- or 64-bit type divided by -1 (both trap on the CPU), give 0.
 * The transcendental operators of an integer type (SIN .. SIGMOID, TANH, and
 * POW through its repeated multiplication) go through double and convert back
 * the way the reference's `(T) std::exp(x)` does: the double becomes an integer
 * of 32 bits (64 for the 64-bit types) of the type's signedness, which is then
 * narrowed.  Where the double does not fit that integer -- EXP of more than 21
 * (signed) or 22 (unsigned), 43 / 44 for the 64-bit types, and SIGMOID of less
 * than minus those -- C++ leaves the conversion undefined and the results are
 * unspecified here too (the device saturates where x86 gives its indefinite
 * value); inside those bounds device and CPU agree. */
enum tcg_dtype
{
	TCG_BAD_TYPE = 0, TCG_DOUBLE = 1, TCG_FLOAT = 2, TCG_INT32 = 3,
	TCG_INT8 = 4, TCG_UINT8 = 5, TCG_INT16 = 6, TCG_UINT16 = 7, TCG_UINT32 = 8,
	TCG_INT64 = 9, TCG_UINT64 = 10, TCG_N_DTYPES
};

enum tcg_opcode
{
	TCG_BAD_OP = 0, TCG_IDENTITY, TCG_ABS, TCG_NEG, TCG_SIN, TCG_COS, TCG_TAN,
	TCG_EXP, TCG_LOG, TCG_SQRT, TCG_ROUND, TCG_SIGMOID, TCG_TANH, TCG_SQUARE,
	TCG_CUBE, TCG_RAND_UNIF, TCG_REVERSE, TCG_REDUCE_SUM, TCG_REDUCE_PROD,
	TCG_REDUCE_MIN, TCG_REDUCE_MAX, TCG_ARGMAX, TCG_PERMUTE, TCG_EXTEND,
	TCG_RESHAPE, TCG_SLICE, TCG_PAD, TCG_STRIDE, TCG_SCATTER, TCG_POW, TCG_ADD,
	TCG_SUB, TCG_MUL, TCG_DIV, TCG_MIN, TCG_MAX, TCG_EQ, TCG_NEQ, TCG_LT,
	TCG_GT, TCG_MATMUL, TCG_CONTRACT, TCG_CONV, TCG_SELECT, TCG_CONCAT,
	TCG_ASSIGN, TCG_ASSIGN_ADD, TCG_ASSIGN_SUB, TCG_ASSIGN_MUL, TCG_ASSIGN_DIV,
	TCG_CAST, TCG_N_OPCODES
};

/* ---- context, memory, transfers -------------------------------------- */

/* Replaces: constructing an eigen::Device (internal/eigen/device.hpp:546-553).
 * Fails with TCG_ERR_HIP when no GPU is visible. */
int tcg_ctx_create (int device, tcg_ctx** out);
int tcg_ctx_destroy (tcg_ctx* ctx);
/* Message of the last failing call on this context ("" if none). With a NULL
 * context: the message of the last failing tcg_ctx_create of this thread. */
const char* tcg_last_error (const tcg_ctx* ctx);
/* Name of the device the context runs on, e.g. "gfx950" */
const char* tcg_device_arch (const tcg_ctx* ctx);

/* Replaces: eigen::iRuntimeMemory::allocate / deallocate
 * (internal/eigen/memory.hpp:14-22), bytes not elements, deallocate receives
 * the original size.  Blocks are recycled in stream order without touching
 * hipMalloc/hipFree on the steady state; 256-byte aligned. */
int tcg_alloc (tcg_ctx* ctx, size_t bytes, void** devptr);
int tcg_free (tcg_ctx* ctx, void* devptr, size_t bytes);
/* Bytes currently handed out / held by the pool (for leak checks in tests) */
int tcg_mem_stats (const tcg_ctx* ctx, uint64_t* in_use, uint64_t* pooled);
/* Device memory the context holds outside the pool until it is destroyed: the
 * row / summed-index tables of convolutions lowered to matrix products, kept
 * by the plan they were computed from so that a pass over the same layers
 * finds them again (at most 256 MiB; recorded launches keep their addresses,
 * so they are never given back earlier). */
int tcg_mem_stats_kept (const tcg_ctx* ctx, uint64_t* conv_tables);

/* Replaces: the memcpy in eigen::SrcRef<T>::assign (internal/eigen/device.hpp:
 * 200-247) and host reads through iDeviceRef::data()
 * (internal/teq/itensor.hpp:22-35).  h2d: the host buffer may be reused as
 * soon as the call returns.  d2h: blocks until the bytes are in `dst`. */
int tcg_h2d (tcg_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes);
int tcg_d2h (tcg_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes);
int tcg_d2d (tcg_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes);
int tcg_fill_zero (tcg_ctx* ctx, void* dst_dev, size_t bytes);
int tcg_sync (tcg_ctx* ctx);

/* Timing on the context's stream with HIP events (for benchmarks):
 * begin records an event, end records a second one, waits for it and returns
 * the milliseconds between them. */
int tcg_timer_begin (tcg_ctx* ctx);
int tcg_timer_end (tcg_ctx* ctx, float* ms);
/* Non-blocking variant: events recorded on the context's stream between
 * launches; tcg_event_elapsed waits for `stop` and returns stop - start. */
int tcg_event_create (tcg_ctx* ctx, void** event);
int tcg_event_destroy (tcg_ctx* ctx, void* event);
int tcg_event_record (tcg_ctx* ctx, void* event);
int tcg_event_elapsed (tcg_ctx* ctx, void* start, void* stop, float* ms);

/* For measurements: everything enqueued on the context's stream after tcg_hold
 * waits until tcg_release, and then runs back to back, so that events recorded
 * in between (tcg_event_record) measure the device and not the pace at which
 * the host enqueues.  tcg_release returns when the held work has run.  Calls
 * that wait for the stream themselves (tcg_sync, tcg_d2h, tcg_timer_end,
 * tcg_event_elapsed) must not be made while it is held: they would wait for
 * the release.  No counterpart in the reference. */
int tcg_hold (tcg_ctx* ctx);
int tcg_release (tcg_ctx* ctx);

/* ---- recorded launch sequences ---------------------------------------- */

/* What one pass of teq::Evaluator::evaluate enqueues (internal/teq/
 * evaluator.hpp:11-61: a post-order walk calling eigen::Device::calc, which
 * runs one operator per functor) can be recorded once and launched again as
 * a whole, without the host walking the graph: between tcg_capture_begin and
 * tcg_capture_end every entry point of this header records its kernels
 * instead of running them, and tcg_alloc hands out memory that belongs to
 * the recording (tcg_free returns it to the recording, never to the pool), so
 * that the addresses baked into the recorded launches stay valid for as long
 * as the graph lives. tcg_h2d, tcg_d2h, tcg_sync and the timers are refused
 * while recording. tcg_graph_launch enqueues the whole sequence on the
 * context's stream; a buffer of the recording that the caller wants to own
 * again afterwards (an output it reads) is taken with tcg_graph_claim and
 * given back with tcg_free as usual. tcg_graph_destroy returns the memory to
 * the pool, except blocks still claimed, which stay with their owner. */
typedef struct tcg_graph tcg_graph;
int tcg_capture_begin (tcg_ctx* ctx);
int tcg_capture_end (tcg_ctx* ctx, tcg_graph** out);
int tcg_capture_abort (tcg_ctx* ctx);
/* The same for a pass over a SMALL graph (a dense layer on a batch of three:
 * tensors of a few dozen elements), whose cost is being launched at all: the
 * sequence is recorded as the steps of ONE kernel, run by a single workgroup
 * with a barrier between steps, and tcg_graph_launch enqueues that one kernel.
 * Entry points that can be steps: tcg_ew_fusedx, tcg_ew_unary/binary/nary/
 * select, tcg_assign, tcg_reduce, tcg_contract, tcg_matmul without batch, and
 * tcg_extend/permute/slice/pad/reverse/stride (gathers into a dense result).
 * Elementwise steps compute exactly what their own launch computes;
 * contractions sum each output in ascending order of the summed index with a
 * fused multiply-add (the order of the generic product kernel), reductions
 * fold each output in ascending index order. Anything else, or more work than
 * one workgroup does in microseconds, fails with TCG_ERR_UNSUPPORTED (at the
 * call or at tcg_capture_end): the caller aborts and records with
 * tcg_capture_begin instead. */
int tcg_capture_begin_small (tcg_ctx* ctx);
/* For such a recording, an input the host rewrites between launches (a leaf
 * of a few dozen elements) can travel with the launch instead of being copied
 * to the device by a launch of its own: tcg_capture_feed, called before
 * tcg_capture_end, says that the `bytes` at device address `devptr` are
 * supplied by the launch (1024 bytes at most in all, no step may write them;
 * `host` is their first content). tcg_graph_feed replaces the content for the
 * launches that follow; it is copied at the call. The device memory at
 * `devptr` is neither read nor written by the recording. */
int tcg_capture_feed (tcg_ctx* ctx, const void* devptr, size_t bytes, const void* host);
int tcg_graph_feed (tcg_ctx* ctx, tcg_graph* graph, const void* devptr, const void* host, size_t bytes);
int tcg_graph_launch (tcg_ctx* ctx, tcg_graph* graph);
/* The small launches of a LONGER sequence, a few at a time (the dense layer and
 * the softmax behind a convolutional network: a dozen launches over a few
 * thousand elements each).  After tcg_batch_begin the entry points named for
 * tcg_capture_begin_small hold their work back as a step when one workgroup
 * does it in a few hundred iterations; tcg_batch_end sends the steps held so
 * far out as ONE kernel on the context's stream (a recording of the stream
 * holds it as one node) and ends the batch.  A call of one of those entry
 * points that cannot be a step sends the held steps out first, ends the batch
 * and runs as itself, so the order of the work is kept; a batch that grows past
 * what one workgroup does in microseconds goes out and a new one starts.  Any
 * OTHER entry point must not be called between begin and end (its launch would
 * overtake the steps held back); tcg_sync, tcg_d2h, tcg_capture_end and
 * tcg_graph_launch end an open batch first.  The buffers the steps name must
 * stay allocated until the batch is sent.  Steps compute what they compute in
 * a single-launch recording (see there for the summation orders), except that
 * a reduction with fewer outputs than lanes folds each output as 2..64
 * interleaved ascending folds combined by halves.  Both calls
 * may be repeated: begin inside a batch and end outside one do nothing.  No
 * counterpart in the reference: its evaluator calls one Eigen expression per
 * node (internal/teq/evaluator.hpp:35-62) and has no launches to save. */
int tcg_batch_begin (tcg_ctx* ctx);
int tcg_batch_end (tcg_ctx* ctx);
/* Work that nothing waits for yet, beside the work that follows it (the two
 * gradients of a convolution, neither of which reads the other: each leaves
 * part of the chip idle at the end of its grid).  tcg_fork: the launches of
 * the calls that follow go to a second stream of the context, which starts
 * when everything enqueued so far has run.  tcg_fork_end: the calls that follow
 * go to the context's own stream again and run BESIDE what was forked.
 * tcg_join: the context's stream waits for the forked launches; memory given
 * back (tcg_free) between tcg_fork and tcg_fork_end returns to the pool only
 * now, because the forked launches use it.  The caller keeps what the forked
 * launches read and write untouched by the calls between tcg_fork_end and
 * tcg_join (no writes to their inputs, no reads of their results, inputs not
 * given back).  One fork at a time.  Inside a recording the second stream is
 * part of the recording (a branch of the graph); tcg_sync, tcg_d2h,
 * tcg_capture_begin/end and tcg_graph_launch join first.  In a single-launch
 * recording (tcg_capture_begin_small) the three calls do nothing.  No
 * counterpart in the reference, whose device runs one expression at a time
 * (internal/eigen/device.hpp:555-570). */
int tcg_fork (tcg_ctx* ctx);
int tcg_fork_end (tcg_ctx* ctx);
int tcg_join (tcg_ctx* ctx);
int tcg_graph_claim (tcg_ctx* ctx, tcg_graph* graph, void* devptr);
int tcg_graph_stats (const tcg_graph* graph, uint64_t* nodes, uint64_t* arena_bytes);
int tcg_graph_destroy (tcg_ctx* ctx, tcg_graph* graph);

/* ---- elementwise ------------------------------------------------------ */

/* ABS..CUBE: `out = eigen::abs<T>(outshape, *in[0])` ... `eigen::cube<T>`
 * (cfg/ops.yml:75-100; internal/eigen/operator.hpp:377-659) */
int tcg_ew_unary (tcg_ctx* ctx, int opcode, int dtype, uint64_t n,
	const void* in, void* out);

/* POW, SUB, DIV, MIN, MAX, EQ, NEQ, LT, GT and two-argument ADD/MUL
 * (cfg/ops.yml:453-493; internal/eigen/operator.hpp:665-987) */
int tcg_ew_binary (tcg_ctx* ctx, int opcode, int dtype, uint64_t n,
	const void* a, const void* b, void* out);

/* ADD / MUL over nargs >= 2 operands, folded left to right
 * (`eigen::add<T>(outshape, in)`, internal/eigen/operator.hpp:694-732,757-795) */
int tcg_ew_nary (tcg_ctx* ctx, int opcode, int dtype, uint64_t n, int nargs,
	const void* const* ins, void* out);

/* SELECT (cfg/ops.yml:608-609; internal/eigen/operator.hpp:1050-1067) */
int tcg_ew_select (tcg_ctx* ctx, int dtype, uint64_t n, const void* cond,
	const void* then, const void* otherwise, void* out);

/* CAST (cfg/ops.yml:681-711; internal/eigen/operator.hpp:1239-1260) */
int tcg_cast (tcg_ctx* ctx, int out_dtype, int in_dtype, uint64_t n,
	const void* in, void* out);

/* ASSIGN, ASSIGN_ADD/SUB/MUL/DIV: target (op)= source in place
 * (cfg/ops.yml:654-680; internal/eigen/operator.hpp:1190-1237) */
int tcg_assign (tcg_ctx* ctx, int opcode, int dtype, uint64_t n,
	void* target, const void* source);

/* RAND_UNIF on the device: out[i] uniform between lo[i] and hi[i]
 * (cfg/ops.yml:101-103; internal/eigen/operator.hpp:989-1044). The reference
 * draws on the host from std::default_random_engine
 * (internal/global/random.hpp:87-99, 143); this generator is Philox4x32-10
 * keyed by `seed`, so the streams differ while the distributions agree: real
 * types lo + u*(hi-lo) with u in [0,1) of 24 (float) or 53 (double) random
 * bits, int32 uniform on the inclusive range lo..hi (multiply-shift of a
 * 32-bit word). Generator block b of the context's stream is
 * philox(counter = {b, 0}, key = seed); a draw of n elements consumes
 * ceil(n/4) blocks (ceil(n/2) for double), element i taking word i%4 of block
 * i/4 (words 2(i%2), 2(i%2)+1 of block i/2). Key and block count live in
 * device memory and are advanced by kernels: a recorded sequence draws new
 * values at every launch. tcg_rand_seed(seed) restarts the stream at block 0
 * (the counterpart of global::seed, internal/global/random.hpp:79);
 * tcg_rand_state returns {seed, blocks drawn} after a synchronisation. */
int tcg_rand_seed (tcg_ctx* ctx, uint64_t seed);
int tcg_rand_state (tcg_ctx* ctx, uint64_t out[2]);
int tcg_rand_uniform (tcg_ctx* ctx, int dtype, uint64_t n, const void* lo,
	const void* hi, void* out);

/* A chain of elementwise nodes evaluated in one pass over memory: what a run
 * of consecutive MatOp/TensOp closures (internal/eigen/device.hpp:304-372)
 * computes, without materialising the intermediates.
 * Three registers (ACC, T0, T1, all zero at the start); operands name a
 * register, a leaf or the instruction's immediate.  The short form of
 * tcg_ew_fusedx for dense operands of one length: it runs as such a group
 * (the kernel is compiled for the program on first use). */
enum tcg_ew_operand
{
	TCG_OPD_NONE = 0, TCG_OPD_ACC = 1, TCG_OPD_T0 = 2, TCG_OPD_T1 = 3,
	TCG_OPD_IMM = 4,
	TCG_OPD_LEAF0 = 8 /* TCG_OPD_LEAF0 + k = leaf k, k < TCG_EW_MAX_LEAVES */
};
#define TCG_EW_MAX_LEAVES 4
#define TCG_EW_MAX_INSTRS 32
typedef struct tcg_ew_instr
{
	uint8_t opcode; /* unary or binary tcg_opcode; TCG_IDENTITY copies `a` */
	uint8_t a;      /* tcg_ew_operand */
	uint8_t b;      /* tcg_ew_operand, TCG_OPD_NONE for unary opcodes */
	uint8_t dst;    /* TCG_OPD_ACC, TCG_OPD_T0 or TCG_OPD_T1 */
	uint32_t pad_;
	double imm;     /* converted to the kernel's dtype */
} tcg_ew_instr;
/* The value of ACC after the last instruction is written to out. */
int tcg_ew_fused (tcg_ctx* ctx, int dtype, uint64_t n, int nleaves,
	const void* const* leaves, int ninstrs, const tcg_ew_instr* program, void* out);

/* A group of elementwise nodes of one shape evaluated in one launch, reading
 * its operands through views and storing several results: what the closures
 * of the group's nodes (internal/eigen/device.hpp:304-372), together with the
 * EXTEND / SLICE / PAD / PERMUTE nodes that only feed them
 * (internal/eigen/operator.hpp:157-275), compute one node at a time.
 * A leaf is addressed as ptr[offset + sum_d c[d] * stride[d]] for the output
 * coordinate c (strides in elements; 0 broadcasts, as EXTEND does); where c[d]
 * lies outside [lo[d], hi[d]) the leaf reads as zero and memory is not
 * touched (PAD). Registers hold one value per element; TCG_FX_STORE writes
 * operand `a` to outs[dst] at the element's position (outputs are dense, of
 * the given shape). TCG_SELECT takes three operands: a != 0 ? b : c. */
enum tcg_fx_operand
{
	TCG_FX_NONE = 0, TCG_FX_IMM = 1,
	TCG_FX_LEAF0 = 8,  /* + k, k < TCG_FX_MAX_LEAVES */
	TCG_FX_REG0 = 32   /* + r, r < TCG_FX_MAX_REGS */
};
#define TCG_FX_MAX_LEAVES 16
#define TCG_FX_MAX_REGS 16
#define TCG_FX_MAX_INSTRS 64
#define TCG_FX_MAX_OUTS 16
#define TCG_FX_STORE 255 /* opcode */
/* opcode: bitwise OR of the two operands' representations. Zero-bordered
 * leaves whose boxes tile the output, OR-ed together, are CONCAT
 * (internal/eigen/operator.hpp:335-368) with every bit kept. */
#define TCG_FX_BITOR 254
typedef struct tcg_fx_leaf
{
	const void* ptr;
	int64_t offset;
	int64_t stride[8];
	uint64_t lo[8];
	uint64_t hi[8];
	/* nsum > 1: the operand's value is the sum, in this order, of the nsum
	 * elements at distances 0, sum_stride, 2 sum_stride, ... (in elements)
	 * from where the fields above point: the K ranges a matrix product left
	 * side by side (tcg_gemm_terms_ranges).  0 and 1 both mean a plain operand. */
	int64_t sum_stride;
	uint32_t nsum;
	/* 1: the operand is (a part of) the result of the matrix product that
	 * tcg_gemm_terms_fx computes in the same launch, never laid out in memory:
	 * ptr is ignored, offset / stride address the M x N result as a row-major
	 * matrix of row length N.  0 everywhere else. */
	uint32_t from_product;
} tcg_fx_leaf;
typedef struct tcg_fx_instr
{
	uint8_t opcode; /* tcg_opcode (unary, binary, TCG_IDENTITY, TCG_SELECT), TCG_FX_BITOR or TCG_FX_STORE */
	uint8_t a, b, c; /* tcg_fx_operand; unused ones TCG_FX_NONE */
	uint8_t dst;    /* TCG_FX_REG0 + r, or the output index of a store */
	uint8_t pad_[3];
	double imm;     /* value of TCG_FX_IMM operands, converted to the dtype */
} tcg_fx_instr;
int tcg_ew_fusedx (tcg_ctx* ctx, int dtype, const uint64_t shape[8],
	int nleaves, const tcg_fx_leaf* leaves, int ninstrs, const tcg_fx_instr* program,
	int nouts, void* const* outs);

/* What the kernels compiled at run time have cost this process so far (groups
 * of elementwise nodes, whole passes of small graphs, products with an
 * epilogue; no counterpart in the reference, whose expressions are compiled
 * with it): kernels compiled here, kernels loaded from the files an earlier
 * process left, and the milliseconds spent on both.  Compiled code is kept
 * under $TCG_FX_CACHE (default ~/.cache/tenncor_amd/fx; TCG_FX_CACHE=0: nowhere),
 * one file per kernel holding the text it was compiled from in front of the
 * code, and is only used for exactly that text, those flags and that compiler. */
int tcg_jit_stats (const tcg_ctx* ctx, uint64_t* compiled, uint64_t* from_disk, double* ms);

/* ---- reductions ------------------------------------------------------- */

/* REDUCE_SUM / REDUCE_PROD / REDUCE_MIN / REDUCE_MAX
 * (`eigen::reduce_sum<T>(outshape, *in[0], attrib)`, cfg/ops.yml:106-151;
 * internal/eigen/operator.hpp:54-132).  Bit i of rankmask = dim i reduced. */
int tcg_reduce (tcg_ctx* ctx, int opcode, int dtype, const uint64_t shape[8],
	unsigned rankmask, const void* in, void* out);

/* The same reduction for callers that cannot allocate device memory (code
 * under HIP graph capture of their own, serving loops, harnesses that forbid
 * hipMalloc).  It has no counterpart in the reference.  tcg_reduce takes its
 * temporaries (partial results of a reduced dim that is split over
 * workgroups, and what is left of the tensor between the steps of a reduction
 * over separated dims) from the context's pool, which may call hipMalloc;
 * this entry point keeps them in a fixed array of device memory that every
 * GPU the library runs on holds from load to exit, and calls no allocating
 * routine.  Same kernels, same launch shapes, same results bit for bit.
 * Limits: the temporaries of one call must fit
 * TCG_REDUCE_NOALLOC_SCRATCH_BYTES (each piece rounded up to 256 bytes),
 * otherwise the call fails with TCG_ERR_ARG and nothing is launched for the
 * step that did not fit; every call on a GPU uses that GPU's one array, so
 * calls that overlap on one GPU (two contexts, two streams) would race --
 * calls on one context are ordered on its stream and do not.  A call from
 * another context while the launches of the context that used the array last
 * are still running is refused with TCG_ERR_ARG (nothing is launched; try
 * again once that context has been synchronised).  Launches that are being
 * recorded -- by tcg_capture_begin or by the caller's own capture of the
 * stream -- run when the recording is launched, which the library cannot
 * order against other users of the array: keeping them apart is then up to
 * the caller.  Not available inside tcg_capture_begin_small. */
#define TCG_REDUCE_NOALLOC_SCRATCH_BYTES ((size_t) 8 << 20)
int tcg_reduce_noalloc (tcg_ctx* ctx, int opcode, int dtype, const uint64_t shape[8],
	unsigned rankmask, const void* in, void* out);

/* ARGMAX (cfg/ops.yml:152-186; internal/eigen/operator.hpp:134-155);
 * return_dim >= 8 gives the flat index of the maximum */
int tcg_argmax (tcg_ctx* ctx, int dtype, const uint64_t shape[8], int return_dim,
	const void* in, void* out);

/* ---- data movement ---------------------------------------------------- */

/* EXTEND (cfg/ops.yml:239-283; internal/eigen/operator.hpp:157-173) */
int tcg_extend (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t bcast[8], const void* in, void* out);
/* PERMUTE (cfg/ops.yml:187-238; internal/eigen/operator.hpp:175-210);
 * `order` is the completed 8-entry permutation: out dim i = in dim order[i] */
int tcg_permute (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t order[8], const void* in, void* out);
/* SLICE (cfg/ops.yml:319-371; internal/eigen/operator.hpp:212-255);
 * offsets/extents are the clamped values of lines 225-230 */
int tcg_slice (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t offsets[8], const uint64_t extents[8], const void* in, void* out);
/* PAD (cfg/ops.yml:372-412; internal/eigen/operator.hpp:257-275) */
int tcg_pad (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t before[8], const uint64_t after[8], const void* in, void* out);
/* PAD without its zero border: copies `in` to its place inside `out` and
 * leaves every other element of `out` as it was. For a padded image whose
 * only readers are tcg_conv_boxed calls clipped to that place (the same
 * reference operator as tcg_pad; the border is what its readers skip) */
int tcg_pad_interior (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t before[8], const uint64_t after[8], const void* in, void* out);
/* REVERSE(cfg/ops.yml:104-105; internal/eigen/operator.hpp:316-333) */
int tcg_reverse (tcg_ctx* ctx, int dtype, const uint64_t shape[8],
	unsigned rankmask, const void* in, void* out);
/* STRIDE (cfg/ops.yml:413-438; internal/eigen/operator.hpp:277-293) */
int tcg_stride (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t incr[8], const uint64_t outshape[8], const void* in, void* out);
/* SCATTER (cfg/ops.yml:439-452; internal/eigen/operator.hpp:295-314) */
int tcg_scatter (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t incr[8], const uint64_t outshape[8], const void* in, void* out);
/* CONCAT (cfg/ops.yml:610-653; internal/eigen/operator.hpp:335-368);
 * shapes = nargs * 8 values */
int tcg_concat (tcg_ctx* ctx, int dtype, int axis, int nargs,
	const uint64_t* shapes, const void* const* ins, void* out);

/* ---- contractions ----------------------------------------------------- */

/* MATMUL (cfg/ops.yml:494-514; internal/eigen/operator.hpp:1107-1139):
 * a{K,M,batch...}, b{N,K,batch...} -> out{N,M,batch...} */
int tcg_matmul (tcg_ctx* ctx, int dtype, const uint64_t ashape[8],
	const uint64_t bshape[8], const void* a, const void* b, void* out);
/* CONTRACT (cfg/ops.yml:515-565; internal/eigen/operator.hpp:1069-1103);
 * pairs = npairs * (a_dim, b_dim); out dims = b's free dims then a's */
int tcg_contract (tcg_ctx* ctx, int dtype, const uint64_t ashape[8],
	const uint64_t bshape[8], int npairs, const uint64_t* pairs,
	const void* a, const void* b, void* out);

/* out = CONTRACT(a[0], b[0]) + CONTRACT(a[1], b[1]) + ... over `nterms` pairs
 * of operands of one pair of shapes: what an ADD node over equal CONTRACT
 * nodes computes.  The gradient builder produces exactly this for a weight
 * that many nodes read: tenncor/eteq/backprop.hpp:563-567 adds the gradients
 * that arrive from each reader (internal/teq/src/derive.cpp:62-160), each of
 * them the CONTRACT of backprop.hpp:269-359 -- sixty-four of them for a
 * recurrent weight unrolled over sixty-four steps.  In fp32, when every
 * operand is a matrix in place, the sum runs as ONE matrix-core product over
 * the concatenated summed index (the operands stay where they are; at most
 * 128 terms, summed extent a multiple of 16): the order of the fp32 additions
 * then differs from product-by-product evaluation (same 1e-4 bar as a
 * contraction).  Otherwise the terms are computed one by one and added in
 * term order, bit for bit what the separate nodes give. */
int tcg_contract_sum (tcg_ctx* ctx, int dtype, const uint64_t ashape[8],
	const uint64_t bshape[8], int npairs, const uint64_t* pairs, int nterms,
	const void* const* a, const void* const* b, void* out);
/* Strided row-major GEMM the two above lower to:
 * C[b][m][n] = sum_k A[b][m][k] * B[b][k][n], element strides given;
 * trans_a: A element (m,k) at m*1 + k*lda instead of m*lda + k, same for B.
 * float and double products whose operands are 16-byte aligned with even
 * (double) or fourfold (float) extents along memory run on the matrix cores
 * (float products whose K is a multiple of 16 take their operands from memory
 * straight into LDS, the fastest route: 4096^3 at 0.86 of the fp32 matrix peak);
 * int32, odd shapes and products too small to fill the chip run on a tiled
 * kernel, or with one lane per result when there are few results and K is
 * long.  Every route sums k in a fixed order: results do not depend on
 * scheduling. */
int tcg_gemm (tcg_ctx* ctx, int dtype, uint64_t M, uint64_t N, uint64_t K,
	uint64_t batch, const void* A, uint64_t lda, uint64_t stride_a, int trans_a,
	const void* B, uint64_t ldb, uint64_t stride_b, int trans_b,
	void* C, uint64_t ldc, uint64_t stride_c);
/* C = sum_t A_t B_t: `nterms` row-major products of one shape M x N x K with
 * the flags of tcg_gemm, every term with operand addresses and leading dims of
 * its own, as ONE product over the concatenated summed index where the
 * matrix cores take the shape (fp32, 16-byte aligned operands, K a multiple
 * of 16, at most 128 terms), else term by term in term order.  What
 * tcg_contract_sum does for whole tensors, for operands that are parts of
 * tensors: a contraction over a dim along which an operand is a CONCAT of
 * tensors (cfg/tenncor/layer.yml:716-768 concatenates input and hidden state
 * in front of the gate product) or an ADD of PADs that tile it (the gradient
 * of the SLICEs that cut the gates back out, tenncor/eteq/backprop.hpp:402-421)
 * reads the parts where they are, each with the rows of the other operand it
 * meets.  C may be a block of a larger matrix (ldc). */
int tcg_gemm_terms (tcg_ctx* ctx, int dtype, uint64_t M, uint64_t N, uint64_t K, int nterms,
	const void* const* A, const uint64_t* lda, int trans_a,
	const void* const* B, const uint64_t* ldb, int trans_b,
	void* C, uint64_t ldc);
/* Sums of products whose operands are concatenations along the dims that
 * survive (the weight gradient of the recurrent cell above: [x_t, h] against
 * the four gate gradients, one term per time step): the result falls into
 * mparts x nparts blocks, block (i, j) = sum_t A[i * nterms + t] B[j * nterms + t]
 * with Mp[i] rows and Np[j] columns, at rows sum(Mp[..i]) and columns
 * sum(Np[..j]) of C.  lda / ldb: one leading dim per part.  Where every part
 * is a multiple of 128 rows / columns (fp32, 16-byte aligned, at most 4 x 8
 * parts and 384 operand addresses) the blocks run as ONE matrix-core product
 * over the whole result, whose tiles look their parts up; otherwise block by
 * block through tcg_gemm_terms.  Same sums per element either way up to the
 * order in which K ranges are added. */
int tcg_gemm_terms_grid (tcg_ctx* ctx, int dtype, int mparts, const uint64_t* Mp, int nparts, const uint64_t* Np,
	uint64_t K, int nterms, const void* const* A, const uint64_t* lda, int trans_a,
	const void* const* B, const uint64_t* ldb, int trans_b, void* C, uint64_t ldc);
/* The same sum of products with its summed index cut into `nranges` equal
 * ranges whose results are left side by side: ranges[r][m][n] (row-major
 * M x N each) is the sum over range r.  The reader adds them up in range
 * order -- an elementwise launch that reads a matrix product backwards
 * through the recurrence of cfg/tenncor/layer.yml:716-768 does so while it
 * loads its operand (tcg_fx_leaf.nsum), which saves the launch that would add
 * the ranges of a product with few results under a long K.  Matrix cores only:
 * fp32, M, N >= 32, K a multiple of 16, nterms * K a multiple of 16 nranges,
 * 2 <= nranges <= 32, 16-byte aligned operands; anything else fails with
 * TCG_ERR_UNSUPPORTED (the caller falls back on tcg_gemm_terms). */
int tcg_gemm_terms_ranges (tcg_ctx* ctx, int dtype, uint64_t M, uint64_t N, uint64_t K, int nterms,
	const void* const* A, const uint64_t* lda, int trans_a,
	const void* const* B, const uint64_t* ldb, int trans_b,
	int nranges, void* ranges);
/* tcg_gemm_terms whose result is read by one group of elementwise nodes and by
 * nothing else, product and group as ONE launch: the product's values go from
 * the matrix cores to the group's arithmetic in registers and are never laid
 * out.  A time step of a recurrent cell is such a pair -- the gate product
 * over [x_t, h] followed by the gate activations and the state update
 * (cfg/tenncor/layer.yml:297-345, 716-768), and backwards the product of the
 * gate gradients with the transposed weight followed by the derivative
 * factors of the step before (tenncor/eteq/backprop.hpp:269-359) -- and as two
 * launches it is bound by being launched, not by arithmetic.
 * The group is given as to tcg_ew_fusedx; the leaves that read the product
 * set from_product and address its M x N result as a row-major matrix with
 * row length N.  Every such leaf must walk the result row by row the way the
 * group walks its own elements: with J = shape[0] and rows = shape[1] * ... *
 * shape[7] = M, group element (j, row) reads result element (row, offset + j),
 * 0 <= offset, offset + J <= N (the SLICEs that cut the gates out of one
 * product are four such leaves with offsets 0, J, 2J, 3J).  Results equal
 * tcg_gemm_terms followed by tcg_ew_fusedx up to the order of the additions
 * over K (each element is summed in a fixed order, in K ranges that are added
 * in range order: results do not depend on scheduling); the group's own
 * arithmetic is the same scalar code in the same order.
 * fp32 only, trans_a = 0, K a multiple of 16, 16-byte aligned operands with
 * leading dims that are multiples of four, at most 8 terms; anything else fails
 * with TCG_ERR_UNSUPPORTED and launches nothing (the caller then runs the two
 * launches).  The kernel is compiled at run time for the shape of the product
 * and the program of the group and kept for the life of the process. */
int tcg_gemm_terms_fx (tcg_ctx* ctx, int dtype, uint64_t M, uint64_t N, uint64_t K, int nterms,
	const void* const* A, const uint64_t* lda, int trans_a,
	const void* const* B, const uint64_t* ldb, int trans_b,
	const uint64_t shape[8], int nleaves, const tcg_fx_leaf* leaves,
	int ninstrs, const tcg_fx_instr* program, int nouts, void* const* outs);
/* CONV (cfg/ops.yml:566-607; internal/eigen/operator.hpp:1141-1187):
 * valid cross-correlation, kernel dim i slides along image dim ranks[i] */
int tcg_conv (tcg_ctx* ctx, int dtype, const uint64_t imgshape[8],
	const uint64_t kshape[8], int nranks, const uint64_t* ranks,
	const void* img, const void* kernel, void* out);
/* The same correlation for the idioms tenncor builds convolutions from
 * (cfg/tenncor/nn.yml:88-93 pads a singleton axis before CONV;
 * tenncor/eteq/backprop.hpp:372-439 pads the upstream gradient and slices one
 * index of the result): the caller promises that `img` is zero outside
 * [img_lo, img_hi) and asks only for the outputs inside [out_lo, out_hi);
 * the rest of `out` is left untouched.  NULL boxes mean "everything". */
int tcg_conv_boxed (tcg_ctx* ctx, int dtype, const uint64_t imgshape[8],
	const uint64_t kshape[8], int nranks, const uint64_t* ranks,
	const uint64_t img_lo[8], const uint64_t img_hi[8],
	const uint64_t out_lo[8], const uint64_t out_hi[8],
	const void* img, const void* kernel, void* out);
/* tcg_conv_boxed for an image that was never laid out with its zero border:
 * `box` holds only the elements inside [img_lo, img_hi), densely, in the same
 * dim order. This is CONV(PAD(x), kernel) (cfg/tenncor/nn.yml:88-93,
 * tenncor/eteq/backprop.hpp:372-399) computed from x itself: box = x,
 * img_lo = the paddings before, img_hi = img_lo + shape of x. Results are
 * those of tcg_conv_boxed on the padded image, bit for bit. */
int tcg_conv_dense_box (tcg_ctx* ctx, int dtype, const uint64_t imgshape[8],
	const uint64_t kshape[8], int nranks, const uint64_t* ranks,
	const uint64_t img_lo[8], const uint64_t img_hi[8],
	const uint64_t out_lo[8], const uint64_t out_hi[8],
	const void* box, const void* kernel, void* out);
/* The same correlation over operands and a result that are laid out in memory
 * otherwise than densely in dim order: the PERMUTE and REVERSE nodes tenncor
 * puts round every convolution (cfg/tenncor/nn.yml:88-93 reverses the kernel
 * and permutes the result; tenncor/eteq/backprop.hpp:372-439 permutes the
 * upstream gradient in front of the correlation and permutes and reverses the
 * kernel gradient behind it) become strides instead of passes over memory.
 * All strides count elements and may be negative (REVERSE):
 *   image element c, img_lo <= c < img_hi:  box[sum_d (c[d] - img_lo[d]) * box_stride[d]]
 *   kernel element w:                        kernel[sum_i w[i] * kernel_stride[i]]
 *   output element c, out_lo <= c < out_hi:  out[sum_d (c[d] - out_lo[d]) * out_stride[d]]
 * (NULL out_lo / out_hi: every output). Nothing else of `out` is written.
 * Values are those of tcg_conv_boxed on the materialised operands; where the
 * result or the kernel already is the row-major matrix of the product that
 * the correlation is lowered to, the product writes or reads it in place. */
int tcg_conv_views (tcg_ctx* ctx, int dtype, const uint64_t imgshape[8],
	const uint64_t kshape[8], int nranks, const uint64_t* ranks,
	const uint64_t img_lo[8], const uint64_t img_hi[8],
	const uint64_t out_lo[8], const uint64_t out_hi[8],
	const void* box, const int64_t box_stride[8],
	const void* kernel, const int64_t kernel_stride[8],
	void* out, const int64_t out_stride[8]);
/* How many of the context's convolutions so far took one of the three special
 * routes of the matrix-product lowering (fp32 only):
 *   patch      the product reads the image out of a patch held in LDS (the summed
 *              index along memory in multiples of 32, 32 or 64 and more result
 *              columns, large enough: the forward pass and the image gradient of
 *              a conv2d layer over 32 and more channels; TCG_CONV_PATCH=0 in the
 *              environment keeps every convolution off it);
 *   short_sum  gather, product and the kernel's layout in one launch (at most 32
 *              summed indices, 16, 32, 48 or 64 columns: a first layer over one
 *              channel; TCG_CONV_SHORT=0 keeps every convolution off it);
 *   few_rows   at most 32 rows under a summed index of 4096 and more (the kernel
 *              gradient of such a first layer): A is gathered while it is
 *              multiplied, stretch by stretch of the summed index, and the
 *              stretches are added up by a second launch (TCG_CONV_FEWROWS=0
 *              keeps every convolution off it).
 * No counterpart in the reference; for tests and for callers who want to know
 * which route their shapes take. */
int tcg_conv_route_counts (const tcg_ctx* ctx, uint64_t* patch, uint64_t* short_sum, uint64_t* few_rows);

#ifdef __cplusplus
}
#endif

#endif /* TCG_H */
