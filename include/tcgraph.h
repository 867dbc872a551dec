/*
 * tcgraph.h -- flat C binding of the host graph layer (libtenncor_host.so).
 *
 * The host layer keeps tenncor's C++ node API (eteq::make_functor, Variable,
 * Constant, tcr::derive, teq::Evaluator + eigen::Device); this header exposes
 * the same calls to languages without C++ linkage, the way the reference's
 * pybind11 module does for Python (tenncor/python/eteq_ext.cpp:130-157 for
 * evaluation and data access, tenncor/python/tenncor_ext.cpp for derive).
 * Nodes are integers local to a tcr_graph; attributes use the nine keys of
 * internal/eigen/packattr.hpp:60-363 with integer-list values.
 *
 * Every function returns 0 on success; tcr_last_error() gives the message of
 * the last failure of the calling thread (the text the reference would have
 * thrown).
 */
#ifndef TCGRAPH_H
#define TCGRAPH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tcr_graph tcr_graph;

const char* tcr_last_error (void);

int tcr_graph_create (tcr_graph** out);
int tcr_graph_destroy (tcr_graph* g);

/* eteq::make_variable<T>(data, shape, label) -- tenncor/eteq/make.hpp:50-56.
 * dtype: a code of enum tcg_dtype (include/tcg.h: 1 double, 2 float, 3 int32,
 * and in the library built for the full type configuration 4 int8 .. 10
 * uint64), the same numbering in both libraries although the C++ enum
 * egen::_GENERATED_DTYPE underneath follows the reference's, which differs
 * between the two configurations; a type the library was not built for is
 * refused.  shape: 8 dims, dim 0 fastest */
int tcr_variable (tcr_graph* g, int dtype, const uint64_t shape[8], const void* data,
	const char* label, int* node);
/* eteq::make_constant<T>(data, shape) -- tenncor/eteq/make.hpp:108-119 */
int tcr_constant (tcr_graph* g, int dtype, const uint64_t shape[8], const void* data, int* node);
/* Variable<T>::assign(data) -- tenncor/eteq/variable.hpp:72-90 */
int tcr_assign (tcr_graph* g, int variable, const void* data);
/* Brings the device copy of a leaf up to date now (one host-to-device copy when
 * the host copy is newer, nothing otherwise) instead of at the next evaluation
 * that reads it: a caller that assigns the next batch while the device still
 * runs the last one keeps the copy out of the evaluation's time.  What the
 * reference has no need for: its leaves are read where they lie. */
int tcr_prefetch (tcr_graph* g, int leaf);

/* eteq::make_funcattr(opcode, children, attrs) -- tenncor/eteq/src/make.cpp:14-29.
 * Attribute i has key keys[i] and the integer list vals[i][0..lens[i]);
 * "rank" takes one value, "dtype" takes one dtype code, "tensor" takes one
 * node id.  The result may be one of the children (build-time elision). */
int tcr_functor (tcr_graph* g, int opcode, int nargs, const int* args, int nattrs,
	const char* const* keys, const int64_t* const* vals, const int* lens, int* node);

/* tcr::derive(root, targets) -- tenncor/src/eteq.cpp:40-76 */
int tcr_derive (tcr_graph* g, int root, int ntargets, const int* targets, int* grads);

/* eteq::DerivativeFuncs::lderive(op, supgrad, arg_idx) --
 * tenncor/eteq/backprop.hpp:58-560: the gradient that functor `op` passes to its
 * argument arg_idx when `supgrad` arrives at it. */
int tcr_local_derivative (tcr_graph* g, int op, int supgrad, int arg_idx, int* grad);

/* teq::get_eval().evaluate(eigen::Device, targets) --
 * tenncor/eteq/src/etens.cpp:46-62 */
int tcr_evaluate (tcr_graph* g, int ntargets, const int* targets);
/* The same with the third argument of iEvaluator::evaluate
 * (internal/teq/ievaluator.hpp:17-25): the walk does not enter the `ignored`
 * nodes, whose readers use the value they already hold
 * (internal/teq/evaluator.hpp:20-24; internal/teq/test/test_evaluator.cpp:75-207) */
int tcr_evaluate_ignoring (tcr_graph* g, int ntargets, const int* targets, int nignored, const int* ignored);
/* Block until the device has finished everything enqueued */
int tcr_sync (tcr_graph* g);

/* teq::set_eval (internal/teq/src/evaluator.cpp:9-20): which evaluator the
 * process uses from now on. TCR_EVAL_DEFAULT removes the registered one, so
 * that teq::get_eval makes its default again: TCR_EVAL_REPLAY, or
 * TCR_EVAL_PLAIN when the environment holds TCR_EVAL_PLAIN=1 (the reference's
 * default is the plain walk; a backend that is dropped in without a call to
 * teq::set_eval should not be the slow one for graphs evaluated again and
 * again, and the replaying evaluator walks a set of targets it sees for the
 * first time exactly like the plain one).
 * TCR_EVAL_PLAIN is teq::Evaluator, the node-by-node
 * walk; TCR_EVAL_REPLAY records the launches of a set of targets the second
 * time it is evaluated and enqueues the recording as a whole afterwards, with
 * elementwise functors that feed one another computed in shared launches, and
 * the whole pass of a graph of small tensors (4096 elements at most each) as
 * the steps of one kernel (tcg_capture_begin_small: sums then run in another
 * order, equal to the walk's within the tolerance of reductions and
 * contractions rather than bit for bit); in a larger graph, runs of launches
 * over at most 16384 elements each (the dense layer and the loss behind a
 * convolutional network) go out as one kernel per run in the same way
 * (tcg_batch_begin; TCR_BATCHES=0 in the environment keeps them apart);
 * TCR_EVAL_REPLAY_LAUNCHES is the same without such single-kernel passes and runs:
 * every value equals the walk's bit for bit;
 * TCR_EVAL_REPLAY_UNFUSED records one launch per functor, as the walk issues. */
#define TCR_EVAL_PLAIN 0
#define TCR_EVAL_REPLAY 1
#define TCR_EVAL_REPLAY_UNFUSED 2
#define TCR_EVAL_REPLAY_LAUNCHES 3
#define TCR_EVAL_DEFAULT 4
/* the launches TCR_EVAL_REPLAY would record, run one after the other with a
 * HIP event in front of and behind each (the slot the reference's debugging
 * evaluator takes, dbg/peval/plugin_eval.hpp:21-42): tcr_evaluator_timing
 * returns the device microseconds per kind of launch as text */
#define TCR_EVAL_TIMING 5
int tcr_set_evaluator (int kind);
int tcr_evaluator_timing (char* out, size_t capacity, size_t* needed);
/* Counters of the replaying evaluator (zeros under TCR_EVAL_PLAIN):
 * out[0] passes walked node by node, out[1] recordings made, out[2] passes
 * served by a recording, out[3] passes with nothing to do, out[4] launches in
 * the latest recording, out[5] device bytes reserved by live recordings */
int tcr_evaluator_stats (uint64_t out[6]);
/* What the most recent recording cost on the host: milliseconds from planning
 * to the finished launch sequence, the part of them spent on kernels compiled
 * at run time, how many of those were compiled and how many came from the
 * files an earlier process left (tcg_jit_stats).  Zeros without a recording. */
int tcr_evaluator_record_cost (double* record_ms, double* jit_ms, uint64_t* jit_compiled, uint64_t* jit_from_disk);
/* How many target sets the replaying evaluator could not record (it walks
 * them node by node instead) and, in `out`, the message of the failure that
 * stopped the latest of them ("" when none, or under TCR_EVAL_PLAIN) */
int tcr_evaluator_record_error (char* out, size_t capacity, uint64_t* failures);

/* Where RAND_UNIF nodes whose operator is built from now on draw their values.
 * TCR_RANDOM_HOST (default): on the host from the seeded std::default_random_engine,
 * as the reference does (internal/eigen/operator.hpp:989-1044,
 * internal/global/random.hpp:87-99,143); such nodes make the replaying evaluator
 * fall back to the node-by-node walk. TCR_RANDOM_DEVICE: on the GPU with the
 * counter-based generator of tcg_rand_uniform (another stream, same
 * distributions); recorded passes then draw new values at every replay. */
#define TCR_RANDOM_HOST 0
#define TCR_RANDOM_DEVICE 1
int tcr_set_random (int where);
/* global::seed (internal/global/random.hpp:79): seeds the host generator and
 * restarts the device generator's stream under the same seed */
int tcr_seed (uint64_t seed);

/* iTensor::shape / get_meta().type_code / device().data() */
int tcr_shape (tcr_graph* g, int node, uint64_t shape[8]);
int tcr_dtype (tcr_graph* g, int node, int* dtype);
/* Copies the node's value (n_elems * type_size bytes) into out; fails when
 * the node has no data (never evaluated or expired) */
int tcr_data (tcr_graph* g, int node, void* out, size_t bytes);
int tcr_version (tcr_graph* g, int node, uint64_t* version);

/* An attribute of a functor as tcr_functor takes them (marsh::iAttributed::
 * get_attr, internal/marsh/attrs.hpp): the integer list under `key`; for
 * "tensor" the node id, for "dtype" the type code.  *len = -1 when the node
 * has no such attribute (or is a leaf); vals may be NULL to ask for the length. */
int tcr_attr (tcr_graph* g, int node, const char* key, int64_t* vals, int capacity, int* len);
/* Structure: opcode (0 for leaves), operands, and the indented dump used by
 * the reference's graph-equality tests (testutil/tutil.hpp) */
int tcr_opcode (tcr_graph* g, int node, int* opcode);
int tcr_nargs (tcr_graph* g, int node, int* nargs);
int tcr_args (tcr_graph* g, int node, int* args, int capacity);
int tcr_to_string (tcr_graph* g, int node, char* out, size_t capacity);
/* Number of distinct functors reachable from the given nodes */
int tcr_count_functors (tcr_graph* g, int nnodes, const int* nodes, int* count);
/* How the replaying evaluator would launch one pass over these targets, as
 * text, one launch per line in launch order (needs no GPU): "node OPCODE" for
 * a functor launched through its own operator, or
 * "group OP+OP+... leaves=L stores=S instrs=I" for elementwise functors sharing
 * a launch, or "swapped CONTRACT+PERMUTE" for a transposed matrix product
 * launched as the product with its operands exchanged, or "padded PAD+CONV"
 * ("padded PAD+CONV+SLICE" when only slices read the result) for a convolution
 * computed from the operand of its PAD node; a line "batch N" says that the N
 * lines behind it are steps over a few thousand elements each that go out as
 * ONE launch (tcg_batch_begin); a last line "folded N" counts the functors that
 * never hold a value of their own. Returns the length the text needs (it is cut to `capacity`). */
int tcr_launch_plan (tcr_graph* g, int ntargets, const int* targets, char* out, size_t capacity, size_t* needed);

/* ---- graph clean-up (tenncor/hone/optimize.hpp:19-38: `hone::optimize(roots, rulestream)`) ----
 * Merges equal subgraphs (tenncor/hone/duplicates.hpp:97-101), then repeats, until
 * nothing changes (50 rounds at most, tenncor/hone/src/optimize.cpp:11,27-31):
 * functors other than IDENTITY whose operands are all constants are evaluated
 * on the GPU and replaced by constants (tenncor/hone/cstrules.hpp:48-65), and the
 * conversions of `rules_json` are applied ({"conversions": [{"srcs": [pattern...],
 * "dest": target}]}, the schema of internal/opt/optimize.proto:7-35 over
 * internal/query/query.proto:7-79; NULL = no conversions). Readers of replaced
 * nodes are rewired in place. out_roots[i] is the node that replaces roots[i].
 * fold = 0 skips the evaluation of constant functors (needs no GPU then).
 * stats = {nodes merged, functors folded, matches converted, rounds}. */
int tcr_optimize (tcr_graph* g, int nroots, const int* roots, const char* rules_json, int fold,
	int* out_roots, uint64_t stats[4]);

#ifdef __cplusplus
}
#endif

#endif /* TCGRAPH_H */
