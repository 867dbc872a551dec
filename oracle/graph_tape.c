/*
 * graph_tape.c -- a whole graph on the host, node by node in the order of
 * teq::Evaluator (internal/teq/evaluator.hpp:33-45: children first, every
 * node into a buffer of its own through eigen::Device::calc,
 * internal/eigen/device.hpp:546-576), each node by the oracle's routine for its
 * opcode.  TEST INFRASTRUCTURE like the rest of this directory: it checks and
 * times the reference's way of evaluating (one core, one node at a time, no
 * python between the nodes -- the recipe of tenncor/bm/benchmark.cpp:334-393
 * re-assigns the input and times evaluate); nothing under tenncor_amd/ uses it.
 *
 * Pinned by tests/test_oracle_tape.py: the reference's whole-graph golden
 * vectors (tenncor/test/test_equation.cpp sigmoid MLP forward and gradients).
 */
#define _POSIX_C_SOURCE 200809L
#include <string.h>
#include <time.h>

#include "tc_oracle.h"

/* one functor; operands and result are indices into the buffer table */
typedef struct orc_tape_op
{
	int32_t opcode, dtype, in_dtype; /* in_dtype: CAST only */
	int32_t nargs, first_arg;        /* operands: arg_ids[first_arg .. first_arg + nargs) */
	int32_t out;
	int32_t nattr;                   /* values of attr[] in use */
	int32_t pad_;
	uint64_t n;                      /* elements of the result */
	uint64_t ashape[8], bshape[8];   /* shapes of the first two operands */
	uint64_t attr[32];               /* per opcode, see orc_tape_step */
} orc_tape_op;

static int orc_tape_step (const orc_tape_op* op, const int32_t* arg_ids, const uint64_t* arg_shapes, void** buf)
{
	const int32_t* ids = arg_ids + op->first_arg;
	void* out = buf[op->out];
	const void* a = op->nargs > 0 ? buf[ids[0]] : 0;
	const void* b = op->nargs > 1 ? buf[ids[1]] : 0;
	const int c = op->opcode;
	if (c >= ORC_ABS && c <= ORC_CUBE) { return orc_unary(c, op->dtype, op->n, a, out); }
	if (c >= ORC_POW && c <= ORC_GT)
	{
		if (op->nargs == 2) { return orc_binary(c, op->dtype, op->n, a, b, out); }
		const void* ins[128];
		if (op->nargs > 128) { return 1; }
		for (int i = 0; i < op->nargs; ++i) { ins[i] = buf[ids[i]]; }
		return orc_nary(c, op->dtype, op->n, op->nargs, ins, out);
	}
	switch (c)
	{
		case ORC_IDENTITY: case ORC_RESHAPE:
			memcpy(out, a, op->n * orc_type_size(op->dtype));
			return 0;
		case ORC_REDUCE_SUM: case ORC_REDUCE_PROD: case ORC_REDUCE_MIN: case ORC_REDUCE_MAX:
			return orc_reduce(c, op->dtype, op->ashape, (unsigned) op->attr[0], 0, a, out);
		case ORC_ARGMAX: return orc_argmax(op->dtype, op->ashape, (int) op->attr[0], a, out);
		case ORC_EXTEND: return orc_extend(op->dtype, op->ashape, op->attr, a, out);
		case ORC_PERMUTE: return orc_permute(op->dtype, op->ashape, op->attr, a, out);
		case ORC_SLICE: return orc_slice(op->dtype, op->ashape, op->attr, op->attr + 8, a, out);
		case ORC_PAD: return orc_pad(op->dtype, op->ashape, op->attr, op->attr + 8, a, out);
		case ORC_REVERSE: return orc_reverse(op->dtype, op->ashape, (unsigned) op->attr[0], a, out);
		case ORC_STRIDE: return orc_stride(op->dtype, op->ashape, op->attr, op->attr + 8, a, out);
		case ORC_SCATTER: return orc_scatter(op->dtype, op->ashape, op->attr, op->attr + 8, a, out);
		case ORC_CONCAT:
		{
			const void* ins[128];
			if (op->nargs > 128) { return 1; }
			for (int i = 0; i < op->nargs; ++i) { ins[i] = buf[ids[i]]; }
			return orc_concat(op->dtype, (int) op->attr[0], op->nargs, arg_shapes + 8 * (size_t) op->first_arg, ins, out);
		}
		case ORC_MATMUL: return orc_matmul(op->dtype, op->ashape, op->bshape, 0, a, b, out);
		case ORC_CONTRACT: return orc_contract(op->dtype, op->ashape, op->bshape, op->nattr / 2, op->attr, 0, a, b, out);
		case ORC_CONV: return orc_conv(op->dtype, op->ashape, op->bshape, op->nattr, op->attr, 0, a, b, out);
		case ORC_SELECT: return orc_select(op->dtype, op->n, a, b, buf[ids[2]], out);
		case ORC_CAST: return orc_cast(op->dtype, op->in_dtype, op->n, a, out);
		default: return 1; /* RAND_UNIF and ASSIGN* are not part of a timed pure pass */
	}
}

/* Runs the tape `reps` times; seconds[r] = wall time of pass r.  arg_shapes holds
 * the shape of every operand (8 values each, parallel to arg_ids). */
int orc_tape_run (const orc_tape_op* ops, int nops, const int32_t* arg_ids, const uint64_t* arg_shapes,
	void** buffers, int reps, double* seconds)
{
	for (int r = 0; r < reps; ++r)
	{
		struct timespec t0, t1;
		clock_gettime(CLOCK_MONOTONIC, &t0);
		for (int i = 0; i < nops; ++i)
		{
			int rc = orc_tape_step(ops + i, arg_ids, arg_shapes, buffers);
			if (rc != 0) { return 1000 + i; }
		}
		clock_gettime(CLOCK_MONOTONIC, &t1);
		if (seconds) { seconds[r] = (double) (t1.tv_sec - t0.tv_sec) + 1e-9 * (double) (t1.tv_nsec - t0.tv_nsec); }
	}
	return 0;
}
