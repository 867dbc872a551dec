/*
 * tc_oracle.h -- CPU restatement of tenncor's Eigen operator semantics.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links or calls
 * this file; it exists so that the tests, the smoke check and the benchmark's
 * cpu_baseline leg have an independent, scalar, obviously-correct statement of
 * what each opcode computes.  Every function cites the reference file:line
 * whose behaviour it restates (paths relative to the tenncor source root).
 *
 * Conventions (internal/teq/shape.hpp:56-59, internal/utils/coord/coord.hpp:19-22):
 *   - a shape is 8 dims, dim 0 is the fastest-varying (contiguous) one;
 *     flat index = c0 + c1*s0 + c2*s0*s1 + ...
 *   - dtype codes follow cfg/mintype.yml:4-13: 1 = double, 2 = float, 3 = int32
 *   - opcode values follow the order of keys in cfg/ops.yml (BAD_OP = 0,
 *     IDENTITY = 1, ABS = 2, ...), see tools/egen/plugins/opcodes.py:16-22
 *   - every function returns 0 on success, non-zero for an argument the
 *     reference would have rejected at node construction.
 *
 * Pinning: each function is checked in tests/test_oracle_golden.py against the
 * hand-computed vectors held by the reference's own tests
 * (internal/eigen/test/test_operator.cpp, tenncor/test/test_api.cpp,
 * tenncor/test/test_equation.cpp) and, where those leave a case open, against
 * numpy routines and brute force.  No function here is "parity unpinned".
 */
#ifndef TC_ORACLE_H
#define TC_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_RANK_CAP 8

enum orc_dtype
{
	ORC_BAD_TYPE = 0, ORC_DOUBLE = 1, ORC_FLOAT = 2, ORC_INT32 = 3,
	/* the integer widths the full build adds (cfg/fulltype.yml:11-34) */
	ORC_INT8 = 4, ORC_UINT8 = 5, ORC_INT16 = 6, ORC_UINT16 = 7, ORC_UINT32 = 8,
	ORC_INT64 = 9, ORC_UINT64 = 10
};

/* cfg/ops.yml key order */
enum orc_opcode {
	ORC_BAD_OP = 0, ORC_IDENTITY, ORC_ABS, ORC_NEG, ORC_SIN, ORC_COS, ORC_TAN,
	ORC_EXP, ORC_LOG, ORC_SQRT, ORC_ROUND, ORC_SIGMOID, ORC_TANH, ORC_SQUARE,
	ORC_CUBE, ORC_RAND_UNIF, ORC_REVERSE, ORC_REDUCE_SUM, ORC_REDUCE_PROD,
	ORC_REDUCE_MIN, ORC_REDUCE_MAX, ORC_ARGMAX, ORC_PERMUTE, ORC_EXTEND,
	ORC_RESHAPE, ORC_SLICE, ORC_PAD, ORC_STRIDE, ORC_SCATTER, ORC_POW, ORC_ADD,
	ORC_SUB, ORC_MUL, ORC_DIV, ORC_MIN, ORC_MAX, ORC_EQ, ORC_NEQ, ORC_LT,
	ORC_GT, ORC_MATMUL, ORC_CONTRACT, ORC_CONV, ORC_SELECT, ORC_CONCAT,
	ORC_ASSIGN, ORC_ASSIGN_ADD, ORC_ASSIGN_SUB, ORC_ASSIGN_MUL, ORC_ASSIGN_DIV,
	ORC_CAST, ORC_N_OPCODES
};

size_t orc_type_size (int dtype);

/* internal/eigen/operator.hpp:377-659 (abs..cube) */
int orc_unary (int opcode, int dtype, uint64_t n, const void* in, void* out);

/* internal/eigen/operator.hpp:665-691 (pow), :738-754 (sub), :801-987
 * (div, eq, neq, lt, gt, min, max); two-argument add/mul :694-732,757-795 */
int orc_binary (int opcode, int dtype, uint64_t n,
	const void* a, const void* b, void* out);

/* internal/eigen/operator.hpp:694-732 (add), :757-795 (mul): left fold */
int orc_nary (int opcode, int dtype, uint64_t n, int nargs,
	const void* const* ins, void* out);

/* internal/eigen/operator.hpp:1050-1067 */
int orc_select (int dtype, uint64_t n, const void* cond,
	const void* then, const void* otherwise, void* out);

/* internal/eigen/operator.hpp:1239-1260 */
int orc_cast (int out_dtype, int in_dtype, uint64_t n, const void* in, void* out);

/* internal/eigen/operator.hpp:1190-1237: target (op)= source, in place */
int orc_assign (int opcode, int dtype, uint64_t n, void* target, const void* source);

/* internal/eigen/operator.hpp:54-132.  rankmask bit i set = dim i reduced.
 * wide_acc != 0 accumulates floating sums/products in double (the accuracy
 * oracle); 0 accumulates in T in coordinate order (what a scalar CPU does). */
int orc_reduce (int opcode, int dtype, const uint64_t shape[8],
	unsigned rankmask, int wide_acc, const void* in, void* out);

/* internal/eigen/operator.hpp:134-155.  return_dim >= 8: flat index of max */
int orc_argmax (int dtype, const uint64_t shape[8], int return_dim,
	const void* in, void* out);

/* internal/eigen/operator.hpp:157-173 */
int orc_extend (int dtype, const uint64_t inshape[8], const uint64_t bcast[8],
	const void* in, void* out);

/* internal/eigen/operator.hpp:175-210.  order must be a full permutation */
int orc_permute (int dtype, const uint64_t inshape[8], const uint64_t order[8],
	const void* in, void* out);

/* internal/eigen/operator.hpp:212-255.  offsets/extents already clamped */
int orc_slice (int dtype, const uint64_t inshape[8], const uint64_t offsets[8],
	const uint64_t extents[8], const void* in, void* out);

/* internal/eigen/operator.hpp:257-275 */
int orc_pad (int dtype, const uint64_t inshape[8], const uint64_t before[8],
	const uint64_t after[8], const void* in, void* out);

/* internal/eigen/operator.hpp:316-333 */
int orc_reverse (int dtype, const uint64_t shape[8], unsigned rankmask,
	const void* in, void* out);

/* internal/eigen/operator.hpp:277-293 */
int orc_stride (int dtype, const uint64_t inshape[8], const uint64_t incr[8],
	const uint64_t outshape[8], const void* in, void* out);

/* internal/eigen/operator.hpp:295-314 */
int orc_scatter (int dtype, const uint64_t inshape[8], const uint64_t incr[8],
	const uint64_t outshape[8], const void* in, void* out);

/* internal/eigen/operator.hpp:335-368.  shapes = nargs*8 values */
int orc_concat (int dtype, int axis, int nargs, const uint64_t* shapes,
	const void* const* ins, void* out);

/* internal/eigen/operator.hpp:1107-1139 (batched over dims >= 2) */
int orc_matmul (int dtype, const uint64_t ashape[8], const uint64_t bshape[8],
	int wide_acc, const void* a, const void* b, void* out);

/* internal/eigen/operator.hpp:1069-1103; pairs = npairs*(a_dim, b_dim) as the
 * caller packs them (cfg/ops.yml:517-565) */
int orc_contract (int dtype, const uint64_t ashape[8], const uint64_t bshape[8],
	int npairs, const uint64_t* pairs, int wide_acc,
	const void* a, const void* b, void* out);

/* internal/eigen/operator.hpp:1141-1187; ranks[i] = image dim kernel dim i
 * slides along, nranks <= 8 (remaining dims are completed ascending) */
int orc_conv (int dtype, const uint64_t imgshape[8], const uint64_t kshape[8],
	int nranks, const uint64_t* ranks, int wide_acc,
	const void* img, const void* kernel, void* out);

/* Philox4x32-10 (Salmon et al., SC'11): ten rounds of
 *   {c0,c1,c2,c3} <- {hi(M1*c2)^c1^k0, lo(M1*c2), hi(M0*c0)^c3^k1, lo(M0*c0)}
 * with M0 = 0xD2511F53, M1 = 0xCD9E8D57, the key advanced by
 * (0x9E3779B9, 0xBB67AE85) after every round.  Not a restatement of the
 * reference (which draws from std::default_random_engine on the host,
 * internal/global/random.hpp:87-99,143) but of the published generator the
 * device RAND_UNIF uses; pinned by the known-answer vectors of the Random123
 * distribution in tests/test_oracle_golden.py. */
void orc_philox4x32_10 (const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]);

/* The device RAND_UNIF stream: element i of a draw that starts at generator
 * block `first_block` (counter {block, 0}, key `seed`): float/int32 take word
 * i%4 of block first_block + i/4, double words 2(i%2), 2(i%2)+1 of block
 * first_block + i/2; real types lo + u*(hi-lo) (one fused multiply-add) with
 * u = top 24 / 53 bits scaled into [0,1), int32 lo + ((word * (hi-lo+1)) >> 32). */
int orc_rand_uniform (int dtype, uint64_t n, uint64_t seed, uint64_t first_block,
	const void* lo, const void* hi, void* out);

#ifdef __cplusplus
}
#endif

#endif /* TC_ORACLE_H */
