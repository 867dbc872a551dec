/*
 * tc_oracle.c -- CPU restatement of tenncor's Eigen operator semantics.
 * TEST INFRASTRUCTURE ONLY (see tc_oracle.h): the shipped library never
 * links this file.
 */
#include "tc_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define T double
#define ACC double
#define SFX f64
#define T_IS_INT 0
#include "tc_oracle_typed.inc"
#undef T
#undef ACC
#undef SFX
#undef T_IS_INT

#define T float
#define ACC double
#define SFX f32
#define T_IS_INT 0
#include "tc_oracle_typed.inc"
#undef T
#undef ACC
#undef SFX
#undef T_IS_INT

#define T int32_t
#define ACC int64_t
#define SFX i32
#define T_IS_INT 1
#include "tc_oracle_typed.inc"
#undef T
#undef ACC
#undef SFX
#undef T_IS_INT

#define DISPATCH(dtype, call_f64, call_f32, call_i32)\
	switch (dtype) {\
		case ORC_DOUBLE: return call_f64;\
		case ORC_FLOAT: return call_f32;\
		case ORC_INT32: return call_i32;\
		default: return 1;\
	}

size_t orc_type_size (int dtype)
{
	switch (dtype)
	{
		case ORC_DOUBLE: return 8;
		case ORC_FLOAT: return 4;
		case ORC_INT32: return 4;
		default: return 0;
	}
}

static uint64_t n_elems (const uint64_t shape[8])
{
	uint64_t n = 1;
	for (int i = 0; i < 8; ++i) { n *= shape[i]; }
	return n;
}

int orc_unary (int opcode, int dtype, uint64_t n, const void* in, void* out)
{
	DISPATCH(dtype,
		unary_f64(opcode, n, (const double*) in, (double*) out),
		unary_f32(opcode, n, (const float*) in, (float*) out),
		unary_i32(opcode, n, (const int32_t*) in, (int32_t*) out))
}

int orc_binary (int opcode, int dtype, uint64_t n,
	const void* a, const void* b, void* out)
{
	DISPATCH(dtype,
		binary_f64(opcode, n, (const double*) a, (const double*) b, (double*) out),
		binary_f32(opcode, n, (const float*) a, (const float*) b, (float*) out),
		binary_i32(opcode, n, (const int32_t*) a, (const int32_t*) b, (int32_t*) out))
}

int orc_nary (int opcode, int dtype, uint64_t n, int nargs,
	const void* const* ins, void* out)
{
	DISPATCH(dtype,
		nary_f64(opcode, n, nargs, (const double* const*) ins, (double*) out),
		nary_f32(opcode, n, nargs, (const float* const*) ins, (float*) out),
		nary_i32(opcode, n, nargs, (const int32_t* const*) ins, (int32_t*) out))
}

int orc_select (int dtype, uint64_t n, const void* cond,
	const void* then, const void* otherwise, void* out)
{
	DISPATCH(dtype,
		select_f64(n, (const double*) cond, (const double*) then, (const double*) otherwise, (double*) out),
		select_f32(n, (const float*) cond, (const float*) then, (const float*) otherwise, (float*) out),
		select_i32(n, (const int32_t*) cond, (const int32_t*) then, (const int32_t*) otherwise, (int32_t*) out))
}

/* internal/eigen/operator.hpp:1239-1260: static_cast per element */
int orc_cast (int out_dtype, int in_dtype, uint64_t n, const void* in, void* out)
{
	for (uint64_t i = 0; i < n; ++i)
	{
		double v;
		int32_t iv = 0;
		int from_int = 0;
		switch (in_dtype)
		{
			case ORC_DOUBLE: v = ((const double*) in)[i]; break;
			case ORC_FLOAT: v = ((const float*) in)[i]; break;
			case ORC_INT32: iv = ((const int32_t*) in)[i]; v = iv; from_int = 1; break;
			default: return 1;
		}
		switch (out_dtype)
		{
			case ORC_DOUBLE: ((double*) out)[i] = v; break;
			case ORC_FLOAT: ((float*) out)[i] = (float) v; break;
			case ORC_INT32:
				if (from_int) { ((int32_t*) out)[i] = iv; }
				else if (v >= 2147483648.0 || v < -2147483648.0 || v != v)
				{
					/* out of range is undefined in C++; pinned to INT32_MIN,
					 * what x86 cvttsd2si yields */
					((int32_t*) out)[i] = INT32_MIN;
				}
				else { ((int32_t*) out)[i] = (int32_t) v; }
				break;
			default: return 1;
		}
	}
	return 0;
}

int orc_assign (int opcode, int dtype, uint64_t n, void* target, const void* source)
{
	DISPATCH(dtype,
		assign_f64(opcode, n, (double*) target, (const double*) source),
		assign_f32(opcode, n, (float*) target, (const float*) source),
		assign_i32(opcode, n, (int32_t*) target, (const int32_t*) source))
}

int orc_reduce (int opcode, int dtype, const uint64_t shape[8],
	unsigned rankmask, int wide_acc, const void* in, void* out)
{
	DISPATCH(dtype,
		reduce_f64(opcode, shape, rankmask, wide_acc, (const double*) in, (double*) out),
		reduce_f32(opcode, shape, rankmask, wide_acc, (const float*) in, (float*) out),
		reduce_i32(opcode, shape, rankmask, 0, (const int32_t*) in, (int32_t*) out))
}

int orc_argmax (int dtype, const uint64_t shape[8], int return_dim,
	const void* in, void* out)
{
	DISPATCH(dtype,
		argmax_f64(shape, return_dim, (const double*) in, (double*) out),
		argmax_f32(shape, return_dim, (const float*) in, (float*) out),
		argmax_i32(shape, return_dim, (const int32_t*) in, (int32_t*) out))
}

#define GATHER(dtype, mode, ishape, oshape, param, in, out)\
	switch (dtype) {\
		case ORC_DOUBLE: gather_f64(mode, ishape, oshape, param, (const double*) in, (double*) out); return 0;\
		case ORC_FLOAT: gather_f32(mode, ishape, oshape, param, (const float*) in, (float*) out); return 0;\
		case ORC_INT32: gather_i32(mode, ishape, oshape, param, (const int32_t*) in, (int32_t*) out); return 0;\
		default: return 1;\
	}

#define SCATTER_TO(dtype, ishape, oshape, scale, off, in, out)\
	switch (dtype) {\
		case ORC_DOUBLE: scatter_to_f64(ishape, oshape, scale, off, (const double*) in, (double*) out); return 0;\
		case ORC_FLOAT: scatter_to_f32(ishape, oshape, scale, off, (const float*) in, (float*) out); return 0;\
		case ORC_INT32: scatter_to_i32(ishape, oshape, scale, off, (const int32_t*) in, (int32_t*) out); return 0;\
		default: return 1;\
	}

/* internal/eigen/operator.hpp:157-173: in.broadcast(coord), out[c] = in[c mod S];
 * cfg/ops.yml:266-283: a factor > 1 needs a singular input dim */
int orc_extend (int dtype, const uint64_t inshape[8], const uint64_t bcast[8],
	const void* in, void* out)
{
	uint64_t oshape[8];
	for (int d = 0; d < 8; ++d)
	{
		if (bcast[d] == 0 || (bcast[d] > 1 && inshape[d] > 1)) { return 1; }
		oshape[d] = inshape[d] * bcast[d];
	}
	GATHER(dtype, MAP_MOD, inshape, oshape, bcast, in, out)
}

/* internal/eigen/operator.hpp:175-210: shuffle, out dim i = in dim order[i] */
int orc_permute (int dtype, const uint64_t inshape[8], const uint64_t order[8],
	const void* in, void* out)
{
	uint64_t oshape[8];
	int seen[8] = {0};
	for (int d = 0; d < 8; ++d)
	{
		if (order[d] >= 8 || seen[order[d]]) { return 1; }
		seen[order[d]] = 1;
		oshape[d] = inshape[order[d]];
	}
	GATHER(dtype, MAP_PERM, inshape, oshape, order, in, out)
}

/* internal/eigen/operator.hpp:212-255 */
int orc_slice (int dtype, const uint64_t inshape[8], const uint64_t offsets[8],
	const uint64_t extents[8], const void* in, void* out)
{
	for (int d = 0; d < 8; ++d)
	{
		if (extents[d] == 0 || offsets[d] + extents[d] > inshape[d]) { return 1; }
	}
	GATHER(dtype, MAP_OFFSET, inshape, extents, offsets, in, out)
}

/* internal/eigen/operator.hpp:257-275: zero fill around the input */
int orc_pad (int dtype, const uint64_t inshape[8], const uint64_t before[8],
	const uint64_t after[8], const void* in, void* out)
{
	uint64_t oshape[8], ones[8];
	for (int d = 0; d < 8; ++d)
	{
		oshape[d] = inshape[d] + before[d] + after[d];
		ones[d] = 1;
	}
	memset(out, 0, n_elems(oshape) * orc_type_size(dtype));
	SCATTER_TO(dtype, inshape, oshape, ones, before, in, out)
}

/* internal/eigen/operator.hpp:316-333 */
int orc_reverse (int dtype, const uint64_t shape[8], unsigned rankmask,
	const void* in, void* out)
{
	uint64_t flip[8];
	for (int d = 0; d < 8; ++d) { flip[d] = rankmask >> d & 1; }
	GATHER(dtype, MAP_FLIP, shape, shape, flip, in, out)
}

/* internal/eigen/operator.hpp:277-293: out[c] = in[c * incr] */
int orc_stride (int dtype, const uint64_t inshape[8], const uint64_t incr[8],
	const uint64_t outshape[8], const void* in, void* out)
{
	for (int d = 0; d < 8; ++d)
	{
		if (incr[d] == 0 || outshape[d] == 0 ||
			(outshape[d] - 1) * incr[d] >= inshape[d]) { return 1; }
	}
	GATHER(dtype, MAP_SCALE, inshape, outshape, incr, in, out)
}

/* internal/eigen/operator.hpp:295-314: zeros, then out[c * incr] = in[c] */
int orc_scatter (int dtype, const uint64_t inshape[8], const uint64_t incr[8],
	const uint64_t outshape[8], const void* in, void* out)
{
	uint64_t zero[8] = {0};
	memset(out, 0, n_elems(outshape) * orc_type_size(dtype));
	SCATTER_TO(dtype, inshape, outshape, incr, zero, in, out)
}

/* internal/eigen/operator.hpp:335-368: two args = concatenate along axis;
 * more = out.chip(i, axis) = arg_i (each of size 1 on the axis) */
int orc_concat (int dtype, int axis, int nargs, const uint64_t* shapes,
	const void* const* ins, void* out)
{
	if (axis < 0 || axis >= 8 || nargs < 1) { return 1; }
	uint64_t oshape[8], ones[8], off[8] = {0};
	for (int d = 0; d < 8; ++d)
	{
		oshape[d] = shapes[d];
		ones[d] = 1;
	}
	oshape[axis] = 0;
	for (int i = 0; i < nargs; ++i)
	{
		for (int d = 0; d < 8; ++d)
		{
			if (d != axis && shapes[i * 8 + d] != oshape[d]) { return 1; }
		}
		oshape[axis] += shapes[i * 8 + axis];
	}
	for (int i = 0; i < nargs; ++i)
	{
		const uint64_t* ishape = shapes + i * 8;
		switch (dtype)
		{
			case ORC_DOUBLE: scatter_to_f64(ishape, oshape, ones, off, (const double*) ins[i], (double*) out); break;
			case ORC_FLOAT: scatter_to_f32(ishape, oshape, ones, off, (const float*) ins[i], (float*) out); break;
			case ORC_INT32: scatter_to_i32(ishape, oshape, ones, off, (const int32_t*) ins[i], (int32_t*) out); break;
			default: return 1;
		}
		off[axis] += ishape[axis];
	}
	return 0;
}

int orc_matmul (int dtype, const uint64_t ashape[8], const uint64_t bshape[8],
	int wide_acc, const void* a, const void* b, void* out)
{
	DISPATCH(dtype,
		matmul_f64(ashape, bshape, wide_acc, (const double*) a, (const double*) b, (double*) out),
		matmul_f32(ashape, bshape, wide_acc, (const float*) a, (const float*) b, (float*) out),
		matmul_i32(ashape, bshape, 0, (const int32_t*) a, (const int32_t*) b, (int32_t*) out))
}

int orc_contract (int dtype, const uint64_t ashape[8], const uint64_t bshape[8],
	int npairs, const uint64_t* pairs, int wide_acc,
	const void* a, const void* b, void* out)
{
	DISPATCH(dtype,
		contract_f64(ashape, bshape, npairs, pairs, wide_acc, (const double*) a, (const double*) b, (double*) out),
		contract_f32(ashape, bshape, npairs, pairs, wide_acc, (const float*) a, (const float*) b, (float*) out),
		contract_i32(ashape, bshape, npairs, pairs, 0, (const int32_t*) a, (const int32_t*) b, (int32_t*) out))
}

int orc_conv (int dtype, const uint64_t imgshape[8], const uint64_t kshape[8],
	int nranks, const uint64_t* ranks, int wide_acc,
	const void* img, const void* kernel, void* out)
{
	DISPATCH(dtype,
		conv_f64(imgshape, kshape, nranks, ranks, wide_acc, (const double*) img, (const double*) kernel, (double*) out),
		conv_f32(imgshape, kshape, nranks, ranks, wide_acc, (const float*) img, (const float*) kernel, (float*) out),
		conv_i32(imgshape, kshape, nranks, ranks, 0, (const int32_t*) img, (const int32_t*) kernel, (int32_t*) out))
}

/* ---- device RAND_UNIF stream ------------------------------------------- */

void orc_philox4x32_10 (const uint32_t counter[4], const uint32_t key[2], uint32_t out[4])
{
	uint32_t c[4] = {counter[0], counter[1], counter[2], counter[3]};
	uint32_t k0 = key[0], k1 = key[1];
	for (int round = 0; round < 10; ++round)
	{
		uint64_t p0 = (uint64_t) 0xD2511F53u * c[0];
		uint64_t p1 = (uint64_t) 0xCD9E8D57u * c[2];
		uint32_t n0 = (uint32_t) (p1 >> 32) ^ c[1] ^ k0;
		uint32_t n1 = (uint32_t) p1;
		uint32_t n2 = (uint32_t) (p0 >> 32) ^ c[3] ^ k1;
		uint32_t n3 = (uint32_t) p0;
		c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
		k0 += 0x9E3779B9u;
		k1 += 0xBB67AE85u;
	}
	memcpy(out, c, sizeof(c));
}

int orc_rand_uniform (int dtype, uint64_t n, uint64_t seed, uint64_t first_block,
	const void* lo, const void* hi, void* out)
{
	const uint32_t key[2] = {(uint32_t) seed, (uint32_t) (seed >> 32)};
	const uint64_t per = dtype == 1 ? 2 : 4;
	if (dtype < 1 || dtype > 3) { return 1; }
	for (uint64_t i = 0; i < n; ++i)
	{
		uint64_t block = first_block + i / per;
		uint32_t ctr[4] = {(uint32_t) block, (uint32_t) (block >> 32), 0, 0}, r[4];
		orc_philox4x32_10(ctr, key, r);
		unsigned k = (unsigned) (i % per);
		if (dtype == 2)
		{
			float a = ((const float*) lo)[i], b = ((const float*) hi)[i];
			float u = (float) (r[k] >> 8) * 0x1p-24f;
			((float*) out)[i] = fmaf(u, b - a, a);
		}
		else if (dtype == 1)
		{
			double a = ((const double*) lo)[i], b = ((const double*) hi)[i];
			uint64_t bits = ((uint64_t) r[2 * k + 1] << 32) | r[2 * k];
			double u = (double) (bits >> 11) * 0x1p-53;
			((double*) out)[i] = fma(u, b - a, a);
		}
		else
		{
			int32_t a = ((const int32_t*) lo)[i], b = ((const int32_t*) hi)[i];
			if (b < a) { ((int32_t*) out)[i] = a; continue; }
			uint64_t range = (uint64_t) ((int64_t) b - (int64_t) a) + 1;
			((int32_t*) out)[i] = (int32_t) ((int64_t) a + (int64_t) (((uint64_t) r[k] * range) >> 32));
		}
	}
	return 0;
}
