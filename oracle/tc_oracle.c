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
#define W uint32_t
#define T_IS_INT 1
#define T_IS_SIGNED 1
#include "tc_oracle_typed.inc"
#undef T
#undef ACC
#undef SFX
#undef W
#undef T_IS_INT
#undef T_IS_SIGNED

#define T int8_t
#define ACC int64_t
#define SFX i8
#define W uint32_t
#define T_IS_INT 1
#define T_IS_SIGNED 1
#include "tc_oracle_typed.inc"
#undef T
#undef ACC
#undef SFX
#undef W
#undef T_IS_INT
#undef T_IS_SIGNED

#define T uint8_t
#define ACC int64_t
#define SFX u8
#define W uint32_t
#define T_IS_INT 1
#define T_IS_SIGNED 0
#include "tc_oracle_typed.inc"
#undef T
#undef ACC
#undef SFX
#undef W
#undef T_IS_INT
#undef T_IS_SIGNED

#define T int16_t
#define ACC int64_t
#define SFX i16
#define W uint32_t
#define T_IS_INT 1
#define T_IS_SIGNED 1
#include "tc_oracle_typed.inc"
#undef T
#undef ACC
#undef SFX
#undef W
#undef T_IS_INT
#undef T_IS_SIGNED

#define T uint16_t
#define ACC int64_t
#define SFX u16
#define W uint32_t
#define T_IS_INT 1
#define T_IS_SIGNED 0
#include "tc_oracle_typed.inc"
#undef T
#undef ACC
#undef SFX
#undef W
#undef T_IS_INT
#undef T_IS_SIGNED

#define T uint32_t
#define ACC int64_t
#define SFX u32
#define W uint32_t
#define T_IS_INT 1
#define T_IS_SIGNED 0
#include "tc_oracle_typed.inc"
#undef T
#undef ACC
#undef SFX
#undef W
#undef T_IS_INT
#undef T_IS_SIGNED

#define T int64_t
#define ACC int64_t
#define SFX i64
#define W uint64_t
#define T_IS_INT 1
#define T_IS_SIGNED 1
#include "tc_oracle_typed.inc"
#undef T
#undef ACC
#undef SFX
#undef W
#undef T_IS_INT
#undef T_IS_SIGNED

#define T uint64_t
#define ACC uint64_t
#define SFX u64
#define W uint64_t
#define T_IS_INT 1
#define T_IS_SIGNED 0
#include "tc_oracle_typed.inc"
#undef T
#undef ACC
#undef SFX
#undef W
#undef T_IS_INT
#undef T_IS_SIGNED

size_t orc_type_size (int dtype)
{
	switch (dtype)
	{
		case ORC_DOUBLE: case ORC_INT64: case ORC_UINT64: return 8;
		case ORC_FLOAT: case ORC_INT32: case ORC_UINT32: return 4;
		case ORC_INT16: case ORC_UINT16: return 2;
		case ORC_INT8: case ORC_UINT8: return 1;
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
	switch (dtype)
	{
		case ORC_DOUBLE: return unary_f64(opcode, n, (const double*) in, (double*) out);
		case ORC_FLOAT: return unary_f32(opcode, n, (const float*) in, (float*) out);
		case ORC_INT32: return unary_i32(opcode, n, (const int32_t*) in, (int32_t*) out);
		case ORC_INT8: return unary_i8(opcode, n, (const int8_t*) in, (int8_t*) out);
		case ORC_UINT8: return unary_u8(opcode, n, (const uint8_t*) in, (uint8_t*) out);
		case ORC_INT16: return unary_i16(opcode, n, (const int16_t*) in, (int16_t*) out);
		case ORC_UINT16: return unary_u16(opcode, n, (const uint16_t*) in, (uint16_t*) out);
		case ORC_UINT32: return unary_u32(opcode, n, (const uint32_t*) in, (uint32_t*) out);
		case ORC_INT64: return unary_i64(opcode, n, (const int64_t*) in, (int64_t*) out);
		case ORC_UINT64: return unary_u64(opcode, n, (const uint64_t*) in, (uint64_t*) out);
		default: return 1;
	}
}

int orc_binary (int opcode, int dtype, uint64_t n,
	const void* a, const void* b, void* out)
{
	switch (dtype)
	{
		case ORC_DOUBLE: return binary_f64(opcode, n, (const double*) a, (const double*) b, (double*) out);
		case ORC_FLOAT: return binary_f32(opcode, n, (const float*) a, (const float*) b, (float*) out);
		case ORC_INT32: return binary_i32(opcode, n, (const int32_t*) a, (const int32_t*) b, (int32_t*) out);
		case ORC_INT8: return binary_i8(opcode, n, (const int8_t*) a, (const int8_t*) b, (int8_t*) out);
		case ORC_UINT8: return binary_u8(opcode, n, (const uint8_t*) a, (const uint8_t*) b, (uint8_t*) out);
		case ORC_INT16: return binary_i16(opcode, n, (const int16_t*) a, (const int16_t*) b, (int16_t*) out);
		case ORC_UINT16: return binary_u16(opcode, n, (const uint16_t*) a, (const uint16_t*) b, (uint16_t*) out);
		case ORC_UINT32: return binary_u32(opcode, n, (const uint32_t*) a, (const uint32_t*) b, (uint32_t*) out);
		case ORC_INT64: return binary_i64(opcode, n, (const int64_t*) a, (const int64_t*) b, (int64_t*) out);
		case ORC_UINT64: return binary_u64(opcode, n, (const uint64_t*) a, (const uint64_t*) b, (uint64_t*) out);
		default: return 1;
	}
}

int orc_nary (int opcode, int dtype, uint64_t n, int nargs,
	const void* const* ins, void* out)
{
	switch (dtype)
	{
		case ORC_DOUBLE: return nary_f64(opcode, n, nargs, (const double* const*) ins, (double*) out);
		case ORC_FLOAT: return nary_f32(opcode, n, nargs, (const float* const*) ins, (float*) out);
		case ORC_INT32: return nary_i32(opcode, n, nargs, (const int32_t* const*) ins, (int32_t*) out);
		case ORC_INT8: return nary_i8(opcode, n, nargs, (const int8_t* const*) ins, (int8_t*) out);
		case ORC_UINT8: return nary_u8(opcode, n, nargs, (const uint8_t* const*) ins, (uint8_t*) out);
		case ORC_INT16: return nary_i16(opcode, n, nargs, (const int16_t* const*) ins, (int16_t*) out);
		case ORC_UINT16: return nary_u16(opcode, n, nargs, (const uint16_t* const*) ins, (uint16_t*) out);
		case ORC_UINT32: return nary_u32(opcode, n, nargs, (const uint32_t* const*) ins, (uint32_t*) out);
		case ORC_INT64: return nary_i64(opcode, n, nargs, (const int64_t* const*) ins, (int64_t*) out);
		case ORC_UINT64: return nary_u64(opcode, n, nargs, (const uint64_t* const*) ins, (uint64_t*) out);
		default: return 1;
	}
}

int orc_select (int dtype, uint64_t n, const void* cond,
	const void* then, const void* otherwise, void* out)
{
	switch (dtype)
	{
		case ORC_DOUBLE: return select_f64(n, (const double*) cond, (const double*) then, (const double*) otherwise, (double*) out);
		case ORC_FLOAT: return select_f32(n, (const float*) cond, (const float*) then, (const float*) otherwise, (float*) out);
		case ORC_INT32: return select_i32(n, (const int32_t*) cond, (const int32_t*) then, (const int32_t*) otherwise, (int32_t*) out);
		case ORC_INT8: return select_i8(n, (const int8_t*) cond, (const int8_t*) then, (const int8_t*) otherwise, (int8_t*) out);
		case ORC_UINT8: return select_u8(n, (const uint8_t*) cond, (const uint8_t*) then, (const uint8_t*) otherwise, (uint8_t*) out);
		case ORC_INT16: return select_i16(n, (const int16_t*) cond, (const int16_t*) then, (const int16_t*) otherwise, (int16_t*) out);
		case ORC_UINT16: return select_u16(n, (const uint16_t*) cond, (const uint16_t*) then, (const uint16_t*) otherwise, (uint16_t*) out);
		case ORC_UINT32: return select_u32(n, (const uint32_t*) cond, (const uint32_t*) then, (const uint32_t*) otherwise, (uint32_t*) out);
		case ORC_INT64: return select_i64(n, (const int64_t*) cond, (const int64_t*) then, (const int64_t*) otherwise, (int64_t*) out);
		case ORC_UINT64: return select_u64(n, (const uint64_t*) cond, (const uint64_t*) then, (const uint64_t*) otherwise, (uint64_t*) out);
		default: return 1;
	}
}

/* internal/eigen/operator.hpp:1239-1260: static_cast per element.  Integer to
 * integer is the value modulo 2^width of the target; floating point to
 * integer truncates towards zero (out of range is undefined in C++: pinned to
 * the lowest value of the target for the 32- and 64-bit signed types, what
 * x86's conversions yield, and not used by the tests for the others) */
int orc_cast (int out_dtype, int in_dtype, uint64_t n, const void* in, void* out)
{
	for (uint64_t i = 0; i < n; ++i)
	{
		double v = 0;
		int64_t iv = 0;      /* the value of an integer source (uint64: its bits) */
		int from_int = 0, from_u64 = 0;
		switch (in_dtype)
		{
			case ORC_DOUBLE: v = ((const double*) in)[i]; break;
			case ORC_FLOAT: v = ((const float*) in)[i]; break;
			case ORC_INT32: iv = ((const int32_t*) in)[i]; from_int = 1; break;
			case ORC_INT8: iv = ((const int8_t*) in)[i]; from_int = 1; break;
			case ORC_UINT8: iv = ((const uint8_t*) in)[i]; from_int = 1; break;
			case ORC_INT16: iv = ((const int16_t*) in)[i]; from_int = 1; break;
			case ORC_UINT16: iv = ((const uint16_t*) in)[i]; from_int = 1; break;
			case ORC_UINT32: iv = ((const uint32_t*) in)[i]; from_int = 1; break;
			case ORC_INT64: iv = ((const int64_t*) in)[i]; from_int = 1; break;
			case ORC_UINT64: iv = (int64_t) ((const uint64_t*) in)[i]; from_int = 1; from_u64 = 1; break;
			default: return 1;
		}
		if (from_int) { v = from_u64 ? (double) (uint64_t) iv : (double) iv; }
		else if (out_dtype != ORC_DOUBLE && out_dtype != ORC_FLOAT)
		{
			if (out_dtype == ORC_UINT64)
			{
				iv = (v >= 18446744073709551616.0 || v <= -1.0 || v != v) ? 0 : (int64_t) (uint64_t) v;
			}
			else if (v >= 9223372036854775808.0 || v < -9223372036854775808.0 || v != v) { iv = INT64_MIN; }
			else { iv = (int64_t) v; }
			if (out_dtype == ORC_INT32 && (v >= 2147483648.0 || v < -2147483648.0 || v != v)) { iv = INT32_MIN; }
		}
		switch (out_dtype)
		{
			case ORC_DOUBLE: ((double*) out)[i] = v; break;
			case ORC_FLOAT: ((float*) out)[i] = from_int ? (from_u64 ? (float) (uint64_t) iv : (float) iv) : (float) v; break;
			case ORC_INT32: ((int32_t*) out)[i] = (int32_t) (uint32_t) (uint64_t) iv; break;
			case ORC_INT8: ((int8_t*) out)[i] = (int8_t) (uint8_t) (uint64_t) iv; break;
			case ORC_UINT8: ((uint8_t*) out)[i] = (uint8_t) (uint64_t) iv; break;
			case ORC_INT16: ((int16_t*) out)[i] = (int16_t) (uint16_t) (uint64_t) iv; break;
			case ORC_UINT16: ((uint16_t*) out)[i] = (uint16_t) (uint64_t) iv; break;
			case ORC_UINT32: ((uint32_t*) out)[i] = (uint32_t) (uint64_t) iv; break;
			case ORC_INT64: ((int64_t*) out)[i] = iv; break;
			case ORC_UINT64: ((uint64_t*) out)[i] = (uint64_t) iv; break;
			default: return 1;
		}
	}
	return 0;
}

int orc_assign (int opcode, int dtype, uint64_t n, void* target, const void* source)
{
	switch (dtype)
	{
		case ORC_DOUBLE: return assign_f64(opcode, n, (double*) target, (const double*) source);
		case ORC_FLOAT: return assign_f32(opcode, n, (float*) target, (const float*) source);
		case ORC_INT32: return assign_i32(opcode, n, (int32_t*) target, (const int32_t*) source);
		case ORC_INT8: return assign_i8(opcode, n, (int8_t*) target, (const int8_t*) source);
		case ORC_UINT8: return assign_u8(opcode, n, (uint8_t*) target, (const uint8_t*) source);
		case ORC_INT16: return assign_i16(opcode, n, (int16_t*) target, (const int16_t*) source);
		case ORC_UINT16: return assign_u16(opcode, n, (uint16_t*) target, (const uint16_t*) source);
		case ORC_UINT32: return assign_u32(opcode, n, (uint32_t*) target, (const uint32_t*) source);
		case ORC_INT64: return assign_i64(opcode, n, (int64_t*) target, (const int64_t*) source);
		case ORC_UINT64: return assign_u64(opcode, n, (uint64_t*) target, (const uint64_t*) source);
		default: return 1;
	}
}

int orc_reduce (int opcode, int dtype, const uint64_t shape[8],
	unsigned rankmask, int wide_acc, const void* in, void* out)
{
	switch (dtype)
	{
		case ORC_DOUBLE: return reduce_f64(opcode, shape, rankmask, wide_acc, (const double*) in, (double*) out);
		case ORC_FLOAT: return reduce_f32(opcode, shape, rankmask, wide_acc, (const float*) in, (float*) out);
		case ORC_INT32: return reduce_i32(opcode, shape, rankmask, 0, (const int32_t*) in, (int32_t*) out);
		case ORC_INT8: return reduce_i8(opcode, shape, rankmask, 0, (const int8_t*) in, (int8_t*) out);
		case ORC_UINT8: return reduce_u8(opcode, shape, rankmask, 0, (const uint8_t*) in, (uint8_t*) out);
		case ORC_INT16: return reduce_i16(opcode, shape, rankmask, 0, (const int16_t*) in, (int16_t*) out);
		case ORC_UINT16: return reduce_u16(opcode, shape, rankmask, 0, (const uint16_t*) in, (uint16_t*) out);
		case ORC_UINT32: return reduce_u32(opcode, shape, rankmask, 0, (const uint32_t*) in, (uint32_t*) out);
		case ORC_INT64: return reduce_i64(opcode, shape, rankmask, 0, (const int64_t*) in, (int64_t*) out);
		case ORC_UINT64: return reduce_u64(opcode, shape, rankmask, 0, (const uint64_t*) in, (uint64_t*) out);
		default: return 1;
	}
}

int orc_argmax (int dtype, const uint64_t shape[8], int return_dim,
	const void* in, void* out)
{
	switch (dtype)
	{
		case ORC_DOUBLE: return argmax_f64(shape, return_dim, (const double*) in, (double*) out);
		case ORC_FLOAT: return argmax_f32(shape, return_dim, (const float*) in, (float*) out);
		case ORC_INT32: return argmax_i32(shape, return_dim, (const int32_t*) in, (int32_t*) out);
		case ORC_INT8: return argmax_i8(shape, return_dim, (const int8_t*) in, (int8_t*) out);
		case ORC_UINT8: return argmax_u8(shape, return_dim, (const uint8_t*) in, (uint8_t*) out);
		case ORC_INT16: return argmax_i16(shape, return_dim, (const int16_t*) in, (int16_t*) out);
		case ORC_UINT16: return argmax_u16(shape, return_dim, (const uint16_t*) in, (uint16_t*) out);
		case ORC_UINT32: return argmax_u32(shape, return_dim, (const uint32_t*) in, (uint32_t*) out);
		case ORC_INT64: return argmax_i64(shape, return_dim, (const int64_t*) in, (int64_t*) out);
		case ORC_UINT64: return argmax_u64(shape, return_dim, (const uint64_t*) in, (uint64_t*) out);
		default: return 1;
	}
}

#define GATHER(dtype, mode, ishape, oshape, param, in, out)\
	switch (dtype) {\
		case ORC_DOUBLE: gather_f64(mode, ishape, oshape, param, (const double*) in, (double*) out); return 0;\
		case ORC_FLOAT: gather_f32(mode, ishape, oshape, param, (const float*) in, (float*) out); return 0;\
		case ORC_INT32: gather_i32(mode, ishape, oshape, param, (const int32_t*) in, (int32_t*) out); return 0;\
		case ORC_INT8: gather_i8(mode, ishape, oshape, param, (const int8_t*) in, (int8_t*) out); return 0;\
		case ORC_UINT8: gather_u8(mode, ishape, oshape, param, (const uint8_t*) in, (uint8_t*) out); return 0;\
		case ORC_INT16: gather_i16(mode, ishape, oshape, param, (const int16_t*) in, (int16_t*) out); return 0;\
		case ORC_UINT16: gather_u16(mode, ishape, oshape, param, (const uint16_t*) in, (uint16_t*) out); return 0;\
		case ORC_UINT32: gather_u32(mode, ishape, oshape, param, (const uint32_t*) in, (uint32_t*) out); return 0;\
		case ORC_INT64: gather_i64(mode, ishape, oshape, param, (const int64_t*) in, (int64_t*) out); return 0;\
		case ORC_UINT64: gather_u64(mode, ishape, oshape, param, (const uint64_t*) in, (uint64_t*) out); return 0;\
		default: return 1;\
	}

#define SCATTER_TO(dtype, ishape, oshape, scale, off, in, out)\
	switch (dtype) {\
		case ORC_DOUBLE: scatter_to_f64(ishape, oshape, scale, off, (const double*) in, (double*) out); return 0;\
		case ORC_FLOAT: scatter_to_f32(ishape, oshape, scale, off, (const float*) in, (float*) out); return 0;\
		case ORC_INT32: scatter_to_i32(ishape, oshape, scale, off, (const int32_t*) in, (int32_t*) out); return 0;\
		case ORC_INT8: scatter_to_i8(ishape, oshape, scale, off, (const int8_t*) in, (int8_t*) out); return 0;\
		case ORC_UINT8: scatter_to_u8(ishape, oshape, scale, off, (const uint8_t*) in, (uint8_t*) out); return 0;\
		case ORC_INT16: scatter_to_i16(ishape, oshape, scale, off, (const int16_t*) in, (int16_t*) out); return 0;\
		case ORC_UINT16: scatter_to_u16(ishape, oshape, scale, off, (const uint16_t*) in, (uint16_t*) out); return 0;\
		case ORC_UINT32: scatter_to_u32(ishape, oshape, scale, off, (const uint32_t*) in, (uint32_t*) out); return 0;\
		case ORC_INT64: scatter_to_i64(ishape, oshape, scale, off, (const int64_t*) in, (int64_t*) out); return 0;\
		case ORC_UINT64: scatter_to_u64(ishape, oshape, scale, off, (const uint64_t*) in, (uint64_t*) out); return 0;\
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
			case ORC_INT8: scatter_to_i8(ishape, oshape, ones, off, (const int8_t*) ins[i], (int8_t*) out); break;
			case ORC_UINT8: scatter_to_u8(ishape, oshape, ones, off, (const uint8_t*) ins[i], (uint8_t*) out); break;
			case ORC_INT16: scatter_to_i16(ishape, oshape, ones, off, (const int16_t*) ins[i], (int16_t*) out); break;
			case ORC_UINT16: scatter_to_u16(ishape, oshape, ones, off, (const uint16_t*) ins[i], (uint16_t*) out); break;
			case ORC_UINT32: scatter_to_u32(ishape, oshape, ones, off, (const uint32_t*) ins[i], (uint32_t*) out); break;
			case ORC_INT64: scatter_to_i64(ishape, oshape, ones, off, (const int64_t*) ins[i], (int64_t*) out); break;
			case ORC_UINT64: scatter_to_u64(ishape, oshape, ones, off, (const uint64_t*) ins[i], (uint64_t*) out); break;
			default: return 1;
		}
		off[axis] += ishape[axis];
	}
	return 0;
}

int orc_matmul (int dtype, const uint64_t ashape[8], const uint64_t bshape[8],
	int wide_acc, const void* a, const void* b, void* out)
{
	switch (dtype)
	{
		case ORC_DOUBLE: return matmul_f64(ashape, bshape, wide_acc, (const double*) a, (const double*) b, (double*) out);
		case ORC_FLOAT: return matmul_f32(ashape, bshape, wide_acc, (const float*) a, (const float*) b, (float*) out);
		case ORC_INT32: return matmul_i32(ashape, bshape, 0, (const int32_t*) a, (const int32_t*) b, (int32_t*) out);
		case ORC_INT8: return matmul_i8(ashape, bshape, 0, (const int8_t*) a, (const int8_t*) b, (int8_t*) out);
		case ORC_UINT8: return matmul_u8(ashape, bshape, 0, (const uint8_t*) a, (const uint8_t*) b, (uint8_t*) out);
		case ORC_INT16: return matmul_i16(ashape, bshape, 0, (const int16_t*) a, (const int16_t*) b, (int16_t*) out);
		case ORC_UINT16: return matmul_u16(ashape, bshape, 0, (const uint16_t*) a, (const uint16_t*) b, (uint16_t*) out);
		case ORC_UINT32: return matmul_u32(ashape, bshape, 0, (const uint32_t*) a, (const uint32_t*) b, (uint32_t*) out);
		case ORC_INT64: return matmul_i64(ashape, bshape, 0, (const int64_t*) a, (const int64_t*) b, (int64_t*) out);
		case ORC_UINT64: return matmul_u64(ashape, bshape, 0, (const uint64_t*) a, (const uint64_t*) b, (uint64_t*) out);
		default: return 1;
	}
}

int orc_contract (int dtype, const uint64_t ashape[8], const uint64_t bshape[8],
	int npairs, const uint64_t* pairs, int wide_acc,
	const void* a, const void* b, void* out)
{
	switch (dtype)
	{
		case ORC_DOUBLE: return contract_f64(ashape, bshape, npairs, pairs, wide_acc, (const double*) a, (const double*) b, (double*) out);
		case ORC_FLOAT: return contract_f32(ashape, bshape, npairs, pairs, wide_acc, (const float*) a, (const float*) b, (float*) out);
		case ORC_INT32: return contract_i32(ashape, bshape, npairs, pairs, 0, (const int32_t*) a, (const int32_t*) b, (int32_t*) out);
		case ORC_INT8: return contract_i8(ashape, bshape, npairs, pairs, 0, (const int8_t*) a, (const int8_t*) b, (int8_t*) out);
		case ORC_UINT8: return contract_u8(ashape, bshape, npairs, pairs, 0, (const uint8_t*) a, (const uint8_t*) b, (uint8_t*) out);
		case ORC_INT16: return contract_i16(ashape, bshape, npairs, pairs, 0, (const int16_t*) a, (const int16_t*) b, (int16_t*) out);
		case ORC_UINT16: return contract_u16(ashape, bshape, npairs, pairs, 0, (const uint16_t*) a, (const uint16_t*) b, (uint16_t*) out);
		case ORC_UINT32: return contract_u32(ashape, bshape, npairs, pairs, 0, (const uint32_t*) a, (const uint32_t*) b, (uint32_t*) out);
		case ORC_INT64: return contract_i64(ashape, bshape, npairs, pairs, 0, (const int64_t*) a, (const int64_t*) b, (int64_t*) out);
		case ORC_UINT64: return contract_u64(ashape, bshape, npairs, pairs, 0, (const uint64_t*) a, (const uint64_t*) b, (uint64_t*) out);
		default: return 1;
	}
}

int orc_conv (int dtype, const uint64_t imgshape[8], const uint64_t kshape[8],
	int nranks, const uint64_t* ranks, int wide_acc,
	const void* img, const void* kernel, void* out)
{
	switch (dtype)
	{
		case ORC_DOUBLE: return conv_f64(imgshape, kshape, nranks, ranks, wide_acc, (const double*) img, (const double*) kernel, (double*) out);
		case ORC_FLOAT: return conv_f32(imgshape, kshape, nranks, ranks, wide_acc, (const float*) img, (const float*) kernel, (float*) out);
		case ORC_INT32: return conv_i32(imgshape, kshape, nranks, ranks, 0, (const int32_t*) img, (const int32_t*) kernel, (int32_t*) out);
		case ORC_INT8: return conv_i8(imgshape, kshape, nranks, ranks, 0, (const int8_t*) img, (const int8_t*) kernel, (int8_t*) out);
		case ORC_UINT8: return conv_u8(imgshape, kshape, nranks, ranks, 0, (const uint8_t*) img, (const uint8_t*) kernel, (uint8_t*) out);
		case ORC_INT16: return conv_i16(imgshape, kshape, nranks, ranks, 0, (const int16_t*) img, (const int16_t*) kernel, (int16_t*) out);
		case ORC_UINT16: return conv_u16(imgshape, kshape, nranks, ranks, 0, (const uint16_t*) img, (const uint16_t*) kernel, (uint16_t*) out);
		case ORC_UINT32: return conv_u32(imgshape, kshape, nranks, ranks, 0, (const uint32_t*) img, (const uint32_t*) kernel, (uint32_t*) out);
		case ORC_INT64: return conv_i64(imgshape, kshape, nranks, ranks, 0, (const int64_t*) img, (const int64_t*) kernel, (int64_t*) out);
		case ORC_UINT64: return conv_u64(imgshape, kshape, nranks, ranks, 0, (const uint64_t*) img, (const uint64_t*) kernel, (uint64_t*) out);
		default: return 1;
	}
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
	const uint64_t per = (dtype == ORC_DOUBLE || dtype == ORC_INT64 || dtype == ORC_UINT64) ? 2 : 4;
	if (dtype < 1 || dtype > ORC_UINT64) { return 1; }
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
		else if (dtype == ORC_INT64 || dtype == ORC_UINT64)
		{
			/* lo + floor(r * (hi - lo + 1) / 2^64) on two words; the full range
			 * (hi - lo + 1 wraps to 0) takes the 64 bits as they are */
			uint64_t a = ((const uint64_t*) lo)[i], b = ((const uint64_t*) hi)[i];
			int less = dtype == ORC_INT64 ? (int64_t) b < (int64_t) a : b < a;
			if (less) { ((uint64_t*) out)[i] = a; continue; }
			uint64_t bits = ((uint64_t) r[2 * k + 1] << 32) | r[2 * k];
			uint64_t range = b - a + 1;
			uint64_t off = range == 0 ? bits : (uint64_t) (((unsigned __int128) bits * range) >> 64);
			((uint64_t*) out)[i] = a + off;
		}
		else
		{
			/* integers of at most 32 bits: lo + floor(r * (hi - lo + 1) / 2^32) */
			int64_t a, b;
			switch (dtype)
			{
				case ORC_INT32: a = ((const int32_t*) lo)[i]; b = ((const int32_t*) hi)[i]; break;
				case ORC_INT8: a = ((const int8_t*) lo)[i]; b = ((const int8_t*) hi)[i]; break;
				case ORC_UINT8: a = ((const uint8_t*) lo)[i]; b = ((const uint8_t*) hi)[i]; break;
				case ORC_INT16: a = ((const int16_t*) lo)[i]; b = ((const int16_t*) hi)[i]; break;
				case ORC_UINT16: a = ((const uint16_t*) lo)[i]; b = ((const uint16_t*) hi)[i]; break;
				default: a = ((const uint32_t*) lo)[i]; b = ((const uint32_t*) hi)[i]; break;
			}
			int64_t v = a;
			if (b >= a)
			{
				uint64_t range = (uint64_t) (b - a) + 1;
				v = a + (int64_t) (((uint64_t) r[k] * range) >> 32);
			}
			switch (dtype)
			{
				case ORC_INT32: case ORC_UINT32: ((uint32_t*) out)[i] = (uint32_t) v; break;
				case ORC_INT8: case ORC_UINT8: ((uint8_t*) out)[i] = (uint8_t) v; break;
				default: ((uint16_t*) out)[i] = (uint16_t) v; break;
			}
		}
	}
	return 0;
}
