// Opcode and dtype tables: what tenncor's `egen` generator emits from
// cfg/ops.yml and cfg/mintype.yml (tools/egen/plugins/opcodes.py:9-68,
// tools/egen/plugins/dtypes.py:8-86).  Enum values are the yaml key order with
// BAD_OP / BAD_TYPE = 0, so codes stored in graphs stay interchangeable.
#ifndef TCH_EGEN_HPP
#define TCH_EGEN_HPP

#include <cstdint>
#include <cstring>
#include <string>

#include "global.hpp"

namespace egen
{

enum _GENERATED_OPCODE
{
	BAD_OP = 0, IDENTITY, ABS, NEG, SIN, COS, TAN, EXP, LOG, SQRT, ROUND,
	SIGMOID, TANH, SQUARE, CUBE, RAND_UNIF, REVERSE, REDUCE_SUM, REDUCE_PROD,
	REDUCE_MIN, REDUCE_MAX, ARGMAX, PERMUTE, EXTEND, RESHAPE, SLICE, PAD,
	STRIDE, SCATTER, POW, ADD, SUB, MUL, DIV, MIN, MAX, EQ, NEQ, LT, GT,
	MATMUL, CONTRACT, CONV, SELECT, CONCAT, ASSIGN, ASSIGN_ADD, ASSIGN_SUB,
	ASSIGN_MUL, ASSIGN_DIV, CAST, _N_GENERATED_OPCODES
};

std::string name_op (_GENERATED_OPCODE code);
_GENERATED_OPCODE get_op (const std::string& name);

/// cfg/ops.yml `commutative: True`: ADD, MUL, MIN, MAX, EQ, NEQ
inline bool is_commutative (_GENERATED_OPCODE code)
{
	switch (code)
	{
		case ADD: case MUL: case MIN: case MAX: case EQ: case NEQ: return true;
		default: return false;
	}
}

/// cfg/ops.yml `idempotent: False`: RAND_UNIF, ASSIGN_ADD/SUB/MUL/DIV, CAST
/// (plain ASSIGN is idempotent)
inline bool is_idempotent (_GENERATED_OPCODE code)
{
	switch (code)
	{
		case RAND_UNIF: case ASSIGN_ADD: case ASSIGN_SUB: case ASSIGN_MUL:
		case ASSIGN_DIV: case CAST: return false;
		default: return true;
	}
}

/// cfg/mintype.yml:4-13
enum _GENERATED_DTYPE { BAD_TYPE = 0, DOUBLE, FLOAT, INT32, _N_GENERATED_DTYPES };

const _GENERATED_DTYPE default_dtype = FLOAT;

std::string name_type (_GENERATED_DTYPE type);
_GENERATED_DTYPE get_type (const std::string& name);

inline uint8_t type_size (_GENERATED_DTYPE type)
{
	switch (type)
	{
		case DOUBLE: return 8;
		case FLOAT: return 4;
		case INT32: return 4;
		default: global::fatal("cannot get size of bad type");
	}
}

/// cfg/mintype.yml: DOUBLE 3, FLOAT 2, INT32 1
inline size_t type_precision (_GENERATED_DTYPE type)
{
	switch (type)
	{
		case DOUBLE: return 3;
		case FLOAT: return 2;
		case INT32: return 1;
		default: return 0;
	}
}

template <typename T> _GENERATED_DTYPE get_type (void) { return BAD_TYPE; }
template <> inline _GENERATED_DTYPE get_type<double> (void) { return DOUBLE; }
template <> inline _GENERATED_DTYPE get_type<float> (void) { return FLOAT; }
template <> inline _GENERATED_DTYPE get_type<int32_t> (void) { return INT32; }

/// static_cast of n elements from `intype` into T
template <typename T>
void type_convert (T* out, const void* input, _GENERATED_DTYPE intype, size_t n)
{
	switch (intype)
	{
		case DOUBLE: for (size_t i = 0; i < n; ++i) { out[i] = (T) ((const double*) input)[i]; } break;
		case FLOAT: for (size_t i = 0; i < n; ++i) { out[i] = (T) ((const float*) input)[i]; } break;
		case INT32: for (size_t i = 0; i < n; ++i) { out[i] = (T) ((const int32_t*) input)[i]; } break;
		default: global::fatalf("invalid input type %s", name_type(intype).c_str());
	}
}

}

// Runs `MACRO(T)` with the C++ type of a dtype code (TYPE_LOOKUP of the
// generated dtype.hpp)
#define TYPE_LOOKUP(MACRO, DTYPE) switch (DTYPE) {\
	case egen::DOUBLE: MACRO(double) break;\
	case egen::FLOAT: MACRO(float) break;\
	case egen::INT32: MACRO(int32_t) break;\
	default: global::fatal("executing bad type"); }

#endif // TCH_EGEN_HPP
