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

// One X-macro row per element type: ENUM, C type, precision (the rank that
// type promotion compares), dtype code of the device library (enum tcg_dtype).
// The codes of the enum follow the key order of the type configuration
// (tools/egen/plugins/dtypes.py:155-159), so the two configurations number
// INT32 differently; the device library has one numbering for both.
#ifdef EGEN_FULLTYPE
/// cfg/fulltype.yml:1-34 (selected like the reference's ETEQ_CFG: define EGEN_FULLTYPE)
#define EGEN_DTYPES(ROW)\
	ROW(DOUBLE, double, 10, 1)\
	ROW(FLOAT, float, 9, 2)\
	ROW(INT8, int8_t, 1, 4)\
	ROW(UINT8, uint8_t, 2, 5)\
	ROW(INT16, int16_t, 3, 6)\
	ROW(UINT16, uint16_t, 4, 7)\
	ROW(INT32, int32_t, 5, 3)\
	ROW(UINT32, uint32_t, 6, 8)\
	ROW(INT64, int64_t, 7, 9)\
	ROW(UINT64, uint64_t, 8, 10)
#else
/// cfg/mintype.yml:4-13
#define EGEN_DTYPES(ROW)\
	ROW(DOUBLE, double, 3, 1)\
	ROW(FLOAT, float, 2, 2)\
	ROW(INT32, int32_t, 1, 3)
#endif

enum _GENERATED_DTYPE
{
	BAD_TYPE = 0,
#define EGEN_ROW(ENUM, CTYPE, PRECISION, DEVICE) ENUM,
	EGEN_DTYPES(EGEN_ROW)
#undef EGEN_ROW
	_N_GENERATED_DTYPES
};

const _GENERATED_DTYPE default_dtype = FLOAT;

std::string name_type (_GENERATED_DTYPE type);
_GENERATED_DTYPE get_type (const std::string& name);

inline uint8_t type_size (_GENERATED_DTYPE type)
{
	switch (type)
	{
#define EGEN_ROW(ENUM, CTYPE, PRECISION, DEVICE) case ENUM: return sizeof(CTYPE);
		EGEN_DTYPES(EGEN_ROW)
#undef EGEN_ROW
		default: global::fatal("cannot get size of bad type");
	}
}

/// The `precision` of the type configuration: the larger wins a promotion
inline size_t type_precision (_GENERATED_DTYPE type)
{
	switch (type)
	{
#define EGEN_ROW(ENUM, CTYPE, PRECISION, DEVICE) case ENUM: return PRECISION;
		EGEN_DTYPES(EGEN_ROW)
#undef EGEN_ROW
		default: return 0;
	}
}

/// The code the device library (include/tcg.h, enum tcg_dtype) knows the type by
inline int device_type (_GENERATED_DTYPE type)
{
	switch (type)
	{
#define EGEN_ROW(ENUM, CTYPE, PRECISION, DEVICE) case ENUM: return DEVICE;
		EGEN_DTYPES(EGEN_ROW)
#undef EGEN_ROW
		default: return 0;
	}
}

template <typename T> _GENERATED_DTYPE get_type (void) { return BAD_TYPE; }
#define EGEN_ROW(ENUM, CTYPE, PRECISION, DEVICE) template <> inline _GENERATED_DTYPE get_type<CTYPE> (void) { return ENUM; }
EGEN_DTYPES(EGEN_ROW)
#undef EGEN_ROW

template <typename T> int device_type (void) { return device_type(get_type<T>()); }

/// static_cast of n elements from `intype` into T
template <typename T>
void type_convert (T* out, const void* input, _GENERATED_DTYPE intype, size_t n)
{
	switch (intype)
	{
#define EGEN_ROW(ENUM, CTYPE, PRECISION, DEVICE) case ENUM: for (size_t i = 0; i < n; ++i) { out[i] = (T) ((const CTYPE*) input)[i]; } break;
		EGEN_DTYPES(EGEN_ROW)
#undef EGEN_ROW
		default: global::fatalf("invalid input type %s", name_type(intype).c_str());
	}
}

}

// Runs `MACRO(T)` with the C++ type of a dtype code (TYPE_LOOKUP of the
// generated dtype.hpp)
#ifdef EGEN_FULLTYPE
#define TYPE_LOOKUP(MACRO, DTYPE) switch (DTYPE) {\
	case egen::DOUBLE: MACRO(double) break;\
	case egen::FLOAT: MACRO(float) break;\
	case egen::INT8: MACRO(int8_t) break;\
	case egen::UINT8: MACRO(uint8_t) break;\
	case egen::INT16: MACRO(int16_t) break;\
	case egen::UINT16: MACRO(uint16_t) break;\
	case egen::INT32: MACRO(int32_t) break;\
	case egen::UINT32: MACRO(uint32_t) break;\
	case egen::INT64: MACRO(int64_t) break;\
	case egen::UINT64: MACRO(uint64_t) break;\
	default: global::fatal("executing bad type"); }
#else
#define TYPE_LOOKUP(MACRO, DTYPE) switch (DTYPE) {\
	case egen::DOUBLE: MACRO(double) break;\
	case egen::FLOAT: MACRO(float) break;\
	case egen::INT32: MACRO(int32_t) break;\
	default: global::fatal("executing bad type"); }
#endif

#endif // TCH_EGEN_HPP
