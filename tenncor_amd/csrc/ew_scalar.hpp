// Scalar semantics of the elementwise operators, shared by every kernel that
// evaluates them (internal/eigen/operator.hpp:377-987).
#ifndef TCG_EW_SCALAR_HPP
#define TCG_EW_SCALAR_HPP

#include "tcg_internal.hpp"

namespace
{

#define TCG_CORE(...) __VA_ARGS__
#include "ew_scalar_core.inc"
#undef TCG_CORE

static inline bool is_unary_op (int op)
{
	return op >= TCG_ABS && op <= TCG_CUBE;
}

static inline bool is_binary_op (int op)
{
	return op >= TCG_POW && op <= TCG_GT;
}

}

#endif // TCG_EW_SCALAR_HPP
