// Scalar semantics of the elementwise operators, shared by every kernel that
// evaluates them (internal/eigen/operator.hpp:377-987).
#ifndef TCG_EW_SCALAR_HPP
#define TCG_EW_SCALAR_HPP

#include "tcg_internal.hpp"

namespace
{

template <typename T> struct is_int { static constexpr bool value = false; };
template <> struct is_int<int32_t> { static constexpr bool value = true; };

template <typename T>
__device__ __forceinline__ T wrap_add (T a, T b)
{
	if constexpr (is_int<T>::value) { return (T) ((uint32_t) a + (uint32_t) b); }
	else { return a + b; }
}

template <typename T>
__device__ __forceinline__ T wrap_sub (T a, T b)
{
	if constexpr (is_int<T>::value) { return (T) ((uint32_t) a - (uint32_t) b); }
	else { return a - b; }
}

template <typename T>
__device__ __forceinline__ T wrap_mul (T a, T b)
{
	if constexpr (is_int<T>::value) { return (T) ((uint32_t) a * (uint32_t) b); }
	else { return a * b; }
}

template <typename T>
__device__ __forceinline__ T safe_div (T a, T b)
{
	if constexpr (is_int<T>::value)
	{
		// the CPU traps on these two; the device returns 0 instead
		if (b == 0 || (a == INT32_MIN && b == -1)) { return 0; }
		return a / b;
	}
	else { return a / b; }
}

// (int) std::pow(a, b) of the CPU path is exact whenever the power is an
// integer that a double holds; the device pow() is not correctly rounded, so
// integer powers are computed by squaring (wrapping like the other int ops)
__device__ __forceinline__ int32_t int_pow (int32_t a, int32_t b)
{
	if (b < 0)
	{
		// |a| > 1: the fraction truncates to 0; a == 0 divides by zero on the CPU
		if (a == 1) { return 1; }
		if (a == -1) { return (b & 1) ? -1 : 1; }
		return 0;
	}
	uint32_t base = (uint32_t) a, r = 1;
	uint32_t e = (uint32_t) b;
	while (e)
	{
		if (e & 1) { r *= base; }
		base *= base;
		e >>= 1;
	}
	return (int32_t) r;
}

// float: single-precision library routines (<= 1-2 ulp, far inside the 1e-5
// budget); int32: through double and truncated, like std::sin(int) on the CPU
template <typename T>
__device__ __forceinline__ T apply_unary (int op, T x)
{
	switch (op)
	{
		case TCG_IDENTITY: return x;
		case TCG_ABS:
			if constexpr (is_int<T>::value) { return x < 0 ? (T) (0u - (uint32_t) x) : x; }
			else if constexpr (sizeof(T) == 4) { return fabsf(x); }
			else { return fabs(x); }
		case TCG_NEG:
			if constexpr (is_int<T>::value) { return (T) (0u - (uint32_t) x); }
			else { return -x; }
		case TCG_SIN:
			if constexpr (sizeof(T) == 4 && !is_int<T>::value) { return sinf(x); }
			else { return (T) sin((double) x); }
		case TCG_COS:
			if constexpr (sizeof(T) == 4 && !is_int<T>::value) { return cosf(x); }
			else { return (T) cos((double) x); }
		case TCG_TAN:
			if constexpr (sizeof(T) == 4 && !is_int<T>::value) { return tanf(x); }
			else { return (T) tan((double) x); }
		case TCG_EXP:
			if constexpr (sizeof(T) == 4 && !is_int<T>::value) { return expf(x); }
			else { return (T) exp((double) x); }
		case TCG_LOG:
			if constexpr (sizeof(T) == 4 && !is_int<T>::value) { return logf(x); }
			else { return (T) log((double) x); }
		case TCG_SQRT:
			if constexpr (sizeof(T) == 4 && !is_int<T>::value) { return sqrtf(x); }
			else { return (T) sqrt((double) x); }
		case TCG_ROUND:
			if constexpr (is_int<T>::value) { return x; }
			else if constexpr (sizeof(T) == 4) { return roundf(x); }
			else { return round(x); }
		case TCG_SIGMOID:
			if constexpr (is_int<T>::value)
			{
				T e = (T) exp(-(double) x);
				T d = (T) (1u + (uint32_t) e);
				return d == 0 ? 0 : (T) (1 / d);
			}
			else if constexpr (sizeof(T) == 4) { return 1.0f / (1.0f + expf(-x)); }
			else { return 1.0 / (1.0 + exp(-x)); }
		case TCG_TANH:
			if constexpr (sizeof(T) == 4 && !is_int<T>::value) { return tanhf(x); }
			else { return (T) tanh((double) x); }
		case TCG_SQUARE: return wrap_mul(x, x);
		case TCG_CUBE: return wrap_mul(wrap_mul(x, x), x);
		default: return x;
	}
}

template <typename T>
__device__ __forceinline__ T apply_binary (int op, T a, T b)
{
	switch (op)
	{
		case TCG_POW:
			if constexpr (is_int<T>::value) { return int_pow(a, b); }
			else if constexpr (sizeof(T) == 4) { return powf(a, b); }
			else { return pow(a, b); }
		case TCG_ADD: return wrap_add(a, b);
		case TCG_SUB: return wrap_sub(a, b);
		case TCG_MUL: return wrap_mul(a, b);
		case TCG_DIV: return safe_div(a, b);
		case TCG_MIN: return a < b ? a : b;
		case TCG_MAX: return a > b ? a : b;
		case TCG_EQ: return (T) (a == b);
		case TCG_NEQ: return (T) (a != b);
		case TCG_LT: return (T) (a < b);
		case TCG_GT: return (T) (a > b);
		default: return a;
	}
}

bool is_unary_op (int op)
{
	return op >= TCG_ABS && op <= TCG_CUBE;
}

bool is_binary_op (int op)
{
	return op >= TCG_POW && op <= TCG_GT;
}

}

#endif // TCG_EW_SCALAR_HPP
