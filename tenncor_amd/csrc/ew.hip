// Elementwise kernels: unary, binary, n-ary, select, cast, in-place assign and
// the fused chain interpreter.  All of them stream memory once with 128-bit
// accesses per lane and are bound by HBM bandwidth.
#include "ew_scalar.hpp"

namespace
{

// ---- streaming kernels ---------------------------------------------------

constexpr int EW_BLOCK = 256;
// launch shape of the streaming kernels: 128-bit accesses in flight per lane,
// workgroups per CU a launch is capped at (a grid-stride loop covers the rest),
// and whether accesses carry the non-temporal hint (bit 0 loads, bit 1 stores).
// Measured on config 2 (np[4096,16384]): operands are read once, so loads are
// non-temporal; results are read by the next node, so stores are not (the
// 256 MiB last-level cache then serves part of the consumer's reads).
// 2 x 64 beat 4 x 16 by 12 % on the binary kernels and 15 % on the unary ones.
#ifndef TCG_EW_UNROLL
#define TCG_EW_UNROLL 2
#endif
#ifndef TCG_EW_BLOCKS_PER_CU
#define TCG_EW_BLOCKS_PER_CU 64
#endif
#ifndef TCG_EW_NONTEMPORAL
#define TCG_EW_NONTEMPORAL 1
#endif
constexpr int EW_UNROLL = TCG_EW_UNROLL;

template <typename T>
__device__ __forceinline__ typename Vec16<T>::type ldv (const T* p, uint64_t vidx)
{
#if TCG_EW_NONTEMPORAL & 1
	return __builtin_nontemporal_load(reinterpret_cast<const typename Vec16<T>::type*>(p) + vidx);
#else
	return reinterpret_cast<const typename Vec16<T>::type*>(p)[vidx];
#endif
}

template <typename T>
__device__ __forceinline__ void stv (T* p, uint64_t vidx, typename Vec16<T>::type v)
{
#if TCG_EW_NONTEMPORAL & 2
	__builtin_nontemporal_store(v, reinterpret_cast<typename Vec16<T>::type*>(p) + vidx);
#else
	reinterpret_cast<typename Vec16<T>::type*>(p)[vidx] = v;
#endif
}

// OP is a compile-time constant so that the switch in apply_* folds away
template <typename T, int OP>
__global__ __launch_bounds__(EW_BLOCK) void ew_unary_vec_k (
	const T* __restrict__ in, T* __restrict__ out, uint64_t n)
{
	constexpr int N = Vec16<T>::N;
	const uint64_t nvec = n / N;
	const uint64_t tile = (uint64_t) EW_BLOCK * EW_UNROLL;
	for (uint64_t base = (uint64_t) blockIdx.x * tile; base < nvec; base += (uint64_t) gridDim.x * tile)
	{
		VecU<T> r[EW_UNROLL];
#pragma unroll
		for (int u = 0; u < EW_UNROLL; ++u)
		{
			uint64_t idx = base + (uint64_t) u * EW_BLOCK + threadIdx.x;
			if (idx < nvec) { r[u].v = ldv(in, idx); }
		}
#pragma unroll
		for (int u = 0; u < EW_UNROLL; ++u)
		{
			uint64_t idx = base + (uint64_t) u * EW_BLOCK + threadIdx.x;
			if (idx < nvec)
			{
#pragma unroll
				for (int e = 0; e < N; ++e) { r[u].e[e] = apply_unary<T>(OP, r[u].e[e]); }
				stv(out, idx, r[u].v);
			}
		}
	}
	if (blockIdx.x == 0)
	{
		uint64_t i = nvec * N + threadIdx.x;
		if (i < n) { out[i] = apply_unary<T>(OP, in[i]); }
	}
}

template <typename T, int OP>
__global__ __launch_bounds__(EW_BLOCK) void ew_binary_vec_k (
	const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ out, uint64_t n)
{
	constexpr int N = Vec16<T>::N;
	const uint64_t nvec = n / N;
	const uint64_t tile = (uint64_t) EW_BLOCK * EW_UNROLL;
	for (uint64_t base = (uint64_t) blockIdx.x * tile; base < nvec; base += (uint64_t) gridDim.x * tile)
	{
		VecU<T> ra[EW_UNROLL], rb[EW_UNROLL];
#pragma unroll
		for (int u = 0; u < EW_UNROLL; ++u)
		{
			uint64_t idx = base + (uint64_t) u * EW_BLOCK + threadIdx.x;
			if (idx < nvec)
			{
				ra[u].v = ldv(a, idx);
				rb[u].v = ldv(b, idx);
			}
		}
#pragma unroll
		for (int u = 0; u < EW_UNROLL; ++u)
		{
			uint64_t idx = base + (uint64_t) u * EW_BLOCK + threadIdx.x;
			if (idx < nvec)
			{
#pragma unroll
				for (int e = 0; e < N; ++e) { ra[u].e[e] = apply_binary<T>(OP, ra[u].e[e], rb[u].e[e]); }
				stv(out, idx, ra[u].v);
			}
		}
	}
	if (blockIdx.x == 0)
	{
		uint64_t i = nvec * N + threadIdx.x;
		if (i < n) { out[i] = apply_binary<T>(OP, a[i], b[i]); }
	}
}

// fallbacks for pointers that are not 16-byte aligned (aliased slices)
template <typename T>
__global__ __launch_bounds__(EW_BLOCK) void ew_unary_scalar_k (int op, const T* in, T* out, uint64_t n)
{
	uint64_t i = (uint64_t) blockIdx.x * EW_BLOCK + threadIdx.x;
	uint64_t step = (uint64_t) gridDim.x * EW_BLOCK;
	for (; i < n; i += step) { out[i] = apply_unary<T>(op, in[i]); }
}

template <typename T>
__global__ __launch_bounds__(EW_BLOCK) void ew_binary_scalar_k (int op, const T* a, const T* b, T* out, uint64_t n)
{
	uint64_t i = (uint64_t) blockIdx.x * EW_BLOCK + threadIdx.x;
	uint64_t step = (uint64_t) gridDim.x * EW_BLOCK;
	for (; i < n; i += step) { out[i] = apply_binary<T>(op, a[i], b[i]); }
}

constexpr int NARY_MAX = 8;
template <typename T>
struct NaryArgs
{
	const T* in[NARY_MAX];
	int nargs;
};

// out = in0 (op) in1 (op) ... folded left to right, one pass over memory
template <typename T, bool VEC>
__global__ __launch_bounds__(EW_BLOCK) void ew_nary_k (int op, NaryArgs<T> args, T* __restrict__ out, uint64_t n)
{
	constexpr int N = VEC ? Vec16<T>::N : 1;
	const uint64_t nvec = n / N;
	uint64_t i = (uint64_t) blockIdx.x * EW_BLOCK + threadIdx.x;
	const uint64_t step = (uint64_t) gridDim.x * EW_BLOCK;
	for (; i < nvec; i += step)
	{
		if constexpr (VEC)
		{
			VecU<T> acc, x;
			acc.v = ldv(args.in[0], i);
			for (int j = 1; j < args.nargs; ++j)
			{
				x.v = ldv(args.in[j], i);
#pragma unroll
				for (int e = 0; e < N; ++e) { acc.e[e] = apply_binary<T>(op, acc.e[e], x.e[e]); }
			}
			stv(out, i, acc.v);
		}
		else
		{
			T acc = args.in[0][i];
			for (int j = 1; j < args.nargs; ++j) { acc = apply_binary<T>(op, acc, args.in[j][i]); }
			out[i] = acc;
		}
	}
	if (VEC && blockIdx.x == 0)
	{
		uint64_t t = nvec * N + threadIdx.x;
		if (t < n)
		{
			T acc = args.in[0][t];
			for (int j = 1; j < args.nargs; ++j) { acc = apply_binary<T>(op, acc, args.in[j][t]); }
			out[t] = acc;
		}
	}
}

template <typename T>
__global__ __launch_bounds__(EW_BLOCK) void ew_select_k (const T* c, const T* a, const T* b, T* out, uint64_t n)
{
	uint64_t i = (uint64_t) blockIdx.x * EW_BLOCK + threadIdx.x;
	uint64_t step = (uint64_t) gridDim.x * EW_BLOCK;
	for (; i < n; i += step) { out[i] = c[i] != 0 ? a[i] : b[i]; }
}

template <typename TO, typename TI>
__global__ __launch_bounds__(EW_BLOCK) void ew_cast_k (const TI* in, TO* out, uint64_t n)
{
	uint64_t i = (uint64_t) blockIdx.x * EW_BLOCK + threadIdx.x;
	uint64_t step = (uint64_t) gridDim.x * EW_BLOCK;
	for (; i < n; i += step) { out[i] = static_cast<TO>(in[i]); }
}

template <typename T>
__global__ __launch_bounds__(EW_BLOCK) void ew_assign_k (int op, T* target, const T* source, uint64_t n)
{
	uint64_t i = (uint64_t) blockIdx.x * EW_BLOCK + threadIdx.x;
	uint64_t step = (uint64_t) gridDim.x * EW_BLOCK;
	for (; i < n; i += step)
	{
		T t = target[i], s = source[i];
		switch (op)
		{
			case TCG_ASSIGN: t = s; break;
			case TCG_ASSIGN_ADD: t = wrap_add(t, s); break;
			case TCG_ASSIGN_SUB: t = wrap_sub(t, s); break;
			case TCG_ASSIGN_MUL: t = wrap_mul(t, s); break;
			case TCG_ASSIGN_DIV: t = safe_div(t, s); break;
		}
		target[i] = t;
	}
}

// ---- host-side launchers ---------------------------------------------------

template <typename T, int OP>
void launch_unary_vec (tcg_ctx* ctx, const T* in, T* out, uint64_t n)
{
	uint64_t nvec = n / Vec16<T>::N;
	unsigned grid = tcg_grid(ctx, nvec, EW_BLOCK * EW_UNROLL, TCG_EW_BLOCKS_PER_CU);
	ew_unary_vec_k<T,OP><<<grid, EW_BLOCK, 0, ctx->stream>>>(in, out, n);
}

template <typename T, int OP>
void launch_binary_vec (tcg_ctx* ctx, const T* a, const T* b, T* out, uint64_t n)
{
	uint64_t nvec = n / Vec16<T>::N;
	unsigned grid = tcg_grid(ctx, nvec, EW_BLOCK * EW_UNROLL, TCG_EW_BLOCKS_PER_CU);
	ew_binary_vec_k<T,OP><<<grid, EW_BLOCK, 0, ctx->stream>>>(a, b, out, n);
}

#define UNARY_CASE(OPC) case OPC: launch_unary_vec<T,OPC>(ctx, in, out, n); break;
#define BINARY_CASE(OPC) case OPC: launch_binary_vec<T,OPC>(ctx, a, b, out, n); break;

template <typename T>
int unary_impl (tcg_ctx* ctx, int op, uint64_t n, const T* in, T* out)
{
	if (tcg_aligned16(in) && tcg_aligned16(out))
	{
		switch (op)
		{
			UNARY_CASE(TCG_ABS) UNARY_CASE(TCG_NEG) UNARY_CASE(TCG_SIN) UNARY_CASE(TCG_COS)
			UNARY_CASE(TCG_TAN) UNARY_CASE(TCG_EXP) UNARY_CASE(TCG_LOG) UNARY_CASE(TCG_SQRT)
			UNARY_CASE(TCG_ROUND) UNARY_CASE(TCG_SIGMOID) UNARY_CASE(TCG_TANH)
			UNARY_CASE(TCG_SQUARE) UNARY_CASE(TCG_CUBE)
		}
	}
	else
	{
		unsigned grid = tcg_grid(ctx, n, EW_BLOCK, 16);
		ew_unary_scalar_k<T><<<grid, EW_BLOCK, 0, ctx->stream>>>(op, in, out, n);
	}
	TCG_LAUNCH_CHECK(ctx, "ew_unary");
	return TCG_OK;
}

template <typename T>
int binary_impl (tcg_ctx* ctx, int op, uint64_t n, const T* a, const T* b, T* out)
{
	if (tcg_aligned16(a) && tcg_aligned16(b) && tcg_aligned16(out))
	{
		switch (op)
		{
			BINARY_CASE(TCG_POW) BINARY_CASE(TCG_ADD) BINARY_CASE(TCG_SUB) BINARY_CASE(TCG_MUL)
			BINARY_CASE(TCG_DIV) BINARY_CASE(TCG_MIN) BINARY_CASE(TCG_MAX) BINARY_CASE(TCG_EQ)
			BINARY_CASE(TCG_NEQ) BINARY_CASE(TCG_LT) BINARY_CASE(TCG_GT)
		}
	}
	else
	{
		unsigned grid = tcg_grid(ctx, n, EW_BLOCK, 16);
		ew_binary_scalar_k<T><<<grid, EW_BLOCK, 0, ctx->stream>>>(op, a, b, out, n);
	}
	TCG_LAUNCH_CHECK(ctx, "ew_binary");
	return TCG_OK;
}

template <typename T>
int nary_impl (tcg_ctx* ctx, int op, uint64_t n, int nargs, const void* const* ins, T* out)
{
	// more than NARY_MAX operands: fold the first NARY_MAX, then keep folding
	// into `out`; the left-to-right order of the reference is preserved
	int done = 0;
	while (done < nargs)
	{
		NaryArgs<T> args;
		int k = 0;
		bool vec = tcg_aligned16(out);
		if (done > 0) { args.in[k++] = out; }
		while (k < NARY_MAX && done < nargs) { args.in[k++] = (const T*) ins[done++]; }
		args.nargs = k;
		for (int j = 0; j < k; ++j) { vec = vec && tcg_aligned16(args.in[j]); }
		if (vec)
		{
			unsigned grid = tcg_grid(ctx, n / Vec16<T>::N, EW_BLOCK, 32);
			ew_nary_k<T,true><<<grid, EW_BLOCK, 0, ctx->stream>>>(op, args, out, n);
		}
		else
		{
			unsigned grid = tcg_grid(ctx, n, EW_BLOCK, 32);
			ew_nary_k<T,false><<<grid, EW_BLOCK, 0, ctx->stream>>>(op, args, out, n);
		}
		TCG_LAUNCH_CHECK(ctx, "ew_nary");
	}
	return TCG_OK;
}

template <typename TO>
int cast_impl (tcg_ctx* ctx, int in_dtype, uint64_t n, const void* in, TO* out)
{
	unsigned grid = tcg_grid(ctx, n, EW_BLOCK, 16);
	switch (in_dtype)
	{
		case TCG_DOUBLE: ew_cast_k<TO,double><<<grid, EW_BLOCK, 0, ctx->stream>>>((const double*) in, out, n); break;
		case TCG_FLOAT: ew_cast_k<TO,float><<<grid, EW_BLOCK, 0, ctx->stream>>>((const float*) in, out, n); break;
		case TCG_INT32: ew_cast_k<TO,int32_t><<<grid, EW_BLOCK, 0, ctx->stream>>>((const int32_t*) in, out, n); break;
		case TCG_INT8: ew_cast_k<TO,int8_t><<<grid, EW_BLOCK, 0, ctx->stream>>>((const int8_t*) in, out, n); break;
		case TCG_UINT8: ew_cast_k<TO,uint8_t><<<grid, EW_BLOCK, 0, ctx->stream>>>((const uint8_t*) in, out, n); break;
		case TCG_INT16: ew_cast_k<TO,int16_t><<<grid, EW_BLOCK, 0, ctx->stream>>>((const int16_t*) in, out, n); break;
		case TCG_UINT16: ew_cast_k<TO,uint16_t><<<grid, EW_BLOCK, 0, ctx->stream>>>((const uint16_t*) in, out, n); break;
		case TCG_UINT32: ew_cast_k<TO,uint32_t><<<grid, EW_BLOCK, 0, ctx->stream>>>((const uint32_t*) in, out, n); break;
		case TCG_INT64: ew_cast_k<TO,int64_t><<<grid, EW_BLOCK, 0, ctx->stream>>>((const int64_t*) in, out, n); break;
		case TCG_UINT64: ew_cast_k<TO,uint64_t><<<grid, EW_BLOCK, 0, ctx->stream>>>((const uint64_t*) in, out, n); break;
		default: return tcg_fail(ctx, TCG_ERR_ARG, "tcg_cast: unknown input dtype %d", in_dtype);
	}
	TCG_LAUNCH_CHECK(ctx, "ew_cast");
	return TCG_OK;
}

} // namespace

extern "C" {

// An elementwise node as a group of one (tcg_ew_fusedx): what such a node is
// while a sequence is recorded as one kernel, and how the integer widths of
// the full type set run (the streaming kernels of this file are built for
// double, float and int32; a group is compiled for its dtype at run time)
static int small_elementwise (tcg_ctx* ctx, int opcode, int dtype, uint64_t n, int nargs,
	const void* const* ins, void* out)
{
	if (nargs > TCG_FX_MAX_LEAVES && tcg_small_mode(ctx))
	{
		TCG_SMALL_RETURN(ctx, tcg_small_unsupported(ctx, "an elementwise node with that many operands"));
	}
	if (nargs > TCG_FX_MAX_LEAVES)
	{
		// a long fold: sixteen operands, then the result so far with fifteen more, ...
		int rc = small_elementwise(ctx, opcode, dtype, n, TCG_FX_MAX_LEAVES, ins, out);
		for (int done = TCG_FX_MAX_LEAVES; done < nargs && rc == TCG_OK;)
		{
			const void* next[TCG_FX_MAX_LEAVES] = {out};
			int take = nargs - done < TCG_FX_MAX_LEAVES - 1 ? nargs - done : TCG_FX_MAX_LEAVES - 1;
			for (int k = 0; k < take; ++k) { next[1 + k] = ins[done + k]; }
			rc = small_elementwise(ctx, opcode, dtype, n, take + 1, next, out);
			done += take;
		}
		return rc;
	}
	uint64_t shape[8] = {n, 1, 1, 1, 1, 1, 1, 1};
	tcg_fx_leaf leaves[TCG_FX_MAX_LEAVES];
	memset(leaves, 0, sizeof(leaves));
	for (int k = 0; k < nargs; ++k)
	{
		leaves[k].ptr = ins[k];
		leaves[k].stride[0] = 1;
		for (int d = 0; d < 8; ++d) { leaves[k].hi[d] = shape[d]; }
	}
	tcg_fx_instr program[TCG_FX_MAX_LEAVES + 1];
	memset(program, 0, sizeof(program));
	int ninstrs = 0;
	auto emit = [&](int op, int a, int b, int c)
	{
		tcg_fx_instr& ins = program[ninstrs++];
		ins.opcode = (uint8_t) op;
		ins.a = (uint8_t) a;
		ins.b = (uint8_t) b;
		ins.c = (uint8_t) c;
		ins.dst = TCG_FX_REG0;
	};
	if (opcode == TCG_SELECT) { emit(opcode, TCG_FX_LEAF0, TCG_FX_LEAF0 + 1, TCG_FX_LEAF0 + 2); }
	else if (opcode == TCG_ASSIGN) { ninstrs = 0; } // the source is stored as it is
	else if (nargs == 1) { emit(opcode, TCG_FX_LEAF0, TCG_FX_NONE, TCG_FX_NONE); }
	else
	{
		emit(opcode, TCG_FX_LEAF0, TCG_FX_LEAF0 + 1, TCG_FX_NONE);
		for (int k = 2; k < nargs; ++k) { emit(opcode, TCG_FX_REG0, TCG_FX_LEAF0 + k, TCG_FX_NONE); }
	}
	tcg_fx_instr& store = program[ninstrs++];
	store.opcode = TCG_FX_STORE;
	store.a = (uint8_t) (opcode == TCG_ASSIGN ? TCG_FX_LEAF0 : TCG_FX_REG0);
	store.b = store.c = TCG_FX_NONE;
	store.dst = 0;
	void* outs[1] = {out};
	return tcg_ew_fusedx(ctx, dtype, shape, nargs, leaves, ninstrs, program, 1, outs);
}

int tcg_ew_unary (tcg_ctx* ctx, int opcode, int dtype, uint64_t n, const void* in, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, is_unary_op(opcode), "tcg_ew_unary: opcode %d is not a unary elementwise op", opcode);
	if (n == 0) { return TCG_OK; }
	TCG_REQUIRE(ctx, in && out, "tcg_ew_unary: NULL pointer");
	if (tcg_small_mode(ctx) || false == tcg_default_dtype(dtype)) { return small_elementwise(ctx, opcode, dtype, n, 1, &in, out); }
	TCG_DISPATCH_TYPE(ctx, dtype, return unary_impl<T>(ctx, opcode, n, (const T*) in, (T*) out));
	return TCG_OK;
}

int tcg_ew_binary (tcg_ctx* ctx, int opcode, int dtype, uint64_t n,
	const void* a, const void* b, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, is_binary_op(opcode), "tcg_ew_binary: opcode %d is not a binary elementwise op", opcode);
	if (n == 0) { return TCG_OK; }
	TCG_REQUIRE(ctx, a && b && out, "tcg_ew_binary: NULL pointer");
	if (tcg_small_mode(ctx) || false == tcg_default_dtype(dtype))
	{
		const void* ins[2] = {a, b};
		return small_elementwise(ctx, opcode, dtype, n, 2, ins, out);
	}
	TCG_DISPATCH_TYPE(ctx, dtype, return binary_impl<T>(ctx, opcode, n, (const T*) a, (const T*) b, (T*) out));
	return TCG_OK;
}

int tcg_ew_nary (tcg_ctx* ctx, int opcode, int dtype, uint64_t n, int nargs,
	const void* const* ins, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, opcode == TCG_ADD || opcode == TCG_MUL, "tcg_ew_nary: opcode %d is not ADD or MUL", opcode);
	TCG_REQUIRE(ctx, nargs >= 2 && ins, "tcg_ew_nary: needs at least 2 operands, got %d", nargs);
	if (n == 0) { return TCG_OK; }
	for (int i = 0; i < nargs; ++i) { TCG_REQUIRE(ctx, ins[i], "tcg_ew_nary: operand %d is NULL", i); }
	TCG_REQUIRE(ctx, out, "tcg_ew_nary: NULL output");
	if (tcg_small_mode(ctx) || false == tcg_default_dtype(dtype)) { return small_elementwise(ctx, opcode, dtype, n, nargs, ins, out); }
	TCG_DISPATCH_TYPE(ctx, dtype, return nary_impl<T>(ctx, opcode, n, nargs, ins, (T*) out));
	return TCG_OK;
}

int tcg_ew_select (tcg_ctx* ctx, int dtype, uint64_t n, const void* cond,
	const void* then, const void* otherwise, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (n == 0) { return TCG_OK; }
	TCG_REQUIRE(ctx, cond && then && otherwise && out, "tcg_ew_select: NULL pointer");
	if (tcg_small_mode(ctx) || false == tcg_default_dtype(dtype))
	{
		const void* ins[3] = {cond, then, otherwise};
		return small_elementwise(ctx, TCG_SELECT, dtype, n, 3, ins, out);
	}
	unsigned grid = tcg_grid(ctx, n, EW_BLOCK, 16);
	TCG_DISPATCH_TYPE(ctx, dtype, (ew_select_k<T><<<grid, EW_BLOCK, 0, ctx->stream>>>(
		(const T*) cond, (const T*) then, (const T*) otherwise, (T*) out, n)));
	TCG_LAUNCH_CHECK(ctx, "ew_select");
	return TCG_OK;
}

int tcg_cast (tcg_ctx* ctx, int out_dtype, int in_dtype, uint64_t n, const void* in, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (n == 0) { return TCG_OK; }
	TCG_REQUIRE(ctx, in && out, "tcg_cast: NULL pointer");
	TCG_DISPATCH_ALL(ctx, out_dtype, return cast_impl<T>(ctx, in_dtype, n, in, (T*) out));
	return TCG_OK;
}

int tcg_assign (tcg_ctx* ctx, int opcode, int dtype, uint64_t n, void* target, const void* source)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, opcode >= TCG_ASSIGN && opcode <= TCG_ASSIGN_DIV, "tcg_assign: opcode %d is not an ASSIGN op", opcode);
	if (n == 0) { return TCG_OK; }
	TCG_REQUIRE(ctx, target && source, "tcg_assign: NULL pointer");
	if (tcg_small_mode(ctx) || false == tcg_default_dtype(dtype))
	{
		if (opcode == TCG_ASSIGN) { return small_elementwise(ctx, TCG_ASSIGN, dtype, n, 1, &source, target); }
		const int fold[] = {TCG_ADD, TCG_SUB, TCG_MUL, TCG_DIV};
		const void* ins[2] = {target, source};
		return small_elementwise(ctx, fold[opcode - TCG_ASSIGN_ADD], dtype, n, 2, ins, target);
	}
	unsigned grid = tcg_grid(ctx, n, EW_BLOCK, 16);
	TCG_DISPATCH_TYPE(ctx, dtype, (ew_assign_k<T><<<grid, EW_BLOCK, 0, ctx->stream>>>(
		opcode, (T*) target, (const T*) source, n)));
	TCG_LAUNCH_CHECK(ctx, "ew_assign");
	return TCG_OK;
}

int tcg_ew_fused (tcg_ctx* ctx, int dtype, uint64_t n, int nleaves,
	const void* const* leaves, int ninstrs, const tcg_ew_instr* program, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, nleaves >= 1 && nleaves <= TCG_EW_MAX_LEAVES, "tcg_ew_fused: %d leaves (1..%d allowed)", nleaves, TCG_EW_MAX_LEAVES);
	TCG_REQUIRE(ctx, ninstrs >= 1 && ninstrs <= TCG_EW_MAX_INSTRS, "tcg_ew_fused: %d instructions (1..%d allowed)", ninstrs, TCG_EW_MAX_INSTRS);
	TCG_REQUIRE(ctx, leaves && program && out, "tcg_ew_fused: NULL pointer");
	auto operand_ok = [nleaves](int k, bool allow_none)
	{
		if (k == TCG_OPD_NONE) { return allow_none; }
		if (k >= TCG_OPD_ACC && k <= TCG_OPD_IMM) { return true; }
		return k >= TCG_OPD_LEAF0 && k < TCG_OPD_LEAF0 + nleaves;
	};
	// the chain is a group of tcg_ew_fusedx over dense operands: ACC, T0, T1
	// become its first three registers, the value of ACC is its one result
	tcg_fx_instr group[TCG_EW_MAX_INSTRS + 4];
	memset(group, 0, sizeof(group));
	int count = 0;
	bool written[3] = {false, false, false};
	auto translate = [](int k) -> uint8_t
	{
		if (k == TCG_OPD_NONE) { return TCG_FX_NONE; }
		if (k == TCG_OPD_IMM) { return TCG_FX_IMM; }
		if (k >= TCG_OPD_LEAF0) { return (uint8_t) (TCG_FX_LEAF0 + (k - TCG_OPD_LEAF0)); }
		return (uint8_t) (TCG_FX_REG0 + (k - TCG_OPD_ACC));
	};
	auto zero = [&](int reg) // registers start at zero
	{
		tcg_fx_instr& ins = group[count++];
		ins.opcode = TCG_IDENTITY;
		ins.a = TCG_FX_IMM;
		ins.b = ins.c = TCG_FX_NONE;
		ins.dst = (uint8_t) (TCG_FX_REG0 + reg);
		ins.imm = 0;
		written[reg] = true;
	};
	for (int i = 0; i < ninstrs; ++i)
	{
		const tcg_ew_instr& ins = program[i];
		bool unary = ins.opcode == TCG_IDENTITY || is_unary_op(ins.opcode);
		TCG_REQUIRE(ctx, unary || is_binary_op(ins.opcode), "tcg_ew_fused: instruction %d has opcode %d", i, (int) ins.opcode);
		TCG_REQUIRE(ctx, operand_ok(ins.a, false) && operand_ok(ins.b, unary) && (unary == (ins.b == TCG_OPD_NONE)),
			"tcg_ew_fused: instruction %d has bad operands (%d, %d)", i, (int) ins.a, (int) ins.b);
		TCG_REQUIRE(ctx, ins.dst >= TCG_OPD_ACC && ins.dst <= TCG_OPD_T1, "tcg_ew_fused: instruction %d has bad destination %d", i, (int) ins.dst);
		for (int k : {(int) ins.a, (int) ins.b})
		{
			if (k >= TCG_OPD_ACC && k <= TCG_OPD_T1 && false == written[k - TCG_OPD_ACC]) { zero(k - TCG_OPD_ACC); }
		}
		tcg_fx_instr& to = group[count++];
		to.opcode = ins.opcode;
		to.a = translate(ins.a);
		to.b = translate(ins.b);
		to.c = TCG_FX_NONE;
		to.dst = translate(ins.dst);
		to.imm = ins.imm;
		written[ins.dst - TCG_OPD_ACC] = true;
	}
	if (false == written[0]) { zero(0); }
	tcg_fx_instr& store = group[count++];
	store.opcode = TCG_FX_STORE;
	store.a = TCG_FX_REG0;
	store.b = store.c = TCG_FX_NONE;
	store.dst = 0;
	if (n == 0) { return TCG_OK; }
	uint64_t shape[8] = {n, 1, 1, 1, 1, 1, 1, 1};
	tcg_fx_leaf views[TCG_EW_MAX_LEAVES];
	memset(views, 0, sizeof(views));
	for (int k = 0; k < nleaves; ++k)
	{
		TCG_REQUIRE(ctx, leaves[k], "tcg_ew_fused: leaf %d is NULL", k);
		views[k].ptr = leaves[k];
		views[k].stride[0] = 1;
		for (int d = 0; d < 8; ++d) { views[k].hi[d] = shape[d]; }
	}
	void* outs[1] = {out};
	return tcg_ew_fusedx(ctx, dtype, shape, nleaves, views, count, group, 1, outs);
}

} // extern "C"
