// A group of elementwise nodes of one shape evaluated in one pass: operands
// are read through strided, offset and zero-bordered views (what EXTEND,
// SLICE, PAD and PERMUTE nodes in front of an elementwise node amount to),
// every node of the group is computed in registers, and the values that
// something outside the group reads are stored.  One launch replaces one
// launch per node (internal/eigen/device.hpp:304-372 materialises each);
// memory traffic drops to the group's inputs and outputs: HBM-bound for large
// shapes, launch-bound for the small per-step shapes of unrolled recurrent
// graphs, where the saving is the launches.
//
// Arithmetic is done by the same scalar routines, in the same order, as the
// one-node kernels: results are bit-identical to the unfused evaluation.
#include "ew_scalar.hpp"

#include <hip/hiprtc.h>

#include <sys/stat.h>
#include <unistd.h>

#include <chrono>
#include <cstdlib>
#include <map>
#include <mutex>
#include <sstream>
#include <unordered_map>

namespace
{

constexpr int FX_BLOCK = 256;
#define FX_MAXD 8
constexpr int FX_SLOTS = TCG_FX_MAX_LEAVES + TCG_FX_MAX_REGS;

#define TCG_CORE(...) __VA_ARGS__
#include "ew_fusedx_args.inc"
#include "pass_args.inc"
#undef TCG_CORE

static_assert(sizeof(FxArgs) <= 4096, "launch arguments must fit the kernel argument segment");

FxDiv fx_make_div (uint32_t d)
{
	FxDiv f = {1, 0, 0, 0};
	f.d = d;
	uint32_t l = 0;
	while (((uint64_t) 1 << l) < d) { ++l; }
	f.m = (uint32_t) ((((uint64_t) 1 << 32) * (((uint64_t) 1 << l) - d)) / d + 1);
	f.s1 = l < 1 ? l : 1;
	f.s2 = l == 0 ? 0 : l - 1;
	return f;
}

// The register file of one lane: leaves first, then registers.  It is only
// ever indexed by constants, so it lives in VGPRs; the slot an instruction
// names is wave-uniform, so picking it is a scalar branch, not a memory access
// (an array indexed by the slot number would be placed in scratch memory).
static_assert(FX_SLOTS == 32, "fx_get / fx_put enumerate the slots");

// ends every case of the slot switches: without it the optimiser merges the
// cases into one access through a selected address, which forces the file
// into memory
#define FX_KEEP_APART asm volatile("")

// one statement per element of the lane's vector, without a loop: every index
// must be a constant before the optimiser decides where the file lives
#define FX_EACH(stmt)\
	{ if constexpr (N > 0) { constexpr int e_ = 0; stmt; }\
	if constexpr (N > 1) { constexpr int e_ = 1; stmt; }\
	if constexpr (N > 2) { constexpr int e_ = 2; stmt; }\
	if constexpr (N > 3) { constexpr int e_ = 3; stmt; } }

template <typename T, int N>
__device__ __forceinline__ void fx_get (const T (&file)[FX_SLOTS][N], int s, T (&v)[N])
{
	switch (s)
	{
		case 0: FX_EACH(v[e_] = file[0][e_]) FX_KEEP_APART; break;
		case 1: FX_EACH(v[e_] = file[1][e_]) FX_KEEP_APART; break;
		case 2: FX_EACH(v[e_] = file[2][e_]) FX_KEEP_APART; break;
		case 3: FX_EACH(v[e_] = file[3][e_]) FX_KEEP_APART; break;
		case 4: FX_EACH(v[e_] = file[4][e_]) FX_KEEP_APART; break;
		case 5: FX_EACH(v[e_] = file[5][e_]) FX_KEEP_APART; break;
		case 6: FX_EACH(v[e_] = file[6][e_]) FX_KEEP_APART; break;
		case 7: FX_EACH(v[e_] = file[7][e_]) FX_KEEP_APART; break;
		case 8: FX_EACH(v[e_] = file[8][e_]) FX_KEEP_APART; break;
		case 9: FX_EACH(v[e_] = file[9][e_]) FX_KEEP_APART; break;
		case 10: FX_EACH(v[e_] = file[10][e_]) FX_KEEP_APART; break;
		case 11: FX_EACH(v[e_] = file[11][e_]) FX_KEEP_APART; break;
		case 12: FX_EACH(v[e_] = file[12][e_]) FX_KEEP_APART; break;
		case 13: FX_EACH(v[e_] = file[13][e_]) FX_KEEP_APART; break;
		case 14: FX_EACH(v[e_] = file[14][e_]) FX_KEEP_APART; break;
		case 15: FX_EACH(v[e_] = file[15][e_]) FX_KEEP_APART; break;
		case 16: FX_EACH(v[e_] = file[16][e_]) FX_KEEP_APART; break;
		case 17: FX_EACH(v[e_] = file[17][e_]) FX_KEEP_APART; break;
		case 18: FX_EACH(v[e_] = file[18][e_]) FX_KEEP_APART; break;
		case 19: FX_EACH(v[e_] = file[19][e_]) FX_KEEP_APART; break;
		case 20: FX_EACH(v[e_] = file[20][e_]) FX_KEEP_APART; break;
		case 21: FX_EACH(v[e_] = file[21][e_]) FX_KEEP_APART; break;
		case 22: FX_EACH(v[e_] = file[22][e_]) FX_KEEP_APART; break;
		case 23: FX_EACH(v[e_] = file[23][e_]) FX_KEEP_APART; break;
		case 24: FX_EACH(v[e_] = file[24][e_]) FX_KEEP_APART; break;
		case 25: FX_EACH(v[e_] = file[25][e_]) FX_KEEP_APART; break;
		case 26: FX_EACH(v[e_] = file[26][e_]) FX_KEEP_APART; break;
		case 27: FX_EACH(v[e_] = file[27][e_]) FX_KEEP_APART; break;
		case 28: FX_EACH(v[e_] = file[28][e_]) FX_KEEP_APART; break;
		case 29: FX_EACH(v[e_] = file[29][e_]) FX_KEEP_APART; break;
		case 30: FX_EACH(v[e_] = file[30][e_]) FX_KEEP_APART; break;
		case 31: FX_EACH(v[e_] = file[31][e_]) FX_KEEP_APART; break;
		default: break;
	}
}

template <typename T, int N>
__device__ __forceinline__ void fx_put (T (&file)[FX_SLOTS][N], int s, const T (&v)[N])
{
	switch (s)
	{
		case 0: FX_EACH(file[0][e_] = v[e_]) FX_KEEP_APART; break;
		case 1: FX_EACH(file[1][e_] = v[e_]) FX_KEEP_APART; break;
		case 2: FX_EACH(file[2][e_] = v[e_]) FX_KEEP_APART; break;
		case 3: FX_EACH(file[3][e_] = v[e_]) FX_KEEP_APART; break;
		case 4: FX_EACH(file[4][e_] = v[e_]) FX_KEEP_APART; break;
		case 5: FX_EACH(file[5][e_] = v[e_]) FX_KEEP_APART; break;
		case 6: FX_EACH(file[6][e_] = v[e_]) FX_KEEP_APART; break;
		case 7: FX_EACH(file[7][e_] = v[e_]) FX_KEEP_APART; break;
		case 8: FX_EACH(file[8][e_] = v[e_]) FX_KEEP_APART; break;
		case 9: FX_EACH(file[9][e_] = v[e_]) FX_KEEP_APART; break;
		case 10: FX_EACH(file[10][e_] = v[e_]) FX_KEEP_APART; break;
		case 11: FX_EACH(file[11][e_] = v[e_]) FX_KEEP_APART; break;
		case 12: FX_EACH(file[12][e_] = v[e_]) FX_KEEP_APART; break;
		case 13: FX_EACH(file[13][e_] = v[e_]) FX_KEEP_APART; break;
		case 14: FX_EACH(file[14][e_] = v[e_]) FX_KEEP_APART; break;
		case 15: FX_EACH(file[15][e_] = v[e_]) FX_KEEP_APART; break;
		case 16: FX_EACH(file[16][e_] = v[e_]) FX_KEEP_APART; break;
		case 17: FX_EACH(file[17][e_] = v[e_]) FX_KEEP_APART; break;
		case 18: FX_EACH(file[18][e_] = v[e_]) FX_KEEP_APART; break;
		case 19: FX_EACH(file[19][e_] = v[e_]) FX_KEEP_APART; break;
		case 20: FX_EACH(file[20][e_] = v[e_]) FX_KEEP_APART; break;
		case 21: FX_EACH(file[21][e_] = v[e_]) FX_KEEP_APART; break;
		case 22: FX_EACH(file[22][e_] = v[e_]) FX_KEEP_APART; break;
		case 23: FX_EACH(file[23][e_] = v[e_]) FX_KEEP_APART; break;
		case 24: FX_EACH(file[24][e_] = v[e_]) FX_KEEP_APART; break;
		case 25: FX_EACH(file[25][e_] = v[e_]) FX_KEEP_APART; break;
		case 26: FX_EACH(file[26][e_] = v[e_]) FX_KEEP_APART; break;
		case 27: FX_EACH(file[27][e_] = v[e_]) FX_KEEP_APART; break;
		case 28: FX_EACH(file[28][e_] = v[e_]) FX_KEEP_APART; break;
		case 29: FX_EACH(file[29][e_] = v[e_]) FX_KEEP_APART; break;
		case 30: FX_EACH(file[30][e_] = v[e_]) FX_KEEP_APART; break;
		case 31: FX_EACH(file[31][e_] = v[e_]) FX_KEEP_APART; break;
		default: break;
	}
}

// operand code -> slot of the register file (leaves first)
__device__ __forceinline__ int fx_slot (int code)
{
	return code >= TCG_FX_REG0 ? code - TCG_FX_REG0 + TCG_FX_MAX_LEAVES : code - TCG_FX_LEAF0;
}

// N > 1: dim 0 is contiguous in every operand that does not broadcast along
// it, and every extent, offset, stride and bound involved is a multiple of N
template <typename T, int N>
__global__ __launch_bounds__(FX_BLOCK) void ew_fusedx_k (FxArgs p)
{
	const uint32_t nvec = (uint32_t) (p.total / N);
	const uint32_t step = gridDim.x * FX_BLOCK;
	for (uint32_t idx = blockIdx.x * FX_BLOCK + threadIdx.x; idx < nvec; idx += step)
	{
		int64_t off[TCG_FX_MAX_LEAVES];
		bool inside[TCG_FX_MAX_LEAVES];
#pragma unroll
		for (int k = 0; k < TCG_FX_MAX_LEAVES; ++k)
		{
			off[k] = k < (int) p.nleaf ? p.leaf[k].off : 0;
			inside[k] = true;
		}
		uint32_t rem = idx;
		for (uint32_t d = 0; d < p.nd; ++d)
		{
			uint32_t c;
			if (d + 1 == p.nd) { c = rem; }
			else
			{
				uint32_t q = fx_div(rem, p.div[d]);
				c = rem - q * p.div[d].d;
				rem = q;
			}
			if (d == 0) { c *= N; }
#pragma unroll
			for (int k = 0; k < TCG_FX_MAX_LEAVES; ++k)
			{
				if (k < (int) p.nleaf)
				{
					off[k] += (int64_t) c * p.leaf[k].stride[d];
					if (p.leaf[k].boxed)
					{
						inside[k] = inside[k] && c >= p.leaf[k].lo[d] && c < p.leaf[k].hi[d];
					}
				}
			}
		}
		T file[FX_SLOTS][N];
#pragma unroll
		for (int k = 0; k < TCG_FX_MAX_LEAVES; ++k)
		{
			if (k < (int) p.nleaf)
			{
				const T* src = (const T*) p.leaf[k].ptr + off[k];
				if (!inside[k])
				{
					FX_EACH(file[k][e_] = (T) 0)
				}
				else if (N > 1 && !p.leaf[k].bcast0)
				{
					VecU<T> v;
					v.v = *reinterpret_cast<const typename Vec16<T>::type*>(src);
					FX_EACH(file[k][e_] = v.e[e_])
					for (uint32_t r = 1; r < p.leaf[k].nsum; ++r)
					{
						v.v = *reinterpret_cast<const typename Vec16<T>::type*>(src + (int64_t) r * p.leaf[k].sum_stride);
						FX_EACH(file[k][e_] += v.e[e_])
					}
				}
				else
				{
					T s = *src;
					for (uint32_t r = 1; r < p.leaf[k].nsum; ++r) { s += src[(int64_t) r * p.leaf[k].sum_stride]; }
					FX_EACH(file[k][e_] = s)
				}
			}
		}
		for (uint32_t i = 0; i < p.ninstr; ++i)
		{
			const FxInstr ins = p.prog[i];
			const T imm = (T) p.imm[i];
			T va[N], vb[N], vc[N], vr[N];
			if (ins.a == TCG_FX_IMM)
			{
#pragma unroll
				for (int e = 0; e < N; ++e) { va[e] = imm; }
			}
			else { fx_get<T,N>(file, fx_slot(ins.a), va); }
			if (ins.opcode == TCG_FX_STORE)
			{
				T* dst = (T*) p.out[ins.dst] + (uint64_t) idx * N;
				if (N > 1)
				{
					VecU<T> v;
#pragma unroll
					for (int e = 0; e < N; ++e) { v.e[e] = va[e]; }
					*reinterpret_cast<typename Vec16<T>::type*>(dst) = v.v;
				}
				else { *dst = va[0]; }
				continue;
			}
			const bool has_b = ins.b != TCG_FX_NONE;
			const bool has_c = ins.c != TCG_FX_NONE;
			if (has_b)
			{
				if (ins.b == TCG_FX_IMM)
				{
#pragma unroll
					for (int e = 0; e < N; ++e) { vb[e] = imm; }
				}
				else { fx_get<T,N>(file, fx_slot(ins.b), vb); }
			}
			if (has_c)
			{
				if (ins.c == TCG_FX_IMM)
				{
#pragma unroll
					for (int e = 0; e < N; ++e) { vc[e] = imm; }
				}
				else { fx_get<T,N>(file, fx_slot(ins.c), vc); }
			}
			if (has_c)
			{
#pragma unroll
				for (int e = 0; e < N; ++e) { vr[e] = va[e] != (T) 0 ? vb[e] : vc[e]; } // SELECT
			}
			else if (has_b)
			{
#pragma unroll
				for (int e = 0; e < N; ++e)
				{
					vr[e] = ins.opcode == TCG_FX_BITOR ? bit_or<T>(va[e], vb[e]) : apply_binary<T>(ins.opcode, va[e], vb[e]);
				}
			}
			else
			{
#pragma unroll
				for (int e = 0; e < N; ++e) { vr[e] = apply_unary<T>(ins.opcode, va[e]); }
			}
			fx_put<T,N>(file, fx_slot(ins.dst), vr);
		}
	}
}

template <typename T>
int fusedx_launch (tcg_ctx* ctx, FxArgs& p, bool vec)
{
	constexpr int N = Vec16<T>::N;
	if (vec)
	{
		p.div[0] = fx_make_div(p.size[0] / N);
		unsigned grid = tcg_grid(ctx, p.total / N, FX_BLOCK, 8);
		ew_fusedx_k<T,N><<<grid, FX_BLOCK, 0, ctx->stream>>>(p);
	}
	else
	{
		unsigned grid = tcg_grid(ctx, p.total, FX_BLOCK, 8);
		ew_fusedx_k<T,1><<<grid, FX_BLOCK, 0, ctx->stream>>>(p);
	}
	TCG_LAUNCH_CHECK(ctx, "ew_fusedx");
	return TCG_OK;
}

// ---- kernels compiled at run time ------------------------------------------
//
// The interpreter above pays for decoding the program in every wave.  A group
// that is evaluated again and again (every step of an unrolled recurrent
// graph, every replay of a recording) is better served by a kernel written
// for it: the program becomes straight-line code over named registers, the
// number of dims and the way each leaf is addressed are fixed in the source.
// Extents, strides, offsets, bounds, immediates and pointers stay launch
// arguments, so one kernel serves every launch of the same program shape.
// The source is built from the same scalar routines (ew_scalar_core.inc) and
// compiled by the runtime compiler with the flags the library is built with.

#define TCG_CORE(...) #__VA_ARGS__
const char* const fx_scalar_src =
#include "ew_scalar_core.inc"
;
const char* const fx_args_src =
#include "ew_fusedx_args.inc"
;
#undef TCG_CORE

struct FxJit
{
	std::mutex mu;
	std::unordered_map<std::string,hipFunction_t> kernels;
	// what the kernels of this process cost (under `mu`): compiled here, loaded
	// from the files an earlier process left, milliseconds spent on either
	uint64_t compiled = 0, from_disk = 0;
	double ms = 0.0;
};

FxJit& fx_jit (void)
{
	// never destroyed: loaded code may be launched until the process ends
	static FxJit* jit = new FxJit();
	return *jit;
}

bool fx_jit_enabled (void)
{
	static const bool on = []
	{
		const char* env = getenv("TCG_FX_JIT");
		return !(env && env[0] == '0');
	}();
	return on;
}

// typedefs, opcode names, the scalar routines and the argument structs
void fx_emit_prelude (std::ostringstream& o)
{
	o << "typedef signed char int8_t; typedef unsigned char uint8_t; typedef short int16_t;\n"
		"typedef unsigned short uint16_t; typedef int int32_t;\n"
		"typedef unsigned int uint32_t; typedef long int64_t; typedef unsigned long uint64_t;\n"
		"#ifndef INT32_MIN\n#define INT32_MIN (-2147483647 - 1)\n#endif\n"
		"#define FX_MAXD " << FX_MAXD << "\n"
		"#define TCG_FX_MAX_LEAVES " << TCG_FX_MAX_LEAVES << "\n"
		"#define TCG_FX_MAX_INSTRS " << TCG_FX_MAX_INSTRS << "\n"
		"#define TCG_FX_MAX_OUTS " << TCG_FX_MAX_OUTS << "\n";
	static const struct { const char* name; int value; } opcodes[] = {
#define FX_OP(n) {#n, n}
		FX_OP(TCG_IDENTITY), FX_OP(TCG_ABS), FX_OP(TCG_NEG), FX_OP(TCG_SIN), FX_OP(TCG_COS), FX_OP(TCG_TAN),
		FX_OP(TCG_EXP), FX_OP(TCG_LOG), FX_OP(TCG_SQRT), FX_OP(TCG_ROUND), FX_OP(TCG_SIGMOID), FX_OP(TCG_TANH),
		FX_OP(TCG_SQUARE), FX_OP(TCG_CUBE), FX_OP(TCG_POW), FX_OP(TCG_ADD), FX_OP(TCG_SUB), FX_OP(TCG_MUL),
		FX_OP(TCG_DIV), FX_OP(TCG_MIN), FX_OP(TCG_MAX), FX_OP(TCG_EQ), FX_OP(TCG_NEQ), FX_OP(TCG_LT), FX_OP(TCG_GT),
#undef FX_OP
	};
	o << "enum {";
	for (auto& op : opcodes) { o << op.name << " = " << op.value << ", "; }
	o << "};\n" << fx_scalar_src << "\n" << fx_args_src << "\n";
}

// What one index `idx` of the iteration space computes: operand loads, the
// program as straight-line code, the stores.  Expects `p` (an FxArgs), `idx`
// and the element type `T` (with N > 1 also VT and VU) in scope.
// dense: the leaf is addressed like the output (offset + linear index)
// Baked launch arguments: the generated code holds extents, strides, offsets,
// bounds and immediates as literals and takes its pointers from these expressions
struct FxBake
{
	std::string leaf_ptr[TCG_FX_MAX_LEAVES];
	std::string out_ptr[TCG_FX_MAX_OUTS];
};

/// The three parts of what one index computes, kept apart so that a caller can
/// put the loads of several indices in front of their arithmetic and their
/// stores behind it (stores may alias later loads as far as the compiler can
/// tell, so it never moves a load across one by itself)
struct FxParts
{
	std::ostringstream load, compute, store;
};

/// `sfx` is appended to every local name (several indices in one scope);
/// `idx` names the index variable; `stream`: leaves whose every element is
/// read exactly once are loaded with the non-temporal hint; `supplied[k]`:
/// leaf k is not loaded -- the caller declares `T l<k><sfx>[N]` itself, between
/// the loads and the arithmetic
void fx_emit_parts (FxParts& parts, int N, const FxArgs& p, const bool* dense, const FxBake* bake,
	const std::string& sfx, const std::string& idx, bool stream, const bool* supplied = nullptr)
{
	std::ostringstream& o = parts.load;
	// how the generated code names a launch argument: a field of `p`, or (baked)
	// the value itself and a pointer expression
	auto num = [](int64_t v) { return "((int64_t) " + std::to_string(v) + "ll)"; };
	auto r_off = [&](uint32_t k) { return bake ? num(p.leaf[k].off) : "p.leaf[" + std::to_string(k) + "].off"; };
	auto r_stride = [&](uint32_t k, uint32_t d)
	{
		return bake ? num(p.leaf[k].stride[d]) : "p.leaf[" + std::to_string(k) + "].stride[" + std::to_string(d) + "]";
	};
	auto r_lo = [&](uint32_t k, uint32_t d)
	{
		return bake ? std::to_string(p.leaf[k].lo[d]) + "u" : "p.leaf[" + std::to_string(k) + "].lo[" + std::to_string(d) + "]";
	};
	auto r_hi = [&](uint32_t k, uint32_t d)
	{
		return bake ? std::to_string(p.leaf[k].hi[d]) + "u" : "p.leaf[" + std::to_string(k) + "].hi[" + std::to_string(d) + "]";
	};
	auto r_sum_stride = [&](uint32_t k) { return bake ? num(p.leaf[k].sum_stride) : "p.leaf[" + std::to_string(k) + "].sum_stride"; };
	auto r_leaf = [&](uint32_t k) { return bake ? bake->leaf_ptr[k] : "p.leaf[" + std::to_string(k) + "].ptr"; };
	auto r_out = [&](uint32_t k) { return bake ? bake->out_ptr[k] : "p.out[" + std::to_string(k) + "]"; };
	auto r_imm = [&](uint32_t i) -> std::string
	{
		if (!bake) { return "p.imm[" + std::to_string(i) + "]"; }
		double v = p.imm[i];
		if (v != v) { return "__builtin_nan(\"\")"; }
		if (v - v != 0.0) { return v > 0 ? "__builtin_inf()" : "(-__builtin_inf())"; }
		char text[64];
		snprintf(text, sizeof(text), "%a", v);
		return std::string("(") + text + ")";
	};
	bool need_coords = false;
	for (uint32_t k = 0; k < p.nleaf; ++k) { need_coords = need_coords || (!dense[k] && !(supplied && supplied[k])); }
	if (need_coords)
	{
		o << "uint32_t rem" << sfx << " = " << idx << ";\n";
		for (uint32_t d = 0; d + 1 < p.nd; ++d)
		{
			if (bake)
			{
				o << "const uint32_t q" << d << sfx << " = rem" << sfx << " / " << p.div[d].d << "u;\n"
					"uint32_t c" << d << sfx << " = rem" << sfx << " - q" << d << sfx << " * " << p.div[d].d << "u;\nrem" << sfx << " = q" << d << sfx << ";\n";
				continue;
			}
			o << "const uint32_t q" << d << sfx << " = fx_div(rem" << sfx << ", p.div[" << d << "]);\n"
				"uint32_t c" << d << sfx << " = rem" << sfx << " - q" << d << sfx << " * p.div[" << d << "].d;\nrem" << sfx << " = q" << d << sfx << ";\n";
		}
		o << "uint32_t c" << p.nd - 1 << sfx << " = rem" << sfx << ";\n";
		if (N > 1) { o << "c0" << sfx << " *= " << N << ";\n"; }
	}
	for (uint32_t k = 0; k < p.nleaf; ++k)
	{
		const FxLeaf& L = p.leaf[k];
		if (supplied && supplied[k]) { continue; }
		// every element read once: no zero stride over an extent above one
		bool once = stream && !L.bcast0 && !L.boxed;
		for (uint32_t d = 0; d < p.nd && once; ++d) { once = dense[k] || p.size[d] == 1 || L.stride[d] != 0; }
		o << "T l" << k << sfx << "[" << N << "];\n{\n";
		if (dense[k])
		{
			o << "const T* src = (const T*) " << r_leaf(k) << " + (" << r_off(k) << " + (int64_t) " << idx << " * " << N << ");\n";
		}
		else
		{
			o << "int64_t off = " << r_off(k);
			for (uint32_t d = 0; d < p.nd; ++d)
			{
				if (d == 0 && L.bcast0) { continue; }
				o << " + (int64_t) c" << d << sfx << " * " << r_stride(k, d);
			}
			o << ";\nconst T* src = (const T*) " << r_leaf(k) << " + off;\n";
		}
		if (L.boxed)
		{
			o << "bool inside = true";
			for (uint32_t d = 0; d < p.nd; ++d)
			{
				o << " && c" << d << sfx << " >= " << r_lo(k, d) << " && c" << d << sfx << " < " << r_hi(k, d);
			}
			o << ";\nif (inside)\n";
		}
		o << "{\n";
		if (N > 1 && !L.bcast0)
		{
			o << "VU v; v.v = " << (once ? "__builtin_nontemporal_load((const VT*) src)" : "*(const VT*) src") << ";\n";
			if (L.nsum > 1)
			{
				// the ranges are added in their order; the loads of several are in flight together
				o << "_Pragma(\"unroll 8\")\nfor (uint32_t r = 1; r < " << L.nsum << "u; ++r)\n{\n"
					"VU w; w.v = *(const VT*) (src + (int64_t) r * " << r_sum_stride(k) << ");\n";
				for (int e = 0; e < N; ++e) { o << "v.e[" << e << "] += w.e[" << e << "];\n"; }
				o << "}\n";
			}
			for (int e = 0; e < N; ++e) { o << "l" << k << sfx << "[" << e << "] = v.e[" << e << "];\n"; }
		}
		else
		{
			o << "T s = *src;\n";
			if (L.nsum > 1)
			{
				o << "_Pragma(\"unroll 8\")\nfor (uint32_t r = 1; r < " << L.nsum << "u; ++r) { s += src[(int64_t) r * " << r_sum_stride(k) << "]; }\n";
			}
			for (int e = 0; e < N; ++e) { o << "l" << k << sfx << "[" << e << "] = s;\n"; }
		}
		o << "}\n";
		if (L.boxed)
		{
			o << "else\n{\n";
			for (int e = 0; e < N; ++e) { o << "l" << k << sfx << "[" << e << "] = (T) 0;\n"; }
			o << "}\n";
		}
		o << "}\n";
	}
	// straight-line program: every write of a register gets a name of its own
	std::ostringstream& c = parts.compute;
	std::ostringstream& st = parts.store;
	std::string reg_name[TCG_FX_MAX_REGS];
	auto operand = [&](int code, uint32_t i, int e) -> std::string
	{
		if (code == TCG_FX_IMM) { return "imm" + std::to_string(i) + sfx; }
		if (code >= TCG_FX_REG0) { return reg_name[code - TCG_FX_REG0] + "[" + std::to_string(e) + "]"; }
		return "l" + std::to_string(code - TCG_FX_LEAF0) + sfx + "[" + std::to_string(e) + "]";
	};
	for (uint32_t i = 0; i < p.ninstr; ++i)
	{
		const FxInstr& ins = p.prog[i];
		bool uses_imm = ins.a == TCG_FX_IMM || ins.b == TCG_FX_IMM || ins.c == TCG_FX_IMM;
		if (uses_imm) { c << "const T imm" << i << sfx << " = (T) " << r_imm(i) << ";\n"; }
		if (ins.opcode == TCG_FX_STORE)
		{
			st << "{\nT* dst = (T*) " << r_out(ins.dst) << " + (uint64_t) " << idx << " * " << N << ";\n";
			if (N > 1)
			{
				st << "VU v;\n";
				for (int e = 0; e < N; ++e) { st << "v.e[" << e << "] = " << operand(ins.a, i, e) << ";\n"; }
				st << "*(VT*) dst = v.v;\n";
			}
			else { st << "*dst = " << operand(ins.a, i, 0) << ";\n"; }
			st << "}\n";
			continue;
		}
		std::string name = "v" + std::to_string(i) + sfx;
		c << "T " << name << "[" << N << "];\n";
		for (int e = 0; e < N; ++e)
		{
			c << name << "[" << e << "] = ";
			if (ins.c != TCG_FX_NONE)
			{
				c << operand(ins.a, i, e) << " != (T) 0 ? " << operand(ins.b, i, e) << " : " << operand(ins.c, i, e);
			}
			else if (ins.opcode == TCG_FX_BITOR)
			{
				c << "bit_or<T>(" << operand(ins.a, i, e) << ", " << operand(ins.b, i, e) << ")";
			}
			else if (ins.b != TCG_FX_NONE)
			{
				c << "apply_binary<T>(" << (int) ins.opcode << ", " << operand(ins.a, i, e) << ", " << operand(ins.b, i, e) << ")";
			}
			else
			{
				c << "apply_unary<T>(" << (int) ins.opcode << ", " << operand(ins.a, i, e) << ")";
			}
			c << ";\n";
		}
		reg_name[ins.dst - TCG_FX_REG0] = name;
	}
}

/// What one index `idx` computes, in program order (loads, arithmetic, stores)
void fx_emit_body (std::ostringstream& o, int N, const FxArgs& p, const bool* dense, const FxBake* bake = nullptr)
{
	FxParts parts;
	fx_emit_parts(parts, N, p, dense, bake, "", "idx", false);
	o << parts.load.str() << parts.compute.str() << parts.store.str();
}

const char* fx_type_name (int dtype)
{
	switch (dtype)
	{
		case TCG_DOUBLE: return "double";
		case TCG_FLOAT: return "float";
		case TCG_INT32: return "int32_t";
		case TCG_INT8: return "int8_t";
		case TCG_UINT8: return "uint8_t";
		case TCG_INT16: return "int16_t";
		case TCG_UINT16: return "uint16_t";
		case TCG_UINT32: return "uint32_t";
		case TCG_INT64: return "int64_t";
		default: return "uint64_t";
	}
}

// `unroll` indices per lane and iteration, their loads issued together in
// front of the arithmetic: a streaming group moves (operands + results) x 4n
// bytes and runs at the rate its loads are kept in flight.  Measured on the
// five-node chain of np[4096,16384] floats (3 operands, 1 result): one index
// per iteration with ordinary loads 5.2 TB/s, with non-temporal loads 6.0,
// two indices in flight 6.8 (what a plain copy reaches); non-temporal stores
// cost 0.5 TB/s.
std::string fx_source (int dtype, int N, const FxArgs& p, const bool* dense, int unroll, bool stream)
{
	std::ostringstream o;
	fx_emit_prelude(o);
	o << "typedef " << fx_type_name(dtype) << " T;\n";
	if (N > 1)
	{
		o << "typedef T VT __attribute__((ext_vector_type(" << N << ")));\n"
			"union VU { VT v; T e[" << N << "]; };\n";
	}
	o << "extern \"C\" __global__ __launch_bounds__(" << FX_BLOCK << ") void fx (FxArgs p)\n{\n"
		"const uint32_t nvec = (uint32_t) (p.total / " << N << ");\n";
	uint32_t tile = FX_BLOCK * (uint32_t) unroll;
	if (unroll > 1)
	{
		// whole tiles of `unroll` indices per lane, then the rest one by one
		o << "const uint32_t nfull = nvec / " << tile << "u * " << tile << "u;\n"
			"for (uint32_t base = blockIdx.x * " << tile << "u + threadIdx.x; base < nfull; base += gridDim.x * " << tile << "u)\n{\n";
		FxParts parts;
		for (int u = 0; u < unroll; ++u)
		{
			std::string sfx = "_" + std::to_string(u);
			parts.load << "const uint32_t idx" << sfx << " = base + " << u * FX_BLOCK << "u;\n";
			fx_emit_parts(parts, N, p, dense, nullptr, sfx, "idx" + sfx, stream);
		}
		o << parts.load.str() << parts.compute.str() << parts.store.str() << "}\n";
		o << "for (uint32_t idx = nfull + blockIdx.x * " << FX_BLOCK << " + threadIdx.x; idx < nvec; idx += gridDim.x * " << FX_BLOCK << ")\n{\n";
	}
	else
	{
		o << "const uint32_t step = gridDim.x * " << FX_BLOCK << ";\n"
			"for (uint32_t idx = blockIdx.x * " << FX_BLOCK << " + threadIdx.x; idx < nvec; idx += step)\n{\n";
	}
	FxParts tail;
	fx_emit_parts(tail, N, p, dense, nullptr, "", "idx", stream);
	o << tail.load.str() << tail.compute.str() << tail.store.str();
	o << "}\n}\n";
	return o.str();
}

// Compiled kernels are kept on disk between processes: a graph of a few thousand
// nodes needs a handful of kernels of 0.1-0.5 s each, which its first recording
// would otherwise pay again in every process.  One file per kernel under
// $TCG_FX_CACHE, else $XDG_CACHE_HOME/tenncor_amd/fx, else ~/.cache/tenncor_amd/fx
// (TCG_FX_CACHE=0: none), named by a hash of what identifies the code -- compiler
// version, kernel name, flags, source text -- and holding that text in full in
// front of the code object, so that a file is only ever used for the text it
// was compiled from.  Written under another name and moved into place.
std::string fx_cache_dir (void)
{
	const char* env = getenv("TCG_FX_CACHE");
	if (env && env[0] == '0' && env[1] == '\0') { return ""; }
	std::string dir;
	if (env && env[0]) { dir = env; }
	else if (const char* xdg = getenv("XDG_CACHE_HOME")) { dir = std::string(xdg) + "/tenncor_amd/fx"; }
	else if (const char* home = getenv("HOME")) { dir = std::string(home) + "/.cache/tenncor_amd/fx"; }
	else { return ""; }
	// every level, ignoring the ones that exist; a directory that cannot be made
	// shows when the file cannot be written, and nothing is cached then
	for (size_t at = 1; at <= dir.size(); ++at)
	{
		if (at == dir.size() || dir[at] == '/') { mkdir(dir.substr(0, at).c_str(), 0700); }
	}
	return dir;
}

std::string fx_cache_path (const std::string& identity)
{
	static const std::string dir = fx_cache_dir();
	if (dir.empty()) { return ""; }
	uint64_t h1 = 1469598103934665603ull, h2 = 0x9e3779b97f4a7c15ull; // two 64-bit hashes of the text
	for (unsigned char c : identity)
	{
		h1 = (h1 ^ c) * 1099511628211ull;
		h2 = (h2 + c) * 0xff51afd7ed558ccdull;
		h2 ^= h2 >> 29;
	}
	char name[64];
	snprintf(name, sizeof(name), "/%016llx%016llx.co", (unsigned long long) h1, (unsigned long long) h2);
	return dir + name;
}

bool fx_cache_read (const std::string& path, const std::string& identity, std::vector<char>& code)
{
	if (path.empty()) { return false; }
	FILE* f = fopen(path.c_str(), "rb");
	if (nullptr == f) { return false; }
	bool ok = false;
	uint64_t lens[2] = {0, 0};
	if (1 == fread(lens, sizeof(lens), 1, f) && lens[0] == identity.size() && lens[1] > 0 && lens[1] < (1ull << 30))
	{
		std::string text(lens[0], '\0');
		code.assign(lens[1], '\0');
		ok = (lens[0] == 0 || 1 == fread(&text[0], lens[0], 1, f)) && text == identity && 1 == fread(code.data(), lens[1], 1, f);
	}
	fclose(f);
	return ok;
}

void fx_cache_write (const std::string& path, const std::string& identity, const std::vector<char>& code)
{
	if (path.empty() || code.empty()) { return; }
	const std::string tmp = path + "." + std::to_string((long) getpid()) + ".tmp";
	FILE* f = fopen(tmp.c_str(), "wb");
	if (nullptr == f) { return; }
	uint64_t lens[2] = {identity.size(), code.size()};
	bool ok = 1 == fwrite(lens, sizeof(lens), 1, f) && 1 == fwrite(identity.data(), identity.size(), 1, f) &&
		1 == fwrite(code.data(), code.size(), 1, f);
	ok = 0 == fclose(f) && ok;
	if (false == ok || 0 != rename(tmp.c_str(), path.c_str())) { remove(tmp.c_str()); }
}

int fx_compile (tcg_ctx* ctx, const std::string& source, hipFunction_t* out, const char* name = "fx")
{
	if (const char* dir = getenv("TCG_FX_DUMP"))
	{
		// the generated sources, for reading: <dir>/<kernel>_<hash of the text>.hip
		char path[512];
		snprintf(path, sizeof(path), "%s/%s_%016zx.hip", dir, name, std::hash<std::string>()(source));
		if (FILE* f = fopen(path, "w"))
		{
			fwrite(source.data(), 1, source.size(), f);
			fclose(f);
		}
	}
	std::string arch = "--offload-arch=" + ctx->arch;
	// the flags libtcg itself is built with (packed fp32 forms stay off), and
	// no contraction: a multiply node feeding an add node must round twice, as
	// it does when the two nodes run as separate kernels
	const char* opts[] = {arch.c_str(), "-O3", "-std=c++17", "-ffp-contract=off",
		"-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
	const auto begun = std::chrono::steady_clock::now();
	FxJit& jit = fx_jit();
	auto spent = [&]
	{
		jit.ms += std::chrono::duration<double,std::milli>(std::chrono::steady_clock::now() - begun).count();
	};
	// code compiled by an earlier process for this text, these flags and this compiler
	std::string identity = "tcg-fx-1\n";
	{
		int major = 0, minor = 0;
		hiprtcVersion(&major, &minor);
		identity += std::to_string(major) + "." + std::to_string(minor) + "\n" + name + "\n";
		for (const char* opt : opts) { identity += std::string(opt) + " "; }
		identity += "\n" + source;
	}
	const std::string cached = fx_cache_path(identity);
	std::vector<char> code;
	if (fx_cache_read(cached, identity, code))
	{
		hipModule_t module;
		if (hipSuccess == hipModuleLoadData(&module, code.data()) && hipSuccess == hipModuleGetFunction(out, module, name))
		{
			++jit.from_disk;
			spent();
			return TCG_OK;
		}
		(void) hipGetLastError(); // a file that does not load is compiled over
	}
	hiprtcProgram prog;
	hiprtcResult rc = hiprtcCreateProgram(&prog, source.c_str(), "fused_group.hip", 0, nullptr, nullptr);
	if (rc != HIPRTC_SUCCESS)
	{
		return tcg_fail(ctx, TCG_ERR_HIP, "tcg_ew_fusedx: hiprtcCreateProgram: %s", hiprtcGetErrorString(rc));
	}
	rc = hiprtcCompileProgram(prog, (int) (sizeof(opts) / sizeof(opts[0])), opts);
	if (rc != HIPRTC_SUCCESS)
	{
		size_t n = 0;
		hiprtcGetProgramLogSize(prog, &n);
		std::string log(n, '\0');
		if (n) { hiprtcGetProgramLog(prog, &log[0]); }
		hiprtcDestroyProgram(&prog);
		if (log.size() > 800) { log.resize(800); }
		return tcg_fail(ctx, TCG_ERR_HIP, "tcg_ew_fusedx: run-time compilation failed: %s", log.c_str());
	}
	size_t size = 0;
	hiprtcGetCodeSize(prog, &size);
	code.assign(size, '\0');
	hiprtcGetCode(prog, code.data());
	hiprtcDestroyProgram(&prog);
	hipModule_t module;
	TCG_HIP(ctx, hipModuleLoadData(&module, code.data()));
	TCG_HIP(ctx, hipModuleGetFunction(out, module, name));
	fx_cache_write(cached, identity, code);
	++jit.compiled;
	spent();
	return TCG_OK;
}

void fx_dense_leaves (const FxArgs& p, bool* dense)
{
	for (uint32_t k = 0; k < p.nleaf; ++k)
	{
		const FxLeaf& L = p.leaf[k];
		dense[k] = !L.boxed;
		int64_t run = 1;
		for (uint32_t d = 0; d < p.nd && dense[k]; ++d)
		{
			dense[k] = L.stride[d] == run;
			run *= (int64_t) p.size[d];
		}
	}
}

int fusedx_jit_launch (tcg_ctx* ctx, int dtype, FxArgs& p, bool vec)
{
	const int N = vec ? (int) (16 / tcg_type_size(dtype)) : 1;
	if (vec) { p.div[0] = fx_make_div(p.size[0] / N); }
	bool dense[TCG_FX_MAX_LEAVES];
	fx_dense_leaves(p, dense);
	// a group that moves more than the caches hold streams: operands read once
	// come in with the non-temporal hint, two indices per lane are in flight
	// and the grid covers the tensor in one sweep where it can
	const bool stream = p.total * tcg_type_size(dtype) >= ((uint64_t) 32 << 20);
	const int unroll = stream ? 2 : 1;
	std::string source = fx_source(dtype, N, p, dense, unroll, stream);
	FxJit& jit = fx_jit();
	hipFunction_t fn = nullptr;
	{
		std::lock_guard<std::mutex> lock(jit.mu);
		auto it = jit.kernels.find(source);
		if (it == jit.kernels.end())
		{
			int rc = fx_compile(ctx, source, &fn);
			if (rc != TCG_OK) { return rc; }
			jit.kernels.emplace(source, fn);
		}
		else { fn = it->second; }
	}
	unsigned grid = tcg_grid(ctx, p.total / N, FX_BLOCK * unroll, stream ? 128 : 16);
	size_t size = sizeof(FxArgs);
	void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &p, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
	TCG_HIP(ctx, hipModuleLaunchKernel(fn, grid, 1, 1, FX_BLOCK, 1, 1, 0, ctx->stream, nullptr, config));
	return TCG_OK;
}

// ---- a whole pass of a small graph as one kernel ------------------------------
//
// A graph of a few dozen functors over tensors of a few dozen elements (a
// dense layer on a batch of three) spends its time being launched: a recorded
// sequence of 13 kernels takes 37 us to enqueue and drain, one kernel 12 us.
// Such a pass is recorded as the steps of ONE kernel: a single workgroup runs
// the steps in order with a barrier between them.  Three kinds of steps:
// elementwise groups (the code a fused group compiles to, so they are bit-exact
// with tcg_ew_fusedx), contractions (each output summed in ascending order of
// the summed index, fused multiply-add: what the generic product kernel does)
// and reductions (each output folded in ascending order).  Work is bounded so
// that one workgroup finishes in microseconds; anything else refuses the
// recording and the caller records the sequence launch by launch.

constexpr int PASS_BLOCK = 256;    // lanes of a whole pass
constexpr int BATCH_BLOCK = 1024;  // lanes of a batch: its steps are a few thousand elements each
constexpr uint64_t PASS_MAX_WORK = 4096;  // iterations of the busiest lane, all steps together
constexpr size_t PASS_MAX_STEPS = 256;

struct PassStep
{
	int kind;  // 0 elementwise, 1 contraction, 2 reduction
	int dtype;
	int opcode;
	FxArgs fx;
	bool dense[TCG_FX_MAX_LEAVES];
	PassContract ct;
	PassReduce rd;
};

} // namespace

struct tcg_small_pass
{
	std::vector<PassStep> steps;
	uint64_t work = 0;
	size_t ptr_bound = 0;  // pointers the steps name, counted with repeats
	// batches: blocks handed out since the batch began (or was last sent): the
	// bytes asked for, whether a caller still owns them, and whether the block
	// had an owner before (it was given back inside the batch by somebody who took
	// it earlier: steps held back may still read what that owner left in memory)
	struct Born { size_t bytes = 0; bool live = false; bool used_before = false; };
	std::map<const void*,Born> born;
	std::set<const void*> given_back; // blocks not born here that were given back here
	hipFunction_t fn = nullptr;
	// the kernel's argument block: pointers, then the bytes of the buffers whose
	// content the caller supplies with every launch
	std::vector<void*> ptrs;
	std::map<const void*,std::pair<size_t,size_t>> feeds; // device address -> (offset, bytes) in feed_data
	std::vector<char> feed_data;
	std::vector<char> kernarg;
};

namespace
{

// lanes of a wave that fold one output of a reduction between them: few outputs,
// each over many elements
uint32_t reduce_share (uint64_t nout, uint64_t R, uint64_t block)
{
	uint32_t share = 1;
	while (share < 64 && share * 2 <= R && nout * share * 2 <= block) { share *= 2; }
	return share;
}

// the steps being collected: those of a batch, or of the single-launch recording
tcg_small_pass* small_current (tcg_ctx* ctx)
{
	return ctx->batch ? ctx->batch : ctx->capturing->pass;
}

// a step of a batch stays below what a launch of its own would cost; a batch that
// is full goes out and the next one starts
constexpr uint64_t BATCH_MAX_STEP_WORK = 512;
constexpr size_t BATCH_MAX_PTRS = 384;

int small_charge (tcg_ctx* ctx, uint64_t items, uint64_t per_item, size_t nptrs)
{
	tcg_small_pass* pass = small_current(ctx);
	const uint64_t lanes = ctx->batch ? BATCH_BLOCK : PASS_BLOCK;
	uint64_t cost = (items + lanes - 1) / lanes * (per_item ? per_item : 1);
	if (ctx->batch)
	{
		if (cost > BATCH_MAX_STEP_WORK)
		{
			return tcg_fail(ctx, TCG_ERR_UNSUPPORTED, "too much work for a step of a batch");
		}
		if (pass->steps.size() >= PASS_MAX_STEPS || pass->work + cost > PASS_MAX_WORK || pass->ptr_bound + nptrs > BATCH_MAX_PTRS)
		{
			int rc = tcg_batch_send(ctx);
			if (rc != TCG_OK) { return rc; }
		}
	}
	else if (pass->steps.size() >= PASS_MAX_STEPS || pass->work + cost > PASS_MAX_WORK)
	{
		return tcg_fail(ctx, TCG_ERR_UNSUPPORTED, "the sequence is too long for a single-launch pass");
	}
	pass->work += cost;
	pass->ptr_bound += nptrs;
	return TCG_OK;
}

int small_append_fx (tcg_ctx* ctx, int dtype, const FxArgs& p)
{
	int rc = small_charge(ctx, p.total, p.ninstr, p.nleaf + p.nout);
	if (rc != TCG_OK) { return rc; }
	PassStep step;
	memset(&step, 0, sizeof(step));
	step.kind = 0;
	step.dtype = dtype;
	step.fx = p;
	fx_dense_leaves(p, step.dense);
	small_current(ctx)->steps.push_back(step);
	return TCG_OK;
}

// resolve: the expression the kernel uses for a device pointer of the recording
template <typename Resolve>
// stage_cap (batches): bytes of LDS into which a contraction's operands are copied
// first when they lie in memory and fit -- one coalesced pass of all lanes instead
// of a round trip to memory per term of every sum
std::string pass_source (const std::vector<PassStep>& steps, size_t nptrs, size_t feed_bytes, size_t lds_bytes, Resolve resolve,
	const int block = PASS_BLOCK, const size_t stage_cap = 0)
{
	std::ostringstream head, o;
	size_t stage_need = 0;
	fx_emit_prelude(head);
	head << "struct PassPtrs { void* p[" << std::max<size_t>(1, nptrs) << "]; char feed[" << std::max<size_t>(16, feed_bytes) << "]; };\n"
		"template <typename T> __device__ __forceinline__ T pass_mac (T a, T b, T acc)\n{\n"
		"if constexpr (is_int<T>::value) { typedef typename wide_unsigned<T>::type W; return (T) ((W) a * (W) b + (W) acc); }\n"
		"else if constexpr (sizeof(T) == 4) { return __builtin_fmaf(a, b, acc); }\n"
		"else { return __builtin_fma(a, b, acc); }\n}\n"
		// the value of lane (lane ^ m) of the wave
		"template <typename T> __device__ __forceinline__ T pass_xor (T v, int m)\n{\n"
		"const int from = (int) (((threadIdx.x & 63u) ^ (uint32_t) m) << 2);\n"
		"if constexpr (sizeof(T) == 8) { union { T t; int w[2]; } u; u.t = v; u.w[0] = __builtin_amdgcn_ds_bpermute(from, u.w[0]); "
		"u.w[1] = __builtin_amdgcn_ds_bpermute(from, u.w[1]); return u.t; }\n"
		"else { union { T t; int w; } u; u.w = 0; u.t = v; u.w = __builtin_amdgcn_ds_bpermute(from, u.w); return u.t; }\n}\n"
		"extern \"C\" __global__ __launch_bounds__(" << block << ") void fx (PassPtrs P)\n{\n";
	if (lds_bytes) { head << "__shared__ __attribute__((aligned(256))) char lds[" << lds_bytes << "];\n"; }
	// fed buffers are read where the launch put them: in the argument block
	head << "const char* feed = (const char*) __builtin_amdgcn_kernarg_segment_ptr() + " << std::max<size_t>(1, nptrs) * sizeof(void*) << ";\n";
	auto lit = [](int64_t v) { return "((int64_t) " + std::to_string(v) + "ll)"; };
	// index -> coordinates over `n` dims with literal extents, accumulating offsets
	auto decompose = [&](const char* index, uint32_t n, const uint32_t* size,
		std::initializer_list<std::pair<const char*,const int64_t*>> sums)
	{
		for (uint32_t d = 0; d < n; ++d)
		{
			o << "{ const uint32_t q = " << index << " / " << size[d] << "u; const int64_t x = " << index << " - q * "
				<< size[d] << "u; " << index << " = q;";
			for (auto& sum : sums) { o << " " << sum.first << " += x * " << lit(sum.second[d]) << ";"; }
			o << " }\n";
		}
	};
	for (size_t i = 0; i < steps.size(); ++i)
	{
		const PassStep& s = steps[i];
		if (i > 0) { o << "__syncthreads();\n"; }
		o << "{\ntypedef " << fx_type_name(s.dtype) << " T;\n";
		if (s.kind == 0)
		{
			FxBake bake;
			for (uint32_t k = 0; k < s.fx.nleaf; ++k) { bake.leaf_ptr[k] = resolve(s.fx.leaf[k].ptr); }
			for (uint32_t k = 0; k < s.fx.nout; ++k) { bake.out_ptr[k] = resolve(s.fx.out[k]); }
			o << "for (uint32_t idx = threadIdx.x; idx < " << s.fx.total << "u; idx += " << block << ")\n{\n";
			fx_emit_body(o, 1, s.fx, s.dense, &bake);
			o << "}\n";
		}
		else if (s.kind == 1)
		{
			const PassContract& c = s.ct;
			// elements an operand spans (0: some stride runs backwards, leave it where it is)
			auto span = [&](const int64_t* ostr, const int64_t* kstr) -> uint64_t
			{
				int64_t last = 0;
				for (uint32_t d = 0; d < c.nod; ++d)
				{
					if (ostr[d] < 0) { return 0; }
					last += (int64_t) (c.osize[d] - 1) * ostr[d];
				}
				for (uint32_t d = 0; d < c.nkd; ++d)
				{
					if (kstr[d] < 0) { return 0; }
					last += (int64_t) (c.ksize[d] - 1) * kstr[d];
				}
				return (uint64_t) last + 1;
			};
			size_t staged = 0;
			auto in_lds = [&](const void* ptr, uint64_t elems) -> std::string
			{
				std::string where = resolve(ptr);
				size_t bytes = (elems * tcg_type_size(s.dtype) + 15) & ~(size_t) 15;
				if (0 == elems || where.compare(0, 4, "P.p[") != 0 || staged + bytes > stage_cap) { return where; }
				o << "for (uint32_t i = threadIdx.x; i < " << elems << "u; i += " << block << ") { ((T*) (stage + " << staged
					<< "))[i] = ((const T*) " << where << ")[i]; }\n";
				where = "((void*) (stage + " + std::to_string(staged) + "))";
				staged += bytes;
				return where;
			};
			const std::string pa = in_lds(c.a, span(c.oastr, c.kastr)), pb = in_lds(c.b, span(c.obstr, c.kbstr));
			if (staged > 0) { o << "__syncthreads();\n"; }
			stage_need = std::max(stage_need, staged);
			o << "const T* a = (const T*) " << pa << "; const T* b = (const T*) " << pb
				<< "; T* out = (T*) " << resolve(c.out) << ";\n"
				"for (uint32_t o = threadIdx.x; o < " << c.nout << "u; o += " << block << ")\n{\n"
				"uint32_t rem = o; int64_t ao = 0, bo = 0;\n";
			decompose("rem", c.nod, c.osize, {{"ao", c.oastr}, {"bo", c.obstr}});
			// unrolled so that the loads of several terms are in flight together; the
			// sum itself stays one chain in ascending order
			o << "T acc = (T) 0;\n"
				"#pragma unroll 16\n"
				"for (uint32_t k = 0; k < " << c.K << "u; ++k)\n{\n"
				"uint32_t r = k; int64_t ak = ao, bk = bo;\n";
			decompose("r", c.nkd, c.ksize, {{"ak", c.kastr}, {"bk", c.kbstr}});
			o << "acc = pass_mac<T>(a[ak], b[bk], acc);\n}\n"
				"out[o] = acc;\n}\n";
		}
		else
		{
			const PassReduce& c = s.rd;
			o << "const T* in = (const T*) " << resolve(c.in) << "; T* out = (T*) " << resolve(c.out) << ";\n";
			// few outputs, each over many elements: `share` lanes of a wave fold one output
			// between them (each every share-th element, ascending) and combine by halves
			// (batches only: a whole pass folds in ascending order, like the kernels its
			// results are compared with bit for bit at these sizes)
			const uint32_t share = block == BATCH_BLOCK ? reduce_share(c.nout, c.R, (uint64_t) block) : 1;
			if (share > 1)
			{
				o << "const uint32_t sub = threadIdx.x % " << share << "u, grp = threadIdx.x / " << share << "u;\n"
					"for (uint32_t o0 = 0; o0 < " << c.nout << "u; o0 += " << block / share << "u)\n{\n"
					"const uint32_t o = o0 + grp; const bool live = o < " << c.nout << "u;\n"
					"T acc = (T) 0;\n"
					"if (live)\n{\n"
					"uint32_t rem = o; int64_t base = 0;\n";
				decompose("rem", c.nod, c.osize, {{"base", c.oistr}});
				o << "#pragma unroll 4\n"
					"for (uint32_t k = sub; k < " << c.R << "u; k += " << share << "u)\n{\n"
					"uint32_t r = k; int64_t off = base;\n";
				decompose("r", c.nrd, c.rsize, {{"off", c.ristr}});
				o << "acc = k == sub ? in[off] : apply_binary<T>(" << s.opcode << ", acc, in[off]);\n}\n}\n"
					"for (int m = " << share / 2 << "; m >= 1; m >>= 1) { acc = apply_binary<T>(" << s.opcode << ", acc, pass_xor<T>(acc, m)); }\n"
					"if (live && sub == 0) { out[o] = acc; }\n}\n";
			}
			else
			{
				o << "for (uint32_t o = threadIdx.x; o < " << c.nout << "u; o += " << block << ")\n{\n"
					"uint32_t rem = o; int64_t base = 0;\n";
				decompose("rem", c.nod, c.osize, {{"base", c.oistr}});
				o << "T acc = in[base];\n"
					"#pragma unroll 8\n"
					"for (uint32_t k = 1; k < " << c.R << "u; ++k)\n{\n"
					"uint32_t r = k; int64_t off = base;\n";
				decompose("r", c.nrd, c.rsize, {{"off", c.ristr}});
				o << "acc = apply_binary<T>(" << s.opcode << ", acc, in[off]);\n}\n"
					"out[o] = acc;\n}\n";
			}
		}
		o << "}\n";
	}
	o << "}\n";
	if (stage_need > 0) { head << "__shared__ __attribute__((aligned(256))) char stage[" << stage_need << "];\n"; }
	return head.str() + o.str();
}

} // namespace

int tcg_small_unsupported (tcg_ctx* ctx, const char* what)
{
	return tcg_fail(ctx, TCG_ERR_UNSUPPORTED, "%s cannot be a step of a single-launch pass", what);
}

int tcg_small_begin (tcg_ctx*, tcg_graph* g)
{
	g->small = true;
	g->pass = new tcg_small_pass();
	return TCG_OK;
}

void tcg_small_release (tcg_graph* g)
{
	if (nullptr == g->pass) { return; }
	delete g->pass;
	g->pass = nullptr;
}

int tcg_small_finish (tcg_ctx* ctx, tcg_graph* g)
{
	tcg_small_pass* pass = g->pass;
	if (pass->steps.empty()) { return TCG_OK; } // nothing to launch
	// A buffer that the recording handed out and took back again is read and
	// written by these steps only: it lives in LDS.  Everything else (leaves,
	// results somebody holds on to) is reached through a pointer argument.
	constexpr size_t lds_cap = 48u << 10;
	std::map<void*,size_t> lds_offset;
	size_t lds_bytes = 0;
	std::map<const void*,size_t> slot;
	auto resolve = [&](const void* ptr) -> std::string
	{
		auto fed = pass->feeds.upper_bound(ptr);
		if (fed != pass->feeds.begin())
		{
			--fed;
			const char* begin = (const char*) fed->first;
			if ((const char*) ptr < begin + fed->second.second)
			{
				return "((void*) (feed + " + std::to_string(fed->second.first + (size_t) ((const char*) ptr - begin)) + "))";
			}
		}
		auto it = g->blocks.upper_bound(const_cast<void*>(ptr));
		if (it != g->blocks.begin())
		{
			--it;
			const char* begin = (const char*) it->first;
			if ((const char*) ptr < begin + it->second && 0 == g->held.count(it->first))
			{
				auto at = lds_offset.find(it->first);
				if (at == lds_offset.end() && lds_bytes + it->second <= lds_cap)
				{
					at = lds_offset.emplace(it->first, lds_bytes).first;
					lds_bytes += it->second;
				}
				if (at != lds_offset.end())
				{
					return "((void*) (lds + " + std::to_string(at->second + (size_t) ((const char*) ptr - begin)) + "))";
				}
			}
		}
		auto at = slot.find(ptr);
		if (at == slot.end()) { at = slot.emplace(ptr, slot.size()).first; }
		return "P.p[" + std::to_string(at->second) + "]";
	};
	// two passes: the first finds out how much LDS and how many pointers there are
	// what the launch supplies is never written by a step
	for (auto& step : pass->steps)
	{
		std::vector<const void*> written;
		if (step.kind == 0) { written.assign(step.fx.out, step.fx.out + step.fx.nout); }
		else { written.push_back(step.kind == 1 ? step.ct.out : step.rd.out); }
		for (const void* w : written)
		{
			auto fed = pass->feeds.upper_bound(w);
			bool hit = fed != pass->feeds.begin() && (const char*) w < (const char*) std::prev(fed)->first + std::prev(fed)->second.second;
			TCG_REQUIRE(ctx, !hit, "tcg_capture_end: a buffer fed by the launch is written by a step");
		}
	}
	(void) pass_source(pass->steps, 1, 0, 0, resolve);
	size_t feed_bytes = (pass->feed_data.size() + 15) & ~(size_t) 15;
	TCG_REQUIRE(ctx, slot.size() * sizeof(void*) + feed_bytes <= 3840,
		"tcg_capture_end: %zu buffers are too many for a single-launch pass", slot.size());
	std::string source = pass_source(pass->steps, slot.size(), feed_bytes, lds_bytes, resolve);
	pass->ptrs.assign(std::max<size_t>(1, slot.size()), nullptr);
	for (auto& kv : slot) { pass->ptrs[kv.second] = const_cast<void*>(kv.first); }
	pass->feed_data.resize(std::max<size_t>(16, feed_bytes), 0);
	pass->kernarg.resize(pass->ptrs.size() * sizeof(void*) + pass->feed_data.size());
	FxJit& jit = fx_jit();
	{
		std::lock_guard<std::mutex> lock(jit.mu);
		auto it = jit.kernels.find(source);
		if (it == jit.kernels.end())
		{
			int rc = fx_compile(ctx, source, &pass->fn);
			if (rc != TCG_OK) { return rc; }
			jit.kernels.emplace(source, pass->fn);
		}
		else { pass->fn = it->second; }
	}
	g->kernels = 1;
	return TCG_OK;
}

// ---- batches: the small launches of a longer sequence, a few at a time ----------
//
// The same steps, collected between tcg_batch_begin and tcg_batch_end wherever
// the caller allows it.  All their buffers are reached through pointers (the
// buffers outlive the batch); the kernel is launched on the context's stream
// like any other, so a recording of the stream holds it as one node.

int tcg_batch_send (tcg_ctx* ctx)
{
	tcg_small_pass* pass = ctx->batch;
	if (nullptr == pass || pass->steps.empty()) { return TCG_OK; }
	// A block that was handed out and taken back since the batch began is read and
	// written by these steps alone: it lives in LDS.  Everything else is reached
	// through a pointer argument.
	constexpr size_t lds_cap = 48u << 10;
	std::map<const void*,size_t> lds_offset;
	size_t lds_bytes = 0;
	std::map<const void*,size_t> slot;
	auto resolve = [&](const void* ptr) -> std::string
	{
		auto it = pass->born.upper_bound(ptr);
		if (it != pass->born.begin())
		{
			--it;
			const char* begin = (const char*) it->first;
			if ((const char*) ptr < begin + it->second.bytes && false == it->second.live && false == it->second.used_before)
			{
				auto at = lds_offset.find(it->first);
				size_t bytes = (it->second.bytes + 255) & ~(size_t) 255;
				if (at == lds_offset.end() && lds_bytes + bytes <= lds_cap)
				{
					at = lds_offset.emplace(it->first, lds_bytes).first;
					lds_bytes += bytes;
				}
				if (at != lds_offset.end())
				{
					return "((void*) (lds + " + std::to_string(at->second + (size_t) ((const char*) ptr - begin)) + "))";
				}
			}
		}
		auto at = slot.find(ptr);
		if (at == slot.end()) { at = slot.emplace(ptr, slot.size()).first; }
		return "P.p[" + std::to_string(at->second) + "]";
	};
	// two passes: the first finds out how much LDS and how many pointers there are
	(void) pass_source(pass->steps, 1, 0, 0, resolve, BATCH_BLOCK);
	// what the temporaries leave of the 64 KiB a workgroup may declare stages operands of contractions
	const size_t stage_cap = ((size_t) 64 << 10) - ((lds_bytes + 255) & ~(size_t) 255) - 256;
	std::string source = pass_source(pass->steps, slot.size(), 0, lds_bytes, resolve, BATCH_BLOCK, stage_cap);
	hipFunction_t fn = nullptr;
	FxJit& jit = fx_jit();
	{
		std::lock_guard<std::mutex> lock(jit.mu);
		auto it = jit.kernels.find(source);
		if (it == jit.kernels.end())
		{
			int rc = fx_compile(ctx, source, &fn);
			if (rc != TCG_OK) { return rc; }
			jit.kernels.emplace(source, fn);
		}
		else { fn = it->second; }
	}
	// the argument block: the pointers, then the (unused) 16 bytes of fed values
	std::vector<void*> args(std::max<size_t>(1, slot.size()) + 2, nullptr);
	for (auto& kv : slot) { args[kv.second] = const_cast<void*>(kv.first); }
	size_t size = args.size() * sizeof(void*);
	void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, args.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
	pass->steps.clear();
	pass->work = 0;
	pass->ptr_bound = 0;
	pass->born.clear(); // what lives on from here holds its values in memory
	pass->given_back.clear();
	TCG_HIP(ctx, hipModuleLaunchKernel(fn, 1, 1, 1, BATCH_BLOCK, 1, 1, 0, ctx->stream, nullptr, config));
	return TCG_OK;
}

int tcg_batch_decline (tcg_ctx* ctx)
{
	int rc = tcg_batch_send(ctx);
	delete ctx->batch;
	ctx->batch = nullptr;
	return rc;
}

void tcg_batch_note_alloc (tcg_ctx* ctx, const void* ptr, size_t bytes)
{
	auto& entry = ctx->batch->born[ptr];
	entry.bytes = std::max(entry.bytes, bytes);
	entry.live = true;
	entry.used_before = entry.used_before || ctx->batch->given_back.count(ptr) > 0;
}

void tcg_batch_note_free (tcg_ctx* ctx, const void* ptr)
{
	auto it = ctx->batch->born.find(ptr);
	if (it != ctx->batch->born.end()) { it->second.live = false; }
	else { ctx->batch->given_back.insert(ptr); }
}

void tcg_batch_discard (tcg_ctx* ctx)
{
	delete ctx->batch;
	ctx->batch = nullptr;
}

extern "C" int tcg_batch_begin (tcg_ctx* ctx)
{
	if (!ctx) { return TCG_ERR_ARG; }
	// a single-launch recording already takes every call as a step
	if (nullptr == ctx->batch && false == (ctx->capturing && ctx->capturing->small)) { ctx->batch = new tcg_small_pass(); }
	return TCG_OK;
}

extern "C" int tcg_batch_end (tcg_ctx* ctx)
{
	if (!ctx) { return TCG_ERR_ARG; }
	return ctx->batch ? tcg_batch_decline(ctx) : TCG_OK;
}

int tcg_small_launch (tcg_ctx* ctx, tcg_graph* g)
{
	tcg_small_pass* pass = g->pass;
	if (nullptr == pass || nullptr == pass->fn) { return TCG_OK; }
	size_t size = pass->kernarg.size(), ptr_bytes = pass->ptrs.size() * sizeof(void*);
	memcpy(pass->kernarg.data(), pass->ptrs.data(), ptr_bytes);
	memcpy(pass->kernarg.data() + ptr_bytes, pass->feed_data.data(), pass->feed_data.size());
	void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, pass->kernarg.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
	TCG_HIP(ctx, hipModuleLaunchKernel(pass->fn, 1, 1, 1, PASS_BLOCK, 1, 1, 0, ctx->stream, nullptr, config));
	return TCG_OK;
}

int tcg_small_declare_feed (tcg_ctx* ctx, const void* devptr, size_t bytes, const void* host)
{
	tcg_small_pass* pass = ctx->capturing->pass;
	TCG_REQUIRE(ctx, devptr && host && bytes > 0, "tcg_capture_feed: NULL pointer or no bytes");
	if (pass->feeds.count(devptr)) { return TCG_OK; }
	size_t offset = (pass->feed_data.size() + 15) & ~(size_t) 15;
	if (offset + bytes > 1024)
	{
		return tcg_fail(ctx, TCG_ERR_UNSUPPORTED, "tcg_capture_feed: more than 1024 bytes fed by the launch");
	}
	pass->feed_data.resize(offset + bytes);
	memcpy(pass->feed_data.data() + offset, host, bytes);
	pass->feeds.emplace(devptr, std::make_pair(offset, bytes));
	return TCG_OK;
}

int tcg_small_feed (tcg_ctx* ctx, tcg_graph* g, const void* devptr, const void* host, size_t bytes)
{
	tcg_small_pass* pass = g->pass;
	TCG_REQUIRE(ctx, pass && host, "tcg_graph_feed: not a single-launch recording");
	auto it = pass->feeds.find(devptr);
	TCG_REQUIRE(ctx, it != pass->feeds.end() && it->second.second == bytes,
		"tcg_graph_feed: %p was not declared with %zu bytes while recording", devptr, bytes);
	memcpy(pass->feed_data.data() + it->second.first, host, bytes);
	return TCG_OK;
}

int tcg_small_contract (tcg_ctx* ctx, int dtype, const uint64_t ashape[8], const uint64_t bshape[8],
	int npairs, const uint64_t* pairs, const void* a, const void* b, void* out)
{
	TCG_REQUIRE(ctx, tcg_type_size(dtype) && a && b && out && npairs >= 0 && npairs <= 8 && (pairs || npairs == 0),
		"tcg_contract: bad arguments");
	PassStep step;
	memset(&step, 0, sizeof(step));
	step.kind = 1;
	step.dtype = dtype;
	PassContract& c = step.ct;
	c.a = a; c.b = b; c.out = out;
	int64_t astr[8], bstr[8];
	astr[0] = bstr[0] = 1;
	for (int d = 1; d < 8; ++d)
	{
		astr[d] = astr[d - 1] * (int64_t) ashape[d - 1];
		bstr[d] = bstr[d - 1] * (int64_t) bshape[d - 1];
	}
	bool acon[8] = {false}, bcon[8] = {false};
	uint64_t K = 1, nout = 1;
	for (int i = 0; i < npairs; ++i)
	{
		uint64_t pa = pairs[2 * i], pb = pairs[2 * i + 1];
		TCG_REQUIRE(ctx, pa < 8 && pb < 8 && !acon[pa] && !bcon[pb] && ashape[pa] == bshape[pb],
			"tcg_contract: invalid shapes or contraction pairs");
		acon[pa] = bcon[pb] = true;
		if (ashape[pa] == 1) { continue; }
		c.ksize[c.nkd] = (uint32_t) ashape[pa];
		c.kastr[c.nkd] = astr[pa];
		c.kbstr[c.nkd] = bstr[pb];
		++c.nkd;
		K *= ashape[pa];
	}
	// output dims: what is left of b, then what is left of a (internal/eigen/operator.hpp:1069-1103)
	for (int side = 0; side < 2; ++side)
	{
		const uint64_t* shape = side == 0 ? bshape : ashape;
		const bool* con = side == 0 ? bcon : acon;
		for (int d = 0; d < 8; ++d)
		{
			if (con[d] || shape[d] == 1) { continue; }
			TCG_REQUIRE(ctx, c.nod < 8, "tcg_contract: the result has more than 8 dims");
			c.osize[c.nod] = (uint32_t) shape[d];
			c.oastr[c.nod] = side == 0 ? 0 : astr[d];
			c.obstr[c.nod] = side == 0 ? bstr[d] : 0;
			++c.nod;
			nout *= shape[d];
		}
	}
	if (nout >= (1ull << 31) || K >= (1ull << 31)) { return tcg_fail(ctx, TCG_ERR_UNSUPPORTED, "tcg_contract: too large for a step"); }
	c.nout = (uint32_t) nout;
	c.K = (uint32_t) K;
	int rc = small_charge(ctx, nout, K, 3);
	if (rc != TCG_OK) { return rc; }
	small_current(ctx)->steps.push_back(step);
	return TCG_OK;
}

int tcg_small_reduce (tcg_ctx* ctx, int opcode, int dtype, const uint64_t shape[8], unsigned rankmask,
	const void* in, void* out)
{
	TCG_REQUIRE(ctx, tcg_type_size(dtype) && in && out, "tcg_reduce: bad arguments");
	int fold = opcode == TCG_REDUCE_SUM ? TCG_ADD : opcode == TCG_REDUCE_PROD ? TCG_MUL :
		opcode == TCG_REDUCE_MIN ? TCG_MIN : opcode == TCG_REDUCE_MAX ? TCG_MAX : 0;
	TCG_REQUIRE(ctx, fold, "tcg_reduce: opcode %d is not a reduction", opcode);
	PassStep step;
	memset(&step, 0, sizeof(step));
	step.kind = 2;
	step.dtype = dtype;
	step.opcode = fold;
	PassReduce& c = step.rd;
	c.in = in; c.out = out;
	uint64_t nout = 1, R = 1;
	int64_t stride = 1;
	for (int d = 0; d < 8; ++d)
	{
		if (shape[d] > 1)
		{
			if (rankmask & (1u << d))
			{
				c.rsize[c.nrd] = (uint32_t) shape[d];
				c.ristr[c.nrd] = stride;
				++c.nrd;
				R *= shape[d];
			}
			else
			{
				c.osize[c.nod] = (uint32_t) shape[d];
				c.oistr[c.nod] = stride;
				++c.nod;
				nout *= shape[d];
			}
		}
		stride *= (int64_t) shape[d];
	}
	if (nout >= (1ull << 31) || R >= (1ull << 31)) { return tcg_fail(ctx, TCG_ERR_UNSUPPORTED, "tcg_reduce: too large for a step"); }
	c.nout = (uint32_t) nout;
	c.R = (uint32_t) R;
	const uint32_t share = ctx->batch ? reduce_share(nout, R, BATCH_BLOCK) : 1;
	int rc = small_charge(ctx, nout * share, (R + share - 1) / share + (share > 1 ? 8 : 0), 2);
	if (rc != TCG_OK) { return rc; }
	small_current(ctx)->steps.push_back(step);
	return TCG_OK;
}

int tcg_small_copy (tcg_ctx* ctx, int dtype, int nd, const uint64_t* shape, const int64_t* stride, int64_t offset,
	const uint64_t* lo, const uint64_t* hi, const void* in, void* out)
{
	uint64_t full[8];
	tcg_fx_leaf leaf;
	memset(&leaf, 0, sizeof(leaf));
	leaf.ptr = in;
	leaf.offset = offset;
	for (int d = 0; d < 8; ++d)
	{
		full[d] = d < nd ? shape[d] : 1;
		leaf.stride[d] = d < nd ? stride[d] : 0;
		leaf.lo[d] = (lo && d < nd) ? lo[d] : 0;
		leaf.hi[d] = (hi && d < nd) ? hi[d] : full[d];
	}
	tcg_fx_instr store;
	memset(&store, 0, sizeof(store));
	store.opcode = TCG_FX_STORE;
	store.a = TCG_FX_LEAF0;
	store.dst = 0;
	void* outs[1] = {out};
	return tcg_ew_fusedx(ctx, dtype, full, 1, &leaf, 1, &store, 1, outs);
}

namespace
{
} // namespace

namespace
{

// Checks a group as tcg_ew_fusedx receives it and turns it into the launch
// arguments of its kernels: iteration dims merged, views per dim, the program.
// `vec`: every operand and result can be moved 16 bytes at a time.
// A leaf whose `from_product` is set has no memory of its own (its values are
// handed to the group by the matrix product the group is the epilogue of):
// its pointer may be NULL and says nothing about alignment.
int fx_prepare (tcg_ctx* ctx, int dtype, const uint64_t shape[8],
	int nleaves, const tcg_fx_leaf* leaves, int ninstrs, const tcg_fx_instr* program,
	int nouts, void* const* outs, FxArgs& p, bool& vec)
{
	TCG_REQUIRE(ctx, shape && leaves && program && outs, "tcg_ew_fusedx: NULL pointer");
	TCG_REQUIRE(ctx, nleaves >= 1 && nleaves <= TCG_FX_MAX_LEAVES, "tcg_ew_fusedx: %d leaves (1..%d allowed)", nleaves, TCG_FX_MAX_LEAVES);
	TCG_REQUIRE(ctx, ninstrs >= 1 && ninstrs <= TCG_FX_MAX_INSTRS, "tcg_ew_fusedx: %d instructions (1..%d allowed)", ninstrs, TCG_FX_MAX_INSTRS);
	TCG_REQUIRE(ctx, nouts >= 1 && nouts <= TCG_FX_MAX_OUTS, "tcg_ew_fusedx: %d outputs (1..%d allowed)", nouts, TCG_FX_MAX_OUTS);
	size_t esz = tcg_type_size(dtype);
	TCG_REQUIRE(ctx, esz, "tcg_ew_fusedx: unknown dtype %d", dtype);
	uint64_t total = 1;
	for (int d = 0; d < 8; ++d)
	{
		TCG_REQUIRE(ctx, shape[d] >= 1 && shape[d] < (1ull << 32), "tcg_ew_fusedx: dim %d has extent %llu", d, (unsigned long long) shape[d]);
		total *= shape[d];
	}
	if (total >= (1ull << 32))
	{
		return tcg_fail(ctx, TCG_ERR_UNSUPPORTED, "tcg_ew_fusedx: %llu elements exceed the 2^32 limit of one launch", (unsigned long long) total);
	}
	for (int k = 0; k < nleaves; ++k) { TCG_REQUIRE(ctx, leaves[k].ptr || leaves[k].from_product, "tcg_ew_fusedx: leaf %d is NULL", k); }
	for (int k = 0; k < nouts; ++k) { TCG_REQUIRE(ctx, outs[k], "tcg_ew_fusedx: output %d is NULL", k); }

	// the program: every operand names a leaf, a register written earlier or
	// the immediate; every output is stored
	memset(&p, 0, sizeof(p));
	bool written[TCG_FX_MAX_REGS] = {false};
	bool stored[TCG_FX_MAX_OUTS] = {false};
	auto readable = [&](int code)
	{
		if (code == TCG_FX_IMM) { return true; }
		if (code >= TCG_FX_LEAF0 && code < TCG_FX_LEAF0 + nleaves) { return true; }
		return code >= TCG_FX_REG0 && code < TCG_FX_REG0 + TCG_FX_MAX_REGS && written[code - TCG_FX_REG0];
	};
	for (int i = 0; i < ninstrs; ++i)
	{
		const tcg_fx_instr& ins = program[i];
		TCG_REQUIRE(ctx, readable(ins.a), "tcg_ew_fusedx: instruction %d reads operand %d", i, (int) ins.a);
		if (ins.opcode == TCG_FX_STORE)
		{
			TCG_REQUIRE(ctx, ins.dst < nouts && ins.b == TCG_FX_NONE && ins.c == TCG_FX_NONE,
				"tcg_ew_fusedx: instruction %d stores to output %d", i, (int) ins.dst);
			stored[ins.dst] = true;
		}
		else
		{
			bool unary = ins.opcode == TCG_IDENTITY || is_unary_op(ins.opcode);
			bool binary = is_binary_op(ins.opcode) || ins.opcode == TCG_FX_BITOR;
			bool select = ins.opcode == TCG_SELECT;
			TCG_REQUIRE(ctx, unary || binary || select, "tcg_ew_fusedx: instruction %d has opcode %d", i, (int) ins.opcode);
			TCG_REQUIRE(ctx, (unary && ins.b == TCG_FX_NONE && ins.c == TCG_FX_NONE) ||
				(binary && readable(ins.b) && ins.c == TCG_FX_NONE) ||
				(select && readable(ins.b) && readable(ins.c)),
				"tcg_ew_fusedx: instruction %d has bad operands (%d, %d, %d)", i, (int) ins.a, (int) ins.b, (int) ins.c);
			TCG_REQUIRE(ctx, ins.dst >= TCG_FX_REG0 && ins.dst < TCG_FX_REG0 + TCG_FX_MAX_REGS,
				"tcg_ew_fusedx: instruction %d has bad destination %d", i, (int) ins.dst);
			written[ins.dst - TCG_FX_REG0] = true;
		}
		p.prog[i].opcode = ins.opcode;
		p.prog[i].a = ins.a;
		p.prog[i].b = ins.b;
		p.prog[i].c = ins.c;
		p.prog[i].dst = ins.dst;
		p.imm[i] = ins.imm;
	}
	for (int k = 0; k < nouts; ++k) { TCG_REQUIRE(ctx, stored[k], "tcg_ew_fusedx: output %d is never stored", k); }

	// iteration dims: extent-1 dims dropped, neighbours merged when every
	// operand steps through them as through one dim
	uint32_t nd = 0;
	for (int d = 0; d < 8; ++d)
	{
		if (shape[d] == 1)
		{
			bool empty = false;
			for (int k = 0; k < nleaves; ++k) { empty = empty || !(leaves[k].lo[d] == 0 && leaves[k].hi[d] >= 1); }
			if (!empty) { continue; } // otherwise some operand is all border: keep the dim
		}
		bool merge = nd > 0;
		for (int k = 0; k < nleaves && merge; ++k)
		{
			const FxLeaf& L = p.leaf[k];
			bool full_prev = L.lo[nd - 1] == 0 && L.hi[nd - 1] >= p.size[nd - 1];
			bool full = leaves[k].lo[d] == 0 && leaves[k].hi[d] >= shape[d];
			merge = full_prev && full && leaves[k].stride[d] == L.stride[nd - 1] * (int64_t) p.size[nd - 1];
		}
		if (merge)
		{
			p.size[nd - 1] *= (uint32_t) shape[d];
			for (int k = 0; k < nleaves; ++k) { p.leaf[k].hi[nd - 1] = p.size[nd - 1]; }
			continue;
		}
		p.size[nd] = (uint32_t) shape[d];
		for (int k = 0; k < nleaves; ++k)
		{
			p.leaf[k].stride[nd] = leaves[k].stride[d];
			p.leaf[k].lo[nd] = (uint32_t) (leaves[k].lo[d] < shape[d] ? leaves[k].lo[d] : shape[d]);
			p.leaf[k].hi[nd] = (uint32_t) (leaves[k].hi[d] < shape[d] ? leaves[k].hi[d] : shape[d]);
		}
		++nd;
	}
	if (nd == 0)
	{
		nd = 1;
		p.size[0] = 1;
		for (int k = 0; k < nleaves; ++k)
		{
			p.leaf[k].stride[0] = 0;
			p.leaf[k].lo[0] = 0;
			p.leaf[k].hi[0] = 1;
		}
	}
	p.nd = nd;
	p.nleaf = (uint32_t) nleaves;
	p.ninstr = (uint32_t) ninstrs;
	p.nout = (uint32_t) nouts;
	p.total = total;
	for (uint32_t d = 0; d < nd; ++d) { p.div[d] = fx_make_div(p.size[d]); }
	const int N = (int) (16 / esz);
	vec = p.size[0] % N == 0;
	for (int k = 0; k < nouts; ++k)
	{
		p.out[k] = outs[k];
		vec = vec && tcg_aligned16(outs[k]);
	}
	for (int k = 0; k < nleaves; ++k)
	{
		FxLeaf& L = p.leaf[k];
		L.ptr = leaves[k].ptr;
		L.off = leaves[k].offset;
		L.nsum = leaves[k].nsum > 1 ? leaves[k].nsum : 1;
		L.sum_stride = L.nsum > 1 ? leaves[k].sum_stride : 0;
		if (L.nsum > 1) { vec = vec && L.sum_stride % N == 0; }
		L.boxed = 0;
		for (uint32_t d = 0; d < nd; ++d) { L.boxed |= !(L.lo[d] == 0 && L.hi[d] >= p.size[d]); }
		L.bcast0 = L.stride[0] == 0;
		if (!L.bcast0)
		{
			vec = vec && L.stride[0] == 1 && L.off % N == 0 && (leaves[k].from_product || tcg_aligned16(L.ptr));
			for (uint32_t d = 1; d < nd; ++d) { vec = vec && L.stride[d] % N == 0; }
		}
		if (L.boxed) { vec = vec && L.lo[0] % N == 0 && L.hi[0] % N == 0; }
	}
	return TCG_OK;
}

} // namespace

extern "C" int tcg_ew_fusedx (tcg_ctx* ctx, int dtype, const uint64_t shape[8],
	int nleaves, const tcg_fx_leaf* leaves, int ninstrs, const tcg_fx_instr* program,
	int nouts, void* const* outs)
{
	if (!ctx) { return TCG_ERR_ARG; }
	FxArgs p;
	bool vec = false;
	int rc = fx_prepare(ctx, dtype, shape, nleaves, leaves, ninstrs, program, nouts, outs, p, vec);
	if (rc != TCG_OK) { return rc; }
	for (int k = 0; k < nleaves; ++k)
	{
		TCG_REQUIRE(ctx, 0 == leaves[k].from_product, "tcg_ew_fusedx: leaf %d names a matrix product (tcg_gemm_terms_fx takes such groups)", k);
	}
	if (tcg_small_mode(ctx)) { TCG_SMALL_RETURN(ctx, small_append_fx(ctx, dtype, p)); }
	if (fx_jit_enabled() || false == tcg_default_dtype(dtype)) { return fusedx_jit_launch(ctx, dtype, p, vec); }
	TCG_DISPATCH_TYPE(ctx, dtype, return fusedx_launch<T>(ctx, p, vec)); // the interpreter: double, float, int32
	return TCG_OK;
}

// ---- a matrix product with the group that reads it as its epilogue -----------
//
// C = sum_t A_t B_t (M x N, fp32) is read by one elementwise group and by
// nothing else; the group's shape is [J, rows = M] and its product leaves read
// C(row, off_g + j).  One workgroup owns TM rows x TJ group columns, that is the
// TM x (G TJ) results the G product leaves need there, and its NW waves split
// the summed index between them: a wave multiplies its range of K for the whole
// tile with v_mfma_f32_16x16x4_f32, operands going from memory to registers in
// the layout the instruction takes (lane l holds row / column l % 16 and the
// four summed indices 4 (l / 16) .. + 3 of a step of 16, one 128-bit load), a
// few steps ahead of the arithmetic: no LDS, no barrier inside the loop.  The
// NW partial tiles meet in LDS and are added in wave order by the lane that
// then runs the group's program on that element, with the other operands of
// the group loaded before the product started.
// The source is generated for the shape (tile, leading dims, terms, layouts) and
// the program; pointers are the only launch arguments.

namespace
{

struct GfxTile
{
	int NW = 0, TM = 0, TJ = 0, N = 1; // waves, rows, group columns per workgroup; elements per lane in the epilogue
};

// the tile with the least operand traffic among those that put a workgroup on every CU
bool gfx_choose_tile (const tcg_ctx* ctx, uint64_t M, uint64_t J, int G, uint64_t ktot, bool trans_b, bool vec, GfxTile& out)
{
	// Eight waves, two on a SIMD.  Sixteen (TCG_GFX_WAVES=16: four on a SIMD, the upper
	// eight handing their partial tiles to the lower eight first) were measured on the
	// steps of a recurrent cell and are slower -- 256 x 2048 x 768: 10.4 -> 11.8 us,
	// 256 x 512 x 2048: 12.2 -> 12.7 us: more loads in flight do not help, as with the
	// loads held further ahead (see gfx_source)
	int nw = 0;
	static const int most = [] { const char* e = getenv("TCG_GFX_WAVES"); return e ? atoi(e) : 8; }();
	for (int w : {16, 8, 4, 2, 1})
	{
		if (w > most || (w == 16 && ktot < 512)) { continue; }
		if (ktot % (16 * (uint64_t) w) == 0) { nw = w; break; }
	}
	if (nw == 0) { return false; }
	const int slots = nw < 8 ? nw : 8; // partial tiles that meet in LDS
	double best = 0.0;
	bool found = false;
	for (int tm : {16, 32, 64})
	{
		for (int tj : {4, 8, 16, 32, 64, 128})
		{
			const int nc = G * tj;
			if (J % (uint64_t) tj != 0) { continue; }
			if (trans_b ? nc % 16 != 0 : nc % 64 != 0) { continue; }
			const int accs = (tm / 16) * (nc / 16) * 4; // accumulator registers per lane
			if (accs > 128) { continue; }
			if ((size_t) slots * tm * nc * sizeof(float) > 65536) { continue; }
			// a lane computes one element of the group, or 16-byte vectors of them when
			// the tile holds more elements than the workgroup lanes; at most 8 per lane
			int n = 1;
			if (tm * tj > 64 * nw && vec && tj % 4 == 0) { n = 4; }
			if (tm * tj / n > 8 * 64 * nw) { continue; }
			const uint64_t groups = ((M + tm - 1) / tm) * (J / tj);
			const double fill = groups >= (uint64_t) ctx->num_cus ? 1.0 : (double) groups / ctx->num_cus;
			// operand elements fetched per result: 1 / rows + 1 / columns of the tile
			const double score = fill * fill / (1.0 / tm + 1.0 / nc);
			if (!found || score > best)
			{
				best = score;
				found = true;
				out.NW = nw;
				out.TM = tm;
				out.TJ = tj;
				out.N = n;
			}
		}
	}
	return found;
}

struct GfxShape
{
	uint32_t M = 0, J = 0, KT = 0, nterms = 0;
	bool trans_b = false;
	uint32_t lda[8], ldb[8];
	int G = 0;
	uint32_t noff[TCG_FX_MAX_LEAVES]; // first column of product leaf g
	int leaf_of[TCG_FX_MAX_LEAVES];   // product leaf g -> leaf of the group
};

// what a profile shows: the layout of B and the number of blocks of the result the group reads
std::string gfx_name (const GfxShape& sh)
{
	return std::string("gemm_fx_") + (sh.trans_b ? "nt" : "nn") + "_" + std::to_string(sh.G);
}

std::string gfx_source (const GfxShape& sh, const GfxTile& t, const FxArgs& p, const bool* dense, const bool* supplied)
{
	const int NT = 64 * t.NW, RB = t.TM / 16, NC = sh.G * t.TJ, CB = NC / 16, CG = NC / 64;
	const uint32_t ktot = sh.KT * sh.nterms, KW = ktot / t.NW, NSTEPS = KW / 16;
	const int BL = sh.trans_b ? CB : 4 * CG; // 128-bit loads of B per step and lane
	const int SLOTS = t.NW < 8 ? t.NW : 8;   // partial tiles in LDS: waves 8.. hand theirs to waves 0..7 first
	// The source names the loads of a step one step ahead of its arithmetic and leaves
	// the order to the compiler, which sinks each load to just before its first use;
	// with two waves on a SIMD that is the fastest form measured for the steps of a
	// recurrent cell.  Holding the loads two to five steps ahead with scheduling
	// barriers made the 256 x 2048 x 768 step slower (10.4 -> 13.0 .. 16.0 us) and left
	// the 256 x 512 x 2048 one where it was (12.2 us): with the arithmetic taken out the
	// loads alone take 8.0 and 12.1 us, so what bounds these tiles is how fast the
	// operands come out of L2, not how long a single load takes.  Steps of 32 summed
	// indices, in which a lane reads whole 128-byte lines of a K-contiguous operand,
	// changed neither (10.1 and 12.3 us); leading dimensions padded by 32 floats, which
	// spread the rows of such an operand over the channels, took the second to 9.0 us,
	// but the operands of a step are the caller's buffers and keep their layout.
	// Loads of four lanes to a row (64 contiguous bytes per row and load, the values
	// changing lanes through ds_bpermute on their way into the matrix instruction)
	// for A, for a K-contiguous B, for both: the recurrent configuration's pass took
	// 2.25-2.33 ms in every one of the four, so the loads stay in the instruction's layout.
	int depth = 2;
	if ((uint32_t) depth > NSTEPS) { depth = (int) NSTEPS; }
	const uint32_t tiles_m = (sh.M + t.TM - 1) / t.TM, tiles_j = sh.J / t.TJ;
	const int items = t.TM * t.TJ / t.N;
	std::ostringstream o;
	fx_emit_prelude(o);
	o << "typedef float T;\ntypedef float f4 __attribute__((ext_vector_type(4)));\n";
	if (t.N > 1) { o << "typedef T VT __attribute__((ext_vector_type(" << t.N << ")));\nunion VU { VT v; T e[" << t.N << "]; };\n"; }
	o << "struct GfxArgs { const float* A[" << sh.nterms << "]; const float* B[" << sh.nterms << "]; const void* leaf["
		<< TCG_FX_MAX_LEAVES << "]; void* out[" << TCG_FX_MAX_OUTS << "]; };\n";
	auto pick = [&](const char* name, const uint32_t* vals)
	{
		// leading dim of the term a step belongs to (wave-uniform)
		o << "__device__ __forceinline__ uint32_t " << name << " (uint32_t term) { return ";
		for (uint32_t k = 0; k + 1 < sh.nterms; ++k) { o << "term == " << k << "u ? " << vals[k] << "u : "; }
		o << vals[sh.nterms - 1] << "u; }\n";
	};
	pick("lda_of", sh.lda);
	pick("ldb_of", sh.ldb);
	o << "__device__ __forceinline__ uint32_t col_of (uint32_t c, uint32_t j0) { const uint32_t g = c / " << t.TJ << "u; return j0 + (c - g * "
		<< t.TJ << "u) + (";
	for (int g = 0; g + 1 < sh.G; ++g) { o << "g == " << g << "u ? " << sh.noff[g] << "u : "; }
	o << sh.noff[sh.G - 1] << "u); }\n";
	// the steps on their way from memory wait in registers: the compiler may use the
	// registers of a CU that holds at most two such workgroups, instead of keeping to
	// the few that the largest number of resident waves would leave each of them
	o << "extern \"C\" __global__ __launch_bounds__(" << NT << ") __attribute__((amdgpu_waves_per_eu(1, " << std::min(4, std::max(2, NT / 128))
		<< "))) void " << gfx_name(sh) << " (GfxArgs a)\n{\n"
		"__shared__ __attribute__((aligned(16))) float red[" << SLOTS * t.TM * NC << "];\n"
		"const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = __builtin_amdgcn_readfirstlane(tid >> 6);\n"
		"const uint32_t r16 = lane & 15u, q = lane >> 4;\n";
	// workgroups are dealt to the eight XCDs in turn: each XCD keeps a band of
	// columns, whose part of B then stays in that XCD's L2 from launch to launch
	// (a split in both directions, 2 x 4 for a recurrent cell's backward step, so that the
	// chip fetches A four times instead of eight and B twice, was measured on the whole
	// pass: 2.11-2.20 against 2.08-2.12 ms, no gain)
	if (tiles_j % 8 == 0)
	{
		o << "const uint32_t local = blockIdx.x >> 3;\n"
			"const uint32_t tj = (blockIdx.x & 7u) * " << tiles_j / 8 << "u + local % " << tiles_j / 8 << "u, tm = local / " << tiles_j / 8 << "u;\n";
	}
	else { o << "const uint32_t tm = blockIdx.x % " << tiles_m << "u, tj = blockIdx.x / " << tiles_m << "u;\n"; }
	o << "const uint32_t m0 = tm * " << t.TM << "u, j0 = tj * " << t.TJ << "u;\n";
	// the elements of the group this lane computes at the end (lane, lane + NT, ...),
	// and their other operands, loaded before the product starts
	const int per_lane = (items + NT - 1) / NT;
	FxBake bake;
	for (uint32_t k = 0; k < p.nleaf; ++k) { bake.leaf_ptr[k] = "a.leaf[" + std::to_string(k) + "]"; }
	for (uint32_t k = 0; k < p.nout; ++k) { bake.out_ptr[k] = "a.out[" + std::to_string(k) + "]"; }
	std::vector<FxParts> parts((size_t) per_lane);
	for (int it = 0; it < per_lane; ++it)
	{
		const std::string x = "_" + std::to_string(it);
		o << "const uint32_t et" << x << " = tid + " << it * NT << "u;\n"
			"const uint32_t er" << x << " = et" << x << " / " << t.TJ / t.N << "u, ej" << x << " = (et" << x << " % " << t.TJ / t.N << "u) * " << t.N << "u;\n"
			"const bool item" << x << " = et" << x << " < " << items << "u && m0 + er" << x << " < " << sh.M << "u;\n"
			"const uint32_t idx" << x << " = item" << x << " ? ((m0 + er" << x << ") * " << sh.J << "u + j0 + ej" << x << ") / " << t.N << "u : 0u;\n";
		fx_emit_parts(parts[(size_t) it], t.N, p, dense, &bake, x, "idx" + x, false, supplied);
		o << parts[(size_t) it].load.str();
	}
	// ---- the product ----
	o << "uint32_t arow[" << RB << "];\n";
	for (int rb = 0; rb < RB; ++rb)
	{
		o << "arow[" << rb << "] = m0 + " << rb * 16 << "u + r16 < " << sh.M << "u ? m0 + " << rb * 16 << "u + r16 : " << sh.M - 1 << "u;\n";
	}
	if (sh.trans_b)
	{
		o << "uint32_t bcol[" << CB << "];\n";
		for (int cb = 0; cb < CB; ++cb) { o << "bcol[" << cb << "] = col_of(" << cb * 16 << "u + r16, j0);\n"; }
	}
	else
	{
		o << "uint32_t bcol[" << CG << "];\n";
		for (int cg = 0; cg < CG; ++cg) { o << "bcol[" << cg << "] = col_of(" << cg * 64 << "u + 4u * r16, j0);\n"; }
	}
	o << "f4 acc[" << RB << "][" << CB << "];\n"
		"_Pragma(\"unroll\") for (int i = 0; i < " << RB << "; ++i) { _Pragma(\"unroll\") for (int j = 0; j < " << CB << "; ++j) { acc[i][j] = (f4) (0.0f); } }\n"
		"f4 ra[" << depth << "][" << RB << "], rb[" << depth << "][" << BL << "];\n"
		"const uint32_t kbase = wave * " << KW << "u;\n";
	auto issue = [&](uint32_t s, int slot)
	{
		o << "{\nconst uint32_t k = kbase + " << s * 16 << "u;\n";
		if (sh.nterms > 1) { o << "const uint32_t term = k / " << sh.KT << "u, kk = k - term * " << sh.KT << "u + 4u * q;\n"; }
		else { o << "const uint32_t term = 0u, kk = k + 4u * q;\n"; }
		o << "const float* __restrict__ A = a.A[term];\nconst float* __restrict__ B = a.B[term];\n"
			"const uint32_t lda = lda_of(term), ldb = ldb_of(term);\n";
		for (int rb = 0; rb < RB; ++rb)
		{
			o << "ra[" << slot << "][" << rb << "] = *(const f4*) (A + (uint64_t) arow[" << rb << "] * lda + kk);\n";
		}
		if (sh.trans_b)
		{
			for (int cb = 0; cb < CB; ++cb)
			{
				o << "rb[" << slot << "][" << cb << "] = *(const f4*) (B + (uint64_t) bcol[" << cb << "] * ldb + kk);\n";
			}
		}
		else
		{
			for (int s4 = 0; s4 < 4; ++s4)
			{
				for (int cg = 0; cg < CG; ++cg)
				{
					o << "rb[" << slot << "][" << s4 * CG + cg << "] = *(const f4*) (B + (uint64_t) (kk + " << s4 << "u) * ldb + bcol[" << cg << "]);\n";
				}
			}
		}
		o << "}\n";
	};
	auto multiply = [&](int slot)
	{
		for (int s4 = 0; s4 < 4; ++s4)
		{
			for (int rb = 0; rb < RB; ++rb)
			{
				for (int cb = 0; cb < CB; ++cb)
				{
					o << "acc[" << rb << "][" << cb << "] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[" << slot << "][" << rb << "][" << s4 << "], ";
					if (sh.trans_b) { o << "rb[" << slot << "][" << cb << "][" << s4 << "]"; }
					else { o << "rb[" << slot << "][" << s4 * CG + cb / 4 << "][" << cb % 4 << "]"; }
					o << ", acc[" << rb << "][" << cb << "], 0, 0, 0);\n";
				}
			}
		}
	};
	if (NSTEPS <= 32)
	{
		for (uint32_t s = 0; s + 1 < (uint32_t) depth; ++s) { issue(s, (int) s); }
		for (uint32_t s = 0; s < NSTEPS; ++s)
		{
			if (s + depth - 1 < NSTEPS) { issue(s + depth - 1, (int) ((s + depth - 1) % depth)); }
			multiply((int) (s % depth));
		}
	}
	else
	{
		// a long K: the steps in a loop, one at a time on its way
		o << "for (uint32_t s = 0; s < " << NSTEPS << "u; ++s)\n{\n"
			"const uint32_t k = kbase + s * 16u;\n";
		if (sh.nterms > 1) { o << "const uint32_t term = k / " << sh.KT << "u, kk = k - term * " << sh.KT << "u + 4u * q;\n"; }
		else { o << "const uint32_t term = 0u, kk = k + 4u * q;\n"; }
		o << "const float* __restrict__ A = a.A[term];\nconst float* __restrict__ B = a.B[term];\n"
			"const uint32_t lda = lda_of(term), ldb = ldb_of(term);\n";
		for (int rb = 0; rb < RB; ++rb) { o << "ra[0][" << rb << "] = *(const f4*) (A + (uint64_t) arow[" << rb << "] * lda + kk);\n"; }
		if (sh.trans_b)
		{
			for (int cb = 0; cb < CB; ++cb) { o << "rb[0][" << cb << "] = *(const f4*) (B + (uint64_t) bcol[" << cb << "] * ldb + kk);\n"; }
		}
		else
		{
			for (int s4 = 0; s4 < 4; ++s4)
			{
				for (int cg = 0; cg < CG; ++cg)
				{
					o << "rb[0][" << s4 * CG + cg << "] = *(const f4*) (B + (uint64_t) (kk + " << s4 << "u) * ldb + bcol[" << cg << "]);\n";
				}
			}
		}
		multiply(0);
		o << "}\n";
	}
	// ---- the partial tiles meet in LDS: red[wave][row][column of the tile] ----
	// park: a wave's partial tile goes to its slot; take: the tile in the slot is
	// added to the wave's own (lane for lane what the other wave's lane left there)
	auto exchange = [&](bool take)
	{
		o << "{\nfloat* mine = red + (wave & 7u) * " << t.TM * NC << "u;\n";
		for (int rb = 0; rb < RB; ++rb)
		{
			for (int i = 0; i < 4; ++i)
			{
				if (sh.trans_b)
				{
					for (int cb = 0; cb < CB; ++cb)
					{
						const std::string at = "mine[(" + std::to_string(rb * 16 + i) + "u + 4u * q) * " + std::to_string(NC) + "u + " +
							std::to_string(cb * 16) + "u + r16]";
						const std::string reg = "acc[" + std::to_string(rb) + "][" + std::to_string(cb) + "][" + std::to_string(i) + "]";
						o << (take ? reg + " += " + at : at + " = " + reg) << ";\n";
					}
				}
				else
				{
					for (int cg = 0; cg < CG; ++cg)
					{
						const std::string at = "*(f4*) (mine + (" + std::to_string(rb * 16 + i) + "u + 4u * q) * " + std::to_string(NC) + "u + " +
							std::to_string(cg * 64) + "u + 4u * r16)";
						o << "{ f4 v; ";
						if (take) { o << "v = " << at << "; "; }
						for (int e = 0; e < 4; ++e)
						{
							const std::string reg = "acc[" + std::to_string(rb) + "][" + std::to_string(cg * 4 + e) + "][" + std::to_string(i) + "]";
							o << (take ? reg + " += v[" + std::to_string(e) + "]; " : "v[" + std::to_string(e) + "] = " + reg + "; ");
						}
						if (!take) { o << at << " = v; "; }
						o << "}\n";
					}
				}
			}
		}
		o << "}\n";
	};
	if (t.NW > 8)
	{
		o << "if (wave >= 8u)\n";
		exchange(false);
		o << "__syncthreads();\nif (wave < 8u)\n";
		exchange(true);
		o << "__syncthreads();\nif (wave < 8u)\n";
		exchange(false);
	}
	else { exchange(false); }
	o << "__syncthreads();\n";
	for (int it = 0; it < per_lane; ++it)
	{
		const std::string x = "_" + std::to_string(it);
		o << "if (item" << x << ")\n{\n";
		for (int g = 0; g < sh.G; ++g)
		{
			const int k = sh.leaf_of[g];
			o << "T l" << k << x << "[" << t.N << "];\n{\nconst float* at = red + er" << x << " * " << NC << "u + " << g * t.TJ << "u + ej" << x << ";\n";
			for (int e = 0; e < t.N; ++e)
			{
				o << "{ float s = at[" << e << "];";
				for (int w = 1; w < SLOTS; ++w) { o << " s += at[" << w * t.TM * NC + e << "];"; }
				o << " l" << k << x << "[" << e << "] = s; }\n";
			}
			o << "}\n";
		}
		o << parts[(size_t) it].compute.str() << parts[(size_t) it].store.str() << "}\n";
	}
	o << "}\n";
	return o.str();
}

} // namespace

extern "C" int tcg_gemm_terms_fx (tcg_ctx* ctx, int dtype, uint64_t M, uint64_t N, uint64_t K, int nterms,
	const void* const* A, const uint64_t* lda, int trans_a,
	const void* const* B, const uint64_t* ldb, int trans_b,
	const uint64_t shape[8], int nleaves, const tcg_fx_leaf* leaves,
	int ninstrs, const tcg_fx_instr* program, int nouts, void* const* outs)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, A && B && lda && ldb, "tcg_gemm_terms_fx: NULL pointer");
	TCG_REQUIRE(ctx, nterms >= 1, "tcg_gemm_terms_fx: %d terms", nterms);
	for (int t = 0; t < nterms; ++t) { TCG_REQUIRE(ctx, A[t] && B[t], "tcg_gemm_terms_fx: operand of term %d is NULL", t); }
	FxArgs p;
	bool vec = false;
	int rc = fx_prepare(ctx, dtype, shape, nleaves, leaves, ninstrs, program, nouts, outs, p, vec);
	if (rc != TCG_OK) { return rc; }
	auto unsupported = [&](const char* why)
	{
		return tcg_fail(ctx, TCG_ERR_UNSUPPORTED, "tcg_gemm_terms_fx: %s", why);
	};
	if (tcg_small_mode(ctx)) { TCG_SMALL_RETURN(ctx, tcg_small_unsupported(ctx, "a matrix product with an epilogue")); }
	if (dtype != TCG_FLOAT || trans_a) { return unsupported("fp32 products with a row-major first operand only"); }
	if (nterms > 8 || K < 16 || K % 16 != 0 || M < 1 || N < 4 || M >= (1ull << 31) || N >= (1ull << 31) || K * (uint64_t) nterms >= (1ull << 31))
	{
		return unsupported("at most 8 terms, K a multiple of 16");
	}
	GfxShape sh;
	sh.M = (uint32_t) M;
	sh.J = (uint32_t) shape[0];
	sh.KT = (uint32_t) K;
	sh.nterms = (uint32_t) nterms;
	sh.trans_b = trans_b != 0;
	for (int t = 0; t < nterms; ++t)
	{
		bool ok = tcg_aligned16(A[t]) && tcg_aligned16(B[t]) && lda[t] % 4 == 0 && ldb[t] % 4 == 0 &&
			lda[t] < (1ull << 31) && ldb[t] < (1ull << 31) && lda[t] >= K && ldb[t] >= (trans_b ? K : N);
		if (!ok) { return unsupported("operands must be 16-byte aligned with leading dims that are multiples of four"); }
		sh.lda[t] = (uint32_t) lda[t];
		sh.ldb[t] = (uint32_t) ldb[t];
	}
	// the group walks [J, rows]; a product leaf reads result element (row, offset + j)
	uint64_t rows = 1;
	for (int d = 1; d < 8; ++d) { rows *= shape[d]; }
	if (rows != M || shape[0] > N) { return unsupported("the group must have one row per row of the product"); }
	bool supplied[TCG_FX_MAX_LEAVES] = {false};
	for (int k = 0; k < nleaves; ++k)
	{
		const tcg_fx_leaf& L = leaves[k];
		if (!L.from_product) { continue; }
		bool ok = L.nsum <= 1 && L.offset >= 0 && (uint64_t) L.offset + shape[0] <= N && L.offset % 4 == 0;
		int64_t run = (int64_t) N;
		for (int d = 0; d < 8 && ok; ++d)
		{
			ok = L.lo[d] == 0 && L.hi[d] >= shape[d];
			if (shape[d] == 1) { continue; }
			ok = ok && L.stride[d] == (d == 0 ? 1 : run);
			if (d > 0) { run *= (int64_t) shape[d]; }
		}
		if (!ok) { return unsupported("a leaf does not walk the product row by row"); }
		supplied[k] = true;
		sh.leaf_of[sh.G] = k;
		sh.noff[sh.G] = (uint32_t) L.offset;
		++sh.G;
	}
	if (sh.G == 0) { return unsupported("no leaf reads the product"); }
	if (M * shape[0] >= (1ull << 31)) { return unsupported("too many elements"); }
	GfxTile tile;
	if (!gfx_choose_tile(ctx, M, shape[0], sh.G, K * (uint64_t) nterms, sh.trans_b, vec, tile))
	{
		return unsupported("no tile fits the shape");
	}
	// offsets go into the pointers, so that launches that differ in them share a kernel
	struct { const float* A[8]; const float* B[8]; const void* leaf[TCG_FX_MAX_LEAVES]; void* out[TCG_FX_MAX_OUTS]; } args;
	static_assert(sizeof(args) <= 4096, "launch arguments must fit the kernel argument segment");
	memset(&args, 0, sizeof(args));
	const size_t esz = tcg_type_size(dtype);
	for (uint32_t k = 0; k < p.nleaf; ++k)
	{
		if (supplied[k]) { continue; }
		args.leaf[k] = (const char*) p.leaf[k].ptr + (int64_t) esz * p.leaf[k].off;
		p.leaf[k].off = 0;
		p.leaf[k].ptr = nullptr;
	}
	for (uint32_t k = 0; k < p.nout; ++k)
	{
		args.out[k] = p.out[k];
		p.out[k] = nullptr;
	}
	if (tile.N > 1) { p.div[0] = fx_make_div(p.size[0] / tile.N); }
	bool dense[TCG_FX_MAX_LEAVES];
	fx_dense_leaves(p, dense);
	std::string source = gfx_source(sh, tile, p, dense, supplied);
	// the kernel's arguments: the term pointers, then the group's
	std::vector<char> packed(sizeof(void*) * (2 * (size_t) nterms + TCG_FX_MAX_LEAVES + TCG_FX_MAX_OUTS));
	{
		char* at = packed.data();
		for (int t = 0; t < nterms; ++t) { memcpy(at, &A[t], sizeof(void*)); at += sizeof(void*); }
		for (int t = 0; t < nterms; ++t) { memcpy(at, &B[t], sizeof(void*)); at += sizeof(void*); }
		memcpy(at, args.leaf, sizeof(args.leaf)); at += sizeof(args.leaf);
		memcpy(at, args.out, sizeof(args.out));
	}
	FxJit& jit = fx_jit();
	hipFunction_t fn = nullptr;
	{
		std::lock_guard<std::mutex> lock(jit.mu);
		auto it = jit.kernels.find(source);
		if (it == jit.kernels.end())
		{
			rc = fx_compile(ctx, source, &fn, gfx_name(sh).c_str());
			if (rc != TCG_OK) { return rc; }
			jit.kernels.emplace(source, fn);
		}
		else { fn = it->second; }
	}
	const unsigned grid = (unsigned) (((M + tile.TM - 1) / tile.TM) * (shape[0] / tile.TJ));
	size_t size = packed.size();
	void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, packed.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
	TCG_HIP(ctx, hipModuleLaunchKernel(fn, grid, 1, 1, 64 * tile.NW, 1, 1, 0, ctx->stream, nullptr, config));
	return TCG_OK;
}

extern "C" int tcg_jit_stats (const tcg_ctx* ctx, uint64_t* compiled, uint64_t* from_disk, double* ms)
{
	if (!ctx) { return TCG_ERR_ARG; }
	FxJit& jit = fx_jit();
	std::lock_guard<std::mutex> lock(jit.mu);
	if (compiled) { *compiled = jit.compiled; }
	if (from_disk) { *from_disk = jit.from_disk; }
	if (ms) { *ms = jit.ms; }
	return TCG_OK;
}
