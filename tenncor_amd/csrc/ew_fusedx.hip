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

#include <cstdlib>
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
				}
				else
				{
					T s = *src;
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

// dense: the leaf is addressed like the output (offset + linear index)
std::string fx_source (int dtype, int N, const FxArgs& p, const bool* dense)
{
	const char* tname = dtype == TCG_DOUBLE ? "double" : dtype == TCG_FLOAT ? "float" : "int";
	std::ostringstream o;
	o << "typedef signed char int8_t; typedef unsigned char uint8_t; typedef int int32_t;\n"
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
	o << "typedef " << tname << " T;\n";
	if (N > 1)
	{
		o << "typedef T VT __attribute__((ext_vector_type(" << N << ")));\n"
			"union VU { VT v; T e[" << N << "]; };\n";
	}
	o << "extern \"C\" __global__ __launch_bounds__(" << FX_BLOCK << ") void fx (FxArgs p)\n{\n"
		"const uint32_t nvec = (uint32_t) (p.total / " << N << ");\n"
		"const uint32_t step = gridDim.x * " << FX_BLOCK << ";\n"
		"for (uint32_t idx = blockIdx.x * " << FX_BLOCK << " + threadIdx.x; idx < nvec; idx += step)\n{\n";
	bool need_coords = false;
	for (uint32_t k = 0; k < p.nleaf; ++k) { need_coords = need_coords || !dense[k]; }
	if (need_coords)
	{
		o << "uint32_t rem = idx;\n";
		for (uint32_t d = 0; d + 1 < p.nd; ++d)
		{
			o << "const uint32_t q" << d << " = fx_div(rem, p.div[" << d << "]);\n"
				"uint32_t c" << d << " = rem - q" << d << " * p.div[" << d << "].d;\nrem = q" << d << ";\n";
		}
		o << "uint32_t c" << p.nd - 1 << " = rem;\n";
		if (N > 1) { o << "c0 *= " << N << ";\n"; }
	}
	for (uint32_t k = 0; k < p.nleaf; ++k)
	{
		const FxLeaf& L = p.leaf[k];
		o << "T l" << k << "[" << N << "];\n{\n";
		if (dense[k])
		{
			o << "const T* src = (const T*) p.leaf[" << k << "].ptr + (p.leaf[" << k << "].off + (int64_t) idx * " << N << ");\n";
		}
		else
		{
			o << "int64_t off = p.leaf[" << k << "].off";
			for (uint32_t d = 0; d < p.nd; ++d)
			{
				if (d == 0 && L.bcast0) { continue; }
				o << " + (int64_t) c" << d << " * p.leaf[" << k << "].stride[" << d << "]";
			}
			o << ";\nconst T* src = (const T*) p.leaf[" << k << "].ptr + off;\n";
		}
		if (L.boxed)
		{
			o << "bool inside = true";
			for (uint32_t d = 0; d < p.nd; ++d)
			{
				o << " && c" << d << " >= p.leaf[" << k << "].lo[" << d << "] && c" << d << " < p.leaf[" << k << "].hi[" << d << "]";
			}
			o << ";\nif (inside)\n";
		}
		o << "{\n";
		if (N > 1 && !L.bcast0)
		{
			o << "VU v; v.v = *(const VT*) src;\n";
			for (int e = 0; e < N; ++e) { o << "l" << k << "[" << e << "] = v.e[" << e << "];\n"; }
		}
		else
		{
			o << "const T s = *src;\n";
			for (int e = 0; e < N; ++e) { o << "l" << k << "[" << e << "] = s;\n"; }
		}
		o << "}\n";
		if (L.boxed)
		{
			o << "else\n{\n";
			for (int e = 0; e < N; ++e) { o << "l" << k << "[" << e << "] = (T) 0;\n"; }
			o << "}\n";
		}
		o << "}\n";
	}
	// straight-line program: every write of a register gets a name of its own
	std::string reg_name[TCG_FX_MAX_REGS];
	auto operand = [&](int code, uint32_t i, int e) -> std::string
	{
		if (code == TCG_FX_IMM) { return "imm" + std::to_string(i); }
		if (code >= TCG_FX_REG0) { return reg_name[code - TCG_FX_REG0] + "[" + std::to_string(e) + "]"; }
		return "l" + std::to_string(code - TCG_FX_LEAF0) + "[" + std::to_string(e) + "]";
	};
	for (uint32_t i = 0; i < p.ninstr; ++i)
	{
		const FxInstr& ins = p.prog[i];
		bool uses_imm = ins.a == TCG_FX_IMM || ins.b == TCG_FX_IMM || ins.c == TCG_FX_IMM;
		if (uses_imm) { o << "const T imm" << i << " = (T) p.imm[" << i << "];\n"; }
		if (ins.opcode == TCG_FX_STORE)
		{
			o << "{\nT* dst = (T*) p.out[" << (int) ins.dst << "] + (uint64_t) idx * " << N << ";\n";
			if (N > 1)
			{
				o << "VU v;\n";
				for (int e = 0; e < N; ++e) { o << "v.e[" << e << "] = " << operand(ins.a, i, e) << ";\n"; }
				o << "*(VT*) dst = v.v;\n";
			}
			else { o << "*dst = " << operand(ins.a, i, 0) << ";\n"; }
			o << "}\n";
			continue;
		}
		std::string name = "v" + std::to_string(i);
		o << "T " << name << "[" << N << "];\n";
		for (int e = 0; e < N; ++e)
		{
			o << name << "[" << e << "] = ";
			if (ins.c != TCG_FX_NONE)
			{
				o << operand(ins.a, i, e) << " != (T) 0 ? " << operand(ins.b, i, e) << " : " << operand(ins.c, i, e);
			}
			else if (ins.opcode == TCG_FX_BITOR)
			{
				o << "bit_or<T>(" << operand(ins.a, i, e) << ", " << operand(ins.b, i, e) << ")";
			}
			else if (ins.b != TCG_FX_NONE)
			{
				o << "apply_binary<T>(" << (int) ins.opcode << ", " << operand(ins.a, i, e) << ", " << operand(ins.b, i, e) << ")";
			}
			else
			{
				o << "apply_unary<T>(" << (int) ins.opcode << ", " << operand(ins.a, i, e) << ")";
			}
			o << ";\n";
		}
		reg_name[ins.dst - TCG_FX_REG0] = name;
	}
	o << "}\n}\n";
	return o.str();
}

int fx_compile (tcg_ctx* ctx, const std::string& source, hipFunction_t* out)
{
	hiprtcProgram prog;
	hiprtcResult rc = hiprtcCreateProgram(&prog, source.c_str(), "fused_group.hip", 0, nullptr, nullptr);
	if (rc != HIPRTC_SUCCESS)
	{
		return tcg_fail(ctx, TCG_ERR_HIP, "tcg_ew_fusedx: hiprtcCreateProgram: %s", hiprtcGetErrorString(rc));
	}
	std::string arch = "--offload-arch=" + ctx->arch;
	// the flags libtcg itself is built with (packed fp32 forms stay off), and
	// no contraction: a multiply node feeding an add node must round twice, as
	// it does when the two nodes run as separate kernels
	const char* opts[] = {arch.c_str(), "-O3", "-std=c++17", "-ffp-contract=off",
		"-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
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
	std::vector<char> code(size);
	hiprtcGetCode(prog, code.data());
	hiprtcDestroyProgram(&prog);
	hipModule_t module;
	TCG_HIP(ctx, hipModuleLoadData(&module, code.data()));
	TCG_HIP(ctx, hipModuleGetFunction(out, module, "fx"));
	return TCG_OK;
}

int fusedx_jit_launch (tcg_ctx* ctx, int dtype, FxArgs& p, bool vec)
{
	const int N = vec ? (int) (16 / tcg_type_size(dtype)) : 1;
	if (vec) { p.div[0] = fx_make_div(p.size[0] / N); }
	bool dense[TCG_FX_MAX_LEAVES];
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
	std::string source = fx_source(dtype, N, p, dense);
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
	unsigned grid = tcg_grid(ctx, p.total / N, FX_BLOCK, 16);
	size_t size = sizeof(FxArgs);
	void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &p, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
	TCG_HIP(ctx, hipModuleLaunchKernel(fn, grid, 1, 1, FX_BLOCK, 1, 1, 0, ctx->stream, nullptr, config));
	return TCG_OK;
}

} // namespace

extern "C" int tcg_ew_fusedx (tcg_ctx* ctx, int dtype, const uint64_t shape[8],
	int nleaves, const tcg_fx_leaf* leaves, int ninstrs, const tcg_fx_instr* program,
	int nouts, void* const* outs)
{
	if (!ctx) { return TCG_ERR_ARG; }
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
	for (int k = 0; k < nleaves; ++k) { TCG_REQUIRE(ctx, leaves[k].ptr, "tcg_ew_fusedx: leaf %d is NULL", k); }
	for (int k = 0; k < nouts; ++k) { TCG_REQUIRE(ctx, outs[k], "tcg_ew_fusedx: output %d is NULL", k); }

	// the program: every operand names a leaf, a register written earlier or
	// the immediate; every output is stored
	FxArgs p;
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
	bool vec = p.size[0] % N == 0;
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
		L.boxed = 0;
		for (uint32_t d = 0; d < nd; ++d) { L.boxed |= !(L.lo[d] == 0 && L.hi[d] >= p.size[d]); }
		L.bcast0 = L.stride[0] == 0;
		if (!L.bcast0)
		{
			vec = vec && L.stride[0] == 1 && L.off % N == 0 && tcg_aligned16(L.ptr);
			for (uint32_t d = 1; d < nd; ++d) { vec = vec && L.stride[d] % N == 0; }
		}
		if (L.boxed) { vec = vec && L.lo[0] % N == 0 && L.hi[0] % N == 0; }
	}
	if (fx_jit_enabled()) { return fusedx_jit_launch(ctx, dtype, p, vec); }
	TCG_DISPATCH_TYPE(ctx, dtype, return fusedx_launch<T>(ctx, p, vec));
	return TCG_OK;
}
