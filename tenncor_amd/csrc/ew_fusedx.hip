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

namespace
{

constexpr int FX_BLOCK = 256;
constexpr int FX_MAXD = 8;
constexpr int FX_SLOTS = TCG_FX_MAX_LEAVES + TCG_FX_MAX_REGS;

struct FxDiv
{
	uint32_t d = 1, m = 0, s1 = 0, s2 = 0;
};

FxDiv fx_make_div (uint32_t d)
{
	FxDiv f;
	f.d = d;
	uint32_t l = 0;
	while (((uint64_t) 1 << l) < d) { ++l; }
	f.m = (uint32_t) ((((uint64_t) 1 << 32) * (((uint64_t) 1 << l) - d)) / d + 1);
	f.s1 = l < 1 ? l : 1;
	f.s2 = l == 0 ? 0 : l - 1;
	return f;
}

__device__ __forceinline__ uint32_t fx_div (uint32_t n, const FxDiv& f)
{
	uint32_t t = __umulhi(f.m, n);
	return (t + ((n - t) >> f.s1)) >> f.s2;
}

struct FxLeaf
{
	const void* ptr;
	int64_t off;               // elements
	int64_t stride[FX_MAXD];   // elements per iteration dim; 0 = broadcast
	uint32_t lo[FX_MAXD];      // with `boxed`: outside [lo, hi) the operand
	uint32_t hi[FX_MAXD];      // reads as zero and memory is not touched
	uint32_t boxed;
	uint32_t bcast0;           // stride[0] == 0
};

struct FxInstr
{
	uint8_t opcode, a, b, c, dst, pad_[3];
};

struct FxArgs
{
	uint32_t nd, nleaf, ninstr, nout;
	uint32_t size[FX_MAXD];    // iteration extents in elements, dim 0 innermost
	FxDiv div[FX_MAXD];        // div[0] divides by size[0] / N
	uint64_t total;            // elements
	FxLeaf leaf[TCG_FX_MAX_LEAVES];
	FxInstr prog[TCG_FX_MAX_INSTRS];
	double imm[TCG_FX_MAX_INSTRS];
	void* out[TCG_FX_MAX_OUTS];
};

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
		T slot[FX_SLOTS][N];
#pragma unroll
		for (int k = 0; k < TCG_FX_MAX_LEAVES; ++k)
		{
			if (k < (int) p.nleaf)
			{
				const T* src = (const T*) p.leaf[k].ptr + off[k];
				if (!inside[k])
				{
#pragma unroll
					for (int e = 0; e < N; ++e) { slot[k][e] = (T) 0; }
				}
				else if (N > 1 && !p.leaf[k].bcast0)
				{
					VecU<T> v;
					v.v = *reinterpret_cast<const typename Vec16<T>::type*>(src);
#pragma unroll
					for (int e = 0; e < N; ++e) { slot[k][e] = v.e[e]; }
				}
				else
				{
					T s = *src;
#pragma unroll
					for (int e = 0; e < N; ++e) { slot[k][e] = s; }
				}
			}
		}
		for (uint32_t i = 0; i < p.ninstr; ++i)
		{
			const FxInstr ins = p.prog[i];
			const T imm = (T) p.imm[i];
			T va[N], vb[N], vc[N];
			{
				const int sa = fx_slot(ins.a);
#pragma unroll
				for (int e = 0; e < N; ++e) { va[e] = ins.a == TCG_FX_IMM ? imm : slot[sa][e]; }
			}
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
				const int sb = fx_slot(ins.b);
#pragma unroll
				for (int e = 0; e < N; ++e) { vb[e] = ins.b == TCG_FX_IMM ? imm : slot[sb][e]; }
			}
			if (has_c)
			{
				const int sc = fx_slot(ins.c);
#pragma unroll
				for (int e = 0; e < N; ++e) { vc[e] = ins.c == TCG_FX_IMM ? imm : slot[sc][e]; }
			}
			const int sd = fx_slot(ins.dst);
#pragma unroll
			for (int e = 0; e < N; ++e)
			{
				T r;
				if (has_c) { r = va[e] != (T) 0 ? vb[e] : vc[e]; } // SELECT
				else if (has_b) { r = apply_binary<T>(ins.opcode, va[e], vb[e]); }
				else { r = apply_unary<T>(ins.opcode, va[e]); }
				slot[sd][e] = r;
			}
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
			bool binary = is_binary_op(ins.opcode);
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
	TCG_DISPATCH_TYPE(ctx, dtype, return fusedx_launch<T>(ctx, p, vec));
	return TCG_OK;
}
