// Data movement: EXTEND, PERMUTE, SLICE, PAD, REVERSE, STRIDE, SCATTER, CONCAT.
//
// Every one of them is "dst[affine(c)] = src[affine(c)] for c in a box", so the
// host lowers each to a CopyPlan (iteration dims, signed element strides on
// both sides, optional zero-filled border) with neighbouring dims merged, and
// one of two kernels runs it:
//   strided_copy_k  lanes along the innermost iteration dim, 128-bit accesses
//                   when both sides are contiguous there;
//   transpose_k     when the source's contiguous dim is not the destination's,
//                   a 64x64 tile goes through LDS so that both the reads and
//                   the writes are coalesced.
// All of them move each byte once: HBM-bound.
#include <type_traits>
#include "tcg_internal.hpp"

namespace
{

// unsigned division by an invariant (Granlund-Montgomery), n < 2^32, d >= 1
struct FastDiv
{
	uint32_t d = 1, m = 0, s1 = 0, s2 = 0;
};

FastDiv make_fastdiv (uint32_t d)
{
	FastDiv f;
	f.d = d;
	uint32_t l = 0;
	while (((uint64_t) 1 << l) < d) { ++l; }
	f.m = (uint32_t) ((((uint64_t) 1 << 32) * (((uint64_t) 1 << l) - d)) / d + 1);
	f.s1 = l < 1 ? l : 1;
	f.s2 = l == 0 ? 0 : l - 1;
	return f;
}

__device__ __forceinline__ uint32_t fdiv (uint32_t n, const FastDiv& f)
{
	uint32_t t = __umulhi(f.m, n);
	return (t + ((n - t) >> f.s1)) >> f.s2;
}

constexpr int MAXD = 8;

struct CopyPlan
{
	int nd = 0;
	uint32_t size[MAXD];    // iteration extents, dim 0 innermost
	int64_t sstride[MAXD];  // source element strides
	int64_t dstride[MAXD];  // destination element strides
	uint32_t lo[MAXD];      // with `box`: coordinates outside [lo, hi) are
	uint32_t hi[MAXD];      // written as zero and never read
	FastDiv div[MAXD];
	int64_t sbase = 0, dbase = 0;
	uint64_t total = 0;
	bool box = false;
};

constexpr int MV_BLOCK = 256;

template <typename T, int V, bool BOX>
__global__ __launch_bounds__(MV_BLOCK) void strided_copy_k (CopyPlan p,
	const T* __restrict__ src, T* __restrict__ dst)
{
	// with V > 1 the innermost dim is contiguous on both sides and every
	// extent/stride/bound involved is a multiple of V
	const uint32_t nvec = (uint32_t) (p.total / V);
	const uint32_t step = gridDim.x * MV_BLOCK;
	for (uint32_t idx = blockIdx.x * MV_BLOCK + threadIdx.x; idx < nvec; idx += step)
	{
		uint32_t rem = idx;
		int64_t so = p.sbase, dof = p.dbase;
		bool inside = true;
#pragma unroll
		for (int d = 0; d < MAXD; ++d)
		{
			if (d < p.nd)
			{
				uint32_t c;
				if (d == p.nd - 1) { c = rem; }
				else
				{
					uint32_t q = fdiv(rem, p.div[d]);
					c = rem - q * p.div[d].d;
					rem = q;
				}
				if (d == 0) { c *= V; }
				so += (int64_t) c * p.sstride[d];
				dof += (int64_t) c * p.dstride[d];
				if (BOX) { inside = inside && c >= p.lo[d] && c < p.hi[d]; }
			}
		}
		if constexpr (V == 1)
		{
			T v = 0;
			if (!BOX || inside) { v = src[so]; }
			dst[dof] = v;
		}
		else
		{
			VecU<T> v;
#pragma unroll
			for (int e = 0; e < V; ++e) { v.e[e] = 0; }
			if (!BOX || inside) { v.v = *reinterpret_cast<const typename Vec16<T>::type*>(src + so); }
			*reinterpret_cast<typename Vec16<T>::type*>(dst + dof) = v.v;
		}
	}
}

constexpr int TR_TILE = 64;

// Plan dims: 0 = destination-contiguous dim (source stride s0 != 1),
// dim j = source-contiguous dim (sstride 1); the rest index the batch.
template <typename T>
__global__ __launch_bounds__(MV_BLOCK) void transpose_k (CopyPlan p, int j,
	uint32_t tiles0, uint32_t tilesj, const T* __restrict__ src, T* __restrict__ dst)
{
	__shared__ T tile[TR_TILE][TR_TILE + 1];
	uint32_t bid = blockIdx.x;
	const uint32_t t0 = bid % tiles0;
	bid /= tiles0;
	const uint32_t tj = bid % tilesj;
	uint32_t rem = bid / tilesj;
	int64_t so = p.sbase, dof = p.dbase;
#pragma unroll
	for (int d = 1; d < MAXD; ++d)
	{
		if (d < p.nd && d != j)
		{
			uint32_t q = fdiv(rem, p.div[d]);
			uint32_t c = rem - q * p.div[d].d;
			rem = q;
			so += (int64_t) c * p.sstride[d];
			dof += (int64_t) c * p.dstride[d];
		}
	}
	const uint32_t i0 = t0 * TR_TILE, j0 = tj * TR_TILE;
	const uint32_t tx = threadIdx.x % TR_TILE, ty = threadIdx.x / TR_TILE;
	constexpr int ROWS = MV_BLOCK / TR_TILE;
	// read: lanes along dim j (contiguous in the source)
#pragma unroll 4
	for (uint32_t r = ty; r < TR_TILE; r += ROWS)
	{
		uint32_t ci = i0 + r, cj = j0 + tx;
		if (ci < p.size[0] && cj < p.size[j])
		{
			tile[r][tx] = src[so + (int64_t) ci * p.sstride[0] + (int64_t) cj * p.sstride[j]];
		}
	}
	__syncthreads();
	// write: lanes along dim 0 (contiguous in the destination)
#pragma unroll 4
	for (uint32_t r = ty; r < TR_TILE; r += ROWS)
	{
		uint32_t ci = i0 + tx, cj = j0 + r;
		if (ci < p.size[0] && cj < p.size[j])
		{
			dst[dof + (int64_t) ci * p.dstride[0] + (int64_t) cj * p.dstride[j]] = tile[tx][r];
		}
	}
}

// The same with 128-bit accesses on both sides: a row of the tile is read by
// TILE / N lanes (N elements each, 16 bytes), so a wave covers several row
// segments per instruction and a quarter of the memory instructions are
// issued.  The tile is written to and read from LDS element by element (odd
// pitch: both walks are free of bank conflicts).  Consecutive workgroups take
// tiles that are neighbours along the source's contiguous dim.  Needs extents
// and strides that are multiples of N and 16-byte aligned bases.
// Measured on fp32 (GB/s of 8 bytes per element): 4096^2 5.8 (scalar, 64) ->
// 6.4 (TILE 32), 64 x 512^2 5.9 -> 6.8; 16384 x 4096, which no cache holds,
// 4.0 -> 6.5 with TILE 128 and non-temporal loads (the hint costs 10 % on the
// sizes the last-level cache holds, so only large copies take it).
template <typename T, int TILE, bool NT>
__global__ __launch_bounds__(MV_BLOCK) void transpose_vec_k (CopyPlan p, int j,
	uint32_t tiles0, uint32_t tilesj, uint32_t group, const T* __restrict__ src, T* __restrict__ dst)
{
	constexpr int N = Vec16<T>::N;
	constexpr int LANES = TILE / N;             // lanes along a row of the tile
	constexpr int ROWS = MV_BLOCK / LANES;      // rows per pass
	constexpr int PASSES = TILE / ROWS;
	__shared__ T tile[TILE][TILE + 1];
	// tiles in groups of GROUP along dim 0: the workgroups in flight together
	// then read GROUP * TILE rows and write as many, in runs of several tiles
	// each, instead of long runs on one side and single tiles on the other
	const uint32_t per_matrix = tiles0 * tilesj;
	uint32_t rem = blockIdx.x / per_matrix;
	const uint32_t in_matrix = blockIdx.x - rem * per_matrix;
	const uint32_t width = group * tilesj;
	const uint32_t first0 = in_matrix / width * group;
	const uint32_t rows = tiles0 - first0 < group ? tiles0 - first0 : group;
	const uint32_t in_group = in_matrix - first0 * tilesj;
	const uint32_t t0 = first0 + in_group % rows, tj = in_group / rows;
	int64_t so = p.sbase, dof = p.dbase;
#pragma unroll
	for (int d = 1; d < MAXD; ++d)
	{
		if (d < p.nd && d != j)
		{
			uint32_t q = fdiv(rem, p.div[d]);
			uint32_t c = rem - q * p.div[d].d;
			rem = q;
			so += (int64_t) c * p.sstride[d];
			dof += (int64_t) c * p.dstride[d];
		}
	}
	const uint32_t i0 = t0 * TILE, j0 = tj * TILE;
	const uint32_t tx = threadIdx.x % LANES, ty = threadIdx.x / LANES;
	// read: lanes along dim j (contiguous in the source); tile[i][j]
	VecU<T> held[PASSES];
#pragma unroll
	for (int k = 0; k < PASSES; ++k)
	{
		uint32_t ci = i0 + ty + k * ROWS, cj = j0 + tx * N;
		if (ci < p.size[0] && cj < p.size[j])
		{
			auto from = reinterpret_cast<const typename Vec16<T>::type*>(src + so + (int64_t) ci * p.sstride[0] + (int64_t) cj);
			held[k].v = NT ? __builtin_nontemporal_load(from) : *from;
		}
	}
#pragma unroll
	for (int k = 0; k < PASSES; ++k)
	{
#pragma unroll
		for (int e = 0; e < N; ++e) { tile[ty + k * ROWS][tx * N + e] = held[k].e[e]; }
	}
	__syncthreads();
	// write: lanes along dim 0 (contiguous in the destination)
#pragma unroll
	for (int k = 0; k < PASSES; ++k)
	{
		uint32_t ci = i0 + tx * N, cj = j0 + ty + k * ROWS;
		if (ci < p.size[0] && cj < p.size[j])
		{
			VecU<T> v;
#pragma unroll
			for (int e = 0; e < N; ++e) { v.e[e] = tile[tx * N + e][ty + k * ROWS]; }
			*reinterpret_cast<typename Vec16<T>::type*>(dst + dof + (int64_t) ci + (int64_t) cj * p.dstride[j]) = v.v;
		}
	}
}

template <typename T, int TILE, bool NT>
void launch_transpose_vec (tcg_ctx* ctx, const CopyPlan& p, int j, uint64_t batch, const T* src, T* dst, bool* launched)
{
	uint32_t tiles0 = (p.size[0] + TILE - 1) / TILE, tilesj = (p.size[j] + TILE - 1) / TILE;
	uint64_t blocks = (uint64_t) tiles0 * tilesj * batch;
	*launched = blocks < (1ull << 31);
	// (4096^2 floats: 5.5 -> 6.0 TB/s with groups of 8; matrices of a few hundred rows gain nothing)
	const uint32_t group = tiles0 >= 32 && tilesj >= 32 ? 8 : 1;
	if (*launched) { transpose_vec_k<T,TILE,NT><<<(unsigned) blocks, MV_BLOCK, 0, ctx->stream>>>(p, j, tiles0, tilesj, group, src, dst); }
}

// ---- plan construction ----------------------------------------------------

void contiguous_strides (const uint64_t shape[8], int64_t stride[8])
{
	stride[0] = 1;
	for (int d = 1; d < 8; ++d) { stride[d] = stride[d - 1] * (int64_t) shape[d - 1]; }
}

// Drops extent-1 dims and merges dims that are contiguous on both sides
void plan_finish (CopyPlan& p, const uint64_t size[8], const int64_t ss[8],
	const int64_t ds[8], const uint64_t* lo, const uint64_t* hi)
{
	p.nd = 0;
	p.total = 1;
	for (int d = 0; d < 8; ++d)
	{
		p.total *= size[d];
		if (size[d] == 1)
		{
			// a singular dim outside its box makes the whole output zero; keep it
			if (!(p.box && !(lo[d] == 0 && hi[d] >= 1))) { continue; }
		}
		bool full = !p.box || (lo[d] == 0 && hi[d] >= size[d]);
		int k = p.nd;
		if (k > 0)
		{
			bool prev_full = !p.box || (p.lo[k - 1] == 0 && p.hi[k - 1] >= p.size[k - 1]);
			if (prev_full && full &&
				ss[d] == p.sstride[k - 1] * (int64_t) p.size[k - 1] &&
				ds[d] == p.dstride[k - 1] * (int64_t) p.size[k - 1])
			{
				p.size[k - 1] *= (uint32_t) size[d];
				p.hi[k - 1] = p.size[k - 1];
				continue;
			}
		}
		p.size[k] = (uint32_t) size[d];
		p.sstride[k] = ss[d];
		p.dstride[k] = ds[d];
		p.lo[k] = p.box ? (uint32_t) lo[d] : 0;
		p.hi[k] = p.box ? (uint32_t) (hi[d] < size[d] ? hi[d] : size[d]) : (uint32_t) size[d];
		++p.nd;
	}
	if (p.nd == 0)
	{
		p.nd = 1;
		p.size[0] = 1;
		p.sstride[0] = 1;
		p.dstride[0] = 1;
		p.lo[0] = 0;
		p.hi[0] = 1;
	}
	for (int d = 0; d < p.nd; ++d) { p.div[d] = make_fastdiv(d == 0 ? p.size[0] : p.size[d]); }
}

template <typename T>
int run_plan (tcg_ctx* ctx, CopyPlan& p, const T* src, T* dst, const char* what)
{
	if (p.total == 0) { return TCG_OK; }
	if (p.total >= (1ull << 32))
	{
		return tcg_fail(ctx, TCG_ERR_UNSUPPORTED, "%s: %llu elements exceed the 2^32 limit of one launch", what, (unsigned long long) p.total);
	}
	if (tcg_small_mode(ctx))
	{
		// a step of a sequence recorded as one kernel: a gather into a dense destination
		int64_t run = 1;
		bool dense_dst = p.dbase == 0;
		uint64_t size[8], lo[8], hi[8];
		for (int d = 0; d < p.nd; ++d)
		{
			dense_dst = dense_dst && p.dstride[d] == run;
			run *= (int64_t) p.size[d];
			size[d] = p.size[d];
			lo[d] = p.box ? p.lo[d] : 0;
			hi[d] = p.box ? p.hi[d] : p.size[d];
		}
		// a copy: any dtype of this element size will do
		int dtype = std::is_same<T,double>::value ? TCG_DOUBLE : std::is_same<T,float>::value ? TCG_FLOAT :
			sizeof(T) == 4 ? TCG_INT32 : sizeof(T) == 2 ? TCG_UINT16 : TCG_UINT8;
		TCG_SMALL_RETURN(ctx, false == dense_dst ? tcg_small_unsupported(ctx, "a copy into a strided destination") :
			tcg_small_copy(ctx, dtype, p.nd, size, p.sstride, p.sbase, lo, hi, src, dst));
	}
	constexpr int N = Vec16<T>::N;
	// transpose path: destination contiguous along dim 0, source along dim j
	if (!p.box && p.nd >= 2 && p.dstride[0] == 1 && p.sstride[0] != 1 && p.size[0] >= 16)
	{
		int j = -1;
		for (int d = 1; d < p.nd; ++d)
		{
			if (p.sstride[d] == 1 && p.size[d] >= 16) { j = d; break; }
		}
		if (j > 0)
		{
			uint64_t batch = 1;
			for (int d = 1; d < p.nd; ++d) { if (d != j) { batch *= p.size[d]; } }
			// 128-bit accesses when every row segment on both sides is aligned
			bool wide = p.size[0] % N == 0 && p.size[j] % N == 0 && p.sbase % N == 0 && p.dbase % N == 0 &&
				tcg_aligned16(src) && tcg_aligned16(dst);
			for (int d = 0; d < p.nd && wide; ++d)
			{
				wide = (d == j || p.sstride[d] % N == 0) && (d == 0 || p.dstride[d] % N == 0);
			}
			bool launched = false;
			if constexpr (sizeof(T) >= 4)
			{
			if (wide)
			{
				// what no cache holds streams through large tiles
				constexpr int BIG = sizeof(T) == 4 ? 128 : 64;
				bool large = p.total * sizeof(T) >= ((uint64_t) 128 << 20) && p.size[0] >= BIG && p.size[j] >= BIG;
				if (large) { launch_transpose_vec<T,BIG,true>(ctx, p, j, batch, src, dst, &launched); }
				else { launch_transpose_vec<T,32,false>(ctx, p, j, batch, src, dst, &launched); }
			}
			}
			if (false == launched)
			{
				uint32_t tiles0 = (p.size[0] + TR_TILE - 1) / TR_TILE;
				uint32_t tilesj = (p.size[j] + TR_TILE - 1) / TR_TILE;
				uint64_t blocks = (uint64_t) tiles0 * tilesj * batch;
				launched = blocks < (1ull << 31);
				if (launched) { transpose_k<T><<<(unsigned) blocks, MV_BLOCK, 0, ctx->stream>>>(p, j, tiles0, tilesj, src, dst); }
			}
			if (launched)
			{
				TCG_LAUNCH_CHECK(ctx, what);
				return TCG_OK;
			}
		}
	}
	bool vec = p.sstride[0] == 1 && p.dstride[0] == 1 && p.size[0] % N == 0 &&
		p.sbase % N == 0 && p.dbase % N == 0 && tcg_aligned16(src) && tcg_aligned16(dst);
	for (int d = 1; d < p.nd && vec; ++d)
	{
		vec = p.sstride[d] % N == 0 && p.dstride[d] % N == 0;
	}
	if (vec && p.box) { vec = p.lo[0] % N == 0 && p.hi[0] % N == 0; }
	if (vec)
	{
		CopyPlan q = p;
		q.size[0] = p.size[0] / N;
		q.div[0] = make_fastdiv(q.size[0]);
		// the kernel scales coordinate 0 by N itself; bounds stay in elements
		unsigned grid = tcg_grid(ctx, p.total / N, MV_BLOCK, 16);
		if (p.box) { strided_copy_k<T,N,true><<<grid, MV_BLOCK, 0, ctx->stream>>>(q, src, dst); }
		else { strided_copy_k<T,N,false><<<grid, MV_BLOCK, 0, ctx->stream>>>(q, src, dst); }
	}
	else
	{
		unsigned grid = tcg_grid(ctx, p.total, MV_BLOCK, 16);
		if (p.box) { strided_copy_k<T,1,true><<<grid, MV_BLOCK, 0, ctx->stream>>>(p, src, dst); }
		else { strided_copy_k<T,1,false><<<grid, MV_BLOCK, 0, ctx->stream>>>(p, src, dst); }
	}
	TCG_LAUNCH_CHECK(ctx, what);
	return TCG_OK;
}

int check_dims (tcg_ctx* ctx, const uint64_t shape[8], const char* what)
{
	for (int d = 0; d < 8; ++d)
	{
		TCG_REQUIRE(ctx, shape[d] >= 1 && shape[d] < (1ull << 32), "%s: dim %d has extent %llu", what, d, (unsigned long long) shape[d]);
	}
	return TCG_OK;
}

#define CHECK_DIMS(ctx, shape, what) do { int rc__ = check_dims(ctx, shape, what); if (rc__ != TCG_OK) { return rc__; } } while (0)

// CONCAT of many operands in one launch: the result seen as
// [outer][along the axis][inner]; every lane finds the operand its group of V
// elements comes from in a table of where each operand starts along the axis
constexpr int CC_MAX = 128;

template <typename T, int V> struct VecOf { typedef T type; };
template <> struct VecOf<uint32_t,4> { typedef uint32_t type __attribute__((ext_vector_type(4))); };

struct ConcatTab
{
	const void* src[CC_MAX];
	uint32_t start[CC_MAX + 1]; // along the axis; start[n] = extent of the result
	uint32_t n;
};

template <typename T, int V>
__global__ __launch_bounds__(MV_BLOCK) void concat_many_k (ConcatTab tab, FastDiv inner_div, FastDiv axis_div,
	uint32_t inner_vecs, uint32_t nvec, T* __restrict__ dst)
{
	typedef typename VecOf<T,V>::type Vec;
	const uint32_t step = gridDim.x * MV_BLOCK;
	for (uint32_t idx = blockIdx.x * MV_BLOCK + threadIdx.x; idx < nvec; idx += step)
	{
		// idx = (outer * axis_total + along) * inner_vecs + within
		const uint32_t row = fdiv(idx, inner_div);
		const uint32_t within = idx - row * inner_vecs;
		const uint32_t outer = fdiv(row, axis_div);
		const uint32_t along = row - outer * axis_div.d;
		// operands are few: halve the table
		uint32_t lo = 0, hi = tab.n;
		while (hi - lo > 1)
		{
			uint32_t mid = (lo + hi) / 2;
			if (tab.start[mid] <= along) { lo = mid; } else { hi = mid; }
		}
		const uint32_t extent = tab.start[lo + 1] - tab.start[lo];
		const uint64_t from = ((uint64_t) outer * extent + (along - tab.start[lo])) * inner_vecs + within;
		reinterpret_cast<Vec*>(dst)[idx] = reinterpret_cast<const Vec*>(tab.src[lo])[from];
	}
}

} // namespace

extern "C" {

int tcg_extend (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t bcast[8], const void* in, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, inshape && bcast && in && out, "tcg_extend: NULL pointer");
	CHECK_DIMS(ctx, inshape, "tcg_extend");
	uint64_t oshape[8];
	int64_t is[8], os[8], ss[8];
	contiguous_strides(inshape, is);
	for (int d = 0; d < 8; ++d)
	{
		TCG_REQUIRE(ctx, bcast[d] >= 1, "tcg_extend: cannot extend using zero dimensions (dim %d)", d);
		TCG_REQUIRE(ctx, !(bcast[d] > 1 && inshape[d] > 1), "tcg_extend: cannot extend non-singular dimension %d", d);
		oshape[d] = inshape[d] * bcast[d];
		// a broadcast dim re-reads the same source element: stride 0
		ss[d] = bcast[d] > 1 ? 0 : is[d];
	}
	CHECK_DIMS(ctx, oshape, "tcg_extend");
	contiguous_strides(oshape, os);
	CopyPlan p;
	plan_finish(p, oshape, ss, os, nullptr, nullptr);
	TCG_DISPATCH_MOVE(ctx, dtype, return run_plan<T>(ctx, p, (const T*) in, (T*) out, "tcg_extend"));
	return TCG_OK;
}

int tcg_permute (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t order[8], const void* in, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, inshape && order && in && out, "tcg_permute: NULL pointer");
	CHECK_DIMS(ctx, inshape, "tcg_permute");
	uint64_t oshape[8];
	int64_t is[8], os[8], ss[8];
	bool seen[8] = {false};
	contiguous_strides(inshape, is);
	for (int d = 0; d < 8; ++d)
	{
		TCG_REQUIRE(ctx, order[d] < 8 && !seen[order[d]], "tcg_permute: permute does not support repeated orders");
		seen[order[d]] = true;
		oshape[d] = inshape[order[d]];
		ss[d] = is[order[d]];
	}
	contiguous_strides(oshape, os);
	CopyPlan p;
	plan_finish(p, oshape, ss, os, nullptr, nullptr);
	TCG_DISPATCH_MOVE(ctx, dtype, return run_plan<T>(ctx, p, (const T*) in, (T*) out, "tcg_permute"));
	return TCG_OK;
}

int tcg_slice (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t offsets[8], const uint64_t extents[8], const void* in, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, inshape && offsets && extents && in && out, "tcg_slice: NULL pointer");
	CHECK_DIMS(ctx, inshape, "tcg_slice");
	int64_t is[8], os[8];
	contiguous_strides(inshape, is);
	CopyPlan p;
	for (int d = 0; d < 8; ++d)
	{
		TCG_REQUIRE(ctx, extents[d] >= 1, "tcg_slice: cannot create slice with 0 dimensions (dim %d)", d);
		TCG_REQUIRE(ctx, offsets[d] + extents[d] <= inshape[d], "tcg_slice: dim %d: offset %llu + extent %llu exceeds %llu", d,
			(unsigned long long) offsets[d], (unsigned long long) extents[d], (unsigned long long) inshape[d]);
		p.sbase += (int64_t) offsets[d] * is[d];
	}
	contiguous_strides(extents, os);
	plan_finish(p, extents, is, os, nullptr, nullptr);
	TCG_DISPATCH_MOVE(ctx, dtype, return run_plan<T>(ctx, p, (const T*) in, (T*) out, "tcg_slice"));
	return TCG_OK;
}

int tcg_pad (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t before[8], const uint64_t after[8], const void* in, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, inshape && before && after && in && out, "tcg_pad: NULL pointer");
	CHECK_DIMS(ctx, inshape, "tcg_pad");
	uint64_t oshape[8], lo[8], hi[8];
	int64_t is[8], os[8];
	contiguous_strides(inshape, is);
	CopyPlan p;
	p.box = true;
	for (int d = 0; d < 8; ++d)
	{
		oshape[d] = inshape[d] + before[d] + after[d];
		lo[d] = before[d];
		hi[d] = before[d] + inshape[d];
		p.sbase -= (int64_t) before[d] * is[d];
	}
	CHECK_DIMS(ctx, oshape, "tcg_pad");
	contiguous_strides(oshape, os);
	plan_finish(p, oshape, is, os, lo, hi);
	TCG_DISPATCH_MOVE(ctx, dtype, return run_plan<T>(ctx, p, (const T*) in, (T*) out, "tcg_pad"));
	return TCG_OK;
}

int tcg_pad_interior (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t before[8], const uint64_t after[8], const void* in, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, inshape && before && after && in && out, "tcg_pad_interior: NULL pointer");
	CHECK_DIMS(ctx, inshape, "tcg_pad_interior");
	uint64_t oshape[8];
	int64_t is[8], os[8];
	contiguous_strides(inshape, is);
	for (int d = 0; d < 8; ++d) { oshape[d] = inshape[d] + before[d] + after[d]; }
	CHECK_DIMS(ctx, oshape, "tcg_pad_interior");
	contiguous_strides(oshape, os);
	CopyPlan p;
	for (int d = 0; d < 8; ++d) { p.dbase += (int64_t) before[d] * os[d]; }
	plan_finish(p, inshape, is, os, nullptr, nullptr);
	TCG_DISPATCH_MOVE(ctx, dtype, return run_plan<T>(ctx, p, (const T*) in, (T*) out, "tcg_pad_interior"));
	return TCG_OK;
}

int tcg_reverse (tcg_ctx* ctx, int dtype, const uint64_t shape[8],
	unsigned rankmask, const void* in, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, shape && in && out, "tcg_reverse: NULL pointer");
	TCG_REQUIRE(ctx, rankmask < 256, "tcg_reverse: rank set 0x%x names a dim >= 8", rankmask);
	CHECK_DIMS(ctx, shape, "tcg_reverse");
	int64_t is[8], ss[8];
	contiguous_strides(shape, is);
	CopyPlan p;
	for (int d = 0; d < 8; ++d)
	{
		if ((rankmask >> d) & 1)
		{
			p.sbase += (int64_t) (shape[d] - 1) * is[d];
			ss[d] = -is[d];
		}
		else { ss[d] = is[d]; }
	}
	plan_finish(p, shape, ss, is, nullptr, nullptr);
	TCG_DISPATCH_MOVE(ctx, dtype, return run_plan<T>(ctx, p, (const T*) in, (T*) out, "tcg_reverse"));
	return TCG_OK;
}

int tcg_stride (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t incr[8], const uint64_t outshape[8], const void* in, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, inshape && incr && outshape && in && out, "tcg_stride: NULL pointer");
	CHECK_DIMS(ctx, inshape, "tcg_stride");
	CHECK_DIMS(ctx, outshape, "tcg_stride");
	int64_t is[8], os[8], ss[8];
	contiguous_strides(inshape, is);
	contiguous_strides(outshape, os);
	for (int d = 0; d < 8; ++d)
	{
		TCG_REQUIRE(ctx, incr[d] >= 1 && (outshape[d] - 1) * incr[d] < inshape[d],
			"tcg_stride: dim %d: %llu steps of %llu leave the input extent %llu", d,
			(unsigned long long) outshape[d], (unsigned long long) incr[d], (unsigned long long) inshape[d]);
		ss[d] = is[d] * (int64_t) incr[d];
	}
	CopyPlan p;
	plan_finish(p, outshape, ss, os, nullptr, nullptr);
	TCG_DISPATCH_MOVE(ctx, dtype, return run_plan<T>(ctx, p, (const T*) in, (T*) out, "tcg_stride"));
	return TCG_OK;
}

int tcg_scatter (tcg_ctx* ctx, int dtype, const uint64_t inshape[8],
	const uint64_t incr[8], const uint64_t outshape[8], const void* in, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, inshape && incr && outshape && in && out, "tcg_scatter: NULL pointer");
	CHECK_DIMS(ctx, inshape, "tcg_scatter");
	CHECK_DIMS(ctx, outshape, "tcg_scatter");
	int64_t is[8], os[8], ds[8];
	uint64_t iter[8];
	contiguous_strides(inshape, is);
	contiguous_strides(outshape, os);
	for (int d = 0; d < 8; ++d)
	{
		TCG_REQUIRE(ctx, incr[d] >= 1, "tcg_scatter: dim %d has increment 0", d);
		// input coordinates whose target falls outside the output are dropped
		uint64_t fit = (outshape[d] + incr[d] - 1) / incr[d];
		iter[d] = inshape[d] < fit ? inshape[d] : fit;
		ds[d] = os[d] * (int64_t) incr[d];
	}
	int rc = tcg_fill_zero(ctx, out, tcg_n_elems(outshape) * tcg_type_size(dtype));
	if (rc != TCG_OK) { return rc; }
	CopyPlan p;
	plan_finish(p, iter, is, ds, nullptr, nullptr);
	TCG_DISPATCH_MOVE(ctx, dtype, return run_plan<T>(ctx, p, (const T*) in, (T*) out, "tcg_scatter"));
	return TCG_OK;
}

int tcg_concat (tcg_ctx* ctx, int dtype, int axis, int nargs,
	const uint64_t* shapes, const void* const* ins, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, shapes && ins && out, "tcg_concat: NULL pointer");
	TCG_REQUIRE(ctx, axis >= 0 && axis < 8, "tcg_concat: axis %d", axis);
	TCG_REQUIRE(ctx, nargs >= 1, "tcg_concat: no operands");
	uint64_t oshape[8];
	for (int d = 0; d < 8; ++d) { oshape[d] = shapes[d]; }
	oshape[axis] = 0;
	for (int i = 0; i < nargs; ++i)
	{
		CHECK_DIMS(ctx, shapes + i * 8, "tcg_concat");
		for (int d = 0; d < 8; ++d)
		{
			TCG_REQUIRE(ctx, d == axis || shapes[i * 8 + d] == oshape[d],
				"tcg_concat: cannot group concat incompatible shapes along axis %d (operand %d, dim %d)", axis, i, d);
		}
		oshape[axis] += shapes[i * 8 + axis];
	}
	CHECK_DIMS(ctx, oshape, "tcg_concat");
	for (int i = 0; i < nargs; ++i) { TCG_REQUIRE(ctx, ins[i], "tcg_concat: operand %d is NULL", i); }
	// many operands (the outputs of an unrolled recurrent layer, one per step,
	// cfg/tenncor/layer.yml:297-345, 716-768): one launch instead of one per operand
	uint64_t inner = 1, outer = 1, total = 1;
	for (int d = 0; d < 8; ++d)
	{
		total *= oshape[d];
		if (d < axis) { inner *= oshape[d]; }
		if (d > axis) { outer *= oshape[d]; }
	}
	const size_t esz = tcg_type_size(dtype);
	if (nargs >= 3 && nargs <= CC_MAX && false == tcg_small_mode(ctx) && esz && total > 0 && total < (1ull << 32) &&
		oshape[axis] < (1ull << 31))
	{
		ConcatTab tab;
		tab.n = (uint32_t) nargs;
		uint32_t at = 0;
		// 16 bytes per lane when every row segment on both sides is aligned
		uint64_t per = 16 / esz;
		bool wide = inner % per == 0 && tcg_aligned16(out);
		for (int i = 0; i < nargs; ++i)
		{
			tab.src[i] = ins[i];
			tab.start[i] = at;
			at += (uint32_t) shapes[i * 8 + axis];
			wide = wide && tcg_aligned16(ins[i]);
		}
		tab.start[nargs] = at;
		if (false == wide) { per = 1; }
		const uint32_t inner_vecs = (uint32_t) (inner / per);
		const uint32_t nvec = (uint32_t) (total / per);
		const unsigned grid = tcg_grid(ctx, nvec, MV_BLOCK, 32);
		const FastDiv idiv = make_fastdiv(inner_vecs), adiv = make_fastdiv((uint32_t) oshape[axis]);
		if (wide)
		{
			concat_many_k<uint32_t,4><<<grid, MV_BLOCK, 0, ctx->stream>>>(tab, idiv, adiv, inner_vecs, nvec, (uint32_t*) out);
		}
		else
		{
			switch (esz)
			{
				case 1: concat_many_k<uint8_t,1><<<grid, MV_BLOCK, 0, ctx->stream>>>(tab, idiv, adiv, inner_vecs, nvec, (uint8_t*) out); break;
				case 2: concat_many_k<uint16_t,1><<<grid, MV_BLOCK, 0, ctx->stream>>>(tab, idiv, adiv, inner_vecs, nvec, (uint16_t*) out); break;
				case 4: concat_many_k<uint32_t,1><<<grid, MV_BLOCK, 0, ctx->stream>>>(tab, idiv, adiv, inner_vecs, nvec, (uint32_t*) out); break;
				default: concat_many_k<uint64_t,1><<<grid, MV_BLOCK, 0, ctx->stream>>>(tab, idiv, adiv, inner_vecs, nvec, (uint64_t*) out); break;
			}
		}
		TCG_LAUNCH_CHECK(ctx, "concat_many_k");
		return TCG_OK;
	}
	int64_t os[8];
	contiguous_strides(oshape, os);
	uint64_t off = 0;
	for (int i = 0; i < nargs; ++i)
	{
		const uint64_t* ishape = shapes + i * 8;
		int64_t is[8];
		contiguous_strides(ishape, is);
		CopyPlan p;
		p.dbase = (int64_t) off * os[axis];
		plan_finish(p, ishape, is, os, nullptr, nullptr);
		TCG_DISPATCH_MOVE(ctx, dtype,
			int rc = run_plan<T>(ctx, p, (const T*) ins[i], (T*) out, "tcg_concat");
			if (rc != TCG_OK) { return rc; });
		off += ishape[axis];
	}
	return TCG_OK;
}

} // extern "C"
