// REDUCE_SUM / PROD / MIN / MAX and ARGMAX.
//
// Any reduction over a set of dims of an 8-D tensor is decomposed on the host
// into steps of the form [A, R, B] -> [A, B] (A = contiguous kept elements,
// R = reduced extent, B = everything outside):
//   A == 1: "inner" kernel, one workgroup (or S of them) per row of R
//           contiguous elements, 128-bit loads, wave shuffle + LDS tree;
//   A  > 1: "outer" kernel, a workgroup owns a strip of columns, lanes run
//           along the contiguous dim, rows are split over the wave rows of
//           the group and over S groups; LDS combines the wave rows.
// When R is split over S workgroups the partial results go to a scratch
// tensor [A, S, B] that a second launch of the same kernel reduces.
// Both kernels read every input byte exactly once: HBM-bound.
#include "tcg_internal.hpp"

#include <limits>
#include <mutex>
#include <type_traits>

// Device memory that exists for as long as the library is loaded, one copy on
// every GPU: the temporaries of tcg_reduce_noalloc.  Host code never uses the
// array's name as an address: the address of each GPU's copy is looked up once
// (tcg_reduce_scratch_init) and kept in g_scratch.
constexpr size_t NOALLOC_SCRATCH_BYTES = TCG_REDUCE_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
static unsigned char* g_scratch[MAX_DEVICES] = {nullptr};
// Every context on a GPU shares that GPU's array, and every call starts at its
// first byte: the context that used it last, with the event recorded behind its
// launches.  Another context is let in once that event has passed.
struct ScratchOwner
{
	tcg_ctx* ctx = nullptr;
	hipEvent_t done = nullptr;
};
static ScratchOwner g_owner[MAX_DEVICES];
static std::mutex g_scratch_mu; // g_scratch and g_owner

namespace
{

template <typename T> struct is_int { static constexpr bool value = std::is_integral<T>::value; };

template <typename T> using Wide = typename std::conditional<sizeof(T) == 8, uint64_t, uint32_t>::type;

template <typename T, int OP>
struct Red
{
	static __device__ __forceinline__ T identity ()
	{
		if constexpr (OP == TCG_REDUCE_SUM) { return (T) 0; }
		else if constexpr (OP == TCG_REDUCE_PROD) { return (T) 1; }
		else if constexpr (OP == TCG_REDUCE_MIN)
		{
			if constexpr (is_int<T>::value) { return std::numeric_limits<T>::max(); }
			else { return (T) INFINITY; }
		}
		else
		{
			if constexpr (is_int<T>::value) { return std::numeric_limits<T>::lowest(); }
			else { return (T) -INFINITY; }
		}
	}

	static __device__ __forceinline__ T combine (T a, T b)
	{
		if constexpr (OP == TCG_REDUCE_SUM)
		{
			// integers wrap modulo 2^width
			if constexpr (is_int<T>::value) { return (T) ((Wide<T>) a + (Wide<T>) b); }
			else { return a + b; }
		}
		else if constexpr (OP == TCG_REDUCE_PROD)
		{
			if constexpr (is_int<T>::value) { return (T) ((Wide<T>) a * (Wide<T>) b); }
			else { return a * b; }
		}
		else if constexpr (OP == TCG_REDUCE_MIN) { return b < a ? b : a; }
		else { return b > a ? b : a; }
	}
};

template <typename T>
__device__ __forceinline__ T shfl_xor_t (T v, int mask)
{
	if constexpr (sizeof(T) < 4) { return (T) __shfl_xor((int) v, mask, TCG_WAVE); }
	else if constexpr (sizeof(T) == 8)
	{
		union { T t; int i[2]; } u;
		u.t = v;
		u.i[0] = __shfl_xor(u.i[0], mask, TCG_WAVE);
		u.i[1] = __shfl_xor(u.i[1], mask, TCG_WAVE);
		return u.t;
	}
	else { return __shfl_xor(v, mask, TCG_WAVE); }
}

template <typename T, int OP>
__device__ __forceinline__ T wave_reduce (T v)
{
#pragma unroll
	for (int m = TCG_WAVE / 2; m >= 1; m >>= 1)
	{
		v = Red<T,OP>::combine(v, shfl_xor_t(v, m));
	}
	return v;
}

constexpr int RED_BLOCK = 256;
constexpr int RED_WAVES = RED_BLOCK / TCG_WAVE;

// launch shape of the column kernel: how many lanes (log2) run along the
// contiguous dim at most, how many workgroups per CU a launch aims for when it
// splits the reduced dim, and how many rows a lane keeps in flight.
// Measured on config 2: 2 workgroups per CU (long row chunks, 8 partial rows)
// beat 8 per CU by 25 % on the column reduction.
#ifndef TCG_RED_TXMAX_LOG2
#define TCG_RED_TXMAX_LOG2 6
#endif
#ifndef TCG_RED_BLOCKS_PER_CU
#define TCG_RED_BLOCKS_PER_CU 2
#endif
#ifndef TCG_RED_OUTER_UNROLL
#define TCG_RED_OUTER_UNROLL 2
#endif
// the operand of a reduction was usually written by the node before it, and
// part of it is still in the last-level cache: plain loads hit there, the
// non-temporal hint measured 4-15 % slower
#ifndef TCG_RED_NONTEMPORAL
#define TCG_RED_NONTEMPORAL 0
#endif
#if TCG_RED_NONTEMPORAL
#define RED_LOAD(ptr) __builtin_nontemporal_load(ptr)
#else
#define RED_LOAD(ptr) (*(ptr))
#endif

// rows of R contiguous elements; block b reduces the part `b % S` of row
// `b / S` and writes out[row * S + part]
template <typename T, int OP, bool VEC>
__global__ __launch_bounds__(RED_BLOCK) void reduce_inner_k (
	const T* __restrict__ in, T* __restrict__ out, uint64_t R, uint32_t S, uint64_t chunk)
{
	constexpr int N = VEC ? Vec16<T>::N : 1;
	const uint64_t row = blockIdx.x / S;
	const uint32_t part = blockIdx.x % S;
	const T* base = in + row * R;
	const uint64_t lo = (uint64_t) part * chunk;
	uint64_t hi = lo + chunk;
	if (hi > R) { hi = R; }

	T acc[4];
#pragma unroll
	for (int u = 0; u < 4; ++u) { acc[u] = Red<T,OP>::identity(); }
	if constexpr (VEC)
	{
		// lo and chunk are multiples of N; the tail of the row is scalar
		const uint64_t vlo = lo / N, vhi = hi / N;
		uint64_t i = vlo + threadIdx.x;
		for (; i + 3 * RED_BLOCK < vhi; i += 4 * RED_BLOCK)
		{
			VecU<T> x[4];
#pragma unroll
			for (int u = 0; u < 4; ++u)
			{
				x[u].v = RED_LOAD(reinterpret_cast<const typename Vec16<T>::type*>(base) + i + u * RED_BLOCK);
			}
#pragma unroll
			for (int u = 0; u < 4; ++u)
			{
#pragma unroll
				for (int e = 0; e < N; ++e) { acc[u] = Red<T,OP>::combine(acc[u], x[u].e[e]); }
			}
		}
		for (; i < vhi; i += RED_BLOCK)
		{
			VecU<T> x;
			x.v = RED_LOAD(reinterpret_cast<const typename Vec16<T>::type*>(base) + i);
#pragma unroll
			for (int e = 0; e < N; ++e) { acc[0] = Red<T,OP>::combine(acc[0], x.e[e]); }
		}
		uint64_t t = vhi * N + threadIdx.x;
		if (t < hi) { acc[1] = Red<T,OP>::combine(acc[1], base[t]); }
	}
	else
	{
		for (uint64_t i = lo + threadIdx.x; i < hi; i += RED_BLOCK)
		{
			acc[0] = Red<T,OP>::combine(acc[0], base[i]);
		}
	}
	T v = Red<T,OP>::combine(Red<T,OP>::combine(acc[0], acc[1]), Red<T,OP>::combine(acc[2], acc[3]));
	v = wave_reduce<T,OP>(v);
	__shared__ T smem[RED_WAVES];
	const int wave = threadIdx.x / TCG_WAVE, lane = threadIdx.x % TCG_WAVE;
	if (lane == 0) { smem[wave] = v; }
	__syncthreads();
	if (threadIdx.x == 0)
	{
		T r = smem[0];
#pragma unroll
		for (int w = 1; w < RED_WAVES; ++w) { r = Red<T,OP>::combine(r, smem[w]); }
		out[row * S + part] = r;
	}
}

// in[a + r*A + b*A*R] -> out[a + s*A + b*A*S]; the group is TX lanes wide
// (each lane N columns) and TY = 256 / TX rows tall
template <typename T, int OP, bool VEC, int BLOCK = RED_BLOCK, int U = TCG_RED_OUTER_UNROLL>
__global__ __launch_bounds__(BLOCK) void reduce_outer_k (
	const T* __restrict__ in, T* __restrict__ out, uint64_t A, uint64_t R,
	uint32_t S, uint64_t chunk, uint32_t txlog2, uint32_t col_tiles)
{
	constexpr int N = VEC ? Vec16<T>::N : 1;
	const uint32_t TX = 1u << txlog2, TY = BLOCK >> txlog2;
	const uint32_t tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> txlog2;
	uint64_t bid = blockIdx.x;
	const uint32_t ctile = bid % col_tiles;
	bid /= col_tiles;
	const uint32_t part = bid % S;
	const uint64_t b = bid / S;
	const uint64_t col = ((uint64_t) ctile * TX + tx) * N;
	const uint64_t lo = (uint64_t) part * chunk;
	uint64_t hi = lo + chunk;
	if (hi > R) { hi = R; }

	T accs[U][N]; // U rows in flight per lane
#pragma unroll
	for (int u = 0; u < U; ++u)
	{
#pragma unroll
		for (int e = 0; e < N; ++e) { accs[u][e] = Red<T,OP>::identity(); }
	}
	if (col < A)
	{
		const T* base = in + col + b * A * R;
		uint64_t r = lo + ty;
		if constexpr (VEC)
		{
			for (; r + (U - 1) * TY < hi; r += U * TY)
			{
				VecU<T> x[U];
#pragma unroll
				for (int u = 0; u < U; ++u)
				{
					x[u].v = RED_LOAD(reinterpret_cast<const typename Vec16<T>::type*>(base + (r + u * TY) * A));
				}
#pragma unroll
				for (int u = 0; u < U; ++u)
				{
#pragma unroll
					for (int e = 0; e < N; ++e) { accs[u][e] = Red<T,OP>::combine(accs[u][e], x[u].e[e]); }
				}
			}
			for (; r < hi; r += TY)
			{
				VecU<T> x;
				x.v = RED_LOAD(reinterpret_cast<const typename Vec16<T>::type*>(base + r * A));
#pragma unroll
				for (int e = 0; e < N; ++e) { accs[0][e] = Red<T,OP>::combine(accs[0][e], x.e[e]); }
			}
		}
		else
		{
			for (; r < hi; r += TY) { accs[0][0] = Red<T,OP>::combine(accs[0][0], base[r * A]); }
		}
	}
	T acc[N];
#pragma unroll
	for (int e = 0; e < N; ++e)
	{
		acc[e] = accs[0][e];
#pragma unroll
		for (int u = 1; u < U; ++u) { acc[e] = Red<T,OP>::combine(acc[e], accs[u][e]); }
	}

	// combine the TY rows of the group through LDS; row stride padded by one
	// element so that the column walk below is conflict-free
	__shared__ T smem[BLOCK * (VEC ? Vec16<T>::N : 1) + BLOCK];
	const uint32_t pitch = TX * N + 1;
#pragma unroll
	for (int e = 0; e < N; ++e) { smem[ty * pitch + tx * N + e] = acc[e]; }
	__syncthreads();
	const uint32_t ncols = TX * N;
	for (uint32_t c = threadIdx.x; c < ncols; c += BLOCK)
	{
		T r = smem[c];
		for (uint32_t y = 1; y < TY; ++y) { r = Red<T,OP>::combine(r, smem[y * pitch + c]); }
		uint64_t gcol = (uint64_t) ctile * TX * N + c;
		if (gcol < A) { out[gcol + (uint64_t) part * A + b * A * S] = r; }
	}
}

// block per output (a, b): value and index of the first maximum along R
template <typename T>
__global__ __launch_bounds__(RED_BLOCK) void argmax_k (
	const T* __restrict__ in, T* __restrict__ out, uint64_t A, uint64_t R)
{
	const uint64_t a = blockIdx.x % A, b = blockIdx.x / A;
	const T* base = in + a + b * A * R;
	uint64_t best_i = ~(uint64_t) 0;
	T best = 0;
	for (uint64_t r = threadIdx.x; r < R; r += RED_BLOCK)
	{
		T v = base[r * A];
		if (best_i == ~(uint64_t) 0 || v > best) { best = v; best_i = r; }
	}
	__shared__ T sval[RED_BLOCK];
	__shared__ uint64_t sidx[RED_BLOCK];
	sval[threadIdx.x] = best;
	sidx[threadIdx.x] = best_i;
	__syncthreads();
	for (int s = RED_BLOCK / 2; s >= 1; s >>= 1)
	{
		if ((int) threadIdx.x < s)
		{
			T ov = sval[threadIdx.x + s];
			uint64_t oi = sidx[threadIdx.x + s];
			uint64_t mi = sidx[threadIdx.x];
			if (oi != ~(uint64_t) 0 && (mi == ~(uint64_t) 0 || ov > sval[threadIdx.x] ||
				(ov == sval[threadIdx.x] && oi < mi)))
			{
				sval[threadIdx.x] = ov;
				sidx[threadIdx.x] = oi;
			}
		}
		__syncthreads();
	}
	if (threadIdx.x == 0) { out[blockIdx.x] = (T) sidx[0]; }
}

// Where the temporaries of a reduction come from: partial results [A, S, B]
// of a reduced dim split over S workgroups, and what is left of the tensor
// between two steps of a reduction over separated dims
struct Scratch
{
	virtual ~Scratch (void) = default;
	virtual int take (tcg_ctx* ctx, size_t bytes, void** out) = 0;
	virtual void give (tcg_ctx* ctx, void* ptr, size_t bytes) = 0;
};

/// The context's pool (or the recording, while one is open)
struct PoolScratch final : public Scratch
{
	int take (tcg_ctx* ctx, size_t bytes, void** out) override { return tcg_alloc(ctx, bytes, out); }
	void give (tcg_ctx* ctx, void* ptr, size_t bytes) override { tcg_free(ctx, ptr, bytes); }
};

/// Hands out at most four 256-byte aligned pieces of one GPU's scratch array
/// at a time (a reduction step holds its operand, its result and its partial
/// results); lowest fitting address first
struct FixedScratch final : public Scratch
{
	FixedScratch (unsigned char* base) : base_(base) {}

	int take (tcg_ctx* ctx, size_t bytes, void** out) override
	{
		size_t need = (bytes + 255) & ~(size_t) 255;
		size_t at = 0;
		for (bool moved = true; moved;)
		{
			moved = false;
			for (int i = 0; i < 4; ++i)
			{
				if (size_[i] > 0 && at < off_[i] + size_[i] && off_[i] < at + need)
				{
					at = off_[i] + size_[i];
					moved = true;
				}
			}
		}
		int slot = 0;
		while (slot < 4 && size_[slot] > 0) { ++slot; }
		if (slot == 4 || at + need > NOALLOC_SCRATCH_BYTES)
		{
			return tcg_fail(ctx, TCG_ERR_ARG,
				"tcg_reduce_noalloc: the temporaries of this reduction (%zu more bytes) do not fit the fixed %zu-byte scratch memory; use tcg_reduce",
				need, NOALLOC_SCRATCH_BYTES);
		}
		off_[slot] = at;
		size_[slot] = need;
		*out = base_ + at;
		return TCG_OK;
	}

	void give (tcg_ctx*, void* ptr, size_t) override
	{
		size_t at = (size_t) ((unsigned char*) ptr - base_);
		for (int i = 0; i < 4; ++i)
		{
			if (size_[i] > 0 && off_[i] == at) { size_[i] = 0; }
		}
	}

	unsigned char* base_;
	size_t off_[4] = {0, 0, 0, 0};
	size_t size_[4] = {0, 0, 0, 0};
};

uint32_t ilog2_floor (uint64_t v)
{
	uint32_t l = 0;
	while (v > 1) { v >>= 1; ++l; }
	return l;
}

template <typename T, int OP>
int launch_inner (tcg_ctx* ctx, const T* in, T* out, uint64_t R, uint64_t K, uint32_t S, uint64_t chunk)
{
	bool vec = tcg_aligned16(in) && (R % Vec16<T>::N == 0);
	uint64_t blocks = K * S;
	TCG_REQUIRE(ctx, blocks < (1ull << 31), "tcg_reduce: %llu rows are too many for one launch", (unsigned long long) blocks);
	if (vec) { reduce_inner_k<T,OP,true><<<(unsigned) blocks, RED_BLOCK, 0, ctx->stream>>>(in, out, R, S, chunk); }
	else { reduce_inner_k<T,OP,false><<<(unsigned) blocks, RED_BLOCK, 0, ctx->stream>>>(in, out, R, S, chunk); }
	TCG_LAUNCH_CHECK(ctx, "reduce_inner");
	return TCG_OK;
}

template <typename T, int OP>
int launch_outer (tcg_ctx* ctx, const T* in, T* out, uint64_t A, uint64_t R, uint64_t B, uint32_t S, uint64_t chunk, uint32_t txlog2, bool vec)
{
	const uint32_t N = vec ? Vec16<T>::N : 1;
	uint64_t col_tiles = (A + ((uint64_t) N << txlog2) - 1) / ((uint64_t) N << txlog2);
	uint64_t blocks = col_tiles * S * B;
	TCG_REQUIRE(ctx, blocks < (1ull << 31) && col_tiles < (1ull << 31), "tcg_reduce: %llu workgroups are too many for one launch", (unsigned long long) blocks);
	if (vec) { reduce_outer_k<T,OP,true><<<(unsigned) blocks, RED_BLOCK, 0, ctx->stream>>>(in, out, A, R, S, chunk, txlog2, (uint32_t) col_tiles); }
	else { reduce_outer_k<T,OP,false><<<(unsigned) blocks, RED_BLOCK, 0, ctx->stream>>>(in, out, A, R, S, chunk, txlog2, (uint32_t) col_tiles); }
	TCG_LAUNCH_CHECK(ctx, "reduce_outer");
	return TCG_OK;
}

// Columns that are too few to fill the chip at full tile width are reduced in
// one pass all the same when narrower tiles (at least 16 lanes: 256-byte row
// segments) give every CU a workgroup: 512 lanes, 32 or 16 row groups, four
// rows in flight per lane.  Measured on np[4096,16384] -> [16384]: 38.9 us
// against 38.2 + 4 us for the split launch and the launch that adds its eight
// partial rows up.
constexpr int RED_WIDE_BLOCK = 512;
constexpr int RED_WIDE_UNROLL = 4;

template <typename T, int OP>
int launch_outer_wide (tcg_ctx* ctx, const T* in, T* out, uint64_t A, uint64_t R, uint64_t B, uint32_t txlog2)
{
	const uint32_t N = Vec16<T>::N;
	uint64_t col_tiles = (A + ((uint64_t) N << txlog2) - 1) / ((uint64_t) N << txlog2);
	uint64_t blocks = col_tiles * B;
	TCG_REQUIRE(ctx, blocks < (1ull << 31), "tcg_reduce: %llu workgroups are too many for one launch", (unsigned long long) blocks);
	reduce_outer_k<T,OP,true,RED_WIDE_BLOCK,RED_WIDE_UNROLL><<<(unsigned) blocks, RED_WIDE_BLOCK, 0, ctx->stream>>>(
		in, out, A, R, 1, R, txlog2, (uint32_t) col_tiles);
	TCG_LAUNCH_CHECK(ctx, "reduce_outer");
	return TCG_OK;
}

// [A, R, B] -> [A, B]
template <typename T, int OP>
int reduce_step (tcg_ctx* ctx, Scratch& mem, const T* in, T* out, uint64_t A, uint64_t R, uint64_t B)
{
	const uint64_t target_blocks = (uint64_t) ctx->num_cus * TCG_RED_BLOCKS_PER_CU;
	if (A == 1)
	{
		// split rows only when there are too few of them to fill the chip
		constexpr uint64_t quantum = (uint64_t) RED_BLOCK * Vec16<T>::N * 4;
		uint64_t S = 1;
		if (B < target_blocks && R >= 4 * quantum)
		{
			S = (target_blocks + B - 1) / B;
			uint64_t maxs = R / (2 * quantum);
			if (S > maxs) { S = maxs; }
			if (S < 1) { S = 1; }
		}
		uint64_t chunk = (R + S - 1) / S;
		chunk = (chunk + quantum - 1) / quantum * quantum;
		S = (R + chunk - 1) / chunk;
		if (S == 1) { return launch_inner<T,OP>(ctx, in, out, R, B, 1, chunk); }
		void* partial = nullptr;
		int rc = mem.take(ctx, sizeof(T) * B * S, &partial);
		if (rc != TCG_OK) { return rc; }
		rc = launch_inner<T,OP>(ctx, in, (T*) partial, R, B, (uint32_t) S, chunk);
		if (rc == TCG_OK) { rc = launch_inner<T,OP>(ctx, (const T*) partial, out, S, B, 1, S); }
		mem.give(ctx, partial, sizeof(T) * B * S);
		return rc;
	}
	bool vec = tcg_aligned16(in) && (A % Vec16<T>::N == 0);
	const uint32_t N = vec ? Vec16<T>::N : 1;
	uint64_t lanes = (A + N - 1) / N;
	uint32_t txlog2 = lanes >= (1u << TCG_RED_TXMAX_LOG2) ? TCG_RED_TXMAX_LOG2 : ilog2_floor(lanes);
	if (((uint64_t) 1 << txlog2) < lanes && txlog2 < TCG_RED_TXMAX_LOG2) { ++txlog2; }
	const uint32_t TY = RED_BLOCK >> txlog2;
	uint64_t col_tiles = (lanes + ((uint64_t) 1 << txlog2) - 1) >> txlog2;
	uint64_t base_blocks = col_tiles * B;
	uint64_t S = 1;
	if (vec && base_blocks < target_blocks && R >= 1024)
	{
		for (uint32_t narrow = txlog2; narrow-- > 4;)
		{
			uint64_t tiles = (lanes + ((uint64_t) 1 << narrow) - 1) >> narrow;
			if (tiles * B >= (uint64_t) ctx->num_cus)
			{
				return launch_outer_wide<T,OP>(ctx, in, out, A, R, B, narrow);
			}
		}
	}
	// (not below 256 KiB per workgroup: the launch that adds the partial rows up
	// then costs more than the split saves -- [64, 400, 128] -> [64, 128] takes
	// 4.5 + 4.8 us in three ranges)
	if (base_blocks < target_blocks && R >= (uint64_t) TY * 16 && A * R * sizeof(T) >= ((uint64_t) 256 << 10))
	{
		S = (target_blocks + base_blocks - 1) / base_blocks;
		uint64_t maxs = R / ((uint64_t) TY * 8);
		if (S > maxs) { S = maxs; }
		if (S < 1) { S = 1; }
	}
	uint64_t chunk = (R + S - 1) / S;
	S = (R + chunk - 1) / chunk;
	if (S == 1) { return launch_outer<T,OP>(ctx, in, out, A, R, B, 1, chunk, txlog2, vec); }
	void* partial = nullptr;
	int rc = mem.take(ctx, sizeof(T) * A * S * B, &partial);
	if (rc != TCG_OK) { return rc; }
	rc = launch_outer<T,OP>(ctx, in, (T*) partial, A, R, B, (uint32_t) S, chunk, txlog2, vec);
	if (rc == TCG_OK) { rc = launch_outer<T,OP>(ctx, (const T*) partial, out, A, S, B, 1, S, txlog2, vec); }
	mem.give(ctx, partial, sizeof(T) * A * S * B);
	return rc;
}

template <typename T, int OP>
int reduce_impl (tcg_ctx* ctx, Scratch& mem, const uint64_t shape[8], unsigned mask, const T* in, T* out)
{
	// merge neighbouring dims of equal kind, dropping singular dims
	uint64_t seg[8];
	bool red[8];
	int nseg = 0;
	for (int d = 0; d < 8; ++d)
	{
		if (shape[d] == 1) { continue; }
		bool r = (mask >> d) & 1;
		if (nseg > 0 && red[nseg - 1] == r) { seg[nseg - 1] *= shape[d]; }
		else { seg[nseg] = shape[d]; red[nseg] = r; ++nseg; }
	}
	int nred = 0;
	uint64_t n = 1;
	for (int i = 0; i < nseg; ++i) { nred += red[i]; n *= seg[i]; }
	if (nred == 0)
	{
		TCG_HIP(ctx, hipMemcpyAsync(out, in, sizeof(T) * n, hipMemcpyDeviceToDevice, ctx->stream));
		return TCG_OK;
	}
	// reduce the innermost reduced segment first; what is left of the tensor
	// shrinks at every step
	const T* cur = in;
	void* tmp_prev = nullptr;
	size_t tmp_prev_bytes = 0;
	int rc = TCG_OK;
	while (nred > 0 && rc == TCG_OK)
	{
		int i = 0;
		while (!red[i]) { ++i; }
		uint64_t A = 1, B = 1;
		for (int j = 0; j < i; ++j) { A *= seg[j]; }
		for (int j = i + 1; j < nseg; ++j) { B *= seg[j]; }
		uint64_t R = seg[i];
		T* dst = out;
		void* tmp = nullptr;
		size_t tmp_bytes = 0;
		if (nred > 1)
		{
			tmp_bytes = sizeof(T) * A * B;
			rc = mem.take(ctx, tmp_bytes, &tmp);
			if (rc != TCG_OK) { break; }
			dst = (T*) tmp;
		}
		rc = reduce_step<T,OP>(ctx, mem, cur, dst, A, R, B);
		if (tmp_prev) { mem.give(ctx, tmp_prev, tmp_prev_bytes); }
		tmp_prev = tmp;
		tmp_prev_bytes = tmp_bytes;
		cur = dst;
		// drop segment i and merge its (kept) neighbours
		for (int j = i; j + 1 < nseg; ++j) { seg[j] = seg[j + 1]; red[j] = red[j + 1]; }
		--nseg;
		--nred;
		if (i > 0 && i < nseg && red[i - 1] == red[i])
		{
			seg[i - 1] *= seg[i];
			for (int j = i; j + 1 < nseg; ++j) { seg[j] = seg[j + 1]; red[j] = red[j + 1]; }
			--nseg;
		}
	}
	if (tmp_prev) { mem.give(ctx, tmp_prev, tmp_prev_bytes); }
	return rc;
}

int reduce_any (tcg_ctx* ctx, Scratch& mem, int opcode, int dtype, const uint64_t shape[8],
	unsigned rankmask, const void* in, void* out)
{
	TCG_DISPATCH_ALL(ctx, dtype,
		switch (opcode)
		{
			case TCG_REDUCE_SUM: return reduce_impl<T,TCG_REDUCE_SUM>(ctx, mem, shape, rankmask, (const T*) in, (T*) out);
			case TCG_REDUCE_PROD: return reduce_impl<T,TCG_REDUCE_PROD>(ctx, mem, shape, rankmask, (const T*) in, (T*) out);
			case TCG_REDUCE_MIN: return reduce_impl<T,TCG_REDUCE_MIN>(ctx, mem, shape, rankmask, (const T*) in, (T*) out);
			default: return reduce_impl<T,TCG_REDUCE_MAX>(ctx, mem, shape, rankmask, (const T*) in, (T*) out);
		});
	return TCG_OK;
}

} // namespace

// Called by tcg_ctx_create with the context's device current: looks up where
// this GPU keeps its copy of the scratch array
int tcg_reduce_scratch_init (tcg_ctx* ctx)
{
	if (ctx->device < 0 || ctx->device >= MAX_DEVICES)
	{
		return tcg_fail(ctx, TCG_ERR_ARG, "device %d: at most %d devices", ctx->device, MAX_DEVICES);
	}
	std::lock_guard<std::mutex> lock(g_scratch_mu);
	if (nullptr == g_scratch[ctx->device])
	{
		unsigned char* ptr = nullptr;
		TCG_HIP(ctx, hipGetSymbolAddress((void**) &ptr, HIP_SYMBOL(scratch)));
		g_scratch[ctx->device] = ptr;
	}
	if (nullptr == ctx->scratch_done) { TCG_HIP(ctx, hipEventCreateWithFlags(&ctx->scratch_done, hipEventDisableTiming)); }
	return TCG_OK;
}

// Called by tcg_ctx_destroy once the context's stream has drained
void tcg_reduce_scratch_release (tcg_ctx* ctx)
{
	std::lock_guard<std::mutex> lock(g_scratch_mu);
	if (ctx->device >= 0 && ctx->device < MAX_DEVICES && g_owner[ctx->device].ctx == ctx) { g_owner[ctx->device] = ScratchOwner(); }
	if (nullptr != ctx->scratch_done)
	{
		(void) hipEventDestroy(ctx->scratch_done);
		ctx->scratch_done = nullptr;
	}
}

extern "C" {

int tcg_reduce (tcg_ctx* ctx, int opcode, int dtype, const uint64_t shape[8],
	unsigned rankmask, const void* in, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, opcode >= TCG_REDUCE_SUM && opcode <= TCG_REDUCE_MAX, "tcg_reduce: opcode %d is not a reduction", opcode);
	TCG_REQUIRE(ctx, shape && in && out, "tcg_reduce: NULL pointer");
	TCG_REQUIRE(ctx, rankmask < 256, "tcg_reduce: rank set 0x%x names a dim >= 8", rankmask);
	if (tcg_n_elems(shape) == 0) { return TCG_OK; }
	if (tcg_small_mode(ctx)) { TCG_SMALL_RETURN(ctx, tcg_small_reduce(ctx, opcode, dtype, shape, rankmask, in, out)); }
	PoolScratch mem;
	return reduce_any(ctx, mem, opcode, dtype, shape, rankmask, in, out);
}

int tcg_reduce_noalloc (tcg_ctx* ctx, int opcode, int dtype, const uint64_t shape[8],
	unsigned rankmask, const void* in, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, opcode >= TCG_REDUCE_SUM && opcode <= TCG_REDUCE_MAX, "tcg_reduce_noalloc: opcode %d is not a reduction", opcode);
	TCG_REQUIRE(ctx, shape && in && out, "tcg_reduce_noalloc: NULL pointer");
	TCG_REQUIRE(ctx, rankmask < 256, "tcg_reduce_noalloc: rank set 0x%x names a dim >= 8", rankmask);
	if (tcg_small_mode(ctx)) { TCG_SMALL_RETURN(ctx, tcg_small_unsupported(ctx, "tcg_reduce_noalloc")); }
	unsigned char* base = ctx->device >= 0 && ctx->device < MAX_DEVICES ? g_scratch[ctx->device] : nullptr;
	if (nullptr == base) { return tcg_fail(ctx, TCG_ERR_HIP, "tcg_reduce_noalloc: no scratch memory on device %d", ctx->device); }
	if (tcg_n_elems(shape) == 0) { return TCG_OK; }
	// Launches that are being recorded (by tcg_capture_begin or by the caller's own
	// capture of this stream) run when their recording is launched, which nothing
	// here can order against other users of the array: no check, and no event.
	hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
	(void) hipStreamIsCapturing(ctx->stream, &capture);
	const bool recorded = nullptr != ctx->capturing || capture != hipStreamCaptureStatusNone;
	if (false == recorded)
	{
		std::lock_guard<std::mutex> lock(g_scratch_mu);
		ScratchOwner& owner = g_owner[ctx->device];
		if (nullptr != owner.ctx && owner.ctx != ctx && hipErrorNotReady == hipEventQuery(owner.done))
		{
			return tcg_fail(ctx, TCG_ERR_ARG, "tcg_reduce_noalloc: another context's reduction is still using "
				"the scratch array of device %d (calls that overlap on one GPU would race)", ctx->device);
		}
		owner.ctx = ctx;
		owner.done = ctx->scratch_done;
	}
	FixedScratch mem(base);
	int rc = reduce_any(ctx, mem, opcode, dtype, shape, rankmask, in, out);
	if (false == recorded) { (void) hipEventRecord(ctx->scratch_done, ctx->stream); }
	return rc;
}

int tcg_argmax (tcg_ctx* ctx, int dtype, const uint64_t shape[8], int return_dim,
	const void* in, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, shape && in && out, "tcg_argmax: NULL pointer");
	TCG_REQUIRE(ctx, return_dim >= 0, "tcg_argmax: negative return_dim");
	uint64_t n = tcg_n_elems(shape);
	if (n == 0) { return TCG_OK; }
	uint64_t A = 1, R = n, B = 1;
	if (return_dim < 8)
	{
		R = shape[return_dim];
		for (int d = 0; d < return_dim; ++d) { A *= shape[d]; }
		for (int d = return_dim + 1; d < 8; ++d) { B *= shape[d]; }
	}
	TCG_REQUIRE(ctx, A * B < (1ull << 31), "tcg_argmax: too many outputs for one launch");
	TCG_DISPATCH_ALL(ctx, dtype, (argmax_k<T><<<(unsigned) (A * B), RED_BLOCK, 0, ctx->stream>>>((const T*) in, (T*) out, A, R)));
	TCG_LAUNCH_CHECK(ctx, "argmax");
	return TCG_OK;
}

} // extern "C"
