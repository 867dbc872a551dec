// fp32 GEMM on the matrix cores: C[b][m][n] = sum_k A[b][m][k] B[b][k][n].
//
// One workgroup of 256 lanes (4 waves, 2x2) owns a BM x BN tile of C; each wave
// owns a (BM/2) x (BN/2) sub-tile built from 32x32 accumulators fed by
// v_mfma_f32_32x32x2_f32.  A and B slabs of BK columns go global -> LDS
// directly where the operands are plain matrices and K is a whole number of
// slabs (gemm_mfma_direct_k: three slabs in LDS, two on their way), and global
// -> registers -> LDS (double buffered, one barrier per slab) everywhere else
// (gemm_mfma_k: sums of products over terms, operands gathered from a
// convolution's image, ragged K).  Workgroup ids are remapped so that the
// workgroups resident on one XCD (ids congruent mod 8) cover a compact patch of
// C and share their A/B panels through that XCD's L2.
// MFMA-bound: 2*M*N*K flops, operands re-read from L2, each C element written once.
#include <type_traits>

#include "tcg_internal.hpp"
#include <cstdlib>

namespace
{

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4v __attribute__((ext_vector_type(4)));

constexpr int BK = 16;
constexpr int NXCD = 8;
constexpr int GROUP_M = 8;

struct GemmArgs
{
	const float* A;
	const float* B;
	float* C;
	uint32_t M, N, K;
	int64_t lda, ldb, ldc;
	int64_t batch_a, batch_b, batch_c;
	uint32_t tiles_m, tiles_n, tiles_per_batch, total_tiles;
	// split K: block id / total_tiles picks a K range of k_per_split columns;
	// with more than one range the C tile goes to partial[range][batch][M][N]
	uint32_t k_per_split;
	float* partial;
	// A read through a convolution's tables (IMPL != 0): A is the image
	const tcg_conv_tab* rows;
	const tcg_conv_tab* sums;
	uint32_t check_ext[4];
	int ncheck;
	const float* zeros; // 16 zero bytes and more in device memory
};

// A sum of products C = sum_t A_t B_t of equal shapes is one product over the
// concatenated summed index: term t supplies the columns [t * k, (t + 1) * k)
// of A and the rows of B with the same numbers.  The operands stay where they
// are; the kernel looks the term's pointers up once per slab (k is a multiple
// of the slab depth, so a slab never straddles two terms).
constexpr int MAX_TERMS = 128;

struct GemmSegs
{
	uint32_t k = 0; // columns of A (rows of B) per term
	const float* a[MAX_TERMS];
	const float* b[MAX_TERMS];
	uint32_t lda[MAX_TERMS]; // the terms may lie in tensors of different row lengths
	uint32_t ldb[MAX_TERMS];
};

struct NoSegs {};

// The same for operands that are concatenations along the dims that survive:
// the result falls into mparts x nparts blocks, block (i, j) being the sum
// over the terms of A[i][t] B[j][t].  Every part is a whole number of tiles,
// so a tile looks its part up once; the operands stay where they are.
constexpr int MAX_GRID_PTRS = 384;
constexpr int MAX_GRID_MPARTS = 4, MAX_GRID_NPARTS = 8;

struct GemmGrid
{
	uint32_t k = 0;      // columns of A (rows of B) per term
	uint32_t terms = 0;
	uint32_t mparts = 0, nparts = 0;
	uint32_t mstart[MAX_GRID_MPARTS + 1]; // first row of each part of A, then M
	uint32_t nstart[MAX_GRID_NPARTS + 1]; // first column of each part of B, then N
	uint32_t lda[MAX_GRID_MPARTS];
	uint32_t ldb[MAX_GRID_NPARTS];
	const float* ptr[MAX_GRID_PTRS];      // a[part][term], then b[part][term]
};

__device__ __forceinline__ bool conv_inside (const GemmArgs& g, const tcg_conv_tab& row, const tcg_conv_tab& col)
{
	bool inside = true;
#pragma unroll
	for (int j = 0; j < 4; ++j)
	{
		if (j < g.ncheck) { inside = inside && (uint32_t) (row.c[j] + col.c[j]) < g.check_ext[j]; }
	}
	return inside;
}

// TA: A(m,k) at m + k*lda (M contiguous) instead of m*lda + k.
// TB: B(k,n) at k + n*ldb (K contiguous) instead of k*ldb + n.
// WGM: waves along M (2: waves 2x2, 4: waves 4x1 for narrow N).
//
// LDS layouts: an operand whose K runs contiguously in memory is kept
// [row][k] with a pitch of BK+4 floats and read four k at a time (one 128-bit
// read per four matrix instructions); an operand whose rows run contiguously
// is kept [k][row] and read one float at a time, consecutive lanes on
// consecutive banks.  Both are written with 128-bit stores straight from the
// 128-bit global loads.  To make the four-at-a-time reads possible the two
// lane halves of a matrix instruction (which supply k and k+1 of its K=2) take
// k = 8*(j/4) + 4*half + j%4 in step j of a slab instead of 2j + half: the
// order in which a slab's sixteen k are summed is a fixed permutation, the
// same for every element.
//
// IMPL: 0 = A is a matrix in memory.  1 = A[m][k] = image[rows[m].off +
// sums[k].off] or zero (a convolution's operand, never materialised); TA then
// says which index runs along memory (consecutive m, or consecutive k), and
// aligned groups of four along that index are contiguous and exist or not
// together: one table lookup and one 128-bit load per group.  A lane's row
// entries stay in registers; the entry of the summed index is fetched one slab
// ahead of the load that needs it.
//
// AHEAD: slabs on their way from memory into registers while one is multiplied.
template <int BM, int BN, int WGM, bool TA, bool TB, int IMPL, int AHEAD = 1>
__global__ __launch_bounds__(256) void gemm_mfma_k (GemmArgs g)
{
	static_assert(AHEAD == 1 || AHEAD == 2, "slabs on their way from memory while one is multiplied");
	static_assert(IMPL == 0 || AHEAD == 2, "a convolution's operand is read two slabs ahead");
	constexpr int WGN = 4 / WGM;
	constexpr int WM = BM / WGM, WN = BN / WGN; // wave tile
	constexpr int TM = WM / 32, TN = WN / 32;   // 32x32 accumulators per wave
	static_assert(WM % 32 == 0 && WN % 32 == 0 && TM >= 1 && TN >= 1, "wave tiles are made of 32x32 blocks");
	constexpr int KP = BK + 4;                  // pitch of a [row][k] tile
	constexpr int AP = TA ? BM + 4 : KP;
	constexpr int BP = TB ? KP : BN + 4;
	constexpr int A_SIZE = TA ? BK * AP : BM * AP;
	constexpr int B_SIZE = TB ? BN * BP : BK * BP;
	constexpr int A_CHUNKS = BM * BK / 4, B_CHUNKS = BN * BK / 4; // float4 per slab
	constexpr int A_VEC = (A_CHUNKS + 255) / 256, B_VEC = (B_CHUNKS + 255) / 256;
	__shared__ __attribute__((aligned(16))) float As[2][A_SIZE];
	__shared__ __attribute__((aligned(16))) float Bs[2][B_SIZE];

	// ---- which tile: XCD-aware, grouped order --------------------------------
	const uint32_t split = blockIdx.x / g.total_tiles;
	uint32_t id = blockIdx.x - split * g.total_tiles;
	const uint32_t k_begin = split * g.k_per_split;
	const uint32_t k_end = g.K - k_begin < g.k_per_split ? g.K : k_begin + g.k_per_split;
	if (g.total_tiles % NXCD == 0)
	{
		id = (id % NXCD) * (g.total_tiles / NXCD) + id / NXCD;
	}
	const uint32_t bz = id / g.tiles_per_batch;
	uint32_t t = id - bz * g.tiles_per_batch;
	const uint32_t group_size = GROUP_M * g.tiles_n;
	const uint32_t group = t / group_size;
	const uint32_t first_m = group * GROUP_M;
	const uint32_t rows_in_group = g.tiles_m - first_m < (uint32_t) GROUP_M ? g.tiles_m - first_m : GROUP_M;
	const uint32_t in_group = t - group * group_size;
	const uint32_t tm = first_m + in_group % rows_in_group;
	const uint32_t tn = in_group / rows_in_group;
	const uint32_t m0 = tm * BM, n0 = tn * BN;
	const float* __restrict__ Abase = g.A + (int64_t) bz * g.batch_a;
	const float* __restrict__ Bbase = g.B + (int64_t) bz * g.batch_b;
	float* __restrict__ C = g.partial ?
		g.partial + ((int64_t) split * (g.total_tiles / g.tiles_per_batch) + bz) * ((int64_t) g.M * g.N) :
		g.C + (int64_t) bz * g.batch_c;
	const int64_t ldc = g.partial ? (int64_t) g.N : g.ldc;

	const int tid = threadIdx.x;
	const int lane = tid & 63, wave = tid >> 6;
	const int wm = wave / WGN, wn = wave % WGN;
	const int l32 = lane & 31, lh = lane >> 5;

	f32x16 acc[TM][TN];
#pragma unroll
	for (int i = 0; i < TM; ++i)
	{
#pragma unroll
		for (int j = 0; j < TN; ++j)
		{
#pragma unroll
			for (int r = 0; r < 16; ++r) { acc[i][j][r] = 0.0f; }
		}
	}

	f32x4v ra[AHEAD][A_VEC], rb[AHEAD][B_VEC];
	const f32x4v zero4 = {0.0f, 0.0f, 0.0f, 0.0f};

	// the table rows a lane gathers from stay the same for every slab
	constexpr int ROW_ENTS = IMPL == 0 ? 1 : (!TA ? A_VEC : 1);
	// ... and with K along memory every chunk of a lane has the same summed indices
	constexpr int COL_ENTS = !TA ? 1 : A_VEC;
	tcg_conv_tab rowent[ROW_ENTS], colent[AHEAD][COL_ENTS];
	// summed index of chunk v in the slab that starts at k0
	auto chunk_k = [&] (uint32_t k0, int v) -> uint32_t
	{
		int idx = tid + v * 256;
		return !TA ? k0 + (idx % (BK / 4)) * 4 : k0 + idx / (BM / 4);
	};
	if constexpr (IMPL != 0)
	{
		static_assert(256 % (BM / 4) == 0, "a lane keeps its rows from slab to slab");
#pragma unroll
		for (int e = 0; e < ROW_ENTS; ++e)
		{
			uint32_t m = !TA ? m0 + (tid + e * 256) / (BK / 4) : m0 + (tid % (BM / 4)) * 4;
			rowent[e] = g.rows[m < g.M ? m : g.M - 1];
		}
#pragma unroll
		for (int v = 0; v < COL_ENTS; ++v)
		{
			uint32_t k = chunk_k(k_begin, v);
			colent[0][v] = g.sums[k < g.K ? k : g.K - 1];
		}
	}

	// AHEAD == 2: two slabs are on their way from memory while one is multiplied.
	// The hardware counts loads that are still out, and they come back in the order
	// they were issued; "slab s + 1 has arrived" can only be waited for as "at most
	// the loads of slab s + 2 are out" when that number is known, so no load sits
	// under a predicate: an element that does not exist is read from the start of
	// the operand instead and replaced by zero (`okm`) on its way into LDS.
	constexpr bool EAGER = AHEAD == 2;
	uint32_t okm[AHEAD];
	auto fetch = [&] (const float* p, bool ok, const float* safe) -> f32x4v
	{
		if constexpr (EAGER) { return *reinterpret_cast<const f32x4v*>(ok ? p : safe); }
		else { return ok ? *reinterpret_cast<const f32x4v*>(p) : zero4; }
	};

	// `set`: the registers the slab waits in (slab x in set x % AHEAD)
	auto load_slab = [&] (uint32_t k0, auto set_c)
	{
		constexpr int set = decltype(set_c)::value;
		if constexpr (IMPL != 0)
		{
			// the table entries of the slab after this one go first: waiting for
			// them later then waits for nothing of this slab
#pragma unroll
			for (int v = 0; v < COL_ENTS; ++v)
			{
				uint32_t kn = chunk_k(k0, v) + BK;
				colent[set ^ 1][v] = g.sums[kn < g.K ? kn : g.K - 1];
			}
		}
		const float* __restrict__ A = Abase;
		const float* __restrict__ B = Bbase;
		const int64_t lda = g.lda, ldb = g.ldb;
		uint32_t oks = 0;
#pragma unroll
		for (int v = 0; v < A_VEC; ++v)
		{
			int idx = tid + v * 256;
			if constexpr (!EAGER)
			{
				if (A_CHUNKS % 256 != 0 && idx >= A_CHUNKS) { break; }
			}
			bool ok = A_CHUNKS % 256 == 0 || idx < A_CHUNKS;
			if constexpr (IMPL != 0)
			{
				// four consecutive k of one row, or four consecutive rows at one k
				uint32_t m = !TA ? m0 + idx / (BK / 4) : m0 + (idx % (BM / 4)) * 4;
				uint32_t k = chunk_k(k0, v);
				const tcg_conv_tab& row = rowent[!TA ? v : 0];
				const tcg_conv_tab& col = colent[set][!TA ? 0 : v];
				ok = ok && m < g.M && k < k_end && conv_inside(g, row, col);
				ra[set][v] = fetch(A + row.off + col.off, ok, g.A);
			}
			else if constexpr (!TA)
			{
				// K contiguous: BK/4 lanes per row
				int mm = idx / (BK / 4), kq = idx % (BK / 4);
				uint32_t m = m0 + mm, k = k0 + kq * 4;
				ok = ok && m < g.M && k < k_end;
				ra[set][v] = fetch(A + (int64_t) m * lda + k, ok, g.A);
			}
			else
			{
				// M contiguous: BM/4 lanes per k
				int kk = idx / (BM / 4), mq = idx % (BM / 4);
				uint32_t m = m0 + mq * 4, k = k0 + kk;
				ok = ok && m < g.M && k < k_end;
				ra[set][v] = fetch(A + (int64_t) k * lda + m, ok, g.A);
			}
			oks |= (uint32_t) ok << v;
		}
#pragma unroll
		for (int v = 0; v < B_VEC; ++v)
		{
			int idx = tid + v * 256;
			if constexpr (!EAGER)
			{
				if (B_CHUNKS % 256 != 0 && idx >= B_CHUNKS) { break; }
			}
			bool ok = B_CHUNKS % 256 == 0 || idx < B_CHUNKS;
			if constexpr (!TB)
			{
				// N contiguous: BN/4 lanes per k
				int kk = idx / (BN / 4), nq = idx % (BN / 4);
				uint32_t n = n0 + nq * 4, k = k0 + kk;
				ok = ok && n < g.N && k < k_end;
				rb[set][v] = fetch(B + (int64_t) k * ldb + n, ok, g.B);
			}
			else
			{
				// K contiguous: BK/4 lanes per n
				int nn = idx / (BK / 4), kq = idx % (BK / 4);
				uint32_t n = n0 + nn, k = k0 + kq * 4;
				ok = ok && n < g.N && k < k_end;
				rb[set][v] = fetch(B + (int64_t) n * ldb + k, ok, g.B);
			}
			oks |= (uint32_t) ok << (16 + v);
		}
		okm[set] = oks;
	};

	auto store_slab = [&] (int buf, auto set_c)
	{
		constexpr int set = decltype(set_c)::value;
		float* as = As[buf];
		float* bs = Bs[buf];
#pragma unroll
		for (int v = 0; v < A_VEC; ++v)
		{
			int idx = tid + v * 256;
			if (A_CHUNKS % 256 != 0 && idx >= A_CHUNKS) { break; }
			f32x4v val = ra[set][v];
			if constexpr (EAGER) { val = (okm[set] >> v & 1u) ? val : zero4; }
			if constexpr (!TA)
			{
				int mm = idx / (BK / 4), kq = idx % (BK / 4);
				*reinterpret_cast<f32x4v*>(as + mm * AP + kq * 4) = val;
			}
			else
			{
				int kk = idx / (BM / 4), mq = idx % (BM / 4);
				*reinterpret_cast<f32x4v*>(as + kk * AP + mq * 4) = val;
			}
		}
#pragma unroll
		for (int v = 0; v < B_VEC; ++v)
		{
			int idx = tid + v * 256;
			if (B_CHUNKS % 256 != 0 && idx >= B_CHUNKS) { break; }
			f32x4v val = rb[set][v];
			if constexpr (EAGER) { val = (okm[set] >> (16 + v) & 1u) ? val : zero4; }
			if constexpr (!TB)
			{
				int kk = idx / (BN / 4), nq = idx % (BN / 4);
				*reinterpret_cast<f32x4v*>(bs + kk * BP + nq * 4) = val;
			}
			else
			{
				int nn = idx / (BK / 4), kq = idx % (BK / 4);
				*reinterpret_cast<f32x4v*>(bs + nn * BP + kq * 4) = val;
			}
		}
	};

	// slab `buf` of LDS times itself into the accumulators
	auto multiply = [&] (int buf)
	{
		const float* as = As[buf];
		const float* bs = Bs[buf];
#pragma unroll
		for (int half = 0; half < BK / 8; ++half)
		{
			const int kb = half * 8 + lh * 4; // this lane's four k of the half slab
			f32x4v a[TM], b[TN];
#pragma unroll
			for (int i = 0; i < TM; ++i)
			{
				const int row = wm * WM + i * 32 + l32;
				if constexpr (!TA) { a[i] = *reinterpret_cast<const f32x4v*>(as + row * AP + kb); }
				else
				{
#pragma unroll
					for (int e = 0; e < 4; ++e) { a[i][e] = as[(kb + e) * AP + row]; }
				}
			}
#pragma unroll
			for (int j = 0; j < TN; ++j)
			{
				const int col = wn * WN + j * 32 + l32;
				if constexpr (TB) { b[j] = *reinterpret_cast<const f32x4v*>(bs + col * BP + kb); }
				else
				{
#pragma unroll
					for (int e = 0; e < 4; ++e) { b[j][e] = bs[(kb + e) * BP + col]; }
				}
			}
#pragma unroll
			for (int e = 0; e < 4; ++e)
			{
#pragma unroll
				for (int i = 0; i < TM; ++i)
				{
#pragma unroll
					for (int j = 0; j < TN; ++j)
					{
						acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][e], b[j][e], acc[i][j], 0, 0, 0);
					}
				}
			}
		}
	};

	const uint32_t nslabs = (k_end - k_begin + BK - 1) / BK;
	using I0 = std::integral_constant<int,0>;
	using I1 = std::integral_constant<int,1>;
	load_slab(k_begin, I0());
	store_slab(0, I0());
	if constexpr (AHEAD == 1)
	{
		__syncthreads();
		for (uint32_t s = 0; s < nslabs; ++s)
		{
			const int buf = s & 1;
			if (s + 1 < nslabs) { load_slab(k_begin + (s + 1) * BK, I0()); }
			multiply(buf);
			if (s + 1 < nslabs) { store_slab(buf ^ 1, I0()); }
			__syncthreads();
		}
	}
	else
	{
		// slab s (s % 2 == par) is multiplied out of LDS while slab s + 2 sets out for the
		// registers slab s came through and slab s + 1 is still on its way; slab s + 1
		// goes into the other half of LDS afterwards.  Past the end the last slab is
		// fetched again and never used, so that every step issues the same loads.
		const uint32_t last = k_begin + (nslabs - 1) * BK;
		auto slab_at = [&] (uint32_t s) -> uint32_t { return s < nslabs ? k_begin + s * BK : last; };
		load_slab(slab_at(1), I1());
		__syncthreads();
		auto step = [&] (uint32_t s, auto par_c)
		{
			constexpr int par = decltype(par_c)::value;
			load_slab(slab_at(s + 2), std::integral_constant<int,par>());
			multiply(par);
			if (s + 1 < nslabs) { store_slab(par ^ 1, std::integral_constant<int,par ^ 1>()); }
			__syncthreads();
		};
		uint32_t s = 0;
		for (; s + 1 < nslabs; s += 2)
		{
			step(s, I0());
			step(s + 1, I1());
		}
		if (s < nslabs) { step(s, I0()); }
	}

	// lane holds column l32; register r is row 8*(r/4) + 4*lh + r%4 of the 32x32 block
#pragma unroll
	for (int i = 0; i < TM; ++i)
	{
#pragma unroll
		for (int j = 0; j < TN; ++j)
		{
			const uint32_t n = n0 + wn * WN + j * 32 + l32;
			if (n >= g.N) { continue; }
#pragma unroll
			for (int r = 0; r < 16; ++r)
			{
				const uint32_t m = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
				if (m < g.M) { C[(int64_t) m * ldc + n] = acc[i][j][r]; }
			}
		}
	}
}

// K a multiple of the slab depth: the slabs go from memory straight into LDS
// (global_load_lds_dwordx4: lane l of a wave's load leaves its 16 bytes at the
// wave's LDS base + 16 l), no registers and no LDS stores in between, three
// slabs in LDS: one being multiplied, two on their way.  A wave's load fills
// 1 KiB of LDS in lane order, so conflict-free reads come from which chunk a
// lane fetches, not from padding.  An operand whose K runs along memory is kept
// [row][16 k], 16 rows x 4 chunks per load, the chunk in slot q of row r being
// q ^ ((r >> 1) & 3); an operand whose rows run along memory is kept
// [k][rows], the rows of k-rows 4..7 and 12..15 exchanged in halves of 32 (the
// two lane halves of a matrix instruction read k and k + 4).  Rows and columns
// past the edge are fetched from the last ones inside and never stored.
// rows exchanged in the k-rows the upper lane half reads: halves of 32, of 16 in a slab of 32 rows
constexpr int direct_swap (int rows) { return rows >= 64 ? 32 : 16; }

template <int ROWS, bool KALONG>
__device__ __forceinline__ void direct_issue (const float* __restrict__ P, int64_t ld, uint32_t first, uint32_t extent,
	uint32_t k0, float* lds, int wave, int lane)
{
	// a slab of 32 rows is two loads: the waves of the second pair repeat them, so
	// that every wave has the same number of loads out
	constexpr int TOTAL = ROWS * BK / 256;          // loads per slab
	constexpr int LOADS = TOTAL >= 4 ? TOTAL / 4 : 1; // per wave
#pragma unroll
	for (int j = 0; j < LOADS; ++j)
	{
		const int load = (wave * LOADS + j) % TOTAL;
		const float* src;
		if constexpr (KALONG)
		{
			const int rows = load * 16;
			const int r = rows + lane / 4, q = lane % 4;
			const int chunk = q ^ ((r >> 1) & 3);
			uint32_t row = first + r;
			row = row < extent ? row : extent - 1;
			src = P + (int64_t) row * ld + k0 + chunk * 4;
		}
		else
		{
			// 256 floats of the [k][rows] slab: 256 / ROWS k-rows
			const int at = load * 256 + lane * 4;
			const int k = at / ROWS, q = (at % ROWS) / 4;
			const int chunk = q ^ (direct_swap(ROWS) / 4 * ((k >> 2) & 1));
			uint32_t row = first + chunk * 4;
			row = row + 4 <= extent ? row : extent - 4;
			src = P + (int64_t) (k0 + k) * ld + row;
		}
		const uint32_t base = __builtin_amdgcn_readfirstlane(
			(uint32_t) (uintptr_t) (const __attribute__((address_space(3))) float*) (lds + load * 256));
		// written as the instruction itself: the compiler keeps one score for every
		// such load it knows of and waits for all of them before any later LDS read,
		// which would leave nothing on its way while a slab is multiplied.  The s_nop is
		// the wait state the hardware wants between a scalar write of M0 and a load into
		// LDS that reads it (the compiler adds it for its builtin, not inside this text)
		asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(base) : "memory", "m0");
	}
}

// IMPL 1: A[m][k] = image[rows[m].off + sums[k].off] or zero, as in gemm_mfma_k.
// The entries of the summed indices of the workgroup's K range wait in LDS
// (direct_tab() of them at most), so that the loop holds no load but the ones that
// go into LDS and the kernel's own count of those stays exact; a lane's row
// entries stay in registers; an element of the zero border is fetched from a
// buffer of zeros.
constexpr int direct_tab (int BM, int BN)
{
	// what the 64 KiB of a workgroup's static LDS leave beside the three slabs, in whole slabs
	int room = (65536 - 3 * (BM + BN) * BK * 4) / (int) sizeof(tcg_conv_tab) / BK * BK;
	return room < 1408 ? room : 1408;
}

template <int BM, int BN, bool TA, bool TB, typename SEGS = NoSegs, int IMPL = 0, int WGM = 2>
__global__ __launch_bounds__(256) void gemm_mfma_direct_k (GemmArgs g, SEGS segs)
{
	// WGM: waves along M (2: waves 2 x 2; 4: waves 4 x 1 for a result of 32 columns)
	constexpr int WGN = 4 / WGM, WM = BM / WGM, WN = BN / WGN;
	static_assert(WM % 32 == 0 && WN % 32 == 0 && WM >= 32 && WN >= 32, "wave tiles are made of 32 x 32 blocks");
	static_assert(IMPL == 0 || (std::is_same<SEGS,NoSegs>::value && !TB), "a convolution's operand against a row-major matrix");
	constexpr bool GRID = std::is_same<SEGS,GemmGrid>::value;
	constexpr bool SEG = !std::is_same<SEGS,NoSegs>::value && !GRID;
	constexpr int TM = WM / 32, TN = WN / 32; // 32 x 32 accumulators per wave
	constexpr int A_SIZE = BM * BK, B_SIZE = BN * BK;
	__shared__ __attribute__((aligned(1024))) float As0[A_SIZE];
	__shared__ __attribute__((aligned(1024))) float As1[A_SIZE];
	__shared__ __attribute__((aligned(1024))) float As2[A_SIZE];
	__shared__ __attribute__((aligned(1024))) float Bs0[B_SIZE];
	__shared__ __attribute__((aligned(1024))) float Bs1[B_SIZE];
	__shared__ __attribute__((aligned(1024))) float Bs2[B_SIZE];

	// block id / total_tiles picks a K range (whole slabs), as in gemm_mfma_k
	const uint32_t split = blockIdx.x / g.total_tiles;
	uint32_t id = blockIdx.x - split * g.total_tiles;
	const uint32_t k_begin = split * g.k_per_split;
	const uint32_t k_end = g.K - k_begin < g.k_per_split ? g.K : k_begin + g.k_per_split;
	if (g.total_tiles % NXCD == 0) { id = (id % NXCD) * (g.total_tiles / NXCD) + id / NXCD; }
	const uint32_t bz = id / g.tiles_per_batch;
	const uint32_t t = id - bz * g.tiles_per_batch;
	const uint32_t group_size = GROUP_M * g.tiles_n;
	const uint32_t group = t / group_size;
	const uint32_t first_m = group * GROUP_M;
	const uint32_t rows_in_group = g.tiles_m - first_m < (uint32_t) GROUP_M ? g.tiles_m - first_m : GROUP_M;
	const uint32_t in_group = t - group * group_size;
	const uint32_t m0 = (first_m + in_group % rows_in_group) * BM, n0 = (in_group / rows_in_group) * BN;
	const float* __restrict__ A = g.A + (int64_t) bz * g.batch_a;
	const float* __restrict__ B = g.B + (int64_t) bz * g.batch_b;
	float* __restrict__ C = g.partial ?
		g.partial + ((int64_t) split * (g.total_tiles / g.tiles_per_batch) + bz) * ((int64_t) g.M * g.N) :
		g.C + (int64_t) bz * g.batch_c;
	const int64_t ldc = g.partial ? (int64_t) g.N : g.ldc;

	const int tid = threadIdx.x;
	const int lane = tid & 63, wave = tid >> 6;
	const int wm = wave / WGN, wn = wave % WGN;
	const int l32 = lane & 31, lh = lane >> 5;

	f32x16 acc[TM][TN];
#pragma unroll
	for (int i = 0; i < TM; ++i)
	{
#pragma unroll
		for (int j = 0; j < TN; ++j)
		{
#pragma unroll
			for (int r = 0; r < 16; ++r) { acc[i][j][r] = 0.0f; }
		}
	}

	// a grid of blocks: the parts this tile lies in, and what takes a row / column
	// of the whole result to a row / column of the part (see gemm_mfma_k)
	uint32_t part_a = 0, part_b = 0;
	int64_t shift_a = 0, shift_b = 0;
	if constexpr (GRID)
	{
		while (part_a + 1 < segs.mparts && m0 >= segs.mstart[part_a + 1]) { ++part_a; }
		while (part_b + 1 < segs.nparts && n0 >= segs.nstart[part_b + 1]) { ++part_b; }
		shift_a = (int64_t) segs.mstart[part_a] * (TA ? 1 : (int64_t) segs.lda[part_a]);
		shift_b = (int64_t) segs.nstart[part_b] * (TB ? (int64_t) segs.ldb[part_b] : 1);
	}
	// a convolution's operand: the entries of this workgroup's summed indices, and the
	// row entries of the chunks this lane fetches (the same for every slab)
	constexpr int A_LOADS = BM / 64;
	__shared__ tcg_conv_tab tab[IMPL != 0 ? direct_tab(BM, BN) : 1];
	tcg_conv_tab rowent[IMPL != 0 ? A_LOADS : 1];
	if constexpr (IMPL != 0)
	{
		for (uint32_t e = tid; e < k_end - k_begin; e += 256) { tab[e] = g.sums[k_begin + e]; }
#pragma unroll
		for (int j = 0; j < A_LOADS; ++j)
		{
			const int load = wave * A_LOADS + j;
			uint32_t m;
			if constexpr (!TA) { m = m0 + load * 16 + lane / 4; }
			else
			{
				const int at = load * 256 + lane * 4;
				const int k = at / BM, q = (at % BM) / 4;
				m = m0 + (q ^ (direct_swap(BM) / 4 * ((k >> 2) & 1))) * 4;
				m = m + 4 <= g.M ? m : g.M - 4;
			}
			rowent[j] = g.rows[m < g.M ? m : g.M - 1];
		}
		__syncthreads();
	}
	auto issue_gathered = [&] (uint32_t k0, float* as)
	{
#pragma unroll
		for (int j = 0; j < A_LOADS; ++j)
		{
			const int load = wave * A_LOADS + j;
			int k; // the summed index of this lane's chunk, counted from the slab's first
			if constexpr (!TA)
			{
				const int r = load * 16 + lane / 4, q = lane % 4;
				k = (q ^ ((r >> 1) & 3)) * 4;
			}
			else { k = (load * 256 + lane * 4) / BM; }
			const tcg_conv_tab col = tab[k0 - k_begin + k];
			const float* src = conv_inside(g, rowent[j], col) ? g.A + rowent[j].off + col.off : g.zeros;
			const uint32_t base = __builtin_amdgcn_readfirstlane(
				(uint32_t) (uintptr_t) (const __attribute__((address_space(3))) float*) (as + load * 256));
			asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(base) : "memory", "m0");
		}
	};
	auto issue = [&] (uint32_t k0, float* as, float* bs)
	{
		// with terms: the operands of the term this slab belongs to, addressed by
		// the summed index counted from the term's first column
		const float* __restrict__ At = A;
		const float* __restrict__ Bt = B;
		int64_t lda = g.lda, ldb = g.ldb;
		if constexpr (SEG)
		{
			const uint32_t term = k0 / segs.k;
			At = segs.a[term];
			Bt = segs.b[term];
			lda = segs.lda[term];
			ldb = segs.ldb[term];
			k0 -= term * segs.k;
		}
		if constexpr (GRID)
		{
			const uint32_t term = k0 / segs.k;
			At = segs.ptr[part_a * segs.terms + term] - shift_a;
			Bt = segs.ptr[(segs.mparts + part_b) * segs.terms + term] - shift_b;
			lda = segs.lda[part_a];
			ldb = segs.ldb[part_b];
			k0 -= term * segs.k;
		}
		if constexpr (IMPL != 0) { issue_gathered(k0, as); }
		else { direct_issue<BM,!TA>(At, lda, m0, g.M, k0, as, wave, lane); }
		direct_issue<BN,TB>(Bt, ldb, n0, g.N, k0, bs, wave, lane);
	};
	auto multiply = [&] (const float* as, const float* bs)
	{
#pragma unroll
		for (int half = 0; half < BK / 8; ++half)
		{
			const int kb = half * 8 + lh * 4; // this lane's four k of the half slab
			f32x4v a[TM], b[TN];
#pragma unroll
			for (int i = 0; i < TM; ++i)
			{
				const int row = wm * WM + i * 32 + l32;
				if constexpr (!TA) { a[i] = *reinterpret_cast<const f32x4v*>(as + row * BK + ((half * 2 + lh) ^ ((row >> 1) & 3)) * 4); }
				else
				{
#pragma unroll
					for (int e = 0; e < 4; ++e) { a[i][e] = as[(kb + e) * BM + (row ^ (direct_swap(BM) * lh))]; }
				}
			}
#pragma unroll
			for (int j = 0; j < TN; ++j)
			{
				const int col = wn * WN + j * 32 + l32;
				if constexpr (TB) { b[j] = *reinterpret_cast<const f32x4v*>(bs + col * BK + ((half * 2 + lh) ^ ((col >> 1) & 3)) * 4); }
				else
				{
#pragma unroll
					for (int e = 0; e < 4; ++e) { b[j][e] = bs[(kb + e) * BN + (col ^ (direct_swap(BN) * lh))]; }
				}
			}
#pragma unroll
			for (int e = 0; e < 4; ++e)
			{
#pragma unroll
				for (int i = 0; i < TM; ++i)
				{
#pragma unroll
					for (int j = 0; j < TN; ++j)
					{
						acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][e], b[j][e], acc[i][j], 0, 0, 0);
					}
				}
			}
		}
	};
	// Every step issues the loads of one slab, so "at most that many loads out"
	// means that everything but the newest slab has landed (loads complete in
	// order); the LDS reads of the step are done as well before the barrier, since
	// the next step's loads overwrite the slab the step before this one read.
	auto landed = [&] ()
	{
		constexpr int PER_SLAB = (BM >= 64 ? BM / 64 : 1) + (BN >= 64 ? BN / 64 : 1);
		static_assert(PER_SLAB < 16, "the count is written into four bits");
		__builtin_amdgcn_s_waitcnt(0x0070 | PER_SLAB); // vmcnt(PER_SLAB) lgkmcnt(0)
		__syncthreads();
	};
	const uint32_t nslabs = (k_end - k_begin) / BK;
	// past the end the last slab is fetched again and never used
	auto slab_at = [&] (uint32_t s) -> uint32_t { return k_begin + (s < nslabs ? s : nslabs - 1) * BK; };
	issue(slab_at(0), As0, Bs0);
	issue(slab_at(1), As1, Bs1);
	landed();
	uint32_t s = 0;
	for (; s + 3 <= nslabs; s += 3)
	{
		issue(slab_at(s + 2), As2, Bs2);
		multiply(As0, Bs0);
		landed();
		issue(slab_at(s + 3), As0, Bs0);
		multiply(As1, Bs1);
		landed();
		issue(slab_at(s + 4), As1, Bs1);
		multiply(As2, Bs2);
		landed();
	}
	if (s < nslabs)
	{
		issue(slab_at(s + 2), As2, Bs2);
		multiply(As0, Bs0);
		landed();
		if (s + 1 < nslabs) { multiply(As1, Bs1); }
	}
	// nothing of this workgroup's is on its way into LDS when it ends
	__builtin_amdgcn_s_waitcnt(0);

#pragma unroll
	for (int i = 0; i < TM; ++i)
	{
#pragma unroll
		for (int j = 0; j < TN; ++j)
		{
			const uint32_t n = n0 + wn * WN + j * 32 + l32;
			if (n >= g.N) { continue; }
#pragma unroll
			for (int r = 0; r < 16; ++r)
			{
				const uint32_t m = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
				if (m < g.M) { C[(int64_t) m * ldc + n] = acc[i][j][r]; }
			}
		}
	}
}

// C[b][m][n] = partial[0][b][m][n] + partial[1][b][m][n] + ... in that order
__global__ __launch_bounds__(256) void gemm_split_sum_k (const float* __restrict__ partial, float* __restrict__ C,
	uint32_t splits, uint32_t M, uint32_t N, uint32_t batch, int64_t ldc, int64_t batch_c)
{
	const uint64_t per_split = (uint64_t) batch * M * N;
	const uint64_t step = (uint64_t) gridDim.x * 256;
	for (uint64_t i = (uint64_t) blockIdx.x * 256 + threadIdx.x; i < per_split; i += step)
	{
		float acc = partial[i];
		for (uint32_t s = 1; s < splits; ++s) { acc += partial[s * per_split + i]; }
		const uint32_t n = (uint32_t) (i % N);
		const uint64_t bm = i / N;
		const uint32_t m = (uint32_t) (bm % M);
		const uint64_t b = bm / M;
		C[b * batch_c + (int64_t) m * ldc + n] = acc;
	}
}

// the same sums for a densely stored C, four elements per lane
__global__ __launch_bounds__(256) void gemm_split_sum_vec_k (const f32x4v* __restrict__ partial,
	f32x4v* __restrict__ C, uint32_t splits, uint64_t per_split_vec)
{
	const uint64_t step = (uint64_t) gridDim.x * 256;
	for (uint64_t i = (uint64_t) blockIdx.x * 256 + threadIdx.x; i < per_split_vec; i += step)
	{
		f32x4v acc = partial[i];
		// eight loads in flight, added in range order
		for (uint32_t s0 = 1; s0 < splits; s0 += 8)
		{
			f32x4v v[8];
#pragma unroll
			for (uint32_t j = 0; j < 8; ++j)
			{
				if (s0 + j < splits) { v[j] = partial[(s0 + j) * per_split_vec + i]; }
			}
#pragma unroll
			for (uint32_t j = 0; j < 8; ++j)
			{
				if (s0 + j < splits) { acc += v[j]; }
			}
		}
		C[i] = acc;
	}
}

// Many ranges over few results (a sliver of a result under a very long K): a
// wave per group of four results; lane l adds the ranges l, l + 64, ... in
// that order, then the 64 lane sums meet in a fixed tree
__global__ __launch_bounds__(256) void gemm_split_sum_wave_k (const f32x4v* __restrict__ partial,
	f32x4v* __restrict__ C, uint32_t splits, uint64_t per_split_vec)
{
	const uint64_t i = (uint64_t) blockIdx.x * 4 + (threadIdx.x >> 6);
	const uint32_t lane = threadIdx.x & 63;
	if (i >= per_split_vec) { return; }
	f32x4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
	for (uint32_t s = lane; s < splits; s += 64) { acc += partial[s * per_split_vec + i]; }
#pragma unroll
	for (int w = 32; w >= 1; w >>= 1)
	{
#pragma unroll
		for (int e = 0; e < 4; ++e) { acc[e] += __shfl_xor(acc[e], w, 64); }
	}
	if (lane == 0) { C[i] = acc; }
}

// `ranges_out`: the K ranges stay side by side there ([range][batch][M][N]) and nothing adds them up
// DIRECT: gemm_mfma_direct_k (plain operands, K a whole number of slabs)
template <int BM, int BN, int WGM, int IMPL, typename SEGS = NoSegs, int AHEAD = 1, bool DIRECT = false>
int launch (tcg_ctx* ctx, const GemmArgs& base, uint64_t batch, int trans_a, int trans_b, uint32_t splits = 1,
	const SEGS& segs = SEGS(), float* ranges_out = nullptr)
{
	GemmArgs g = base;
	uint64_t tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
	uint64_t total = tiles_m * tiles_n * batch;
	TCG_REQUIRE(ctx, total < (1ull << 31), "tcg_gemm: too many tiles for one launch");
	g.tiles_m = (uint32_t) tiles_m;
	g.tiles_n = (uint32_t) tiles_n;
	g.tiles_per_batch = (uint32_t) (tiles_m * tiles_n);
	g.total_tiles = (uint32_t) total;
	g.k_per_split = g.K;
	g.partial = nullptr;
	size_t partial_bytes = 0;
	if (splits > 1)
	{
		// ranges are whole slabs; the last one may be shorter
		g.k_per_split = ((g.K + splits - 1) / splits + BK - 1) / BK * BK;
		splits = (g.K + g.k_per_split - 1) / g.k_per_split;
	}
	if (ranges_out)
	{
		TCG_REQUIRE(ctx, splits > 1 && total * splits < (1ull << 31), "tcg_gemm: %u ranges of K", splits);
		g.partial = ranges_out;
	}
	else if (splits > 1)
	{
		TCG_REQUIRE(ctx, total * splits < (1ull << 31), "tcg_gemm: too many tiles for one launch");
		partial_bytes = sizeof(float) * splits * batch * g.M * g.N;
		void* buf = nullptr;
		int rc = tcg_alloc(ctx, partial_bytes, &buf);
		if (rc != TCG_OK) { return rc; }
		g.partial = (float*) buf;
	}
	else { splits = 1; }
	// (Few tiles under many ranges -- the kernel gradient of a convolution, 13 tiles x 39
	// ranges, whose counters show 172 MiB fetched for 22 MiB of operands because the
	// tiles of a range land on all eight XCDs: sending the tiles of one range to one XCD
	// instead took 100 us against 66; thirteen CUs then ask one L2 for the same lines at
	// the same time.)
	const unsigned grid = g.total_tiles * splits;
	if constexpr (DIRECT)
	{
		if constexpr (IMPL != 0)
		{
			// (the caller has seen to it that a K range fits the table in LDS)
			if (trans_b) { return tcg_fail(ctx, TCG_ERR_ARG, "gemm_mfma: a convolution's B operand is row-major"); }
			if (!trans_a) { gemm_mfma_direct_k<BM,BN,false,false,SEGS,IMPL,WGM><<<grid, 256, 0, ctx->stream>>>(g, segs); }
			else { gemm_mfma_direct_k<BM,BN,true,false,SEGS,IMPL,WGM><<<grid, 256, 0, ctx->stream>>>(g, segs); }
		}
		else if (!trans_a && !trans_b) { gemm_mfma_direct_k<BM,BN,false,false,SEGS,0,WGM><<<grid, 256, 0, ctx->stream>>>(g, segs); }
		else if (trans_a && !trans_b) { gemm_mfma_direct_k<BM,BN,true,false,SEGS,0,WGM><<<grid, 256, 0, ctx->stream>>>(g, segs); }
		else if (!trans_a) { gemm_mfma_direct_k<BM,BN,false,true,SEGS,0,WGM><<<grid, 256, 0, ctx->stream>>>(g, segs); }
		else { gemm_mfma_direct_k<BM,BN,true,true,SEGS,0,WGM><<<grid, 256, 0, ctx->stream>>>(g, segs); }
	}
	else
	{
		static_assert(DIRECT || std::is_same<SEGS,NoSegs>::value, "sums over terms take the direct kernel");
		if (!trans_a && !trans_b) { gemm_mfma_k<BM,BN,WGM,false,false,IMPL,AHEAD><<<grid, 256, 0, ctx->stream>>>(g); }
		else if (trans_a && !trans_b) { gemm_mfma_k<BM,BN,WGM,true,false,IMPL,AHEAD><<<grid, 256, 0, ctx->stream>>>(g); }
		else if constexpr (IMPL == 0)
		{
			if (!trans_a) { gemm_mfma_k<BM,BN,WGM,false,true,0><<<grid, 256, 0, ctx->stream>>>(g); }
			else { gemm_mfma_k<BM,BN,WGM,true,true,0><<<grid, 256, 0, ctx->stream>>>(g); }
		}
		else { return tcg_fail(ctx, TCG_ERR_ARG, "gemm_mfma: a convolution's B operand is row-major"); }
	}
	if (g.partial && !ranges_out)
	{
		uint64_t n = batch * g.M * g.N;
		bool dense = g.ldc == (int64_t) g.N && (batch == 1 || g.batch_c == (int64_t) g.M * g.N);
		if (dense && n % 4 == 0 && tcg_aligned16(g.C) && splits >= 32 && n / 4 <= 16384)
		{
			gemm_split_sum_wave_k<<<(unsigned) ((n / 4 + 3) / 4), 256, 0, ctx->stream>>>((const f32x4v*) g.partial,
				(f32x4v*) g.C, splits, n / 4);
		}
		else if (dense && n % 4 == 0 && tcg_aligned16(g.C))
		{
			unsigned rgrid = tcg_grid(ctx, n / 4, 256, 8);
			gemm_split_sum_vec_k<<<rgrid, 256, 0, ctx->stream>>>((const f32x4v*) g.partial, (f32x4v*) g.C, splits, n / 4);
		}
		else
		{
			unsigned rgrid = tcg_grid(ctx, n, 256, 8);
			gemm_split_sum_k<<<rgrid, 256, 0, ctx->stream>>>(g.partial, g.C, splits, g.M, g.N, (uint32_t) batch, g.ldc, g.batch_c);
		}
		tcg_free(ctx, g.partial, partial_bytes);
	}
	TCG_LAUNCH_CHECK(ctx, "gemm_mfma");
	return TCG_OK;
}

// Few results under a long K (the products of a recurrent layer's time steps:
// a batch of a few hundred rows): small tiles so that the grid covers the
// chip, and the four waves of a workgroup split K between them instead of
// splitting the tile.  TMW x TNW waves tile the (32 TMW) x (32 TNW) results,
// KW waves share each 32 x 32 block: in every round the workgroup stages
// 16 KW columns of K and wave q multiplies columns [16 q, 16 q + 16) of them.
// At the end the KW partial blocks meet in LDS and are added in wave order, so
// the sum does not depend on scheduling and no second kernel is needed.
template <int TMW, int TNW, int KW, int KPW, bool TA, bool TB, typename SEGS = NoSegs>
__global__ __launch_bounds__(64 * TMW * TNW * KW) void gemm_mfma_kw_k (GemmArgs g, SEGS segs)
{
	constexpr bool SEG = !std::is_same<SEGS,NoSegs>::value;
	constexpr int NT = 64 * TMW * TNW * KW; // threads of a workgroup
	static_assert(NT == 256 || NT == 512, "four or eight waves");
	constexpr int BM = 32 * TMW, BN = 32 * TNW, BKW = KPW * KW;
	constexpr int KP = BKW + 4;
	constexpr int AP = TA ? BM + 4 : KP;
	constexpr int BP = TB ? KP : BN + 4;
	constexpr int A_SIZE = TA ? BKW * AP : BM * AP;
	constexpr int B_SIZE = TB ? BN * BP : BKW * BP;
	constexpr int A_CHUNKS = BM * BKW / 4, B_CHUNKS = BN * BKW / 4;
	constexpr int A_VEC = (A_CHUNKS + NT - 1) / NT, B_VEC = (B_CHUNKS + NT - 1) / NT;
	constexpr int RED = (KW - 1) * TMW * TNW * 1024; // partial blocks parked for the final sum
	constexpr int STAGE = 2 * (A_SIZE + B_SIZE);
	__shared__ __attribute__((aligned(16))) float lds[STAGE > RED ? STAGE : RED];

	uint32_t id = blockIdx.x;
	if (g.total_tiles % NXCD == 0) { id = (id % NXCD) * (g.total_tiles / NXCD) + id / NXCD; }
	const uint32_t bz = id / g.tiles_per_batch;
	const uint32_t t = id - bz * g.tiles_per_batch;
	const uint32_t tm = t % g.tiles_m, tn = t / g.tiles_m;
	const uint32_t m0 = tm * BM, n0 = tn * BN;
	const float* __restrict__ Abase = g.A + (int64_t) bz * g.batch_a;
	const float* __restrict__ Bbase = g.B + (int64_t) bz * g.batch_b;
	float* __restrict__ C = g.C + (int64_t) bz * g.batch_c;

	const int tid = threadIdx.x;
	const int lane = tid & 63, wave = tid >> 6;
	const int wk = wave % KW, wt = wave / KW;
	const int wm = wt / TNW, wn = wt % TNW;
	const int l32 = lane & 31, lh = lane >> 5;

	f32x16 acc;
#pragma unroll
	for (int r = 0; r < 16; ++r) { acc[r] = 0.0f; }
	f32x4v ra[A_VEC], rb[B_VEC];
	const f32x4v zero4 = {0.0f, 0.0f, 0.0f, 0.0f};

	auto load_round = [&] (uint32_t k0)
	{
		// with terms: a round never straddles two of them (their depth is a multiple of a round's)
		const float* __restrict__ A = Abase;
		const float* __restrict__ B = Bbase;
		uint32_t kfirst = 0;
		int64_t lda = g.lda, ldb = g.ldb;
		if constexpr (SEG)
		{
			const uint32_t term = k0 / segs.k;
			A = segs.a[term];
			B = segs.b[term];
			lda = segs.lda[term];
			ldb = segs.ldb[term];
			kfirst = term * segs.k;
		}
#pragma unroll
		for (int v = 0; v < A_VEC; ++v)
		{
			int idx = tid + v * NT;
			if (A_CHUNKS % NT != 0 && idx >= A_CHUNKS) { break; }
			if constexpr (!TA)
			{
				int mm = idx / (BKW / 4), kq = idx % (BKW / 4);
				uint32_t m = m0 + mm, k = k0 + kq * 4;
				ra[v] = (m < g.M && k < g.K) ? *reinterpret_cast<const f32x4v*>(A + (int64_t) m * lda + (k - kfirst)) : zero4;
			}
			else
			{
				int kk = idx / (BM / 4), mq = idx % (BM / 4);
				uint32_t m = m0 + mq * 4, k = k0 + kk;
				ra[v] = (m < g.M && k < g.K) ? *reinterpret_cast<const f32x4v*>(A + (int64_t) (k - kfirst) * lda + m) : zero4;
			}
		}
#pragma unroll
		for (int v = 0; v < B_VEC; ++v)
		{
			int idx = tid + v * NT;
			if (B_CHUNKS % NT != 0 && idx >= B_CHUNKS) { break; }
			if constexpr (!TB)
			{
				int kk = idx / (BN / 4), nq = idx % (BN / 4);
				uint32_t n = n0 + nq * 4, k = k0 + kk;
				rb[v] = (n < g.N && k < g.K) ? *reinterpret_cast<const f32x4v*>(B + (int64_t) (k - kfirst) * ldb + n) : zero4;
			}
			else
			{
				int nn = idx / (BKW / 4), kq = idx % (BKW / 4);
				uint32_t n = n0 + nn, k = k0 + kq * 4;
				rb[v] = (n < g.N && k < g.K) ? *reinterpret_cast<const f32x4v*>(B + (int64_t) n * ldb + (k - kfirst)) : zero4;
			}
		}
	};

	auto store_round = [&] (int buf)
	{
		float* as = lds + buf * A_SIZE;
		float* bs = lds + 2 * A_SIZE + buf * B_SIZE;
#pragma unroll
		for (int v = 0; v < A_VEC; ++v)
		{
			int idx = tid + v * NT;
			if (A_CHUNKS % NT != 0 && idx >= A_CHUNKS) { break; }
			if constexpr (!TA)
			{
				int mm = idx / (BKW / 4), kq = idx % (BKW / 4);
				*reinterpret_cast<f32x4v*>(as + mm * AP + kq * 4) = ra[v];
			}
			else
			{
				int kk = idx / (BM / 4), mq = idx % (BM / 4);
				*reinterpret_cast<f32x4v*>(as + kk * AP + mq * 4) = ra[v];
			}
		}
#pragma unroll
		for (int v = 0; v < B_VEC; ++v)
		{
			int idx = tid + v * NT;
			if (B_CHUNKS % NT != 0 && idx >= B_CHUNKS) { break; }
			if constexpr (!TB)
			{
				int kk = idx / (BN / 4), nq = idx % (BN / 4);
				*reinterpret_cast<f32x4v*>(bs + kk * BP + nq * 4) = rb[v];
			}
			else
			{
				int nn = idx / (BKW / 4), kq = idx % (BKW / 4);
				*reinterpret_cast<f32x4v*>(bs + nn * BP + kq * 4) = rb[v];
			}
		}
	};

	const uint32_t rounds = (g.K + BKW - 1) / BKW;
	load_round(0);
	store_round(0);
	__syncthreads();
	for (uint32_t s = 0; s < rounds; ++s)
	{
		const int buf = s & 1;
		if (s + 1 < rounds) { load_round((s + 1) * BKW); }
		const float* as = lds + buf * A_SIZE;
		const float* bs = lds + 2 * A_SIZE + buf * B_SIZE;
		const int row = wm * 32 + l32, col = wn * 32 + l32;
#pragma unroll
		for (int half = 0; half < KPW / 8; ++half)
		{
			const int kb = wk * KPW + half * 8 + lh * 4; // this lane's four k of these eight
			f32x4v a, b;
			if constexpr (!TA) { a = *reinterpret_cast<const f32x4v*>(as + row * AP + kb); }
			else
			{
#pragma unroll
				for (int e = 0; e < 4; ++e) { a[e] = as[(kb + e) * AP + row]; }
			}
			if constexpr (TB) { b = *reinterpret_cast<const f32x4v*>(bs + col * BP + kb); }
			else
			{
#pragma unroll
				for (int e = 0; e < 4; ++e) { b[e] = bs[(kb + e) * BP + col]; }
			}
#pragma unroll
			for (int e = 0; e < 4; ++e) { acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], acc, 0, 0, 0); }
		}
		if (s + 1 < rounds) { store_round(buf ^ 1); }
		__syncthreads();
	}

	// the KW partial blocks of each 32 x 32 block: waves 1.. park theirs, wave 0 adds them in order
	if constexpr (KW > 1)
	{
		if (wk > 0)
		{
			float* park = lds + ((wt * (KW - 1) + (wk - 1)) * 1024);
#pragma unroll
			for (int r = 0; r < 16; ++r) { park[r * 64 + lane] = acc[r]; }
		}
		__syncthreads();
		if (wk == 0)
		{
#pragma unroll
			for (int q = 1; q < KW; ++q)
			{
				const float* park = lds + ((wt * (KW - 1) + (q - 1)) * 1024);
#pragma unroll
				for (int r = 0; r < 16; ++r) { acc[r] += park[r * 64 + lane]; }
			}
		}
	}
	if (wk == 0)
	{
		// lane holds column l32; register r is row 8*(r/4) + 4*lh + r%4 of the 32x32 block
		const uint32_t n = n0 + wn * 32 + l32;
		if (n < g.N)
		{
#pragma unroll
			for (int r = 0; r < 16; ++r)
			{
				const uint32_t m = m0 + wm * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
				if (m < g.M) { C[(int64_t) m * g.ldc + n] = acc[r]; }
			}
		}
	}
}

template <int TMW, int TNW, int KW, int KPW, typename SEGS = NoSegs>
int launch_kw (tcg_ctx* ctx, const GemmArgs& base, uint64_t batch, int trans_a, int trans_b, const SEGS& segs = SEGS())
{
	GemmArgs g = base;
	constexpr int BM = 32 * TMW, BN = 32 * TNW, NT = 64 * TMW * TNW * KW;
	uint64_t tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
	uint64_t total = tiles_m * tiles_n * batch;
	TCG_REQUIRE(ctx, total < (1ull << 31), "tcg_gemm: too many tiles for one launch");
	g.tiles_m = (uint32_t) tiles_m;
	g.tiles_n = (uint32_t) tiles_n;
	g.tiles_per_batch = (uint32_t) (tiles_m * tiles_n);
	g.total_tiles = (uint32_t) total;
	g.k_per_split = g.K;
	g.partial = nullptr;
	const unsigned grid = g.total_tiles;
	if (!trans_a && !trans_b) { gemm_mfma_kw_k<TMW,TNW,KW,KPW,false,false,SEGS><<<grid, NT, 0, ctx->stream>>>(g, segs); }
	else if (trans_a && !trans_b) { gemm_mfma_kw_k<TMW,TNW,KW,KPW,true,false,SEGS><<<grid, NT, 0, ctx->stream>>>(g, segs); }
	else if (!trans_a) { gemm_mfma_kw_k<TMW,TNW,KW,KPW,false,true,SEGS><<<grid, NT, 0, ctx->stream>>>(g, segs); }
	else { gemm_mfma_kw_k<TMW,TNW,KW,KPW,true,true,SEGS><<<grid, NT, 0, ctx->stream>>>(g, segs); }
	TCG_LAUNCH_CHECK(ctx, "gemm_mfma_kw");
	return TCG_OK;
}

// How many ranges of K for `tiles` large tiles: the fewest that put at least
// two workgroups on every CU and leave the last round of workgroups at least
// nine tenths full (96 tiles on 256 CUs: 6 ranges make 2.25 rounds, of which
// the last quarter runs alone; 8 make three full ones), every range keeping
// 256 summed indices
uint32_t ranges_for_tiles (uint64_t tiles, uint64_t cus, uint64_t depth)
{
	uint64_t most = depth / 256 < 32 ? depth / 256 : 32;
	if (most < 2 || tiles >= 2 * cus) { return 1; }
	uint64_t best = 1;
	double best_fill = 0.0;
	for (uint64_t r = 2; r <= most; ++r)
	{
		uint64_t groups = tiles * r;
		if (groups < 2 * cus && r < most) { continue; }
		uint64_t rounds = (groups + cus - 1) / cus;
		double fill = (double) groups / (double) (rounds * cus);
		if (fill >= 0.9) { return (uint32_t) r; }
		if (fill > best_fill)
		{
			best_fill = fill;
			best = r;
		}
	}
	return (uint32_t) best;
}

// Tile shapes by problem shape
template <int IMPL>
int dispatch (tcg_ctx* ctx, const GemmArgs& g, uint64_t batch, int trans_a, int trans_b)
{
	const uint64_t M = g.M, N = g.N, K = g.K;
	// narrow results (the column count of a convolution lowered to a product is
	// its channel count): tiles as wide as N, so that no lane multiplies padding
	const uint64_t cus = (uint64_t) ctx->num_cus;
	// a convolution's operand read through its tables: two slabs on their way (64-column
	// products 91 -> 84 us, 32-column 111 -> 106, kernel gradient 96 -> 76); plain operands
	// gain nothing from it (4096^3, and the products of a recurrent layer's steps)
	constexpr int AHEAD = IMPL == 1 ? 2 : 1;
	if (N <= 32 && (M + 127) / 128 * batch >= cus)
	{
		if ((M + 255) / 256 * batch >= 2 * cus) { return launch<256,32,4,IMPL,NoSegs,AHEAD>(ctx, g, batch, trans_a, trans_b); }
		// two workgroups per CU hide little of a slab's load latency behind its eight
		// matrix instructions per wave: up to four ranges of a long K fill the CUs
		// (the image gradient of a convolution, 73728 x 32 x 1600: 156 -> 111 + 10 us)
		uint64_t ranges = (M + 127) / 128 * batch < 4 * cus ? 4 : 1;
		if (ranges > K / 256) { ranges = K / 256; }
		if (ranges < 2 || batch != 1) { ranges = 1; }
		// plain operands under a K of whole slabs go straight into LDS here too (73728 x 32 x 1600:
		// 147 -> 139 us); the gathering form of this tile gains nothing from it and stays as it is
		if constexpr (IMPL == 0)
		{
			if (K % BK == 0 && M >= 4 && N >= 4) { return launch<128,32,4,0,NoSegs,1,true>(ctx, g, batch, trans_a, trans_b, (uint32_t) ranges); }
		}
		return launch<128,32,4,IMPL,NoSegs,AHEAD>(ctx, g, batch, trans_a, trans_b, (uint32_t) ranges);
	}
	// plain operands under a K of whole slabs go from memory straight into LDS (4096^3:
	// 129 -> 136 TFLOP/s, 51200 x 64 x 800: 72 -> 65 us, 512 x 4096 x 1024: 53 -> 45 us);
	// rows and columns past the edge are read from the last four inside
	const bool direct = IMPL == 0 && K % BK == 0 && M >= 4 && N >= 4;
	if (N <= 64 && (M + 127) / 128 * batch >= cus)
	{
		if constexpr (IMPL == 0)
		{
			if (direct) { return launch<128,64,2,0,NoSegs,1,true>(ctx, g, batch, trans_a, trans_b); }
		}
		else
		{
			// the gathered operand goes straight into LDS as well when the table entries of K
			// fit beside the slabs (a 5 x 5 x 32 convolution forwards: 84 -> 71 us)
			if (K % BK == 0 && K <= (uint64_t) direct_tab(128, 64) && M >= 4 && N >= 4 && batch == 1)
			{
				return launch<128,64,2,1,NoSegs,1,true>(ctx, g, batch, trans_a, trans_b);
			}
		}
		return launch<128,64,2,IMPL,NoSegs,AHEAD>(ctx, g, batch, trans_a, trans_b);
	}
	// small problems: smaller tiles so that the grid still covers the chip
	uint64_t big_tiles = ((M + 127) / 128) * ((N + 127) / 128) * batch;
	auto large = [&] (uint32_t ranges)
	{
		if constexpr (IMPL == 0)
		{
			if (direct) { return launch<128,128,2,0,NoSegs,1,true>(ctx, g, batch, trans_a, trans_b, ranges); }
		}
		return launch<128,128,2,IMPL,NoSegs,AHEAD>(ctx, g, batch, trans_a, trans_b, ranges);
	};
	if (big_tiles >= 2 * cus) { return large(1); }
	// fewer large tiles than two per CU under a long K: ranges of K chosen so that the
	// workgroups come in full rounds (768 x 2048 x 16384: 72 -> 110 TFLOP/s, 1024 x 1024 x 4096:
	// 63 -> 85, 512 x 512 x 8192: 57 -> 76; with K = 1024 the small tiles below stay ahead)
	if (big_tiles >= 16 && K >= 1536 && batch < (1ull << 16))
	{
		// (a single full round of tiles that go straight into LDS needs no ranges)
		if (direct && big_tiles == cus) { return large(1); }
		return large(ranges_for_tiles(big_tiles, cus, K));
	}
	if (big_tiles >= cus) { return large(1); }
	// still too few tiles for the chip and a long K: several workgroups share a
	// tile, each summing a range of K, and a second kernel adds the ranges up
	// in a fixed order (so that results do not depend on scheduling)
	uint64_t tiles = ((M + 63) / 64) * ((N + 63) / 64) * batch;
	uint64_t splits = 2 * (uint64_t) ctx->num_cus / tiles;
	if (splits > K / 64) { splits = K / 64; }
	// a sliver of a result under a very long K (the kernel gradient of a
	// convolution's first layer: 25 x 32 results, K = 73728) may take a
	// workgroup per CU and more, as long as every range keeps 256 summed indices
	uint64_t cap = K / 256 > 32 ? K / 256 : 32;
	if (cap > 256) { cap = 256; }
	if (splits > cap) { splits = cap; }
	if (splits < 2 || batch >= (1ull << 16)) { splits = 1; }
	if constexpr (IMPL == 0)
	{
		// row-major operands with enough 32 x 32 blocks for the chip: the waves of a
		// workgroup share K between them and no second kernel adds ranges up
		// (256 x 2048 x 768: 13.9 us against 19.3 us for both kernels of the split form;
		// with a transposed operand the split form stays ahead)
		if (!trans_a && !trans_b && splits >= 2 && K >= 256 && ((M + 31) / 32) * ((N + 31) / 32) * batch >= cus)
		{
			return launch_kw<1,1,4,32>(ctx, g, batch, trans_a, trans_b);
		}
	}
	if constexpr (IMPL == 0)
	{
		if (direct) { return launch<64,64,2,0,NoSegs,1,true>(ctx, g, batch, trans_a, trans_b, (uint32_t) splits); }
	}
	else
	{
		// a K range is K / splits rounded up to whole slabs (the kernel gradient of that
		// convolution, 800 x 64 x 51200 in 39 ranges: 76 -> 65 us)
		uint64_t range = ((K + splits - 1) / splits + BK - 1) / BK * BK;
		if (K % BK == 0 && range <= (uint64_t) direct_tab(64, 64) && M >= 4 && N >= 4 && batch == 1)
		{
			return launch<64,64,2,1,NoSegs,1,true>(ctx, g, batch, trans_a, trans_b, (uint32_t) splits);
		}
	}
	return launch<64,64,2,IMPL,NoSegs,AHEAD>(ctx, g, batch, trans_a, trans_b, (uint32_t) splits);
}

} // namespace

int tcg_gemm_f32_mfma (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t K, uint64_t batch,
	const float* A, uint64_t lda, uint64_t stride_a, int trans_a,
	const float* B, uint64_t ldb, uint64_t stride_b, int trans_b,
	float* C, uint64_t ldc, uint64_t stride_c, bool* handled)
{
	*handled = false;
	// 128-bit operand loads: every row start and every slab offset must be
	// 16-byte aligned; anything else goes to the generic kernel
	// (a sliver of a tile still pays when K is long: the K ranges spread it over the chip)
	bool ok = M >= 8 && N >= 8 && K >= 8 && ((M >= 32 && N >= 32) || K >= 512) &&
		M < (1ull << 31) && N < (1ull << 31) && K < (1ull << 31) &&
		tcg_aligned16(A) && tcg_aligned16(B) &&
		lda % 4 == 0 && ldb % 4 == 0 && stride_a % 4 == 0 && stride_b % 4 == 0 &&
		((trans_a ? M : K) % 4 == 0) && ((trans_b ? K : N) % 4 == 0);
	if (!ok) { return TCG_OK; }
	GemmArgs g;
	g.A = A; g.B = B; g.C = C;
	g.M = (uint32_t) M; g.N = (uint32_t) N; g.K = (uint32_t) K;
	g.lda = (int64_t) lda; g.ldb = (int64_t) ldb; g.ldc = (int64_t) ldc;
	g.batch_a = (int64_t) stride_a; g.batch_b = (int64_t) stride_b; g.batch_c = (int64_t) stride_c;
	g.tiles_m = g.tiles_n = g.tiles_per_batch = g.total_tiles = 0;
	g.rows = g.sums = nullptr;
	g.zeros = nullptr;
	g.ncheck = 0;
	*handled = true;
	return dispatch<0>(ctx, g, batch, trans_a, trans_b);
}

// C[m][n] = sum_t sum_k A_t[m][k] B_t[k][n]: `terms` products of one shape
// (K columns each, same layouts; each term with its own leading dims) as one
// product of depth terms * K; *handled = false when the shapes do not fit
int tcg_gemm_f32_mfma_terms (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t K, uint32_t terms,
	const float* const* A, const uint64_t* lda, int trans_a, const float* const* B, const uint64_t* ldb, int trans_b,
	float* C, uint64_t ldc, bool* handled)
{
	*handled = false;
	bool ok = terms >= 1 && terms <= (uint32_t) MAX_TERMS && M >= 32 && N >= 32 && K >= BK && K % BK == 0 &&
		M < (1ull << 31) && N < (1ull << 31) && K * terms < (1ull << 31) &&
		((trans_a ? M : K) % 4 == 0) && ((trans_b ? K : N) % 4 == 0);
	for (uint32_t t = 0; t < terms && ok; ++t)
	{
		ok = tcg_aligned16(A[t]) && tcg_aligned16(B[t]) && lda[t] % 4 == 0 && ldb[t] % 4 == 0 &&
			lda[t] < (1ull << 32) && ldb[t] < (1ull << 32);
	}
	if (!ok) { return TCG_OK; }
	GemmArgs g;
	g.A = A[0]; g.B = B[0]; g.C = C;
	g.M = (uint32_t) M; g.N = (uint32_t) N; g.K = (uint32_t) (K * terms);
	g.lda = (int64_t) lda[0]; g.ldb = (int64_t) ldb[0]; g.ldc = (int64_t) ldc;
	g.batch_a = g.batch_b = g.batch_c = 0;
	g.tiles_m = g.tiles_n = g.tiles_per_batch = g.total_tiles = 0;
	g.rows = g.sums = nullptr;
	g.zeros = nullptr;
	g.ncheck = 0;
	GemmSegs segs;
	segs.k = (uint32_t) K;
	for (uint32_t t = 0; t < terms; ++t)
	{
		segs.a[t] = A[t];
		segs.b[t] = B[t];
		segs.lda[t] = (uint32_t) lda[t];
		segs.ldb[t] = (uint32_t) ldb[t];
	}
	*handled = true;
	// few results (a time step of a recurrent layer): the waves of a workgroup share K
	const uint64_t cus = (uint64_t) ctx->num_cus;
	if (!trans_a && !trans_b && K % 128 == 0 && g.K >= 256 && ((M + 31) / 32) * ((N + 31) / 32) >= cus &&
		((M + 127) / 128) * ((N + 127) / 128) < cus)
	{
		return launch_kw<1,1,4,32,GemmSegs>(ctx, g, 1, trans_a, trans_b, segs);
	}
	// large tiles; ranges of the long summed index spread the tiles over the chip
	uint64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
	if (tiles * (g.K / 256 < 32 ? g.K / 256 : 32) < cus)
	{
		// not enough of them even so: smaller tiles, ranges as for a plain product of this shape
		uint64_t small = ((M + 63) / 64) * ((N + 63) / 64);
		uint64_t ranges = 2 * cus / small;
		if (ranges > g.K / 64) { ranges = g.K / 64; }
		if (ranges > 32) { ranges = 32; }
		if (ranges < 2) { ranges = 1; }
		return launch<64,64,2,0,GemmSegs,1,true>(ctx, g, 1, trans_a, trans_b, (uint32_t) ranges, segs);
	}
	return launch<128,128,2,0,GemmSegs,1,true>(ctx, g, 1, trans_a, trans_b, ranges_for_tiles(tiles, cus, g.K), segs);
}

// C = the mparts x nparts blocks sum_t A[i][t] B[j][t] as one product of
// (sum of the parts' rows) x (sum of the parts' columns) x (terms * K)
int tcg_gemm_f32_mfma_grid (tcg_ctx* ctx, uint32_t mparts, const uint64_t* Mp, uint32_t nparts, const uint64_t* Np,
	uint64_t K, uint32_t terms, const float* const* A, const uint64_t* lda, int trans_a,
	const float* const* B, const uint64_t* ldb, int trans_b, float* C, uint64_t ldc, bool* handled)
{
	*handled = false;
	bool ok = mparts >= 1 && mparts <= (uint32_t) MAX_GRID_MPARTS && nparts >= 1 && nparts <= (uint32_t) MAX_GRID_NPARTS &&
		terms >= 1 && (uint64_t) (mparts + nparts) * terms <= (uint64_t) MAX_GRID_PTRS &&
		K >= BK && K % BK == 0 && K * terms < (1ull << 31) && ldc % 4 == 0 && tcg_aligned16(C);
	uint64_t M = 0, N = 0;
	GemmGrid grid;
	for (uint32_t i = 0; i < mparts && ok; ++i)
	{
		ok = Mp[i] >= 128 && Mp[i] % 128 == 0 && lda[i] % 4 == 0 && lda[i] < (1ull << 32);
		grid.mstart[i] = (uint32_t) M;
		grid.lda[i] = (uint32_t) lda[i];
		M += Mp[i];
		for (uint32_t t = 0; t < terms && ok; ++t)
		{
			ok = tcg_aligned16(A[i * terms + t]);
			grid.ptr[i * terms + t] = A[i * terms + t];
		}
	}
	for (uint32_t j = 0; j < nparts && ok; ++j)
	{
		ok = Np[j] >= 128 && Np[j] % 128 == 0 && ldb[j] % 4 == 0 && ldb[j] < (1ull << 32);
		grid.nstart[j] = (uint32_t) N;
		grid.ldb[j] = (uint32_t) ldb[j];
		N += Np[j];
		for (uint32_t t = 0; t < terms && ok; ++t)
		{
			ok = tcg_aligned16(B[j * terms + t]);
			grid.ptr[(mparts + j) * terms + t] = B[j * terms + t];
		}
	}
	ok = ok && M < (1ull << 31) && N < (1ull << 31) && ldc >= N;
	if (!ok) { return TCG_OK; }
	grid.mstart[mparts] = (uint32_t) M;
	grid.nstart[nparts] = (uint32_t) N;
	grid.k = (uint32_t) K;
	grid.terms = terms;
	grid.mparts = mparts;
	grid.nparts = nparts;
	GemmArgs g;
	g.A = A[0]; g.B = B[0]; g.C = C;
	g.M = (uint32_t) M; g.N = (uint32_t) N; g.K = (uint32_t) (K * terms);
	g.lda = (int64_t) lda[0]; g.ldb = (int64_t) ldb[0]; g.ldc = (int64_t) ldc;
	g.batch_a = g.batch_b = g.batch_c = 0;
	g.tiles_m = g.tiles_n = g.tiles_per_batch = g.total_tiles = 0;
	g.rows = g.sums = nullptr;
	g.zeros = nullptr;
	g.ncheck = 0;
	*handled = true;
	const uint32_t splits = ranges_for_tiles((M / 128) * (N / 128), (uint64_t) ctx->num_cus, g.K);
	return launch<128,128,2,0,GemmGrid,1,true>(ctx, g, 1, trans_a, trans_b, splits, grid);
}

// The same sum of products with its K ranges left side by side:
// ranges[r][m][n] = sum over the r-th of `nranges` equal parts of the
// concatenated summed index; whoever reads them adds them up in range order
int tcg_gemm_f32_mfma_ranges (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t K, uint32_t terms,
	const float* const* A, const uint64_t* lda, int trans_a, const float* const* B, const uint64_t* ldb, int trans_b,
	uint32_t nranges, float* ranges, bool* handled)
{
	*handled = false;
	bool ok = terms >= 1 && terms <= (uint32_t) MAX_TERMS && M >= 32 && N >= 32 && K >= BK && K % BK == 0 &&
		M < (1ull << 31) && N < (1ull << 31) && K * terms < (1ull << 31) &&
		((trans_a ? M : K) % 4 == 0) && ((trans_b ? K : N) % 4 == 0) &&
		nranges >= 2 && nranges <= 32 && (K * terms) % ((uint64_t) nranges * BK) == 0 && tcg_aligned16(ranges);
	for (uint32_t t = 0; t < terms && ok; ++t)
	{
		ok = tcg_aligned16(A[t]) && tcg_aligned16(B[t]) && lda[t] % 4 == 0 && ldb[t] % 4 == 0 &&
			lda[t] < (1ull << 32) && ldb[t] < (1ull << 32);
	}
	if (!ok) { return TCG_OK; }
	GemmArgs g;
	g.A = A[0]; g.B = B[0]; g.C = ranges;
	g.M = (uint32_t) M; g.N = (uint32_t) N; g.K = (uint32_t) (K * terms);
	g.lda = (int64_t) lda[0]; g.ldb = (int64_t) ldb[0]; g.ldc = (int64_t) N;
	g.batch_a = g.batch_b = g.batch_c = 0;
	g.tiles_m = g.tiles_n = g.tiles_per_batch = g.total_tiles = 0;
	g.rows = g.sums = nullptr;
	g.zeros = nullptr;
	g.ncheck = 0;
	GemmSegs segs;
	segs.k = (uint32_t) K;
	for (uint32_t t = 0; t < terms; ++t)
	{
		segs.a[t] = A[t];
		segs.b[t] = B[t];
		segs.lda[t] = (uint32_t) lda[t];
		segs.ldb[t] = (uint32_t) ldb[t];
	}
	*handled = true;
	return launch<64,64,2,0,GemmSegs,1,true>(ctx, g, 1, trans_a, trans_b, nranges, segs, ranges);
}

int tcg_gemm_f32_mfma_sum (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t K, uint32_t terms,
	const float* const* A, uint64_t lda, int trans_a, const float* const* B, uint64_t ldb, int trans_b,
	float* C, uint64_t ldc, bool* handled)
{
	*handled = false;
	if (terms > (uint32_t) MAX_TERMS) { return TCG_OK; }
	uint64_t ldas[MAX_TERMS], ldbs[MAX_TERMS];
	for (uint32_t t = 0; t < terms; ++t)
	{
		ldas[t] = lda;
		ldbs[t] = ldb;
	}
	return tcg_gemm_f32_mfma_terms(ctx, M, N, K, terms, A, ldas, trans_a, B, ldbs, trans_b, C, ldc, handled);
}

int tcg_gemm_f32_mfma_conv (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t S,
	const float* image, const tcg_conv_operand& op, const float* B, uint64_t ldb,
	float* C, uint64_t ldc, bool* handled)
{
	*handled = false;
	bool ok = M >= 8 && N >= 8 && S >= 8 && ((M >= 32 && N >= 32) || S >= 512) &&
		M < (1ull << 31) && N < (1ull << 31) && S < (1ull << 31) &&
		tcg_aligned16(B) && ldb % 4 == 0 && N % 4 == 0 && op.rows && op.sums && op.ncheck >= 0 && op.ncheck <= 4 &&
		op.vec4 && tcg_aligned16(image) && (op.along_m ? M : S) % 4 == 0;
	if (!ok) { return TCG_OK; }
	GemmArgs g;
	g.A = image; g.B = B; g.C = C;
	g.M = (uint32_t) M; g.N = (uint32_t) N; g.K = (uint32_t) S;
	g.lda = 0; g.ldb = (int64_t) ldb; g.ldc = (int64_t) ldc;
	g.batch_a = g.batch_b = g.batch_c = 0;
	g.tiles_m = g.tiles_n = g.tiles_per_batch = g.total_tiles = 0;
	g.rows = op.rows;
	g.sums = op.sums;
	g.zeros = ctx->zeros;
	g.ncheck = op.ncheck;
	for (int j = 0; j < 4; ++j) { g.check_ext[j] = op.check_ext[j]; }
	*handled = true;
	return dispatch<1>(ctx, g, 1, op.along_m, 0);
}
