// fp64 GEMM on the matrix cores: C[b][m][n] = sum_k A[b][m][k] B[b][k][n].
//
// tenncor's goldens and many of its graphs are double (DOUBLE is the widest
// dtype of cfg/mintype.yml); the products behind MATMUL / CONTRACT
// (internal/eigen/operator.hpp:1069-1139) then run here.  One workgroup of 256
// lanes (4 waves, 2x2) owns a BM x BN tile of C, each wave a quarter of it built
// from 16x16 accumulators fed by v_mfma_f64_16x16x4_f64 (lane i + 16 k supplies
// A[i][k] and B[k][i]; a lane holds C[4 r + lane / 16][lane % 16], r = 0..3).
// A and B slabs of BK = 8 columns go global -> LDS directly when K is a whole
// number of slabs (dgemm_mfma_direct_k: three slabs in LDS, two on their way),
// else global -> registers -> LDS (dgemm_mfma_k: double buffered, one barrier
// per slab, both operands kept [k][row] so that the sixteen lanes of a k read
// sixteen consecutive doubles; an operand whose K runs along memory is kept
// [row][k], see the kernel).  Sums run over k in ascending order in both.
// MFMA-bound: 2*M*N*K flops against 78.6 TFLOP/s.
#include "tcg_internal.hpp"
#include <type_traits>

namespace
{

typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));

constexpr int DBK = 8;
constexpr int DNXCD = 8;
constexpr int DGROUP_M = 8;

struct DGemmArgs
{
	const double* A;
	const double* B;
	double* C;
	uint32_t M, N, K;
	int64_t lda, ldb, ldc;
	int64_t batch_a, batch_b, batch_c;
	uint32_t tiles_m, tiles_n, tiles_per_batch, total_tiles;
};

// TA: A(m,k) at m + k*lda (M contiguous) instead of m*lda + k.
// TB: B(k,n) at k + n*ldb (K contiguous) instead of k*ldb + n.
template <int BM, int BN, bool TA, bool TB>
__global__ __launch_bounds__(256) void dgemm_mfma_k (DGemmArgs g)
{
	constexpr int WM = BM / 2, WN = BN / 2;   // wave tile
	constexpr int TM = WM / 16, TN = WN / 16; // 16x16 accumulators per wave
	// pitches of the [k][row] tiles: a 64-bit read goes out in two halves of 32
	// lanes (two k, sixteen rows each), which land on disjoint banks when the
	// pitch is 32 dwords past a multiple of 64
	constexpr int AP = BM + 16, BP = BN + 16;
	constexpr int A_CHUNKS = BM * DBK / 2, B_CHUNKS = BN * DBK / 2; // double2 per slab
	constexpr int A_VEC = (A_CHUNKS + 255) / 256, B_VEC = (B_CHUNKS + 255) / 256;
	// an operand whose K runs along memory is kept [row][k] instead, pitch 10:
	// written with the 128-bit values as they were loaded, and the sixteen rows
	// times two k of a half-wave read fall on 32 distinct bank pairs
	constexpr int KP = DBK + 2;
	constexpr int A_SIZE = TA ? DBK * AP : BM * KP;
	constexpr int B_SIZE = TB ? BN * KP : DBK * BP;
	__shared__ __attribute__((aligned(16))) double As[2][A_SIZE];
	__shared__ __attribute__((aligned(16))) double Bs[2][B_SIZE];

	// workgroups resident on one XCD (ids congruent mod 8) take consecutive
	// tiles, and consecutive tiles walk down groups of eight tile rows: what an
	// XCD works on at a time is a compact patch of C whose panels its L2 holds
	uint32_t id = blockIdx.x;
	if (g.total_tiles % DNXCD == 0)
	{
		id = (id % DNXCD) * (g.total_tiles / DNXCD) + id / DNXCD;
	}
	const uint32_t bz = id / g.tiles_per_batch;
	const uint32_t t = id - bz * g.tiles_per_batch;
	const uint32_t group_size = DGROUP_M * g.tiles_n;
	const uint32_t group = t / group_size;
	const uint32_t first_m = group * DGROUP_M;
	const uint32_t rows_in_group = g.tiles_m - first_m < (uint32_t) DGROUP_M ? g.tiles_m - first_m : DGROUP_M;
	const uint32_t in_group = t - group * group_size;
	const uint32_t tm = first_m + in_group % rows_in_group;
	const uint32_t tn = in_group / rows_in_group;
	const uint32_t m0 = tm * BM, n0 = tn * BN;
	const double* __restrict__ A = g.A + (int64_t) bz * g.batch_a;
	const double* __restrict__ B = g.B + (int64_t) bz * g.batch_b;
	double* __restrict__ C = g.C + (int64_t) bz * g.batch_c;

	const int tid = threadIdx.x;
	const int lane = tid & 63, wave = tid >> 6;
	const int wm = wave >> 1, wn = wave & 1;
	const int l16 = lane & 15, lk = lane >> 4;

	f64x4 acc[TM][TN];
#pragma unroll
	for (int i = 0; i < TM; ++i)
	{
#pragma unroll
		for (int j = 0; j < TN; ++j)
		{
#pragma unroll
			for (int r = 0; r < 4; ++r) { acc[i][j][r] = 0.0; }
		}
	}

	f64x2 ra[A_VEC], rb[B_VEC];
	const f64x2 zero2 = {0.0, 0.0};

	auto load_slab = [&] (uint32_t k0)
	{
#pragma unroll
		for (int v = 0; v < A_VEC; ++v)
		{
			int idx = tid + v * 256;
			if (A_CHUNKS % 256 != 0 && idx >= A_CHUNKS) { break; }
			if constexpr (!TA)
			{
				int mm = idx / (DBK / 2), kq = idx % (DBK / 2);
				uint32_t m = m0 + mm, k = k0 + kq * 2;
				ra[v] = (m < g.M && k < g.K) ? *reinterpret_cast<const f64x2*>(A + (int64_t) m * g.lda + k) : zero2;
			}
			else
			{
				int kk = idx / (BM / 2), mq = idx % (BM / 2);
				uint32_t m = m0 + mq * 2, k = k0 + kk;
				ra[v] = (m < g.M && k < g.K) ? *reinterpret_cast<const f64x2*>(A + (int64_t) k * g.lda + m) : zero2;
			}
		}
#pragma unroll
		for (int v = 0; v < B_VEC; ++v)
		{
			int idx = tid + v * 256;
			if (B_CHUNKS % 256 != 0 && idx >= B_CHUNKS) { break; }
			if constexpr (!TB)
			{
				int kk = idx / (BN / 2), nq = idx % (BN / 2);
				uint32_t n = n0 + nq * 2, k = k0 + kk;
				rb[v] = (n < g.N && k < g.K) ? *reinterpret_cast<const f64x2*>(B + (int64_t) k * g.ldb + n) : zero2;
			}
			else
			{
				int nn = idx / (DBK / 2), kq = idx % (DBK / 2);
				uint32_t n = n0 + nn, k = k0 + kq * 2;
				rb[v] = (n < g.N && k < g.K) ? *reinterpret_cast<const f64x2*>(B + (int64_t) n * g.ldb + k) : zero2;
			}
		}
	};

	auto store_slab = [&] (int buf)
	{
		double* as = As[buf];
		double* bs = Bs[buf];
#pragma unroll
		for (int v = 0; v < A_VEC; ++v)
		{
			int idx = tid + v * 256;
			if (A_CHUNKS % 256 != 0 && idx >= A_CHUNKS) { break; }
			if constexpr (!TA)
			{
				int mm = idx / (DBK / 2), kq = idx % (DBK / 2);
				*reinterpret_cast<f64x2*>(as + mm * KP + kq * 2) = ra[v];
			}
			else
			{
				int kk = idx / (BM / 2), mq = idx % (BM / 2);
				*reinterpret_cast<f64x2*>(as + kk * AP + mq * 2) = ra[v];
			}
		}
#pragma unroll
		for (int v = 0; v < B_VEC; ++v)
		{
			int idx = tid + v * 256;
			if (B_CHUNKS % 256 != 0 && idx >= B_CHUNKS) { break; }
			if constexpr (!TB)
			{
				int kk = idx / (BN / 2), nq = idx % (BN / 2);
				*reinterpret_cast<f64x2*>(bs + kk * BP + nq * 2) = rb[v];
			}
			else
			{
				int nn = idx / (DBK / 2), kq = idx % (DBK / 2);
				*reinterpret_cast<f64x2*>(bs + nn * KP + kq * 2) = rb[v];
			}
		}
	};

	const uint32_t nslabs = (g.K + DBK - 1) / DBK;
	load_slab(0);
	store_slab(0);
	__syncthreads();
	for (uint32_t s = 0; s < nslabs; ++s)
	{
		const int buf = s & 1;
		if (s + 1 < nslabs) { load_slab((s + 1) * DBK); }
		const double* as = TA ? As[buf] + lk * AP + wm * WM + l16 : As[buf] + (wm * WM + l16) * KP + lk;
		const double* bs = TB ? Bs[buf] + (wn * WN + l16) * KP + lk : Bs[buf] + lk * BP + wn * WN + l16;
#pragma unroll
		for (int ks = 0; ks < DBK / 4; ++ks)
		{
			double a[TM], b[TN];
#pragma unroll
			for (int i = 0; i < TM; ++i) { a[i] = TA ? as[ks * 4 * AP + i * 16] : as[i * 16 * KP + ks * 4]; }
#pragma unroll
			for (int j = 0; j < TN; ++j) { b[j] = TB ? bs[j * 16 * KP + ks * 4] : bs[ks * 4 * BP + j * 16]; }
#pragma unroll
			for (int i = 0; i < TM; ++i)
			{
#pragma unroll
				for (int j = 0; j < TN; ++j)
				{
					acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], b[j], acc[i][j], 0, 0, 0);
				}
			}
		}
		if (s + 1 < nslabs) { store_slab(buf ^ 1); }
		__syncthreads();
	}

	// lane holds column l16; register r is row 4*r + lk of the 16x16 block
#pragma unroll
	for (int i = 0; i < TM; ++i)
	{
#pragma unroll
		for (int j = 0; j < TN; ++j)
		{
			const uint32_t n = n0 + wn * WN + j * 16 + l16;
			if (n >= g.N) { continue; }
#pragma unroll
			for (int r = 0; r < 4; ++r)
			{
				const uint32_t m = m0 + wm * WM + i * 16 + 4 * r + lk;
				if (m < g.M) { C[(int64_t) m * g.ldc + n] = acc[i][j][r]; }
			}
		}
	}
}

// K a multiple of the slab depth: the slabs go from memory straight into LDS
// (global_load_lds_dwordx4: lane l of a wave's load leaves its two doubles at
// the wave's LDS base + 16 l), no registers and no LDS stores in between, three
// slabs in LDS: one being multiplied, two on their way.  A wave's load fills
// 1 KiB of LDS in lane order, so conflict-free reads come from which chunk a
// lane fetches: an operand whose K runs along memory is kept [row][8 k], 16
// rows x 4 chunks per load, the chunk in slot q of row r being q ^ ((r >> 2) & 3)
// (the sixteen rows times two k of a half-wave's 64-bit read then fall on 32
// distinct bank pairs); an operand whose rows run along memory is kept
// [k][rows] with the halves of 32 rows exchanged in the odd k-rows.  Rows and
// columns past the edge are fetched from the last ones inside and never stored.
template <int ROWS, bool KALONG>
__device__ __forceinline__ void ddirect_issue (const double* __restrict__ P, int64_t ld, uint32_t first, uint32_t extent,
	uint32_t k0, double* lds, int wave, int lane)
{
	constexpr int LOADS = ROWS / 64; // per wave and slab
#pragma unroll
	for (int j = 0; j < LOADS; ++j)
	{
		const int load = wave * LOADS + j;
		const double* src;
		if constexpr (KALONG)
		{
			const int r = load * 16 + lane / 4, q = lane % 4;
			const int chunk = q ^ ((r >> 2) & 3);
			uint32_t row = first + r;
			row = row < extent ? row : extent - 1;
			src = P + (int64_t) row * ld + k0 + chunk * 2;
		}
		else
		{
			// 128 doubles of the [k][rows] slab: 128 / ROWS k-rows
			const int at = load * 128 + lane * 2;
			const int k = at / ROWS, q = (at % ROWS) / 2;
			const int chunk = q ^ (8 * (k & 1));
			uint32_t row = first + chunk * 2;
			row = row + 2 <= extent ? row : extent - 2;
			src = P + (int64_t) (k0 + k) * ld + row;
		}
		const uint32_t base = __builtin_amdgcn_readfirstlane(
			(uint32_t) (uintptr_t) (const __attribute__((address_space(3))) double*) (lds + load * 128));
		// written as the instruction itself, and counted by the kernel: through the
		// builtin the compiler waits for every such load before any later LDS read
		asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(base) : "memory", "m0");
	}
}

template <int BM, int BN, bool TA, bool TB>
__global__ __launch_bounds__(256) void dgemm_mfma_direct_k (DGemmArgs g)
{
	constexpr int WM = BM / 2, WN = BN / 2;   // wave tile
	constexpr int TM = WM / 16, TN = WN / 16; // 16x16 accumulators per wave
	constexpr int A_SIZE = BM * DBK, B_SIZE = BN * DBK;
	__shared__ __attribute__((aligned(1024))) double As[3][A_SIZE];
	__shared__ __attribute__((aligned(1024))) double Bs[3][B_SIZE];

	uint32_t id = blockIdx.x;
	if (g.total_tiles % DNXCD == 0) { id = (id % DNXCD) * (g.total_tiles / DNXCD) + id / DNXCD; }
	const uint32_t bz = id / g.tiles_per_batch;
	const uint32_t t = id - bz * g.tiles_per_batch;
	const uint32_t group_size = DGROUP_M * g.tiles_n;
	const uint32_t group = t / group_size;
	const uint32_t first_m = group * DGROUP_M;
	const uint32_t rows_in_group = g.tiles_m - first_m < (uint32_t) DGROUP_M ? g.tiles_m - first_m : DGROUP_M;
	const uint32_t in_group = t - group * group_size;
	const uint32_t m0 = (first_m + in_group % rows_in_group) * BM, n0 = (in_group / rows_in_group) * BN;
	const double* __restrict__ A = g.A + (int64_t) bz * g.batch_a;
	const double* __restrict__ B = g.B + (int64_t) bz * g.batch_b;
	double* __restrict__ C = g.C + (int64_t) bz * g.batch_c;

	const int tid = threadIdx.x;
	const int lane = tid & 63, wave = tid >> 6;
	const int wm = wave >> 1, wn = wave & 1;
	const int l16 = lane & 15, lk = lane >> 4;

	f64x4 acc[TM][TN];
#pragma unroll
	for (int i = 0; i < TM; ++i)
	{
#pragma unroll
		for (int j = 0; j < TN; ++j)
		{
#pragma unroll
			for (int r = 0; r < 4; ++r) { acc[i][j][r] = 0.0; }
		}
	}

	auto issue = [&] (uint32_t k0, int buf)
	{
		ddirect_issue<BM,!TA>(A, g.lda, m0, g.M, k0, As[buf], wave, lane);
		ddirect_issue<BN,TB>(B, g.ldb, n0, g.N, k0, Bs[buf], wave, lane);
	};
	// element (row, k) of a slab as the loads left it
	auto at = [&] (bool kalong, int rows, int row, int k) -> int
	{
		return kalong ? row * DBK + (((k >> 1) ^ ((row >> 2) & 3)) << 1) + (k & 1) : k * rows + (row ^ (16 * (k & 1)));
	};
	// where this lane reads its operands of each accumulator and k-step, once for all slabs
	int aoff[TM][DBK / 4], boff[TN][DBK / 4];
#pragma unroll
	for (int ks = 0; ks < DBK / 4; ++ks)
	{
#pragma unroll
		for (int i = 0; i < TM; ++i) { aoff[i][ks] = at(!TA, BM, wm * WM + i * 16 + l16, ks * 4 + lk); }
#pragma unroll
		for (int j = 0; j < TN; ++j) { boff[j][ks] = at(TB, BN, wn * WN + j * 16 + l16, ks * 4 + lk); }
	}
	// live: false for the steps past the last slab (the loop runs in threes), whose
	// operands count as zero on both sides (what is in LDS then may hold infinities)
	auto multiply = [&] (auto buf_c, bool live)
	{
		constexpr int buf = decltype(buf_c)::value;
#pragma unroll
		for (int ks = 0; ks < DBK / 4; ++ks)
		{
			double a[TM], b[TN];
#pragma unroll
			for (int i = 0; i < TM; ++i) { a[i] = live ? As[buf][aoff[i][ks]] : 0.0; }
#pragma unroll
			for (int j = 0; j < TN; ++j) { b[j] = live ? Bs[buf][boff[j][ks]] : 0.0; }
#pragma unroll
			for (int i = 0; i < TM; ++i)
			{
#pragma unroll
				for (int j = 0; j < TN; ++j)
				{
					acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], b[j], acc[i][j], 0, 0, 0);
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
		constexpr int PER_SLAB = (BM + BN) / 64;
		static_assert(PER_SLAB < 16, "the count is written into four bits");
		__builtin_amdgcn_s_waitcnt(0x0070 | PER_SLAB); // vmcnt(PER_SLAB) lgkmcnt(0)
		__syncthreads();
	};
	const uint32_t nslabs = g.K / DBK;
	// past the end the last slab is fetched again and never used
	auto slab_at = [&] (uint32_t s) -> uint32_t { return (s < nslabs ? s : nslabs - 1) * DBK; };
	using I0 = std::integral_constant<int,0>;
	using I1 = std::integral_constant<int,1>;
	using I2 = std::integral_constant<int,2>;
	issue(slab_at(0), 0);
	issue(slab_at(1), 1);
	landed();
	// one body for every three slabs, also for the last one or two: a branch round
	// part of it would have the accumulators copied where the paths meet
	for (uint32_t s = 0; s < nslabs; s += 3)
	{
		issue(slab_at(s + 2), 2);
		multiply(I0(), true);
		landed();
		issue(slab_at(s + 3), 0);
		multiply(I1(), s + 1 < nslabs);
		landed();
		issue(slab_at(s + 4), 1);
		multiply(I2(), s + 2 < nslabs);
		landed();
	}
	// nothing of this workgroup's is on its way into LDS when it ends
	__builtin_amdgcn_s_waitcnt(0);

	// lane holds column l16; register r is row 4*r + lk of the 16x16 block
#pragma unroll
	for (int i = 0; i < TM; ++i)
	{
#pragma unroll
		for (int j = 0; j < TN; ++j)
		{
			const uint32_t n = n0 + wn * WN + j * 16 + l16;
			if (n >= g.N) { continue; }
#pragma unroll
			for (int r = 0; r < 4; ++r)
			{
				const uint32_t m = m0 + wm * WM + i * 16 + 4 * r + lk;
				if (m < g.M) { C[(int64_t) m * g.ldc + n] = acc[i][j][r]; }
			}
		}
	}
}

template <int BM, int BN>
int dlaunch (tcg_ctx* ctx, DGemmArgs g, uint64_t batch, int trans_a, int trans_b)
{
	uint64_t tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
	uint64_t total = tiles_m * tiles_n * batch;
	TCG_REQUIRE(ctx, total < (1ull << 31), "tcg_gemm: too many tiles for one launch");
	g.tiles_m = (uint32_t) tiles_m;
	g.tiles_n = (uint32_t) tiles_n;
	g.tiles_per_batch = (uint32_t) (tiles_m * tiles_n);
	g.total_tiles = (uint32_t) total;
	const unsigned grid = (unsigned) total;
	// K a whole number of slabs: from memory straight into LDS (4096^3: 61.8 -> 66.3 TFLOP/s)
	if (g.K % DBK == 0 && g.M >= 2 && g.N >= 2)
	{
		if (!trans_a && !trans_b) { dgemm_mfma_direct_k<BM,BN,false,false><<<grid, 256, 0, ctx->stream>>>(g); }
		else if (trans_a && !trans_b) { dgemm_mfma_direct_k<BM,BN,true,false><<<grid, 256, 0, ctx->stream>>>(g); }
		else if (!trans_a && trans_b) { dgemm_mfma_direct_k<BM,BN,false,true><<<grid, 256, 0, ctx->stream>>>(g); }
		else { dgemm_mfma_direct_k<BM,BN,true,true><<<grid, 256, 0, ctx->stream>>>(g); }
		TCG_LAUNCH_CHECK(ctx, "dgemm_mfma_direct");
		return TCG_OK;
	}
	if (!trans_a && !trans_b) { dgemm_mfma_k<BM,BN,false,false><<<grid, 256, 0, ctx->stream>>>(g); }
	else if (trans_a && !trans_b) { dgemm_mfma_k<BM,BN,true,false><<<grid, 256, 0, ctx->stream>>>(g); }
	else if (!trans_a && trans_b) { dgemm_mfma_k<BM,BN,false,true><<<grid, 256, 0, ctx->stream>>>(g); }
	else { dgemm_mfma_k<BM,BN,true,true><<<grid, 256, 0, ctx->stream>>>(g); }
	TCG_LAUNCH_CHECK(ctx, "dgemm_mfma");
	return TCG_OK;
}

} // namespace

int tcg_gemm_f64_mfma (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t K, uint64_t batch,
	const double* A, uint64_t lda, uint64_t stride_a, int trans_a,
	const double* B, uint64_t ldb, uint64_t stride_b, int trans_b,
	double* C, uint64_t ldc, uint64_t stride_c, bool* handled)
{
	*handled = false;
	// 128-bit operand loads: every row start and every slab offset 16-byte aligned;
	// problems too small to fill the chip with 64x64 tiles stay on the generic kernel
	bool ok = M >= 32 && N >= 32 && K >= 8 &&
		M < (1ull << 31) && N < (1ull << 31) && K < (1ull << 31) &&
		((M + 63) / 64) * ((N + 63) / 64) * batch >= (uint64_t) ctx->num_cus / 2 &&
		tcg_aligned16(A) && tcg_aligned16(B) &&
		lda % 2 == 0 && ldb % 2 == 0 && stride_a % 2 == 0 && stride_b % 2 == 0 &&
		((trans_a ? M : K) % 2 == 0) && ((trans_b ? K : N) % 2 == 0);
	if (!ok) { return TCG_OK; }
	DGemmArgs g;
	g.A = A; g.B = B; g.C = C;
	g.M = (uint32_t) M; g.N = (uint32_t) N; g.K = (uint32_t) K;
	g.lda = (int64_t) lda; g.ldb = (int64_t) ldb; g.ldc = (int64_t) ldc;
	g.batch_a = (int64_t) stride_a; g.batch_b = (int64_t) stride_b; g.batch_c = (int64_t) stride_c;
	g.tiles_m = g.tiles_n = g.tiles_per_batch = g.total_tiles = 0;
	*handled = true;
	uint64_t big_tiles = ((M + 127) / 128) * ((N + 127) / 128) * batch;
	if (big_tiles >= (uint64_t) ctx->num_cus) { return dlaunch<128,128>(ctx, g, batch, trans_a, trans_b); }
	return dlaunch<64,64>(ctx, g, batch, trans_a, trans_b);
}
