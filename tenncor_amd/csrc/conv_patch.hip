// CONV as a matrix product whose A operand is read out of a patch of the image
// held in LDS (internal/eigen/operator.hpp:1141-1187 is the operator; conv.hip
// lowers it to out[rows, cols] = A[rows, sums] * B[sums, cols] with
// A[m][s] = image[rows[m].off + sums[s].off]).
//
// The address of A[m][s] is a sum of a row part and a summed part, so the rows
// of a tile meet the same image elements again and again (a 5x5 window: 25
// times).  The product kernels of gemm_mfma.hip fetch every A[m][s] from L2;
// for narrow results (32 or 64 columns) that traffic, not the matrix pipes,
// bounds them.  Here a workgroup copies the stretch of memory that its rows can
// touch -- [min row offset + min sum offset, max + max] -- into LDS once and
// reads every A fragment from there; B streams from memory into registers.
//
// Layout in LDS: the image stretch as it lies in memory, with 4 floats of
// padding after every 2^pad_shift floats (the distance between neighbouring
// rows), so that the sixteen rows of a matrix instruction's operand fall into
// different banks.  Instruction: v_mfma_f32_16x16x4_f32; a lane holds four
// consecutive summed indices of its row (one 128-bit LDS read feeds four
// instructions).
#include "tcg_internal.hpp"

#include <climits>
#include <cstdint>
#include <cstdlib>

namespace
{

typedef float f4 __attribute__((ext_vector_type(4)));

constexpr int SB = 32; // the summed index comes in multiples of this

struct PatchArgs
{
	const float* img;
	const float* B;
	float* C;
	const tcg_conv_tab* rows;
	const tcg_conv_tab* sums;
	uint32_t M, N, S;
	int64_t ldb, ldc;
	int32_t smin, smax;    // least and greatest offset of the summed index
	int32_t vlo, vhi;      // image elements [vlo, vhi) exist (multiples of four)
	uint32_t pad_shift;
	uint32_t patch_floats; // floats of LDS the padded stretch may take
	uint32_t check_ext[2];
	uint32_t tiles_m, tiles;
};

__device__ __forceinline__ int padded (int x, uint32_t shift)
{
	return x + ((x >> shift) << 2);
}

// A workgroup of NW waves computes RBT x CBT blocks of 16 x 16 results.  The waves
// share the summed index between them (wave w takes the steps of sixteen summed
// indices w, w + NW, ...) and every wave holds a partial sum of the whole tile:
// a step then is RBT reads of A from LDS and one short read of B from memory for
// 4 RBT CBT matrix instructions, and B is read once per workgroup, not once per
// wave.  The partial sums are added up through LDS in wave order at the end.
// Column n0 + CBT r + cb of the result is column r of block cb: a lane's four B
// rows are then CBT consecutive floats each, and so are its results.
constexpr int NW = 4;

template <int CBT> struct BVec;
template <> struct BVec<2> { typedef float type __attribute__((ext_vector_type(2))); };
template <> struct BVec<4> { typedef float type __attribute__((ext_vector_type(4))); };

template <int RBT, int CBT, int NCHECK>
__global__ __launch_bounds__(64 * NW) void conv_patch_k (PatchArgs a)
{
	constexpr int NT = 64 * NW, TM = 16 * RBT, TN = 16 * CBT;
	typedef typename BVec<CBT>::type bvec;
	extern __shared__ __attribute__((aligned(16))) float lds[];
	__shared__ int range[2];
	float* patch = lds;
	int* stab = (int*) (lds + a.patch_floats);
	const uint32_t S4 = a.S >> 2;
	const int tid = (int) threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int r16 = lane & 15, q = lane >> 4;
	// neighbouring tiles (which share rows of the image between them) on one XCD
	uint32_t tile = blockIdx.x;
	if (a.tiles % 8 == 0) { tile = (blockIdx.x & 7u) * (a.tiles >> 3) + (blockIdx.x >> 3); }
	const uint32_t tm = tile % a.tiles_m, tn = tile / a.tiles_m;
	const uint32_t m0 = tm * TM, n0 = tn * TN;
	int rbase[RBT];
	int rc[RBT][NCHECK > 0 ? NCHECK : 1];
	bool rok[RBT];
	int least = INT_MAX, most = INT_MIN;
#pragma unroll
	for (int rb = 0; rb < RBT; ++rb)
	{
		const uint32_t m = m0 + (uint32_t) (rb * 16 + r16);
		rok[rb] = m < a.M;
		const tcg_conv_tab e = a.rows[rok[rb] ? m : m0];
		rbase[rb] = (int) e.off;
#pragma unroll
		for (int k = 0; k < NCHECK; ++k) { rc[rb][k] = e.c[k]; }
		least = rbase[rb] < least ? rbase[rb] : least;
		most = rbase[rb] > most ? rbase[rb] : most;
	}
	// (every wave holds every row of the tile: wave 0 says where they begin and end)
#pragma unroll
	for (int d = 1; d < 16; d <<= 1)
	{
		const int l2 = __shfl_xor(least, d), m2 = __shfl_xor(most, d);
		least = l2 < least ? l2 : least;
		most = m2 > most ? m2 : most;
	}
	if (tid == 0)
	{
		range[0] = least;
		range[1] = most;
	}
	for (uint32_t f = (uint32_t) tid; f < S4; f += NT)
	{
		const tcg_conv_tab e = a.sums[4 * f];
		stab[f] = (int) e.off;
#pragma unroll
		for (int k = 0; k < NCHECK; ++k) { stab[(k + 1) * S4 + f] = e.c[k]; }
	}
	__syncthreads();
	const int lo = range[0] + a.smin;
	{
		int from = lo > a.vlo ? lo : a.vlo;
		int to = range[1] + a.smax + 4;
		if (to > a.vhi) { to = a.vhi; }
#pragma unroll 4
		for (int p = from + 4 * tid; p < to; p += 4 * NT)
		{
			const f4 v = *(const f4*) (a.img + p);
			*(f4*) (patch + padded(p - lo, a.pad_shift)) = v;
		}
	}
#pragma unroll
	for (int rb = 0; rb < RBT; ++rb) { rbase[rb] -= lo; }
	__syncthreads();
	f4 acc[RBT][CBT];
#pragma unroll
	for (int rb = 0; rb < RBT; ++rb)
	{
#pragma unroll
		for (int cb = 0; cb < CBT; ++cb) { acc[rb][cb] = f4{0.f, 0.f, 0.f, 0.f}; }
	}
	const float* bcol = a.B + n0 + (uint32_t) (CBT * r16);
	auto load_b = [&] (uint32_t jj, bvec (&bv)[4])
	{
		const float* from = bcol + (int64_t) (16 * jj + 4 * q) * a.ldb;
#pragma unroll
		for (int i = 0; i < 4; ++i) { bv[i] = *(const bvec*) (from + i * a.ldb); }
	};
	auto load_a = [&] (uint32_t jj, f4 (&av)[RBT])
	{
		const uint32_t s4 = 4 * jj + q;
		const int so = stab[s4];
		int sc[NCHECK > 0 ? NCHECK : 1];
#pragma unroll
		for (int k = 0; k < NCHECK; ++k) { sc[k] = stab[(k + 1) * S4 + s4]; }
#pragma unroll
		for (int rb = 0; rb < RBT; ++rb)
		{
			bool ok = rok[rb];
#pragma unroll
			for (int k = 0; k < NCHECK; ++k) { ok = ok & ((uint32_t) (rc[rb][k] + sc[k]) < a.check_ext[k]); }
			const f4 v = *(const f4*) (patch + padded(rbase[rb] + so, a.pad_shift));
			av[rb] = ok ? v : f4{0.f, 0.f, 0.f, 0.f};
		}
	};
	// (Leaving out the sixteen-row blocks that lie wholly in the zero border for a step --
	// 15% of the matrix instructions of a 5x5 image gradient -- was measured: the branches
	// round each block's instructions took the kernel from 78 to 116 us, branches round
	// three blocks at a time to 106 us.)
	auto multiply = [&] (const f4 (&av)[RBT], const bvec (&bv)[4])
	{
#pragma unroll
		for (int rb = 0; rb < RBT; ++rb)
		{
#pragma unroll
			for (int cb = 0; cb < CBT; ++cb)
			{
				acc[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[rb].x, bv[0][cb], acc[rb][cb], 0, 0, 0);
				acc[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[rb].y, bv[1][cb], acc[rb][cb], 0, 0, 0);
				acc[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[rb].z, bv[2][cb], acc[rb][cb], 0, 0, 0);
				acc[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[rb].w, bv[3][cb], acc[rb][cb], 0, 0, 0);
			}
		}
	};
	// both operands a step ahead: asked for before the matrix instructions of a step, needed after them
	const uint32_t nsteps = a.S >> 4;
	{
		bvec bnow[4], bnext[4];
		f4 anow[RBT], anext[RBT];
		uint32_t jj = (uint32_t) wave;
		if (jj < nsteps)
		{
			load_b(jj, bnow);
			load_a(jj, anow);
		}
		for (; jj < nsteps; jj += NW)
		{
			if (jj + NW < nsteps)
			{
				load_b(jj + NW, bnext);
				load_a(jj + NW, anext);
			}
			multiply(anow, bnow);
#pragma unroll
			for (int i = 0; i < 4; ++i) { bnow[i] = bnext[i]; }
#pragma unroll
			for (int rb = 0; rb < RBT; ++rb) { anow[rb] = anext[rb]; }
		}
	}
	// the partial sums of the waves, added in wave order where the patch was
	__syncthreads();
	f4* sum = (f4*) lds;
	for (int w = 0; w < NW; ++w)
	{
		if (wave == w && w + 1 < NW)
		{
#pragma unroll
			for (int rb = 0; rb < RBT; ++rb)
			{
#pragma unroll
				for (int cb = 0; cb < CBT; ++cb)
				{
					f4* at = sum + (rb * CBT + cb) * 64 + lane;
					*at = w == 0 ? acc[rb][cb] : *at + acc[rb][cb];
				}
			}
		}
		if (w + 1 < NW) { __syncthreads(); }
	}
	if (wave != NW - 1) { return; }
	// a lane holds rows 4 q .. 4 q + 3 and columns CBT r16 .. CBT r16 + CBT - 1
#pragma unroll
	for (int rb = 0; rb < RBT; ++rb)
	{
		f4 total[CBT];
#pragma unroll
		for (int cb = 0; cb < CBT; ++cb) { total[cb] = sum[(rb * CBT + cb) * 64 + lane] + acc[rb][cb]; }
		const uint32_t mrow = m0 + (uint32_t) (rb * 16 + 4 * q);
		float* to = a.C + (int64_t) mrow * a.ldc + n0 + (uint32_t) (CBT * r16);
#pragma unroll
		for (int i = 0; i < 4; ++i)
		{
			if (mrow + i < a.M)
			{
				bvec out;
#pragma unroll
				for (int cb = 0; cb < CBT; ++cb) { out[cb] = total[cb][i]; }
				*(bvec*) (to + (int64_t) i * a.ldc) = out;
			}
		}
	}
}

struct Shape
{
	int rbt, cbt;
};

// the tiles there are kernels for: rows x columns = 16 rbt x 16 cbt
// (tiles twice as tall, one workgroup and so one wave per SIMD on every CU, were measured on the
// second layer of the reference's CNN: 208 x 64 forwards 59.6 against 57-59 us, 288 x 32 for the
// image gradient 93 against 77 us)
constexpr Shape SHAPES[] = {
	{9, 2}, // 144 x 32
	{6, 2}, //  96 x 32
	{7, 4}, // 112 x 64
	{5, 4}, //  80 x 64
};
constexpr int NSHAPES = (int) (sizeof(SHAPES) / sizeof(SHAPES[0]));

template <int RBT, int CBT>
int launch_shape (tcg_ctx* ctx, const PatchArgs& a, int ncheck, size_t lds_bytes)
{
	const unsigned threads = 64 * NW;
	auto go = [&] (auto kernel) -> int
	{
		// (more than 64 KiB of LDS per workgroup has to be asked for, once per kernel)
		static bool asked = false;
		if (lds_bytes > 65536 && false == asked)
		{
			if (hipFuncSetAttribute((const void*) kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int) TCG_CONV_PATCH_LDS) != hipSuccess)
			{
				(void) hipGetLastError();
				return TCG_ERR_UNSUPPORTED;
			}
			asked = true;
		}
		kernel<<<a.tiles, threads, lds_bytes, ctx->stream>>>(a);
		return TCG_OK;
	};
	if (ncheck == 0) { return go(conv_patch_k<RBT,CBT,0>); }
	return go(conv_patch_k<RBT,CBT,2>);
}

} // namespace

int tcg_conv_patch_shapes (void) { return NSHAPES; }

void tcg_conv_patch_shape (int which, uint32_t* rows, uint32_t* cols, uint32_t* threads)
{
	const Shape& s = SHAPES[which];
	*rows = (uint32_t) (16 * s.rbt);
	*cols = (uint32_t) (16 * s.cbt);
	*threads = (uint32_t) (64 * NW);
}

size_t tcg_conv_patch_lds (int which, uint32_t patch_floats, uint64_t S, int ncheck)
{
	// the padded stretch of the image, or the partial sums of all waves but the last that take its place
	const Shape& s = SHAPES[which];
	const size_t sums = (size_t) 256 * s.rbt * s.cbt;
	const size_t first = patch_floats > sums ? patch_floats : sums;
	return sizeof(float) * first + sizeof(int) * (size_t) (1 + (ncheck > 0 ? 2 : 0)) * (S / 4);
}

int tcg_conv_patch_f32 (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t S, const float* image,
	const tcg_conv_operand& op, const tcg_conv_patch& pp, const float* B, uint64_t ldb, float* C, uint64_t ldc, bool* handled)
{
	*handled = false;
	if (pp.shape < 0 || pp.shape >= NSHAPES) { return TCG_OK; }
	uint32_t tm = 0, tn = 0, threads = 0;
	tcg_conv_patch_shape(pp.shape, &tm, &tn, &threads);
	bool ok = M >= 1 && M < (1ull << 31) && N >= tn && N % tn == 0 && N < (1ull << 31) && S >= SB && S % SB == 0 && S <= 8192 &&
		op.rows && op.sums && op.ncheck >= 0 && op.ncheck <= 2 && op.vec4 && false == op.along_m &&
		tcg_aligned16(image) && tcg_aligned16(B) && tcg_aligned16(C) && ldb % 4 == 0 && ldc % 4 == 0 && ldb >= N && ldc >= N &&
		pp.vlo % 4 == 0 && pp.vhi % 4 == 0 && pp.vlo < pp.vhi && pp.pad_shift >= 4 && pp.pad_shift <= 31;
	if (false == ok) { return TCG_OK; }
	PatchArgs a;
	a.img = image; a.B = B; a.C = C;
	a.rows = op.rows; a.sums = op.sums;
	a.M = (uint32_t) M; a.N = (uint32_t) N; a.S = (uint32_t) S;
	a.ldb = (int64_t) ldb; a.ldc = (int64_t) ldc;
	a.smin = pp.smin; a.smax = pp.smax; a.vlo = pp.vlo; a.vhi = pp.vhi;
	a.pad_shift = pp.pad_shift;
	a.patch_floats = pp.patch_floats;
	// one check is run as two, the second of which every element passes
	a.check_ext[0] = op.ncheck >= 1 ? op.check_ext[0] : 0xffffffffu;
	a.check_ext[1] = op.ncheck >= 2 ? op.check_ext[1] : 0xffffffffu;
	a.tiles_m = (uint32_t) ((M + tm - 1) / tm);
	const uint64_t tiles = (uint64_t) a.tiles_m * (N / tn);
	if (tiles >= (1ull << 31)) { return TCG_OK; }
	a.tiles = (uint32_t) tiles;
	const size_t lds_bytes = tcg_conv_patch_lds(pp.shape, pp.patch_floats, S, op.ncheck);
	if (lds_bytes > TCG_CONV_PATCH_LDS) { return TCG_OK; }
	int rc = TCG_ERR_UNSUPPORTED;
	switch (pp.shape)
	{
		case 0: rc = launch_shape<9,2>(ctx, a, op.ncheck, lds_bytes); break;
		case 1: rc = launch_shape<6,2>(ctx, a, op.ncheck, lds_bytes); break;
		case 2: rc = launch_shape<7,4>(ctx, a, op.ncheck, lds_bytes); break;
		case 3: rc = launch_shape<5,4>(ctx, a, op.ncheck, lds_bytes); break;
		default: break;
	}
	if (rc == TCG_ERR_UNSUPPORTED) { return TCG_OK; }
	if (rc != TCG_OK) { return rc; }
	TCG_LAUNCH_CHECK(ctx, "conv_patch");
	++ctx->conv_patch_launches;
	*handled = true;
	return TCG_OK;
}

extern "C" int tcg_conv_route_counts (const tcg_ctx* ctx, uint64_t* patch, uint64_t* short_sum, uint64_t* few_rows)
{
	if (!ctx || !patch || !short_sum || !few_rows) { return TCG_ERR_ARG; }
	*patch = ctx->conv_patch_launches;
	*short_sum = ctx->conv_short_launches;
	*few_rows = ctx->conv_fewrows_launches;
	return TCG_OK;
}
