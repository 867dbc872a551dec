// CONV: N-d valid cross-correlation (internal/eigen/operator.hpp:1141-1187),
//   out[c] = sum_k img[c + e(k)] * kernel[k],  kernel dim i sliding along image
//   dim ranks[i].
//
// The way tenncor's conv2d and its gradients are written (PAD of a singleton
// axis, correlate, SLICE one index back out) most of the image operand is
// padding and most of the output is thrown away, so the kernel takes two
// boxes: the image is promised to be zero outside [img_lo, img_hi) and only
// outputs inside [out_lo, out_hi) are produced.  Summation ranges are clipped
// to the image box per output coordinate, which removes the work on padding
// exactly (terms that are skipped are exact zeros).  With full boxes this is
// the plain correlation and the parity reference of anything faster.
//
// Two mappings: one lane per output (many outputs, short sums) or one
// workgroup per output with the lanes striding over the clipped kernel box and
// an LDS tree at the end (few outputs, long sums: kernel gradients).
#include "tcg_internal.hpp"

#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <string>
#include <type_traits>
#include <vector>

namespace
{

template <typename T> struct is_int { static constexpr bool value = false; };
template <> struct is_int<int32_t> { static constexpr bool value = true; };
template <> struct is_int<int8_t> { static constexpr bool value = true; };
template <> struct is_int<uint8_t> { static constexpr bool value = true; };
template <> struct is_int<int16_t> { static constexpr bool value = true; };
template <> struct is_int<uint16_t> { static constexpr bool value = true; };
template <> struct is_int<uint32_t> { static constexpr bool value = true; };
template <> struct is_int<int64_t> { static constexpr bool value = true; };
template <> struct is_int<uint64_t> { static constexpr bool value = true; };

// integers wrap modulo 2^width: summed in 32 (64) unsigned bits and truncated
template <typename T> using Wide = typename std::conditional<sizeof(T) == 8, uint64_t, uint32_t>::type;

template <typename T>
__device__ __forceinline__ T mac (T acc, T x, T w)
{
	if constexpr (is_int<T>::value) { return (T) ((Wide<T>) acc + (Wide<T>) x * (Wide<T>) w); }
	else { return acc + x * w; }
}

struct ConvPlan
{
	// everything indexed by IMAGE dim d; the kernel dim sliding along d has
	// extent ksize[d] (1 when none does) and kernel-memory stride kstr[d]
	uint32_t wsize[8];   // output window extents
	uint32_t wlo[8];     // output window offsets
	int64_t istr[8];     // image strides
	int64_t ostr[8];     // output strides
	uint32_t ksize[8];
	int64_t kstr[8];
	int32_t ilo[8];      // image non-zero box
	int32_t ihi[8];
	uint64_t nwin = 1;   // outputs in the window
	int64_t ioff0 = 0;   // image offset of coordinate 0 (negative when `img` holds the box only)
	int64_t ooff0 = 0;   // output offset of coordinate 0 (negative when `out` starts at the window)
};

constexpr int CV_BLOCK = 256;

template <typename T, bool GROUP_PER_OUTPUT>
__global__ __launch_bounds__(CV_BLOCK) void conv_boxed_k (ConvPlan p,
	const T* __restrict__ img, const T* __restrict__ ker, T* __restrict__ out)
{
	uint64_t o = GROUP_PER_OUTPUT ? (uint64_t) blockIdx.x : (uint64_t) blockIdx.x * CV_BLOCK + threadIdx.x;
	if (o >= p.nwin) { return; }
	// output coordinate, and per image dim the clipped kernel range [k0, k0 + kr)
	int64_t ibase = p.ioff0, obase = p.ooff0, kbase = 0;
	uint32_t kr[8];
	uint64_t nterms = 1;
	uint32_t rem = (uint32_t) o; // the host keeps nwin below 2^32
#pragma unroll
	for (int d = 0; d < 8; ++d)
	{
		uint32_t q = rem / p.wsize[d];
		int32_t c = (int32_t) (rem - q * p.wsize[d]) + (int32_t) p.wlo[d];
		rem = q;
		int32_t lo = p.ilo[d] - c, hi = p.ihi[d] - c;
		if (lo < 0) { lo = 0; }
		if (hi > (int32_t) p.ksize[d]) { hi = (int32_t) p.ksize[d]; }
		int32_t r = hi - lo;
		if (r < 0) { r = 0; }
		kr[d] = (uint32_t) r;
		nterms *= (uint32_t) r;
		ibase += (int64_t) (c + lo) * p.istr[d];
		kbase += (int64_t) lo * p.kstr[d];
		obase += (int64_t) c * p.ostr[d];
	}
	T acc = 0;
	if constexpr (!GROUP_PER_OUTPUT)
	{
		// odometer over the clipped box
		uint32_t kc[8];
#pragma unroll
		for (int d = 0; d < 8; ++d) { kc[d] = 0; }
		int64_t ioff = ibase, koff = kbase;
		for (uint64_t t = 0; t < nterms; ++t)
		{
			acc = mac(acc, img[ioff], ker[koff]);
			bool carry = true;
#pragma unroll
			for (int d = 0; d < 8; ++d)
			{
				if (carry && kr[d] > 1)
				{
					++kc[d];
					ioff += p.istr[d];
					koff += p.kstr[d];
					if (kc[d] == kr[d])
					{
						ioff -= (int64_t) kr[d] * p.istr[d];
						koff -= (int64_t) kr[d] * p.kstr[d];
						kc[d] = 0;
					}
					else { carry = false; }
				}
			}
		}
		out[obase] = acc;
	}
	else
	{
		for (uint64_t t = threadIdx.x; t < nterms; t += CV_BLOCK)
		{
			uint64_t r2 = t;
			int64_t ioff = ibase, koff = kbase;
#pragma unroll
			for (int d = 0; d < 8; ++d)
			{
				if (kr[d] > 1)
				{
					uint64_t q = r2 / kr[d];
					uint32_t k = (uint32_t) (r2 - q * kr[d]);
					r2 = q;
					ioff += (int64_t) k * p.istr[d];
					koff += (int64_t) k * p.kstr[d];
				}
			}
			acc = mac(acc, img[ioff], ker[koff]);
		}
		__shared__ T smem[CV_BLOCK];
		smem[threadIdx.x] = acc;
		__syncthreads();
		for (int s = CV_BLOCK / 2; s >= 1; s >>= 1)
		{
			if ((int) threadIdx.x < s)
			{
				T a = smem[threadIdx.x], b = smem[threadIdx.x + s];
				if constexpr (is_int<T>::value) { smem[threadIdx.x] = (T) ((Wide<T>) a + (Wide<T>) b); }
				else { smem[threadIdx.x] = a + b; }
			}
			__syncthreads();
		}
		if (threadIdx.x == 0) { out[obase] = smem[0]; }
	}
}

// ---- lowering to a matrix product ------------------------------------------
//
// Per image dim d (kernel extent K_d, image non-zero box [lo, hi), output
// window W_d) the correlation does one of three things:
//   K_d == 1            the output coordinate indexes the image directly:
//                       a row dim of the product (batch-like);
//   hi - lo == 1        only one kernel index per output coordinate meets the
//                       box (w = lo - x): no sum, the output coordinate picks
//                       the kernel slice: a column dim (this is how conv2d
//                       spells "output channels": a singleton axis padded to
//                       2*O - 1 and correlated with the O filters);
//   otherwise           the output coordinate is a row dim and the kernel
//                       coordinate a summed dim (spatial dims; a dim whose
//                       output extent is 1 is a plain summed channel dim).
// So out[rows, cols] = A[rows, sums] * B[sums, cols] with A gathered from the
// image (zero outside its box) and B gathered from the kernel.  A and B are
// materialised (A in row chunks of bounded size), the product runs on the GEMM
// path (matrix cores for fp32), and the result is scattered to the window.
// Reads of A are the dominant traffic: rows*sums elements written and read once.

struct ConvDiv
{
	uint32_t d, m, s1, s2;
};

ConvDiv conv_make_div (uint32_t d)
{
	ConvDiv f = {d, 0, 0, 0};
	uint32_t l = 0;
	while (((uint64_t) 1 << l) < d) { ++l; }
	f.m = (uint32_t) ((((uint64_t) 1 << 32) * (((uint64_t) 1 << l) - d)) / d + 1);
	f.s1 = l < 1 ? l : 1;
	f.s2 = l == 0 ? 0 : l - 1;
	return f;
}

__device__ __forceinline__ uint32_t conv_div (uint32_t n, const ConvDiv& f)
{
	uint32_t t = __umulhi(f.m, n);
	return (t + ((n - t) >> f.s1)) >> f.s2;
}

struct ConvGemmPlan
{
	// The bytes of a plan are the key under which its tables are kept
	// (tcg_ctx::conv_tables): every byte, padding included, starts at zero.
	ConvGemmPlan (void) { memset((void*) this, 0, sizeof(*this)); }

	// per image dim: extents of its row, summed and column component (1 = none)
	uint32_t msize[8], ssize[8], nsize[8];
	ConvDiv mdiv[8], sdiv[8], ndiv[8];
	int32_t xlo[8];     // first output coordinate of the window, in image coordinates
	int32_t oxlo[8];    // the same in output coordinates (they differ when the
	                    // image has been cut down to its non-zero box)
	int32_t slo[8];     // first summed kernel coordinate
	uint32_t is_col[8]; // column dim: image coordinate fixed at ilo, kernel index ilo - x
	int32_t ilo[8], ihi[8];
	uint32_t ksize[8];
	int64_t istr[8], ostr[8], kstr[8];
	uint32_t M, N, S;   // rows, columns, summed
	uint32_t Sp, Np;    // padded to multiples of 4 (leading dims of A / B and C)
	// dims where a row coordinate and a summed coordinate (or the box) decide
	// together whether the image element exists; -1 pads the list
	int32_t check_dim[4];
	uint32_t check_ext[4];
	int32_t ncheck;     // -1: more than four, the general gather handles them
	// The order in which the row / summed / column index decomposes into image
	// dims, fastest first (each lists all eight dims; a dim of extent 1 is a
	// no-op).  Any order gives the same product as long as A, B and C agree on
	// it, so each index runs first along the dim that lies closest in memory:
	// the summed index along the image, rows and columns along the result.
	// Without tables (ncheck < 0) all three are the identity.
	uint32_t mord[8], sord[8], nord[8];
	uint32_t nflip[8];  // column dim counted from its last output coordinate down
};

// Per row / per summed index: image offset and, for the checked dims, the
// coordinate relative to the box start (row part and summed part add up)
using ConvTabEntry = tcg_conv_tab;

constexpr int CG_BLOCK = 256;

// A[m - m0][s] for m in [m0, m0 + rows)
template <typename T>
__global__ __launch_bounds__(CG_BLOCK) void conv_gather_image_k (ConvGemmPlan p, uint32_t m0, uint32_t rows,
	const T* __restrict__ img, T* __restrict__ A)
{
	const uint64_t total = (uint64_t) rows * p.Sp;
	const uint64_t step = (uint64_t) gridDim.x * CG_BLOCK;
	for (uint64_t i = (uint64_t) blockIdx.x * CG_BLOCK + threadIdx.x; i < total; i += step)
	{
		uint32_t r = (uint32_t) (i / p.Sp);
		uint32_t s = (uint32_t) (i - (uint64_t) r * p.Sp);
		T v = 0;
		if (s < p.S)
		{
			uint32_t rm = m0 + r, rs = s;
			int64_t off = 0;
			bool inside = true;
#pragma unroll
			for (int d = 0; d < 8; ++d)
			{
				uint32_t qm = conv_div(rm, p.mdiv[d]);
				int32_t x = (int32_t) (rm - qm * p.msize[d]);
				rm = qm;
				uint32_t qs = conv_div(rs, p.sdiv[d]);
				int32_t w = (int32_t) (rs - qs * p.ssize[d]);
				rs = qs;
				int32_t c = p.is_col[d] ? p.ilo[d] : p.xlo[d] + x + p.slo[d] + w;
				inside = inside && c >= p.ilo[d] && c < p.ihi[d];
				off += (int64_t) c * p.istr[d];
			}
			if (inside) { v = img[off]; }
		}
		A[i] = v;
	}
}

constexpr int64_t CONV_NO_KERNEL = INT64_MIN;

// rows: entry m describes output row m; sums: entry s describes summed index s
__global__ __launch_bounds__(CG_BLOCK) void conv_tables_k (ConvGemmPlan p, ConvTabEntry* __restrict__ rows,
	ConvTabEntry* __restrict__ sums)
{
	const uint32_t i = blockIdx.x * CG_BLOCK + threadIdx.x;
	if (i < p.M)
	{
		uint32_t rm = i;
		ConvTabEntry e;
		e.off = 0;
		e.c[0] = e.c[1] = e.c[2] = e.c[3] = 0;
		for (int j = 0; j < 8; ++j)
		{
			const uint32_t d = p.mord[j];
			uint32_t qm = conv_div(rm, p.mdiv[d]);
			int32_t x = (int32_t) (rm - qm * p.msize[d]);
			rm = qm;
			int32_t c = p.is_col[d] ? p.ilo[d] : p.xlo[d] + x;
			e.off += (int64_t) c * p.istr[d];
#pragma unroll
			for (int k = 0; k < 4; ++k)
			{
				if (p.check_dim[k] == (int32_t) d) { e.c[k] = c - p.ilo[d]; }
			}
		}
		rows[i] = e;
	}
	if (i < p.Sp)
	{
		uint32_t rs = i;
		ConvTabEntry e;
		e.off = 0;
		e.c[0] = e.c[1] = e.c[2] = e.c[3] = 0;
		for (int j = 0; j < 8; ++j)
		{
			const uint32_t d = p.sord[j];
			uint32_t qs = conv_div(rs, p.sdiv[d]);
			int32_t w = (int32_t) (rs - qs * p.ssize[d]) + p.slo[d];
			rs = qs;
			e.off += (int64_t) w * p.istr[d];
#pragma unroll
			for (int k = 0; k < 4; ++k)
			{
				if (p.check_dim[k] == (int32_t) d) { e.c[k] = w; }
			}
		}
		// padding columns of A: a coordinate no row can complete into the box
		if (i >= p.S) { e.c[0] = INT32_MIN / 2; }
		sums[i] = e;
	}
	// behind the sums: where B[s][n] lies in the kernel, as a part that follows from s
	// and a part that follows from n (CONV_NO_KERNEL: no such element, B[s][n] = 0)
	int64_t* ktab = (int64_t*) (sums + p.Sp);
	if (i < p.Sp)
	{
		uint32_t rs = i;
		int64_t off = 0;
		bool valid = i < p.S;
		for (int j = 0; j < 8; ++j)
		{
			const uint32_t d = p.sord[j];
			uint32_t qs = conv_div(rs, p.sdiv[d]);
			int32_t w = (int32_t) (rs - qs * p.ssize[d]) + p.slo[d];
			rs = qs;
			if (p.is_col[d]) { continue; }
			valid = valid && w >= 0 && w < (int32_t) p.ksize[d];
			off += (int64_t) w * p.kstr[d];
		}
		ktab[i] = valid ? off : CONV_NO_KERNEL;
	}
	if (i < p.Np)
	{
		uint32_t rn = i;
		int64_t off = 0;
		bool valid = i < p.N;
		for (int j = 0; j < 8; ++j)
		{
			const uint32_t d = p.nord[j];
			uint32_t qn = conv_div(rn, p.ndiv[d]);
			uint32_t xq = rn - qn * p.nsize[d];
			rn = qn;
			if (0 == p.is_col[d]) { continue; }
			if (p.nflip[d]) { xq = p.nsize[d] - 1 - xq; }
			int32_t w = p.ilo[d] - (p.xlo[d] + (int32_t) xq);
			valid = valid && w >= 0 && w < (int32_t) p.ksize[d];
			off += (int64_t) w * p.kstr[d];
		}
		ktab[p.Sp + i] = valid ? off : CONV_NO_KERNEL;
	}
}

// B[s][n], elements first, first + step, ...
template <typename T>
__device__ __forceinline__ void conv_gather_kernel_part (const ConvGemmPlan& p, const T* __restrict__ ker, T* __restrict__ B,
	uint64_t first, uint64_t step)
{
	const uint64_t total = (uint64_t) p.Sp * p.Np;
	for (uint64_t i = first; i < total; i += step)
	{
		uint32_t s = (uint32_t) (i / p.Np);
		uint32_t n = (uint32_t) (i - (uint64_t) s * p.Np);
		T v = 0;
		if (s < p.S && n < p.N)
		{
			uint32_t rs = s, rn = n;
			int64_t off = 0;
			bool valid = true;
			// a dim is a column dim (its kernel index follows from the column)
			// or it is not (its kernel index is the summed one): never both
			for (int j = 0; j < 8; ++j)
			{
				const uint32_t d = p.sord[j];
				uint32_t qs = conv_div(rs, p.sdiv[d]);
				int32_t w = (int32_t) (rs - qs * p.ssize[d]) + p.slo[d];
				rs = qs;
				if (p.is_col[d]) { continue; }
				valid = valid && w >= 0 && w < (int32_t) p.ksize[d];
				off += (int64_t) w * p.kstr[d];
			}
			for (int j = 0; j < 8; ++j)
			{
				const uint32_t d = p.nord[j];
				uint32_t qn = conv_div(rn, p.ndiv[d]);
				uint32_t xq = rn - qn * p.nsize[d];
				rn = qn;
				if (0 == p.is_col[d]) { continue; }
				if (p.nflip[d]) { xq = p.nsize[d] - 1 - xq; }
				int32_t w = p.ilo[d] - (p.xlo[d] + (int32_t) xq);
				valid = valid && w >= 0 && w < (int32_t) p.ksize[d];
				off += (int64_t) w * p.kstr[d];
			}
			if (valid) { v = ker[off]; }
		}
		B[i] = v;
	}
}

template <typename T>
__global__ __launch_bounds__(CG_BLOCK) void conv_gather_kernel_k (ConvGemmPlan p,
	const T* __restrict__ ker, T* __restrict__ B)
{
	conv_gather_kernel_part<T>(p, ker, B, (uint64_t) blockIdx.x * CG_BLOCK + threadIdx.x, (uint64_t) gridDim.x * CG_BLOCK);
}

// the same from the offsets kept behind the sum table (conv_tables_k): two table reads and one of the kernel per element
template <typename T>
__global__ __launch_bounds__(CG_BLOCK) void conv_gather_kernel_tab_k (uint32_t Sp, uint32_t Np, const int64_t* __restrict__ ktab,
	const T* __restrict__ ker, T* __restrict__ B)
{
	const uint32_t total = Sp * Np;
	for (uint32_t i = blockIdx.x * CG_BLOCK + threadIdx.x; i < total; i += gridDim.x * CG_BLOCK)
	{
		const uint32_t s = i / Np, n = i - s * Np;
		const int64_t ks = ktab[s], kn = ktab[Sp + n];
		T v = 0;
		if (ks != CONV_NO_KERNEL && kn != CONV_NO_KERNEL) { v = ker[ks + kn]; }
		B[i] = v;
	}
}

constexpr int CG_ROWS = 16;
constexpr int CG_NARROW_ROWS = 128; // rows per workgroup when the summed index is at most CG_BLOCK / 2 long

// A[m - m0][s] from the two tables: one summed index per lane, CG_ROWS rows per workgroup.
// With `B`: the workgroups behind those of the rows (blockIdx.y >= row_blocks, blockIdx.x == 0)
// gather the kernel as well, which saves its launch where both operands are laid out
template <typename T, int NCHECK>
__global__ __launch_bounds__(CG_BLOCK) void conv_gather_tab_k (ConvGemmPlan p, uint32_t m0, uint32_t rows,
	const ConvTabEntry* __restrict__ rowtab, const ConvTabEntry* __restrict__ sumtab,
	const T* __restrict__ img, T* __restrict__ A, uint32_t row_blocks, const T* __restrict__ ker, T* __restrict__ B)
{
	if (blockIdx.y >= row_blocks)
	{
		if (blockIdx.x == 0)
		{
			conv_gather_kernel_part<T>(p, ker, B, (uint64_t) (blockIdx.y - row_blocks) * CG_BLOCK + threadIdx.x,
				(uint64_t) (gridDim.y - row_blocks) * CG_BLOCK);
		}
		return;
	}
	if (p.Sp <= CG_BLOCK / 2)
	{
		// a short summed index (a 5x5 window over one channel: 28 columns) would leave
		// most lanes of a workgroup without a column: the lanes walk the CG_ROWS x Sp
		// elements of the workgroup's rows in memory order instead
		// (CG_NARROW_ROWS rows per workgroup: every lane has several independent elements in flight)
		const uint32_t r0 = blockIdx.y * CG_NARROW_ROWS;
		const uint32_t count = (rows - r0 < (uint32_t) CG_NARROW_ROWS ? rows - r0 : (uint32_t) CG_NARROW_ROWS) * p.Sp;
#pragma unroll 4
		for (uint32_t i = threadIdx.x; i < count; i += CG_BLOCK)
		{
			const uint32_t r = i / p.Sp, s = i - r * p.Sp;
			const ConvTabEntry row = rowtab[m0 + r0 + r];
			const ConvTabEntry col = sumtab[s];
			bool inside = s < p.S;
#pragma unroll
			for (int j = 0; j < NCHECK; ++j)
			{
				inside = inside && (uint32_t) (row.c[j] + col.c[j]) < p.check_ext[j];
			}
			T v = 0;
			if (inside) { v = img[row.off + col.off]; }
			A[(uint64_t) (r0 + r) * p.Sp + s] = v;
		}
		return;
	}
	const uint32_t s = blockIdx.x * CG_BLOCK + threadIdx.x;
	if (s >= p.Sp) { return; }
	const ConvTabEntry col = sumtab[s];
	const bool pad_col = s >= p.S;
	const uint32_t r0 = blockIdx.y * CG_ROWS;
#pragma unroll 4
	for (uint32_t r = r0; r < r0 + CG_ROWS && r < rows; ++r)
	{
		const ConvTabEntry row = rowtab[m0 + r];
		bool inside = !pad_col;
#pragma unroll
		for (int j = 0; j < NCHECK; ++j)
		{
			inside = inside && (uint32_t) (row.c[j] + col.c[j]) < p.check_ext[j];
		}
		T v = 0;
		if (inside) { v = img[row.off + col.off]; }
		A[(uint64_t) r * p.Sp + s] = v;
	}
}

// The whole product for a short summed index (a 5x5 window over one channel: 25
// terms) and few columns, in one launch: B is small enough for every wave to hold
// its share of it in registers for good (v_mfma_f32_16x16x4_f32: SP4 x CB values per
// lane), gathered from the kernel itself through the offsets kept behind the sum
// table (`ker`) or read from the matrix (`Bmat`); a wave then gathers the rows of A
// that belong to 64 output rows straight into the lanes that multiply them.  A is
// never written to memory, B needs no launch of its own, nothing goes through LDS.
typedef float conv_f4 __attribute__((ext_vector_type(4)));
constexpr int CS_MAX_S = 32, CS_MAX_N = 64, CS_RB = 4;

template <int SP4, int CB>
__global__ __launch_bounds__(CG_BLOCK) void conv_short_k (ConvGemmPlan p, uint32_t m0, uint32_t rows,
	const ConvTabEntry* __restrict__ rowtab, const ConvTabEntry* __restrict__ sumtab, const float* __restrict__ img,
	const float* __restrict__ ker, const float* __restrict__ Bmat, int64_t ldb, float* __restrict__ C, int64_t ldc, int64_t safe)
{
	const uint32_t lane = threadIdx.x & 63u, r16 = lane & 15u, q = lane >> 4;
	const uint32_t wave = blockIdx.x * (CG_BLOCK / 64) + (threadIdx.x >> 6);
	const uint32_t first = wave * (16 * CS_RB);
	if (first >= rows) { return; }
	// checks beyond the plan's own pass everything (their table entries are zero)
	uint32_t ext[4];
#pragma unroll
	for (int j = 0; j < 4; ++j) { ext[j] = j < p.ncheck ? p.check_ext[j] : 0xffffffffu; }
	// this lane's summed indices 4 j + q and its share of B: every offset first, then
	// every element (no load waits for another of its kind)
	ConvTabEntry col[SP4];
	float b[SP4][CB];
	{
		const int64_t* ktab = (const int64_t*) (sumtab + p.Sp);
		const float* from = ker ? ker : Bmat;
		int64_t ks[SP4], kn[CB];
#pragma unroll
		for (int j = 0; j < SP4; ++j)
		{
			const uint32_t s = 4 * j + q;
			col[j] = sumtab[s];
			ks[j] = ker ? ktab[s] : (int64_t) s * ldb;
		}
#pragma unroll
		for (int cb = 0; cb < CB; ++cb)
		{
			const uint32_t n = 16 * cb + r16;
			kn[cb] = ker ? ktab[p.Sp + n] : (int64_t) n;
		}
#pragma unroll
		for (int j = 0; j < SP4; ++j)
		{
#pragma unroll
			for (int cb = 0; cb < CB; ++cb)
			{
				const bool there = nullptr == ker || (ks[j] != CONV_NO_KERNEL && kn[cb] != CONV_NO_KERNEL);
				const float v = from[there ? ks[j] + kn[cb] : 0];
				b[j][cb] = there ? v : 0.f;
			}
		}
	}
	conv_f4 acc[CS_RB][CB];
	float a[CS_RB][SP4];
#pragma unroll
	for (int rb = 0; rb < CS_RB; ++rb)
	{
		const uint32_t r = first + 16 * rb + r16;
		const bool real = r < rows;
		const ConvTabEntry row = rowtab[m0 + (real ? r : first)];
#pragma unroll
		for (int j = 0; j < SP4; ++j)
		{
			bool inside = real & (4 * j + q < p.S);
#pragma unroll
			for (int k = 0; k < 4; ++k) { inside = inside & ((uint32_t) (row.c[k] + col[j].c[k]) < ext[k]); }
			// (every lane loads, from an element that exists when its own lies in the zero border)
			const float v = img[inside ? row.off + col[j].off : safe];
			a[rb][j] = inside ? v : 0.f;
		}
	}
#pragma unroll
	for (int rb = 0; rb < CS_RB; ++rb)
	{
#pragma unroll
		for (int cb = 0; cb < CB; ++cb)
		{
			acc[rb][cb] = conv_f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
			for (int j = 0; j < SP4; ++j) { acc[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[rb][j], b[j][cb], acc[rb][cb], 0, 0, 0); }
		}
	}
	// a lane holds rows 4 q .. 4 q + 3 of column r16 of each block
#pragma unroll
	for (int rb = 0; rb < CS_RB; ++rb)
	{
		const uint32_t r = first + 16 * rb + 4 * q;
		float* to = C + (int64_t) r * ldc + r16;
#pragma unroll
		for (int cb = 0; cb < CB; ++cb)
		{
			if (r < rows) { to[16 * cb] = acc[rb][cb].x; }
			if (r + 1 < rows) { to[ldc + 16 * cb] = acc[rb][cb].y; }
			if (r + 2 < rows) { to[2 * ldc + 16 * cb] = acc[rb][cb].z; }
			if (r + 3 < rows) { to[3 * ldc + 16 * cb] = acc[rb][cb].w; }
		}
	}
}

template <int SP4>
void conv_short_launch (tcg_ctx* ctx, const ConvGemmPlan& g, uint32_t m0, uint32_t rows, const ConvTabEntry* rt, const ConvTabEntry* st,
	const float* img, const float* ker, const float* Bmat, int64_t ldb, float* C, int64_t ldc)
{
	// an element of the image that exists: the first of its box
	int64_t safe = 0;
	for (int d = 0; d < 8; ++d) { safe += (int64_t) g.ilo[d] * g.istr[d]; }
	const uint32_t per_group = 16 * CS_RB * (CG_BLOCK / 64);
	const uint32_t groups = (rows + per_group - 1) / per_group;
	switch (g.Np / 16)
	{
		case 1: conv_short_k<SP4,1><<<groups, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, rt, st, img, ker, Bmat, ldb, C, ldc, safe); break;
		case 2: conv_short_k<SP4,2><<<groups, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, rt, st, img, ker, Bmat, ldb, C, ldc, safe); break;
		case 3: conv_short_k<SP4,3><<<groups, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, rt, st, img, ker, Bmat, ldb, C, ldc, safe); break;
		default: conv_short_k<SP4,4><<<groups, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, rt, st, img, ker, Bmat, ldb, C, ldc, safe); break;
	}
}

// Few rows under a very long summed index (the kernel gradient of a first layer:
// 25 x 32 results, each a sum over 73728 pixels): a workgroup takes a stretch of the
// summed index, its four waves a quarter each; a lane gathers A[m][s] for its row
// and its summed index of the step and reads B[s][n] beside it, nothing is laid out
// in memory first.  The waves' sums meet in LDS in wave order; the workgroups' sums
// go side by side into `partial` ([workgroup][m][Np]) for conv_ranges_sum_k.
constexpr int CF_MAX_M = 32, CF_STRETCH = 256;

template <int RB, int CB>
__global__ __launch_bounds__(CG_BLOCK) void conv_fewrows_k (ConvGemmPlan p,
	const ConvTabEntry* __restrict__ rowtab, const ConvTabEntry* __restrict__ sumtab, const float* __restrict__ img,
	const float* __restrict__ Bmat, int64_t ldb, float* __restrict__ partial, int64_t safe)
{
	__shared__ conv_f4 meet[3][RB * CB][64];
	const uint32_t lane = threadIdx.x & 63u, r16 = lane & 15u, q = lane >> 4, wave = threadIdx.x >> 6;
	uint32_t ext[4];
#pragma unroll
	for (int j = 0; j < 4; ++j) { ext[j] = j < p.ncheck ? p.check_ext[j] : 0xffffffffu; }
	ConvTabEntry row[RB];
	bool real[RB];
#pragma unroll
	for (int rb = 0; rb < RB; ++rb)
	{
		const uint32_t m = 16 * rb + r16;
		real[rb] = m < p.M;
		row[rb] = rowtab[real[rb] ? m : 0];
	}
	conv_f4 acc[RB][CB];
#pragma unroll
	for (int rb = 0; rb < RB; ++rb)
	{
#pragma unroll
		for (int cb = 0; cb < CB; ++cb) { acc[rb][cb] = conv_f4{0.f, 0.f, 0.f, 0.f}; }
	}
	// a wave's sixteen steps in three sweeps, so that it waits for memory twice, not
	// twice per step: the table entries of its summed indices, then every element of A
	// and B, then the matrix instructions
	constexpr int STEPS = CF_STRETCH / 4 / 4;
	const uint32_t begin = blockIdx.x * CF_STRETCH + wave * (CF_STRETCH / 4);
	ConvTabEntry col[STEPS];
#pragma unroll
	for (int j = 0; j < STEPS; ++j)
	{
		const uint32_t s = begin + 4 * j + q;
		col[j] = sumtab[s < p.S ? s : 0];
	}
	float a[STEPS][RB], b[STEPS][CB];
#pragma unroll
	for (int j = 0; j < STEPS; ++j)
	{
		const uint32_t s = begin + 4 * j + q;
		const bool there = s < p.S;
#pragma unroll
		for (int rb = 0; rb < RB; ++rb)
		{
			bool inside = real[rb] & there;
#pragma unroll
			for (int k = 0; k < 4; ++k) { inside = inside & ((uint32_t) (row[rb].c[k] + col[j].c[k]) < ext[k]); }
			const float v = img[inside ? row[rb].off + col[j].off : safe];
			a[j][rb] = inside ? v : 0.f;
		}
#pragma unroll
		for (int cb = 0; cb < CB; ++cb)
		{
			const float v = Bmat[(int64_t) (there ? s : 0) * ldb + 16 * cb + r16];
			b[j][cb] = there ? v : 0.f;
		}
	}
#pragma unroll
	for (int j = 0; j < STEPS; ++j)
	{
#pragma unroll
		for (int rb = 0; rb < RB; ++rb)
		{
#pragma unroll
			for (int cb = 0; cb < CB; ++cb) { acc[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j][rb], b[j][cb], acc[rb][cb], 0, 0, 0); }
		}
	}
	if (wave > 0)
	{
#pragma unroll
		for (int rb = 0; rb < RB; ++rb)
		{
#pragma unroll
			for (int cb = 0; cb < CB; ++cb) { meet[wave - 1][rb * CB + cb][lane] = acc[rb][cb]; }
		}
	}
	__syncthreads();
	if (wave > 0) { return; }
	float* to = partial + (uint64_t) blockIdx.x * p.M * p.Np;
#pragma unroll
	for (int rb = 0; rb < RB; ++rb)
	{
#pragma unroll
		for (int cb = 0; cb < CB; ++cb)
		{
			conv_f4 sum = acc[rb][cb];
#pragma unroll
			for (int w = 0; w < 3; ++w) { sum += meet[w][rb * CB + cb][lane]; }
			// a lane holds rows 4 q .. 4 q + 3 of column r16 of the block
			const uint32_t m = 16 * rb + 4 * q, n = 16 * cb + r16;
			if (m < p.M) { to[m * p.Np + n] = sum.x; }
			if (m + 1 < p.M) { to[(m + 1) * p.Np + n] = sum.y; }
			if (m + 2 < p.M) { to[(m + 2) * p.Np + n] = sum.z; }
			if (m + 3 < p.M) { to[(m + 3) * p.Np + n] = sum.w; }
		}
	}
}

// C[m][n] = the sum of partial[g][m][n] over g: a wave per result; lane l adds the
// workgroups l, l + 64, ... in that order, then the 64 lane sums meet in a fixed tree
__global__ __launch_bounds__(CG_BLOCK) void conv_ranges_sum_k (const float* __restrict__ partial, uint32_t groups, uint32_t M, uint32_t Np,
	float* __restrict__ C, int64_t ldc)
{
	const uint32_t i = blockIdx.x * (CG_BLOCK / 64) + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
	if (i >= M * Np) { return; }
	float acc = 0.f;
	for (uint32_t g = lane; g < groups; g += 64) { acc += partial[(uint64_t) g * M * Np + i]; }
#pragma unroll
	for (int w = 32; w >= 1; w >>= 1) { acc += __shfl_xor(acc, w, 64); }
	if (lane == 0) { C[(int64_t) (i / Np) * ldc + i % Np] = acc; }
}

template <int RB>
void conv_fewrows_launch (tcg_ctx* ctx, const ConvGemmPlan& g, uint32_t groups, const ConvTabEntry* rt, const ConvTabEntry* st,
	const float* img, const float* Bmat, int64_t ldb, float* partial)
{
	int64_t safe = 0;
	for (int d = 0; d < 8; ++d) { safe += (int64_t) g.ilo[d] * g.istr[d]; }
	switch (g.Np / 16)
	{
		case 1: conv_fewrows_k<RB,1><<<groups, CG_BLOCK, 0, ctx->stream>>>(g, rt, st, img, Bmat, ldb, partial, safe); break;
		case 2: conv_fewrows_k<RB,2><<<groups, CG_BLOCK, 0, ctx->stream>>>(g, rt, st, img, Bmat, ldb, partial, safe); break;
		case 3: conv_fewrows_k<RB,3><<<groups, CG_BLOCK, 0, ctx->stream>>>(g, rt, st, img, Bmat, ldb, partial, safe); break;
		default: conv_fewrows_k<RB,4><<<groups, CG_BLOCK, 0, ctx->stream>>>(g, rt, st, img, Bmat, ldb, partial, safe); break;
	}
}

// out[window coordinate of (m, n)] = C[m - m0][n]
template <typename T>
__global__ __launch_bounds__(CG_BLOCK) void conv_scatter_k (ConvGemmPlan p, uint32_t m0, uint32_t rows,
	const T* __restrict__ C, T* __restrict__ out)
{
	const uint64_t total = (uint64_t) rows * p.N;
	const uint64_t step = (uint64_t) gridDim.x * CG_BLOCK;
	for (uint64_t i = (uint64_t) blockIdx.x * CG_BLOCK + threadIdx.x; i < total; i += step)
	{
		uint32_t r = (uint32_t) (i / p.N);
		uint32_t n = (uint32_t) (i - (uint64_t) r * p.N);
		uint32_t rm = m0 + r, rn = n;
		int64_t off = 0;
		for (int j = 0; j < 8; ++j)
		{
			const uint32_t d = p.mord[j];
			uint32_t qm = conv_div(rm, p.mdiv[d]);
			int32_t xm = (int32_t) (rm - qm * p.msize[d]);
			rm = qm;
			if (0 == p.is_col[d]) { off += (int64_t) (p.oxlo[d] + xm) * p.ostr[d]; }
		}
		for (int j = 0; j < 8; ++j)
		{
			const uint32_t d = p.nord[j];
			uint32_t qn = conv_div(rn, p.ndiv[d]);
			uint32_t xq = rn - qn * p.nsize[d];
			rn = qn;
			if (0 == p.is_col[d]) { continue; }
			if (p.nflip[d]) { xq = p.nsize[d] - 1 - xq; }
			off += (int64_t) (p.oxlo[d] + (int32_t) xq) * p.ostr[d];
		}
		out[off] = C[(uint64_t) r * p.Np + n];
	}
}

// Whether the product form pays: enough columns to fill matrix tiles and
// enough work to amortise materialising the operands
bool conv_gemm_plan (const ConvPlan& c, ConvGemmPlan& g)
{
	uint64_t M = 1, N = 1, S = 1;
	for (int d = 0; d < 8; ++d)
	{
		g.msize[d] = g.ssize[d] = g.nsize[d] = 1;
		g.xlo[d] = (int32_t) c.wlo[d];
		g.oxlo[d] = (int32_t) c.wlo[d];
		g.slo[d] = 0;
		g.is_col[d] = 0;
		g.ilo[d] = c.ilo[d];
		g.ihi[d] = c.ihi[d];
		g.ksize[d] = c.ksize[d];
		g.istr[d] = c.istr[d];
		g.ostr[d] = c.ostr[d];
		g.kstr[d] = c.kstr[d];
		if (c.ksize[d] == 1) { g.msize[d] = c.wsize[d]; }
		else if (c.ihi[d] - c.ilo[d] == 1)
		{
			g.nsize[d] = c.wsize[d];
			g.is_col[d] = 1;
		}
		else
		{
			g.msize[d] = c.wsize[d];
			// kernel coordinates that meet the box for some output of the window
			int32_t first = c.ilo[d] - (int32_t) (c.wlo[d] + c.wsize[d] - 1);
			int32_t last = c.ihi[d] - (int32_t) c.wlo[d]; // exclusive
			if (first < 0) { first = 0; }
			if (last > (int32_t) c.ksize[d]) { last = (int32_t) c.ksize[d]; }
			if (last <= first) { return false; } // nothing to sum: the direct kernel writes the zeros
			g.slo[d] = first;
			g.ssize[d] = (uint32_t) (last - first);
		}
		g.mdiv[d] = conv_make_div(g.msize[d]);
		g.sdiv[d] = conv_make_div(g.ssize[d]);
		g.ndiv[d] = conv_make_div(g.nsize[d]);
		g.mord[d] = g.sord[d] = g.nord[d] = (uint32_t) d;
		g.nflip[d] = 0;
		M *= g.msize[d];
		N *= g.nsize[d];
		S *= g.ssize[d];
	}
	// a sum of 25 terms (a 5x5 window over one channel) still goes through the product:
	// the direct kernel took 78.7 us where the product takes 53 us on 100x28x28 images
	if (N < 8 || S < 8 || M < 8 || M >= (1ull << 31) || N >= (1ull << 31) || S >= (1ull << 31)) { return false; }
	if (M * N * S < (1ull << 22)) { return false; }
	g.M = (uint32_t) M;
	g.N = (uint32_t) N;
	g.S = (uint32_t) S;
	g.Sp = (g.S + 3) & ~3u;
	g.Np = (g.N + 3) & ~3u;
	g.ncheck = 0;
	for (int j = 0; j < 4; ++j)
	{
		g.check_dim[j] = -1;
		g.check_ext[j] = 0;
	}
	for (int d = 0; d < 8; ++d)
	{
		if (g.is_col[d]) { continue; }
		// coordinates this dim can take against the box
		int64_t first = (int64_t) g.xlo[d] + g.slo[d];
		int64_t last = first + (g.msize[d] - 1) + (g.ssize[d] - 1);
		if (first >= g.ilo[d] && last < g.ihi[d]) { continue; } // always inside
		if (g.ncheck >= 0 && g.ncheck < 4)
		{
			g.check_dim[g.ncheck] = d;
			g.check_ext[g.ncheck] = (uint32_t) (g.ihi[d] - g.ilo[d]);
			++g.ncheck;
		}
		else { g.ncheck = -1; }
	}
	return true;
}

// Orders of the three indices once the strides are final (see ConvGemmPlan).
// (Rows enumerated batch first, so that the rows of a tile of the product sit at
// one position of the padded dims and the tile can leave out the slabs of the
// summed index that meet nothing but zero border -- 31% of them for the image
// gradient of a 5x5 convolution over 20x20 outputs -- were measured slower than
// multiplying the zeros: 111.4 against 104.7 us.  The rows of such a tile lie a
// whole image apart, and nothing a slab loads is found in L1 again by the next
// kernel position, as it is when neighbouring rows are neighbouring pixels.)
void conv_choose_orders (ConvGemmPlan& g)
{
	if (g.ncheck < 0) { return; } // the general gather decomposes in dim order
	auto mag = [](int64_t v) { return v < 0 ? -v : v; };
	auto sorted = [&](uint32_t* ord, const uint32_t* extent, const int64_t* stride)
	{
		for (int d = 0; d < 8; ++d) { ord[d] = (uint32_t) d; }
		std::stable_sort(ord, ord + 8, [&](uint32_t x, uint32_t y)
		{
			bool sx = extent[x] == 1, sy = extent[y] == 1;
			if (sx != sy) { return sy; }
			return false == sx && mag(stride[x]) < mag(stride[y]);
		});
	};
	sorted(g.sord, g.ssize, g.istr);
	sorted(g.mord, g.msize, g.ostr);
	sorted(g.nord, g.nsize, g.ostr);
	for (int d = 0; d < 8; ++d) { g.nflip[d] = g.is_col[d] && g.nsize[d] > 1 && g.ostr[d] < 0; }
}

// The product's C is the result itself when the result, restricted to the
// window, is a row-major [rows][columns] matrix in the chosen orders; *base:
// offset of C[0][0] from the address of output coordinate 0
bool conv_result_in_place (const ConvGemmPlan& g, int64_t* base, int64_t* ldc)
{
	if (g.ncheck < 0 || g.N % 4 != 0) { return false; }
	int64_t run = 1;
	for (int j = 0; j < 8; ++j)
	{
		uint32_t d = g.nord[j];
		if (g.nsize[d] == 1) { continue; }
		if ((g.nflip[d] ? -g.ostr[d] : g.ostr[d]) != run) { return false; }
		run *= g.nsize[d];
	}
	int64_t ld = 0, expect = 0;
	for (int j = 0; j < 8; ++j)
	{
		uint32_t d = g.mord[j];
		if (g.msize[d] == 1) { continue; }
		if (0 == ld)
		{
			ld = g.ostr[d];
			if (ld < (int64_t) g.N) { return false; }
			expect = ld;
		}
		else if (g.ostr[d] != expect) { return false; }
		expect *= g.msize[d];
	}
	if (0 == ld) { return false; }
	int64_t off = 0;
	for (int d = 0; d < 8; ++d)
	{
		off += (int64_t) (g.oxlo[d] + (g.nflip[d] ? (int32_t) g.nsize[d] - 1 : 0)) * g.ostr[d];
	}
	*base = off;
	*ldc = ld;
	return true;
}

// The product's B is the kernel itself when the kernel elements B[s][n] names
// form a row-major matrix in the chosen orders
bool conv_kernel_in_place (const ConvGemmPlan& g, int64_t* base, int64_t* ldb)
{
	if (g.ncheck < 0 || g.N % 4 != 0 || g.S % 4 != 0) { return false; }
	int64_t run = 1, off = 0;
	for (int j = 0; j < 8; ++j)
	{
		uint32_t d = g.nord[j];
		if (0 == g.is_col[d]) { continue; }
		// the kernel index of column component q is ilo - x(q)
		int32_t xfirst = g.xlo[d] + (g.nflip[d] ? (int32_t) g.nsize[d] - 1 : 0);
		int32_t xlast = g.xlo[d] + (g.nflip[d] ? 0 : (int32_t) g.nsize[d] - 1);
		int32_t wfirst = g.ilo[d] - xfirst, wlast = g.ilo[d] - xlast;
		if (wfirst < 0 || wlast < 0 || wfirst >= (int32_t) g.ksize[d] || wlast >= (int32_t) g.ksize[d]) { return false; }
		if (g.nsize[d] > 1)
		{
			if ((g.nflip[d] ? g.kstr[d] : -g.kstr[d]) != run) { return false; }
			run *= g.nsize[d];
		}
		off += (int64_t) wfirst * g.kstr[d];
	}
	int64_t ld = 0, expect = 0;
	for (int j = 0; j < 8; ++j)
	{
		uint32_t d = g.sord[j];
		if (g.is_col[d]) { continue; }
		if (g.slo[d] < 0 || g.slo[d] + (int32_t) g.ssize[d] > (int32_t) g.ksize[d]) { return false; }
		off += (int64_t) g.slo[d] * g.kstr[d];
		if (g.ssize[d] == 1) { continue; }
		if (0 == ld)
		{
			ld = g.kstr[d];
			if (ld < (int64_t) g.N || ld % 4 != 0) { return false; }
			expect = ld;
		}
		else if (g.kstr[d] != expect) { return false; }
		expect *= g.ssize[d];
	}
	if (0 == ld) { return false; }
	*base = off;
	*ldb = ld;
	return true;
}

// How the matrix-core kernel can read A straight from the image: along which
// index memory runs, and whether aligned groups of four along it are
// contiguous, 16-byte aligned and inside or outside the box together
void conv_operand_mode (const ConvGemmPlan& g, tcg_conv_operand& op)
{
	op.ncheck = g.ncheck;
	for (int j = 0; j < 4; ++j) { op.check_ext[j] = j < g.ncheck ? g.check_ext[j] : 0; }
	op.along_m = false;
	op.vec4 = false;
	// the dim that lies along memory
	int f = -1;
	for (int d = 0; d < 8 && f < 0; ++d)
	{
		if (0 == g.is_col[d] && (g.msize[d] > 1 || g.ssize[d] > 1) && g.istr[d] == 1) { f = d; }
	}
	if (f < 0) { return; }
	// both indices may step along the contiguous dim (a spatial dim carries an
	// output coordinate and a kernel coordinate): the longer run wins, and it
	// must be the first dim its index steps along
	op.along_m = g.msize[f] >= g.ssize[f];
	const uint32_t* ord = op.along_m ? g.mord : g.sord;
	const uint32_t* extent = op.along_m ? g.msize : g.ssize;
	for (int j = 0; j < 8; ++j)
	{
		if (extent[ord[j]] == 1) { continue; }
		if ((int) ord[j] != f) { return; }
		break;
	}
	bool checked = false;
	for (int j = 0; j < g.ncheck; ++j) { checked = checked || g.check_dim[j] == f; }
	uint32_t run = op.along_m ? g.msize[f] : g.ssize[f], other = op.along_m ? g.ssize[f] : g.msize[f];
	bool vec = false == checked && run % 4 == 0 && other == 1 && (g.xlo[f] + g.slo[f]) % 4 == 0;
	for (int d = 0; d < 8 && vec; ++d)
	{
		if (d == f || g.istr[d] % 4 == 0) { continue; }
		// a dim with an odd stride may only add a constant multiple of four
		int64_t fixed = g.is_col[d] ? g.ilo[d] : g.xlo[d] + g.slo[d];
		vec = g.msize[d] == 1 && g.ssize[d] == 1 && (fixed * g.istr[d]) % 4 == 0;
	}
	op.vec4 = vec;
}

// Whether the product can read its A operand out of a patch of the image in LDS
// (conv_patch.hip), and with which of that kernel's tiles: worked out on the host
// from the same formulas as the tables.  It pays when the rows of a tile meet
// the same image elements many times over and the tiles fill the chip evenly.
tcg_conv_patch conv_patch_prepare (const tcg_ctx* ctx, const ConvGemmPlan& g, const tcg_conv_operand& op)
{
	tcg_conv_patch none, pp;
	if (op.along_m || false == op.vec4 || g.ncheck < 0 || g.ncheck > 2 || g.S != g.Sp || g.S % 32 != 0 || g.S < 128 || g.S > 8192 ||
		g.N % 32 != 0 || g.N != g.Np || (uint64_t) g.M * g.N * g.S < (1ull << 28) || g.M > (1u << 22)) // (the row offsets are worked out here, once per plan)
	{
		return none;
	}
	const int64_t limit = (int64_t) 1 << 30;
	// image elements that exist
	int64_t vlo = 0, vhi = 1;
	for (int d = 0; d < 8; ++d)
	{
		const int64_t first = g.ilo[d], last = g.is_col[d] ? g.ilo[d] : g.ihi[d] - 1;
		if (g.istr[d] < 0) { return none; }
		vlo += first * g.istr[d];
		vhi += last * g.istr[d];
	}
	if (vlo % 4 != 0 || vhi % 4 != 0 || vlo < -limit || vhi > limit) { return none; }
	// offsets of the summed index at the multiples of four
	int64_t smin = INT64_MAX, smax = INT64_MIN;
	for (uint32_t s = 0; s < g.S; s += 4)
	{
		uint32_t rs = s;
		int64_t off = 0;
		for (int j = 0; j < 8; ++j)
		{
			const uint32_t d = g.sord[j];
			const int64_t w = (int64_t) (rs % g.ssize[d]) + g.slo[d];
			rs /= g.ssize[d];
			off += w * g.istr[d];
		}
		smin = std::min(smin, off);
		smax = std::max(smax, off);
	}
	// offsets of the rows
	std::vector<int64_t> rowoff(g.M);
	for (uint32_t m = 0; m < g.M; ++m)
	{
		uint32_t rm = m;
		int64_t off = 0;
		for (int j = 0; j < 8; ++j)
		{
			const uint32_t d = g.mord[j];
			const int64_t x = rm % g.msize[d];
			rm /= g.msize[d];
			off += (g.is_col[d] ? (int64_t) g.ilo[d] : (int64_t) g.xlo[d] + x) * g.istr[d];
		}
		if (off < -limit || off > limit || (off + smin) % 4 != 0) { return none; }
		rowoff[m] = off;
	}
	if (smin < -limit || smax > limit) { return none; }
	// neighbouring rows a power of two apart: padding behind every such stretch keeps
	// the sixteen rows of a matrix instruction in different banks
	uint32_t pad_shift = 31;
	if (g.M > 1)
	{
		const int64_t step = rowoff[1] > rowoff[0] ? rowoff[1] - rowoff[0] : rowoff[0] - rowoff[1];
		if (step >= 16 && step <= 4096 && (step & (step - 1)) == 0)
		{
			pad_shift = 0;
			while (((int64_t) 1 << pad_shift) < step) { ++pad_shift; }
		}
	}
	double best = 0;
	for (int which = 0; which < tcg_conv_patch_shapes(); ++which)
	{
		uint32_t tm = 0, tn = 0, threads = 0;
		tcg_conv_patch_shape(which, &tm, &tn, &threads);
		if (g.N % tn != 0) { continue; }
		int64_t span = 0;
		for (uint32_t m0 = 0; m0 < g.M; m0 += tm)
		{
			const uint32_t m1 = std::min(g.M, m0 + tm);
			const auto mm = std::minmax_element(rowoff.begin() + m0, rowoff.begin() + m1);
			span = std::max(span, *mm.second - *mm.first);
		}
		const int64_t stretch = span + (smax - smin) + 4;
		if (stretch > (int64_t) (TCG_CONV_PATCH_LDS / sizeof(float))) { continue; }
		const uint32_t floats = (uint32_t) (stretch + ((stretch >> pad_shift) << 2) + 4);
		const size_t lds = tcg_conv_patch_lds(which, floats, g.S, g.ncheck);
		if (lds > TCG_CONV_PATCH_LDS) { continue; }
		// elements of A a tile reads per element it copies
		if ((double) tm * g.S < 4.0 * (double) stretch) { continue; }
		const uint64_t tiles = (uint64_t) ((g.M + tm - 1) / tm) * (g.N / tn);
		// how evenly the tiles fall on the CUs (the tiles of a CU share its matrix pipes,
		// so the CU with the most tiles sets the time); wider tiles read B less often
		const uint64_t cus = (uint64_t) ctx->num_cus;
		const uint64_t most = (tiles + cus - 1) / cus;
		// (a tile as wide as the result copies the stretch of the image once, not once per column of tiles:
		// 51200 x 64 x 800 took 59.5 us with tiles of 112 x 64 and 66.5 us with 144 x 32)
		double score = (double) tiles / (double) (most * cus) * (1.0 + tm / 2048.0) * (tn == g.N ? 1.15 : 1.0);
		if (const char* force = getenv("TCG_CONV_PATCH_SHAPE")) { score = atoi(force) == which ? 10.0 : score * 0.01; } // for measurements and tests
		if (score > best)
		{
			best = score;
			pp.shape = which;
			pp.patch_floats = floats;
		}
	}
	if (pp.shape < 0) { return none; }
	pp.smin = (int32_t) smin;
	pp.smax = (int32_t) smax;
	pp.vlo = (int32_t) vlo;
	pp.vhi = (int32_t) vhi;
	pp.pad_shift = pad_shift;
	return pp;
}

template <typename T>
int conv_gemm_run (tcg_ctx* ctx, int dtype, const ConvGemmPlan& g, const T* img, const T* ker, T* out)
{
	// rows of A per pass: at most 512 MiB of gathered image at a time
	uint64_t max_rows = ((512ull << 20) / sizeof(T)) / g.Sp;
	if (const char* env = getenv("TCG_CONV_CHUNK_ROWS")) // for tests of the chunked path
	{
		uint64_t forced = strtoull(env, nullptr, 10);
		if (forced) { max_rows = forced; }
	}
	if (max_rows < 64) { max_rows = 64; }
	max_rows &= ~(uint64_t) 63;
	uint32_t chunk = (uint32_t) (g.M < max_rows ? g.M : max_rows);
	const bool tables = g.ncheck >= 0;
	// operands and results that already are the matrices of the product stay where they are
	const char* place_env = getenv("TCG_CONV_IN_PLACE"); // "0": always gather B and scatter C (for tests)
	const bool in_place = !(place_env && place_env[0] == '0');
	int64_t b_base = 0, b_ld = 0, c_base = 0, c_ld = 0;
	bool direct_b = in_place && conv_kernel_in_place(g, &b_base, &b_ld) && tcg_aligned16(ker + b_base);
	bool direct_c = in_place && conv_result_in_place(g, &c_base, &c_ld);
	size_t a_bytes = sizeof(T) * (size_t) chunk * g.Sp;
	size_t b_bytes = sizeof(T) * (size_t) g.Sp * g.Np;
	size_t c_bytes = sizeof(T) * (size_t) chunk * g.Np;
	size_t rt_bytes = sizeof(ConvTabEntry) * (size_t) g.M;
	size_t st_bytes = sizeof(ConvTabEntry) * (size_t) g.Sp + sizeof(int64_t) * ((size_t) g.Sp + g.Np); // sums, then kernel offsets
	void *A = nullptr, *B = nullptr, *C = nullptr, *RT = nullptr, *ST = nullptr;
	// fp32: the product reads A through the tables, nothing is gathered
	const char* impl_env = getenv("TCG_CONV_IMPLICIT"); // "0": always materialise A (the parity reference)
	bool implicit = std::is_same<T,float>::value && tables && !(impl_env && impl_env[0] == '0');
	int rc = TCG_OK;
	if (false == direct_b) { rc = tcg_alloc(ctx, b_bytes, &B); }
	if (rc == TCG_OK && false == direct_c) { rc = tcg_alloc(ctx, c_bytes, &C); }
	// the tables depend on the plan alone: kept with the context, filled once
	bool kept_tables = false, fill_tables = tables;
	tcg_ctx::ConvTables* kept_entry = nullptr;
	if (rc == TCG_OK && tables)
	{
		std::string key((const char*) &g, sizeof(g));
		auto it = ctx->conv_tables.find(key);
		if (it != ctx->conv_tables.end())
		{
			RT = it->second.rows;
			ST = it->second.sums;
			kept_tables = true;
			fill_tables = false;
			kept_entry = &it->second;
		}
		else if (ctx->conv_table_bytes + rt_bytes + st_bytes <= tcg_ctx::conv_table_limit)
		{
			tcg_ctx::ConvTables kept;
			if (hipMalloc(&kept.rows, rt_bytes) == hipSuccess && hipMalloc(&kept.sums, st_bytes) == hipSuccess)
			{
				RT = kept.rows;
				ST = kept.sums;
				kept_tables = true;
				kept_entry = &ctx->conv_tables.emplace(key, kept).first->second;
				ctx->conv_table_bytes += rt_bytes + st_bytes;
			}
			else
			{
				(void) hipGetLastError();
				if (kept.rows) { (void) hipFree(kept.rows); }
			}
		}
	}
	if (rc == TCG_OK && tables && false == kept_tables) { rc = tcg_alloc(ctx, rt_bytes, &RT); }
	if (rc == TCG_OK && tables && false == kept_tables) { rc = tcg_alloc(ctx, st_bytes, &ST); }
	if (rc == TCG_OK)
	{
		unsigned grid = 0;
		const T* Bmat = direct_b ? ker + b_base : (const T*) B;
		const uint64_t ldb = direct_b ? (uint64_t) b_ld : g.Np;
		const uint64_t ldc = direct_c ? (uint64_t) c_ld : g.Np;
		if (fill_tables)
		{
			uint32_t longest = g.M > g.Sp ? g.M : g.Sp;
			if (g.Np > longest) { longest = g.Np; }
			hipStream_t where = ctx->stream;
			if (kept_tables && ctx->capturing)
			{
				// kept tables are filled once, now, not by the recording at every replay
				where = ctx->side_stream;
			}
			conv_tables_k<<<(longest + CG_BLOCK - 1) / CG_BLOCK, CG_BLOCK, 0, where>>>(g,
				(ConvTabEntry*) RT, (ConvTabEntry*) ST);
			if (where != ctx->stream) { rc = hipStreamSynchronize(where) == hipSuccess ? TCG_OK : tcg_fail(ctx, TCG_ERR_HIP, "conv tables: %s", hipGetErrorString(hipGetLastError())); }
		}
		tcg_conv_operand operand;
		if (implicit)
		{
			conv_operand_mode(g, operand);
			// only where the gathers can be 128 bits wide: gathering element by
			// element inside the product measured slower than materialising A with
			// the coalesced gather kernel (image gradient of a 5x5 convolution:
			// 285 vs 300 us for both steps, but 214-253 vs 76 us on a kernel gradient
			// with 25 rows, whichever index ran along the lanes)
			implicit = operand.vec4;
		}
		// the image's patch in LDS where that pays (TCG_CONV_PATCH=0: never, for tests)
		tcg_conv_patch patch;
		const char* patch_env = getenv("TCG_CONV_PATCH");
		if (implicit && chunk == g.M && !(patch_env && patch_env[0] == '0'))
		{
			if (kept_entry && kept_entry->patch_known)
			{
				patch.shape = kept_entry->patch_shape;
				patch.smin = kept_entry->patch_smin; patch.smax = kept_entry->patch_smax;
				patch.vlo = kept_entry->patch_vlo; patch.vhi = kept_entry->patch_vhi;
				patch.pad_shift = kept_entry->patch_pad_shift; patch.patch_floats = kept_entry->patch_floats;
			}
			else
			{
				patch = conv_patch_prepare(ctx, g, operand);
				if (kept_entry)
				{
					kept_entry->patch_known = true;
					kept_entry->patch_shape = patch.shape;
					kept_entry->patch_smin = patch.smin; kept_entry->patch_smax = patch.smax;
					kept_entry->patch_vlo = patch.vlo; kept_entry->patch_vhi = patch.vhi;
					kept_entry->patch_pad_shift = patch.pad_shift; kept_entry->patch_floats = patch.patch_floats;
				}
			}
		}
		// the kernel laid out as B: by a launch of its own, or by the workgroups that the
		// launch which lays out the first rows of A has left over
		// (the latter only for a small kernel behind a launch one workgroup wide: the extra
		// workgroups are counted along y, and a launch many workgroups wide would start that
		// many idle ones for each of them -- 498 us for a kernel of 73728 x 32 elements)
		bool gather_b = false == direct_b;
		const bool fold_b = tables && g.Sp <= (uint32_t) CG_BLOCK && (uint64_t) g.Sp * g.Np <= ((uint64_t) 1 << 16);
		if (gather_b && (implicit || false == fold_b))
		{
			grid = tcg_grid(ctx, (uint64_t) g.Sp * g.Np, CG_BLOCK, 16);
			if (tables && (uint64_t) g.Sp * g.Np < (1ull << 32))
			{
				const int64_t* ktab = (const int64_t*) ((const ConvTabEntry*) ST + g.Sp);
				conv_gather_kernel_tab_k<T><<<grid, CG_BLOCK, 0, ctx->stream>>>(g.Sp, g.Np, ktab, ker, (T*) B);
			}
			else { conv_gather_kernel_k<T><<<grid, CG_BLOCK, 0, ctx->stream>>>(g, ker, (T*) B); }
			gather_b = false;
		}
		for (uint32_t m0 = 0; m0 < g.M && rc == TCG_OK; m0 += chunk)
		{
			uint32_t rows = g.M - m0 < chunk ? g.M - m0 : chunk;
			T* Cmat = direct_c ? out + c_base + (int64_t) m0 * c_ld : (T*) C;
			if constexpr (std::is_same<T,float>::value)
			{
				if (implicit)
				{
					operand.rows = (const ConvTabEntry*) RT + m0;
					operand.sums = (const ConvTabEntry*) ST;
					bool handled = false;
					if (patch.shape >= 0 && rows == g.M)
					{
						rc = tcg_conv_patch_f32(ctx, rows, g.Np, g.S, img, operand, patch, (const float*) Bmat, ldb,
							(float*) Cmat, ldc, &handled);
						if (rc != TCG_OK) { break; }
					}
					if (false == handled)
					{
						rc = tcg_gemm_f32_mfma_conv(ctx, rows, g.Np, g.S, img, operand, (const float*) Bmat, ldb,
							(float*) Cmat, ldc, &handled);
					}
					if (rc != TCG_OK) { break; }
					if (handled)
					{
						if (false == direct_c)
						{
							grid = tcg_grid(ctx, (uint64_t) rows * g.N, CG_BLOCK, 16);
							conv_scatter_k<T><<<grid, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, (const T*) C, out);
						}
						continue;
					}
					implicit = false; // shapes the matrix-core kernel does not take: gather as below
				}
			}
			if constexpr (std::is_same<T,float>::value)
			{
				// a short summed index and few columns: gather, product and the kernel's layout in one launch
				const char* short_env = getenv("TCG_CONV_SHORT"); // "0": gather and multiply (for tests)
				if (tables && g.Sp <= (uint32_t) CS_MAX_S && g.Np <= (uint32_t) CS_MAX_N && g.Np % 16 == 0 &&
					!(short_env && short_env[0] == '0'))
				{
					const ConvTabEntry* rt = (const ConvTabEntry*) RT;
					const ConvTabEntry* st = (const ConvTabEntry*) ST;
					const float* kb = gather_b ? (const float*) ker : nullptr;
					switch (g.Sp / 4)
					{
						case 1: conv_short_launch<1>(ctx, g, m0, rows, rt, st, img, kb, (const float*) Bmat, (int64_t) ldb, (float*) Cmat, (int64_t) ldc); break;
						case 2: conv_short_launch<2>(ctx, g, m0, rows, rt, st, img, kb, (const float*) Bmat, (int64_t) ldb, (float*) Cmat, (int64_t) ldc); break;
						case 3: conv_short_launch<3>(ctx, g, m0, rows, rt, st, img, kb, (const float*) Bmat, (int64_t) ldb, (float*) Cmat, (int64_t) ldc); break;
						case 4: conv_short_launch<4>(ctx, g, m0, rows, rt, st, img, kb, (const float*) Bmat, (int64_t) ldb, (float*) Cmat, (int64_t) ldc); break;
						case 5: conv_short_launch<5>(ctx, g, m0, rows, rt, st, img, kb, (const float*) Bmat, (int64_t) ldb, (float*) Cmat, (int64_t) ldc); break;
						case 6: conv_short_launch<6>(ctx, g, m0, rows, rt, st, img, kb, (const float*) Bmat, (int64_t) ldb, (float*) Cmat, (int64_t) ldc); break;
						case 7: conv_short_launch<7>(ctx, g, m0, rows, rt, st, img, kb, (const float*) Bmat, (int64_t) ldb, (float*) Cmat, (int64_t) ldc); break;
						default: conv_short_launch<8>(ctx, g, m0, rows, rt, st, img, kb, (const float*) Bmat, (int64_t) ldb, (float*) Cmat, (int64_t) ldc); break;
					}
					++ctx->conv_short_launches;
					if (false == direct_c)
					{
						grid = tcg_grid(ctx, (uint64_t) rows * g.N, CG_BLOCK, 16);
						conv_scatter_k<T><<<grid, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, (const T*) C, out);
					}
					continue;
				}
			}
			if constexpr (std::is_same<T,float>::value)
			{
				// few rows under a very long summed index: gathered and multiplied stretch by stretch, then summed
				const char* few_env = getenv("TCG_CONV_FEWROWS"); // "0": gather and multiply (for tests)
				if (tables && rows == g.M && g.M <= (uint32_t) CF_MAX_M && g.Np <= (uint32_t) CS_MAX_N && g.Np % 16 == 0 &&
					g.S >= 4096 && false == gather_b && !(few_env && few_env[0] == '0'))
				{
					const uint32_t groups = (g.S + CF_STRETCH - 1) / CF_STRETCH;
					const size_t partial_bytes = sizeof(float) * (size_t) groups * g.M * g.Np;
					void* partial = nullptr;
					rc = tcg_alloc(ctx, partial_bytes, &partial);
					if (rc != TCG_OK) { break; }
					const ConvTabEntry* rt = (const ConvTabEntry*) RT;
					const ConvTabEntry* st = (const ConvTabEntry*) ST;
					if (g.M <= 16) { conv_fewrows_launch<1>(ctx, g, groups, rt, st, img, (const float*) Bmat, (int64_t) ldb, (float*) partial); }
					else { conv_fewrows_launch<2>(ctx, g, groups, rt, st, img, (const float*) Bmat, (int64_t) ldb, (float*) partial); }
					const uint32_t results = g.M * g.Np;
					conv_ranges_sum_k<<<(results + CG_BLOCK / 64 - 1) / (CG_BLOCK / 64), CG_BLOCK, 0, ctx->stream>>>((const float*) partial, groups,
						g.M, g.Np, (float*) Cmat, (int64_t) ldc);
					tcg_free(ctx, partial, partial_bytes);
					++ctx->conv_fewrows_launches;
					if (false == direct_c)
					{
						grid = tcg_grid(ctx, (uint64_t) rows * g.N, CG_BLOCK, 16);
						conv_scatter_k<T><<<grid, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, (const T*) C, out);
					}
					continue;
				}
			}
			if (nullptr == A)
			{
				rc = tcg_alloc(ctx, a_bytes, &A);
				if (rc != TCG_OK) { break; }
			}
			if (tables)
			{
				const uint32_t per_block = g.Sp <= CG_BLOCK / 2 ? CG_NARROW_ROWS : CG_ROWS;
				const uint32_t row_blocks = (rows + per_block - 1) / per_block;
				uint32_t kernel_blocks = 0;
				if (gather_b)
				{
					kernel_blocks = (uint32_t) (((uint64_t) g.Sp * g.Np + CG_BLOCK - 1) / CG_BLOCK);
					if (kernel_blocks > 1024) { kernel_blocks = 1024; }
				}
				dim3 tgrid((g.Sp + CG_BLOCK - 1) / CG_BLOCK, row_blocks + kernel_blocks);
				const ConvTabEntry* rt = (const ConvTabEntry*) RT;
				const ConvTabEntry* st = (const ConvTabEntry*) ST;
				const T* kb = gather_b ? ker : nullptr;
				switch (g.ncheck)
				{
					case 0: conv_gather_tab_k<T,0><<<tgrid, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, rt, st, img, (T*) A, row_blocks, kb, (T*) B); break;
					case 1: conv_gather_tab_k<T,1><<<tgrid, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, rt, st, img, (T*) A, row_blocks, kb, (T*) B); break;
					case 2: conv_gather_tab_k<T,2><<<tgrid, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, rt, st, img, (T*) A, row_blocks, kb, (T*) B); break;
					case 3: conv_gather_tab_k<T,3><<<tgrid, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, rt, st, img, (T*) A, row_blocks, kb, (T*) B); break;
					default: conv_gather_tab_k<T,4><<<tgrid, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, rt, st, img, (T*) A, row_blocks, kb, (T*) B); break;
				}
				gather_b = false;
			}
			else
			{
				grid = tcg_grid(ctx, (uint64_t) rows * g.Sp, CG_BLOCK, 32);
				conv_gather_image_k<T><<<grid, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, img, (T*) A);
			}
			// (a kernel read in place has S rows: S is then a multiple of four and equals Sp)
			rc = tcg_gemm(ctx, dtype, rows, g.Np, g.Sp, 1, A, g.Sp, 0, 0, Bmat, ldb, 0, 0, Cmat, ldc, 0);
			if (rc != TCG_OK) { break; }
			if (false == direct_c)
			{
				grid = tcg_grid(ctx, (uint64_t) rows * g.N, CG_BLOCK, 16);
				conv_scatter_k<T><<<grid, CG_BLOCK, 0, ctx->stream>>>(g, m0, rows, (const T*) C, out);
			}
		}
	}
	if (A) { tcg_free(ctx, A, a_bytes); }
	if (B) { tcg_free(ctx, B, b_bytes); }
	if (C) { tcg_free(ctx, C, c_bytes); }
	if (RT && false == kept_tables) { tcg_free(ctx, RT, rt_bytes); }
	if (ST && false == kept_tables) { tcg_free(ctx, ST, st_bytes); }
	if (rc != TCG_OK) { return rc; }
	TCG_LAUNCH_CHECK(ctx, "conv_gemm");
	return TCG_OK;
}

} // namespace

extern "C" {

// dense_box: `img` holds only the elements inside [img_lo, img_hi), densely,
// or with the element strides `box_stride` when those are given.
// kernel_stride (per kernel dim) / out_stride (per output dim; `out` is then
// the address of the first output of the window): element strides of the
// kernel and of the result when they are not the dense ones.
static int conv_boxed_impl (tcg_ctx* ctx, int dtype, const uint64_t imgshape[8],
	const uint64_t kshape[8], int nranks, const uint64_t* ranks,
	const uint64_t img_lo[8], const uint64_t img_hi[8],
	const uint64_t out_lo[8], const uint64_t out_hi[8],
	const void* img, const void* kernel, void* out, bool dense_box,
	const int64_t* box_stride = nullptr, const int64_t* kernel_stride = nullptr, const int64_t* out_stride = nullptr)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, imgshape && kshape && img && kernel && out && (ranks || nranks == 0), "tcg_conv: NULL pointer");
	if (nranks > 8) { nranks = 8; }
	uint64_t order[8];
	bool visited[8] = {false};
	for (int i = 0; i < nranks; ++i)
	{
		TCG_REQUIRE(ctx, ranks[i] < 8, "tcg_conv: rank %llu >= 8", (unsigned long long) ranks[i]);
		TCG_REQUIRE(ctx, !visited[ranks[i]], "tcg_conv: convolution does not support repeated kernel dimensions");
		visited[ranks[i]] = true;
		order[i] = ranks[i];
	}
	for (int i = nranks; i < 8; ++i)
	{
		TCG_REQUIRE(ctx, kshape[i] <= 1, "tcg_conv: unspecified non-singular kernel dimension %d is undefined", i);
	}
	for (int i = 0, j = nranks; i < 8; ++i)
	{
		if (!visited[i]) { order[j++] = i; }
	}
	ConvPlan p;
	uint64_t oshape[8];
	int64_t kmem[8];
	kmem[0] = 1;
	for (int i = 1; i < 8; ++i) { kmem[i] = kmem[i - 1] * (int64_t) kshape[i - 1]; }
	for (int d = 0; d < 8; ++d)
	{
		TCG_REQUIRE(ctx, imgshape[d] >= 1 && imgshape[d] < (1ull << 31) && kshape[d] >= 1,
			"tcg_conv: dim %d is empty or too large", d);
		oshape[d] = imgshape[d];
	}
	// kernel dim i slides along image dim order[i]
	for (int i = 0; i < 8; ++i)
	{
		uint64_t d = order[i];
		TCG_REQUIRE(ctx, kshape[i] <= oshape[d], "tcg_conv: cannot convolve a kernel against a smaller image (kernel dim %d)", i);
		oshape[d] -= kshape[i] - 1;
		p.ksize[d] = (uint32_t) kshape[i];
		p.kstr[d] = kernel_stride ? kernel_stride[i] : kmem[i];
	}
	p.istr[0] = p.ostr[0] = 1;
	for (int d = 1; d < 8; ++d)
	{
		p.istr[d] = p.istr[d - 1] * (int64_t) imgshape[d - 1];
		p.ostr[d] = p.ostr[d - 1] * (int64_t) oshape[d - 1];
	}
	uint64_t max_terms = 1;
	for (int d = 0; d < 8; ++d)
	{
		uint64_t ilo = img_lo ? img_lo[d] : 0, ihi = img_hi ? img_hi[d] : imgshape[d];
		uint64_t olo = out_lo ? out_lo[d] : 0, ohi = out_hi ? out_hi[d] : oshape[d];
		TCG_REQUIRE(ctx, ilo <= ihi && ihi <= imgshape[d], "tcg_conv: image box [%llu,%llu) leaves dim %d of extent %llu",
			(unsigned long long) ilo, (unsigned long long) ihi, d, (unsigned long long) imgshape[d]);
		TCG_REQUIRE(ctx, olo < ohi && ohi <= oshape[d], "tcg_conv: output window [%llu,%llu) leaves dim %d of extent %llu",
			(unsigned long long) olo, (unsigned long long) ohi, d, (unsigned long long) oshape[d]);
		p.ilo[d] = (int32_t) ilo;
		p.ihi[d] = (int32_t) ihi;
		p.wlo[d] = (uint32_t) olo;
		p.wsize[d] = (uint32_t) (ohi - olo);
		p.nwin *= p.wsize[d];
		uint64_t span = ihi - ilo < p.ksize[d] ? ihi - ilo : p.ksize[d];
		max_terms *= span;
	}
	if (out_stride)
	{
		for (int d = 0; d < 8; ++d)
		{
			p.ostr[d] = out_stride[d];
			p.ooff0 -= (int64_t) p.wlo[d] * out_stride[d];
		}
	}
	ConvGemmPlan gp; // (zeroed by its constructor: its bytes name the tables computed from it)
	const char* gemm_env = getenv("TCG_CONV_GEMM"); // "0": direct kernels only (the parity reference)
	// (the product route exists for the three default types)
	if (!(gemm_env && gemm_env[0] == '0') && tcg_default_dtype(dtype) && conv_gemm_plan(p, gp))
	{
		// An image that is mostly padding (conv2d's image gradient pads the
		// fastest dim from 1 to 2*C - 1) scatters its non-zero elements over
		// memory: cut the box out into a dense buffer first, unless the box is
		// one contiguous slab already (only the slowest dim is cut)
		uint64_t box[8], lo[8], box_elems = 1, img_elems = 1;
		int last_sig = 0, first_cut = 8;
		for (int d = 0; d < 8; ++d)
		{
			lo[d] = (uint64_t) p.ilo[d];
			box[d] = (uint64_t) (p.ihi[d] - p.ilo[d]);
			box_elems *= box[d];
			img_elems *= imgshape[d];
			if (imgshape[d] > 1) { last_sig = d; }
			if (box[d] < imgshape[d] && d < first_cut) { first_cut = d; }
		}
		size_t esz = tcg_type_size(dtype);
		bool compact = false == dense_box && esz && box_elems > 0 && first_cut < last_sig &&
			box_elems * 2 <= img_elems && box_elems * esz <= (1ull << 30);
		void* dense = nullptr;
		if (compact)
		{
			int rc = tcg_alloc(ctx, box_elems * esz, &dense);
			if (rc == TCG_OK) { rc = tcg_slice(ctx, dtype, imgshape, lo, box, img, dense); }
			if (rc != TCG_OK)
			{
				if (dense) { tcg_free(ctx, dense, box_elems * esz); }
				return rc;
			}
			img = dense;
		}
		if (compact || dense_box)
		{
			int64_t run = 1;
			for (int d = 0; d < 8; ++d)
			{
				gp.xlo[d] -= p.ilo[d];
				gp.ilo[d] = 0;
				gp.ihi[d] = (int32_t) box[d];
				gp.istr[d] = (dense_box && box_stride) ? box_stride[d] : run;
				run *= (int64_t) box[d];
			}
		}
		if (out_stride)
		{
			// `out` starts at the window
			for (int d = 0; d < 8; ++d) { gp.oxlo[d] = 0; }
		}
		conv_choose_orders(gp);
		int rc = TCG_OK;
		TCG_DISPATCH_TYPE(ctx, dtype, rc = conv_gemm_run<T>(ctx, dtype, gp, (const T*) img, (const T*) kernel, (T*) out));
		if (dense) { tcg_free(ctx, dense, box_elems * esz); }
		return rc;
	}
	if (dense_box)
	{
		int64_t run = 1;
		for (int d = 0; d < 8; ++d)
		{
			p.istr[d] = box_stride ? box_stride[d] : run;
			p.ioff0 -= (int64_t) p.ilo[d] * p.istr[d];
			run *= (int64_t) (p.ihi[d] - p.ilo[d]);
		}
	}
	// few outputs with long sums: give each output a whole workgroup
	bool group = p.nwin < (uint64_t) ctx->num_cus * 64 * 16 && max_terms >= 2048;
	uint64_t blocks = group ? p.nwin : (p.nwin + CV_BLOCK - 1) / CV_BLOCK;
	TCG_REQUIRE(ctx, blocks < (1ull << 31) && p.nwin < (1ull << 32), "tcg_conv: %llu outputs are too many for one launch", (unsigned long long) p.nwin);
	if (group)
	{
		TCG_DISPATCH_ALL(ctx, dtype, (conv_boxed_k<T,true><<<(unsigned) blocks, CV_BLOCK, 0, ctx->stream>>>(
			p, (const T*) img, (const T*) kernel, (T*) out)));
	}
	else
	{
		TCG_DISPATCH_ALL(ctx, dtype, (conv_boxed_k<T,false><<<(unsigned) blocks, CV_BLOCK, 0, ctx->stream>>>(
			p, (const T*) img, (const T*) kernel, (T*) out)));
	}
	TCG_LAUNCH_CHECK(ctx, "conv_boxed");
	return TCG_OK;
}

int tcg_conv_boxed (tcg_ctx* ctx, int dtype, const uint64_t imgshape[8],
	const uint64_t kshape[8], int nranks, const uint64_t* ranks,
	const uint64_t img_lo[8], const uint64_t img_hi[8],
	const uint64_t out_lo[8], const uint64_t out_hi[8],
	const void* img, const void* kernel, void* out)
{
	return conv_boxed_impl(ctx, dtype, imgshape, kshape, nranks, ranks, img_lo, img_hi, out_lo, out_hi,
		img, kernel, out, false);
}

int tcg_conv_dense_box (tcg_ctx* ctx, int dtype, const uint64_t imgshape[8],
	const uint64_t kshape[8], int nranks, const uint64_t* ranks,
	const uint64_t img_lo[8], const uint64_t img_hi[8],
	const uint64_t out_lo[8], const uint64_t out_hi[8],
	const void* box, const void* kernel, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, img_lo && img_hi, "tcg_conv_dense_box: the box is required");
	return conv_boxed_impl(ctx, dtype, imgshape, kshape, nranks, ranks, img_lo, img_hi, out_lo, out_hi,
		box, kernel, out, true);
}

int tcg_conv_views (tcg_ctx* ctx, int dtype, const uint64_t imgshape[8],
	const uint64_t kshape[8], int nranks, const uint64_t* ranks,
	const uint64_t img_lo[8], const uint64_t img_hi[8],
	const uint64_t out_lo[8], const uint64_t out_hi[8],
	const void* box, const int64_t box_stride[8],
	const void* kernel, const int64_t kernel_stride[8],
	void* out, const int64_t out_stride[8])
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, img_lo && img_hi && box_stride && kernel_stride && out_stride,
		"tcg_conv_views: the box and the three stride lists are required");
	return conv_boxed_impl(ctx, dtype, imgshape, kshape, nranks, ranks, img_lo, img_hi, out_lo, out_hi,
		box, kernel, out, true, box_stride, kernel_stride, out_stride);
}

int tcg_conv (tcg_ctx* ctx, int dtype, const uint64_t imgshape[8],
	const uint64_t kshape[8], int nranks, const uint64_t* ranks,
	const void* img, const void* kernel, void* out)
{
	return tcg_conv_boxed(ctx, dtype, imgshape, kshape, nranks, ranks,
		nullptr, nullptr, nullptr, nullptr, img, kernel, out);
}

} // extern "C"
