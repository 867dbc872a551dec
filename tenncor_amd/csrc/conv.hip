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

namespace
{

template <typename T> struct is_int { static constexpr bool value = false; };
template <> struct is_int<int32_t> { static constexpr bool value = true; };

template <typename T>
__device__ __forceinline__ T mac (T acc, T x, T w)
{
	if constexpr (is_int<T>::value) { return (T) ((uint32_t) acc + (uint32_t) x * (uint32_t) w); }
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
};

constexpr int CV_BLOCK = 256;

template <typename T, bool GROUP_PER_OUTPUT>
__global__ __launch_bounds__(CV_BLOCK) void conv_boxed_k (ConvPlan p,
	const T* __restrict__ img, const T* __restrict__ ker, T* __restrict__ out)
{
	uint64_t o = GROUP_PER_OUTPUT ? (uint64_t) blockIdx.x : (uint64_t) blockIdx.x * CV_BLOCK + threadIdx.x;
	if (o >= p.nwin) { return; }
	// output coordinate, and per image dim the clipped kernel range [k0, k0 + kr)
	int64_t ibase = 0, obase = 0, kbase = 0;
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
				if constexpr (is_int<T>::value) { smem[threadIdx.x] = (T) ((uint32_t) a + (uint32_t) b); }
				else { smem[threadIdx.x] = a + b; }
			}
			__syncthreads();
		}
		if (threadIdx.x == 0) { out[obase] = smem[0]; }
	}
}

} // namespace

extern "C" {

int tcg_conv_boxed (tcg_ctx* ctx, int dtype, const uint64_t imgshape[8],
	const uint64_t kshape[8], int nranks, const uint64_t* ranks,
	const uint64_t img_lo[8], const uint64_t img_hi[8],
	const uint64_t out_lo[8], const uint64_t out_hi[8],
	const void* img, const void* kernel, void* out)
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
		p.kstr[d] = kmem[i];
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
	// few outputs with long sums: give each output a whole workgroup
	bool group = p.nwin < (uint64_t) ctx->num_cus * 64 * 16 && max_terms >= 2048;
	uint64_t blocks = group ? p.nwin : (p.nwin + CV_BLOCK - 1) / CV_BLOCK;
	TCG_REQUIRE(ctx, blocks < (1ull << 31) && p.nwin < (1ull << 32), "tcg_conv: %llu outputs are too many for one launch", (unsigned long long) p.nwin);
	if (group)
	{
		TCG_DISPATCH_TYPE(ctx, dtype, (conv_boxed_k<T,true><<<(unsigned) blocks, CV_BLOCK, 0, ctx->stream>>>(
			p, (const T*) img, (const T*) kernel, (T*) out)));
	}
	else
	{
		TCG_DISPATCH_TYPE(ctx, dtype, (conv_boxed_k<T,false><<<(unsigned) blocks, CV_BLOCK, 0, ctx->stream>>>(
			p, (const T*) img, (const T*) kernel, (T*) out)));
	}
	TCG_LAUNCH_CHECK(ctx, "conv_boxed");
	return TCG_OK;
}

int tcg_conv (tcg_ctx* ctx, int dtype, const uint64_t imgshape[8],
	const uint64_t kshape[8], int nranks, const uint64_t* ranks,
	const void* img, const void* kernel, void* out)
{
	return tcg_conv_boxed(ctx, dtype, imgshape, kshape, nranks, ranks,
		nullptr, nullptr, nullptr, nullptr, img, kernel, out);
}

} // extern "C"
