// CONV: N-d valid cross-correlation (internal/eigen/operator.hpp:1141-1187).
//
// conv_direct_k is the general kernel: one lane per output element walking the
// kernel's significant dims with an odometer.  It is the parity reference for
// any specialised path and the fallback for every shape.
#include "tcg_internal.hpp"

namespace
{

template <typename T> struct is_int { static constexpr bool value = false; };
template <> struct is_int<int32_t> { static constexpr bool value = true; };

struct ConvPlan
{
	int nod = 0;             // significant output dims
	uint32_t osize[8];
	int64_t oistr[8];        // image stride of each output dim
	uint32_t odiv[8];
	int nkd = 0;             // significant kernel dims
	uint32_t ksize[8];
	int64_t kistr[8];        // image stride of the dim each kernel dim slides along
	uint64_t nk = 1;
	uint64_t nout = 1;
};

template <typename T>
__global__ __launch_bounds__(256) void conv_direct_k (ConvPlan p,
	const T* __restrict__ img, const T* __restrict__ ker, T* __restrict__ out)
{
	uint64_t o = (uint64_t) blockIdx.x * 256 + threadIdx.x;
	if (o >= p.nout) { return; }
	uint64_t rem = o;
	int64_t base = 0;
#pragma unroll
	for (int d = 0; d < 8; ++d)
	{
		if (d < p.nod)
		{
			uint64_t q = rem / p.osize[d];
			uint32_t c = (uint32_t) (rem - q * p.osize[d]);
			rem = q;
			base += (int64_t) c * p.oistr[d];
		}
	}
	uint32_t kc[8];
#pragma unroll
	for (int d = 0; d < 8; ++d) { kc[d] = 0; }
	int64_t off = base;
	T acc = 0;
	for (uint64_t k = 0; k < p.nk; ++k)
	{
		T x = img[off], w = ker[k];
		if constexpr (is_int<T>::value) { acc = (T) ((uint32_t) acc + (uint32_t) x * (uint32_t) w); }
		else { acc += x * w; }
		bool carry = true;
#pragma unroll
		for (int d = 0; d < 8; ++d)
		{
			if (d < p.nkd && carry)
			{
				++kc[d];
				off += p.kistr[d];
				if (kc[d] == p.ksize[d])
				{
					off -= (int64_t) p.ksize[d] * p.kistr[d];
					kc[d] = 0;
				}
				else { carry = false; }
			}
		}
	}
	out[o] = acc;
}

} // namespace

extern "C" {

int tcg_conv (tcg_ctx* ctx, int dtype, const uint64_t imgshape[8],
	const uint64_t kshape[8], int nranks, const uint64_t* ranks,
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
	uint64_t oshape[8];
	int64_t istr[8];
	istr[0] = 1;
	for (int d = 1; d < 8; ++d) { istr[d] = istr[d - 1] * (int64_t) imgshape[d - 1]; }
	for (int d = 0; d < 8; ++d)
	{
		TCG_REQUIRE(ctx, imgshape[d] >= 1 && kshape[d] >= 1, "tcg_conv: dim %d is empty", d);
		oshape[d] = imgshape[d];
	}
	ConvPlan p;
	for (int i = 0; i < 8; ++i)
	{
		TCG_REQUIRE(ctx, kshape[i] <= oshape[order[i]], "tcg_conv: cannot convolve a kernel against a smaller image (kernel dim %d)", i);
		oshape[order[i]] -= kshape[i] - 1;
		p.nk *= kshape[i];
	}
	// kernel dims in memory order; singular ones drop out of the odometer
	for (int i = 0; i < 8; ++i)
	{
		if (kshape[i] == 1) { continue; }
		p.ksize[p.nkd] = (uint32_t) kshape[i];
		p.kistr[p.nkd] = istr[order[i]];
		++p.nkd;
	}
	for (int d = 0; d < 8; ++d)
	{
		p.nout *= oshape[d];
		if (oshape[d] == 1) { continue; }
		p.osize[p.nod] = (uint32_t) oshape[d];
		p.oistr[p.nod] = istr[d];
		++p.nod;
	}
	uint64_t blocks = (p.nout + 255) / 256;
	TCG_REQUIRE(ctx, blocks < (1ull << 31), "tcg_conv: %llu outputs are too many for one launch", (unsigned long long) p.nout);
	TCG_DISPATCH_TYPE(ctx, dtype, (conv_direct_k<T><<<(unsigned) blocks, 256, 0, ctx->stream>>>(
		p, (const T*) img, (const T*) kernel, (T*) out)));
	TCG_LAUNCH_CHECK(ctx, "conv_direct");
	return TCG_OK;
}

} // extern "C"
