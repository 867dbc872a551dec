// Device generator for RAND_UNIF: Philox4x32-10 (Salmon, Moraes, Dror, Shaw:
// "Parallel random numbers: as easy as 1, 2, 3", SC'11), a counter-based
// generator, so element i of draw d depends on (key, counter) only and every
// lane computes its own block without shared state.  The key and the number of
// blocks drawn so far live in device memory and are read and advanced by
// kernels, which lets a recorded launch sequence draw fresh values at every
// replay.  The reference draws on the host from std::default_random_engine
// (internal/eigen/operator.hpp:989-1044, internal/global/random.hpp:87-99);
// the two streams differ by construction, the distributions agree:
// real types uniform on [lo, hi), int32 uniform on the inclusive range.
#include "tcg_internal.hpp"

#include <type_traits>

namespace
{

constexpr int RAND_BLOCK = 256;

struct Philox4 final
{
	uint32_t v[4];
};

__device__ __forceinline__ Philox4 philox4x32_10 (uint64_t counter, uint64_t key)
{
	uint32_t c0 = (uint32_t) counter, c1 = (uint32_t) (counter >> 32), c2 = 0, c3 = 0;
	uint32_t k0 = (uint32_t) key, k1 = (uint32_t) (key >> 32);
#pragma unroll
	for (int round = 0; round < 10; ++round)
	{
		uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
		uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
		c0 = hi1 ^ c1 ^ k0;
		c1 = lo1;
		c2 = hi0 ^ c3 ^ k1;
		c3 = lo0;
		k0 += 0x9E3779B9u; // Weyl sequence of the key schedule
		k1 += 0xBB67AE85u;
	}
	return Philox4{{c0, c1, c2, c3}};
}

// one generator block per 4 elements, or 2 elements of 8 bytes
template <typename T> struct PerBlock { static constexpr int N = sizeof(T) == 8 ? 2 : 4; };

__device__ __forceinline__ float draw (const Philox4& r, int k, float lo, float hi)
{
	float u = (float) (r.v[k] >> 8) * 0x1p-24f;
	return fmaf(u, hi - lo, lo);
}

__device__ __forceinline__ double draw (const Philox4& r, int k, double lo, double hi)
{
	uint64_t bits = ((uint64_t) r.v[2 * k + 1] << 32) | r.v[2 * k];
	double u = (double) (bits >> 11) * 0x1p-53;
	return fma(u, hi - lo, lo);
}

// integers of at most 32 bits: lo + floor(r * (hi - lo + 1) / 2^32)
template <typename T, typename std::enable_if<std::is_integral<T>::value && sizeof(T) <= 4, int>::type = 0>
__device__ __forceinline__ T draw (const Philox4& r, int k, T lo, T hi)
{
	if (hi < lo) { return lo; }
	uint64_t range = (uint64_t) ((int64_t) hi - (int64_t) lo) + 1;
	return (T) ((int64_t) lo + (int64_t) (((uint64_t) r.v[k] * range) >> 32));
}

// 64-bit integers: two words per draw, lo + floor(r * (hi - lo + 1) / 2^64);
// the full range (hi - lo + 1 wraps to 0) takes the 64 bits as they are
template <typename T, typename std::enable_if<std::is_integral<T>::value && sizeof(T) == 8, int>::type = 0>
__device__ __forceinline__ T draw (const Philox4& r, int k, T lo, T hi)
{
	if (hi < lo) { return lo; }
	uint64_t bits = ((uint64_t) r.v[2 * k + 1] << 32) | r.v[2 * k];
	uint64_t range = (uint64_t) hi - (uint64_t) lo + 1;
	uint64_t off = range == 0 ? bits : __umul64hi(bits, range);
	return (T) ((uint64_t) lo + off);
}

template <typename T>
__global__ __launch_bounds__(RAND_BLOCK) void rand_uniform_k (const uint64_t* __restrict__ state,
	const T* __restrict__ lo, const T* __restrict__ hi, T* __restrict__ out, uint64_t n)
{
	constexpr int N = PerBlock<T>::N;
	const uint64_t key = state[0], first = state[1];
	const uint64_t nblocks = (n + N - 1) / N;
	for (uint64_t b = (uint64_t) blockIdx.x * RAND_BLOCK + threadIdx.x; b < nblocks;
		b += (uint64_t) gridDim.x * RAND_BLOCK)
	{
		Philox4 r = philox4x32_10(first + b, key);
		uint64_t base = b * N;
#pragma unroll
		for (int k = 0; k < N; ++k)
		{
			if (base + k < n) { out[base + k] = draw(r, k, lo[base + k], hi[base + k]); }
		}
	}
}

__global__ void rand_advance_k (uint64_t* state, uint64_t nblocks)
{
	if (threadIdx.x == 0 && blockIdx.x == 0) { state[1] += nblocks; }
}

__global__ void rand_seed_k (uint64_t* state, uint64_t key)
{
	if (threadIdx.x == 0 && blockIdx.x == 0) { state[0] = key; state[1] = 0; }
}

template <typename T>
int launch (tcg_ctx* ctx, uint64_t n, const void* lo, const void* hi, void* out)
{
	const uint64_t nblocks = (n + PerBlock<T>::N - 1) / PerBlock<T>::N;
	uint64_t grid = (nblocks + RAND_BLOCK - 1) / RAND_BLOCK;
	const uint64_t cap = (uint64_t) ctx->num_cus * 32;
	if (grid > cap) { grid = cap; }
	hipLaunchKernelGGL(rand_uniform_k<T>, dim3((unsigned) grid), dim3(RAND_BLOCK), 0, ctx->stream,
		ctx->rng_state, (const T*) lo, (const T*) hi, (T*) out, n);
	TCG_LAUNCH_CHECK(ctx, "rand_uniform_k");
	hipLaunchKernelGGL(rand_advance_k, dim3(1), dim3(64), 0, ctx->stream, ctx->rng_state, nblocks);
	TCG_LAUNCH_CHECK(ctx, "rand_advance_k");
	return TCG_OK;
}

}

extern "C" {

int tcg_rand_seed (tcg_ctx* ctx, uint64_t seed)
{
	if (!ctx) { return TCG_ERR_ARG; }
	hipLaunchKernelGGL(rand_seed_k, dim3(1), dim3(64), 0, ctx->stream, ctx->rng_state, seed);
	TCG_LAUNCH_CHECK(ctx, "rand_seed_k");
	return TCG_OK;
}

int tcg_rand_state (tcg_ctx* ctx, uint64_t out[2])
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, out, "tcg_rand_state: NULL pointer");
	TCG_REQUIRE(ctx, !ctx->capturing, "tcg_rand_state: host transfers cannot be part of a captured sequence");
	TCG_HIP(ctx, hipMemcpyAsync(out, ctx->rng_state, 2 * sizeof(uint64_t), hipMemcpyDeviceToHost, ctx->stream));
	TCG_HIP(ctx, hipStreamSynchronize(ctx->stream));
	return TCG_OK;
}

int tcg_rand_uniform (tcg_ctx* ctx, int dtype, uint64_t n, const void* lo, const void* hi, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (n == 0) { return TCG_OK; }
	TCG_REQUIRE(ctx, lo && hi && out, "tcg_rand_uniform: NULL pointer");
	switch (dtype)
	{
		case TCG_DOUBLE: return launch<double>(ctx, n, lo, hi, out);
		case TCG_FLOAT: return launch<float>(ctx, n, lo, hi, out);
		case TCG_INT32: return launch<int32_t>(ctx, n, lo, hi, out);
		case TCG_INT8: return launch<int8_t>(ctx, n, lo, hi, out);
		case TCG_UINT8: return launch<uint8_t>(ctx, n, lo, hi, out);
		case TCG_INT16: return launch<int16_t>(ctx, n, lo, hi, out);
		case TCG_UINT16: return launch<uint16_t>(ctx, n, lo, hi, out);
		case TCG_UINT32: return launch<uint32_t>(ctx, n, lo, hi, out);
		case TCG_INT64: return launch<int64_t>(ctx, n, lo, hi, out);
		case TCG_UINT64: return launch<uint64_t>(ctx, n, lo, hi, out);
		default: return tcg_fail(ctx, TCG_ERR_ARG, "tcg_rand_uniform: unknown dtype %d", dtype);
	}
}

}
