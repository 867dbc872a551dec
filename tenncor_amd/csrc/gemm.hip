// MATMUL / CONTRACT lowering and the generic strided GEMM.
//
// tcg_matmul and tcg_contract reduce to batched row-major GEMMs
// C[b][m][n] = sum_k A[b][m][k] B[b][k][n].  fp32 problems whose operands are
// 16-byte aligned go to the MFMA kernel (gemm_mfma.hip), such fp64 problems to
// gemm_mfma_f64.hip; everything else (int32, odd strides, small problems) runs
// the LDS-tiled kernel below.
#include <type_traits>
#include <vector>

#include "tcg_internal.hpp"

int tcg_gemm_f32_mfma (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t K, uint64_t batch,
	const float* A, uint64_t lda, uint64_t stride_a, int trans_a,
	const float* B, uint64_t ldb, uint64_t stride_b, int trans_b,
	float* C, uint64_t ldc, uint64_t stride_c, bool* handled);

int tcg_gemm_f64_mfma (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t K, uint64_t batch,
	const double* A, uint64_t lda, uint64_t stride_a, int trans_a,
	const double* B, uint64_t ldb, uint64_t stride_b, int trans_b,
	double* C, uint64_t ldc, uint64_t stride_c, bool* handled);

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
__device__ __forceinline__ T fma_wrap (T a, T b, T c)
{
	if constexpr (is_int<T>::value) { return (T) ((Wide<T>) a * (Wide<T>) b + (Wide<T>) c); }
	else if constexpr (sizeof(T) == 4) { return __builtin_fmaf(a, b, c); }
	else { return __builtin_fma(a, b, c); }
}

constexpr int GT = 64;  // tile of C per workgroup
constexpr int GK = 16;  // depth per step

// element (m,k) of A at m*sam + k*sak, (k,n) of B at k*sbk + n*sbn
template <typename T>
__global__ __launch_bounds__(256) void gemm_generic_k (
	uint32_t M, uint32_t N, uint32_t K,
	const T* __restrict__ A, int64_t sam, int64_t sak, int64_t batch_a,
	const T* __restrict__ B, int64_t sbk, int64_t sbn, int64_t batch_b,
	T* __restrict__ C, int64_t ldc, int64_t batch_c, uint32_t tiles_n, uint32_t tiles_m)
{
	__shared__ T As[GK][GT + 1];
	__shared__ T Bs[GK][GT + 1];
	uint32_t bid = blockIdx.x;
	const uint32_t tn = bid % tiles_n;
	bid /= tiles_n;
	const uint32_t tm = bid % tiles_m;
	const uint32_t bz = bid / tiles_m;
	A += (int64_t) bz * batch_a;
	B += (int64_t) bz * batch_b;
	C += (int64_t) bz * batch_c;
	const uint32_t m0 = tm * GT, n0 = tn * GT;
	const uint32_t tx = threadIdx.x % 16, ty = threadIdx.x / 16;
	// lanes run along whichever index is contiguous in memory
	const bool a_kfast = sak == 1 || sam != 1;
	const bool b_nfast = sbn == 1 || sbk != 1;
	T acc[4][4];
#pragma unroll
	for (int i = 0; i < 4; ++i)
	{
#pragma unroll
		for (int j = 0; j < 4; ++j) { acc[i][j] = 0; }
	}
	for (uint32_t k0 = 0; k0 < K; k0 += GK)
	{
#pragma unroll
		for (int e = 0; e < 4; ++e)
		{
			uint32_t idx = threadIdx.x + e * 256;
			uint32_t kk = a_kfast ? idx % GK : idx / GT;
			uint32_t mm = a_kfast ? idx / GK : idx % GT;
			T v = 0;
			if (m0 + mm < M && k0 + kk < K) { v = A[(int64_t) (m0 + mm) * sam + (int64_t) (k0 + kk) * sak]; }
			As[kk][mm] = v;
			uint32_t nn = b_nfast ? idx % GT : idx / GK;
			uint32_t kb = b_nfast ? idx / GT : idx % GK;
			T w = 0;
			if (n0 + nn < N && k0 + kb < K) { w = B[(int64_t) (k0 + kb) * sbk + (int64_t) (n0 + nn) * sbn]; }
			Bs[kb][nn] = w;
		}
		__syncthreads();
#pragma unroll
		for (int kk = 0; kk < GK; ++kk)
		{
			T a[4], b[4];
#pragma unroll
			for (int i = 0; i < 4; ++i) { a[i] = As[kk][ty * 4 + i]; }
#pragma unroll
			for (int j = 0; j < 4; ++j) { b[j] = Bs[kk][tx * 4 + j]; }
#pragma unroll
			for (int i = 0; i < 4; ++i)
			{
#pragma unroll
				for (int j = 0; j < 4; ++j) { acc[i][j] = fma_wrap(a[i], b[j], acc[i][j]); }
			}
		}
		__syncthreads();
	}
#pragma unroll
	for (int i = 0; i < 4; ++i)
	{
		uint32_t m = m0 + ty * 4 + i;
		if (m >= M) { continue; }
#pragma unroll
		for (int j = 0; j < 4; ++j)
		{
			uint32_t n = n0 + tx * 4 + j;
			if (n < N) { C[(int64_t) m * ldc + n] = acc[i][j]; }
		}
	}
}

// A few thousand results with a long K (a dense head on a batch, its weight
// gradient): the tiled kernel would run a handful of workgroups through one
// memory latency per 16 columns of K.  Here every lane owns one result and
// walks K itself, sixteen pairs of loads in flight; the sum runs in the same order with
// the same fused multiply-add, so the value equals the tiled kernel's bit for bit.
template <typename T>
__global__ __launch_bounds__(256) void gemm_small_k (
	uint32_t M, uint32_t N, uint32_t K, uint32_t batch,
	const T* __restrict__ A, int64_t sam, int64_t sak, int64_t batch_a,
	const T* __restrict__ B, int64_t sbk, int64_t sbn, int64_t batch_b,
	T* __restrict__ C, int64_t ldc, int64_t batch_c)
{
	const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
	if (idx >= M * N * batch) { return; }
	const uint32_t n = idx % N, m = (idx / N) % M, bz = idx / (N * M);
	const T* a = A + (int64_t) bz * batch_a + (int64_t) m * sam;
	const T* b = B + (int64_t) bz * batch_b + (int64_t) n * sbn;
	T acc = 0;
	uint32_t k = 0;
	for (; k + 16 <= K; k += 16)
	{
		T av[16], bv[16];
#pragma unroll
		for (int e = 0; e < 16; ++e)
		{
			av[e] = a[(int64_t) (k + e) * sak];
			bv[e] = b[(int64_t) (k + e) * sbk];
		}
#pragma unroll
		for (int e = 0; e < 16; ++e) { acc = fma_wrap(av[e], bv[e], acc); }
	}
	for (; k < K; ++k) { acc = fma_wrap(a[(int64_t) k * sak], b[(int64_t) k * sbk], acc); }
	C[(int64_t) bz * batch_c + (int64_t) m * ldc + n] = acc;
}

template <typename T>
int gemm_generic (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t K, uint64_t batch,
	const T* A, uint64_t lda, uint64_t stride_a, int trans_a,
	const T* B, uint64_t ldb, uint64_t stride_b, int trans_b,
	T* C, uint64_t ldc, uint64_t stride_c)
{
	uint64_t tiles_m = (M + GT - 1) / GT, tiles_n = (N + GT - 1) / GT;
	uint64_t blocks = tiles_m * tiles_n * batch;
	TCG_REQUIRE(ctx, M < (1ull << 31) && N < (1ull << 31) && K < (1ull << 31) && blocks < (1ull << 31),
		"tcg_gemm: problem %llux%llux%llu (batch %llu) is too large for one launch",
		(unsigned long long) M, (unsigned long long) N, (unsigned long long) K, (unsigned long long) batch);
	int64_t sam = trans_a ? 1 : (int64_t) lda, sak = trans_a ? (int64_t) lda : 1;
	int64_t sbk = trans_b ? 1 : (int64_t) ldb, sbn = trans_b ? (int64_t) ldb : 1;
	if (K >= 32 && M * N * batch <= 16384)
	{
		const unsigned grid = (unsigned) ((M * N * batch + 255) / 256);
		gemm_small_k<T><<<grid, 256, 0, ctx->stream>>>((uint32_t) M, (uint32_t) N, (uint32_t) K, (uint32_t) batch,
			A, sam, sak, (int64_t) stride_a, B, sbk, sbn, (int64_t) stride_b, C, (int64_t) ldc, (int64_t) stride_c);
		TCG_LAUNCH_CHECK(ctx, "gemm_small");
		return TCG_OK;
	}
	gemm_generic_k<T><<<(unsigned) blocks, 256, 0, ctx->stream>>>((uint32_t) M, (uint32_t) N, (uint32_t) K,
		A, sam, sak, (int64_t) stride_a, B, sbk, sbn, (int64_t) stride_b, C, (int64_t) ldc, (int64_t) stride_c,
		(uint32_t) tiles_n, (uint32_t) tiles_m);
	TCG_LAUNCH_CHECK(ctx, "gemm_generic");
	return TCG_OK;
}

// One operand of a contraction seen as a matrix: its significant dims must be
// [all contracted..., all free...] (inner = contracted) or the reverse.
struct Operand
{
	bool direct = false;
	bool contracted_inner = false; // contracted dims are the fastest ones
};

Operand classify (const uint64_t shape[8], const bool com[8])
{
	Operand o;
	int switches = 0, first = -1, prev = -1;
	for (int d = 0; d < 8; ++d)
	{
		if (shape[d] == 1) { continue; }
		int kind = com[d] ? 1 : 0;
		if (first < 0) { first = kind; }
		if (prev >= 0 && kind != prev) { ++switches; }
		prev = kind;
	}
	o.direct = switches <= 1;
	o.contracted_inner = first != 0; // no significant dim at all: either way
	return o;
}

// C[m][n] += T[m][n] for a C whose rows are ldc apart (terms of a sum of
// products added in term order on the routes that compute term by term)
template <typename T>
__global__ __launch_bounds__(256) void add_rows_k (uint32_t M, uint32_t N, const T* __restrict__ term, T* __restrict__ C, int64_t ldc)
{
	const uint64_t total = (uint64_t) M * N;
	for (uint64_t i = (uint64_t) blockIdx.x * 256 + threadIdx.x; i < total; i += (uint64_t) gridDim.x * 256)
	{
		const uint64_t m = i / N, n = i - m * N;
		T& c = C[(int64_t) m * ldc + n];
		if constexpr (is_int<T>::value) { c = (T) ((Wide<T>) c + (Wide<T>) term[i]); }
		else { c = c + term[i]; }
	}
}

} // namespace

extern "C" {

int tcg_gemm (tcg_ctx* ctx, int dtype, uint64_t M, uint64_t N, uint64_t K,
	uint64_t batch, const void* A, uint64_t lda, uint64_t stride_a, int trans_a,
	const void* B, uint64_t ldb, uint64_t stride_b, int trans_b,
	void* C, uint64_t ldc, uint64_t stride_c)
{
	if (!ctx) { return TCG_ERR_ARG; }
	if (M == 0 || N == 0 || batch == 0) { return TCG_OK; }
	TCG_REQUIRE(ctx, A && B && C, "tcg_gemm: NULL pointer");
	TCG_REQUIRE(ctx, ldc >= N, "tcg_gemm: ldc %llu < N %llu", (unsigned long long) ldc, (unsigned long long) N);
	if (dtype == TCG_FLOAT)
	{
		bool handled = false;
		int rc = tcg_gemm_f32_mfma(ctx, M, N, K, batch, (const float*) A, lda, stride_a, trans_a,
			(const float*) B, ldb, stride_b, trans_b, (float*) C, ldc, stride_c, &handled);
		if (rc != TCG_OK || handled) { return rc; }
	}
	else if (dtype == TCG_DOUBLE)
	{
		bool handled = false;
		int rc = tcg_gemm_f64_mfma(ctx, M, N, K, batch, (const double*) A, lda, stride_a, trans_a,
			(const double*) B, ldb, stride_b, trans_b, (double*) C, ldc, stride_c, &handled);
		if (rc != TCG_OK || handled) { return rc; }
	}
	TCG_DISPATCH_ALL(ctx, dtype, return gemm_generic<T>(ctx, M, N, K, batch,
		(const T*) A, lda, stride_a, trans_a, (const T*) B, ldb, stride_b, trans_b, (T*) C, ldc, stride_c));
	return TCG_OK;
}

int tcg_matmul (tcg_ctx* ctx, int dtype, const uint64_t ashape[8],
	const uint64_t bshape[8], const void* a, const void* b, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, ashape && bshape && a && b && out, "tcg_matmul: NULL pointer");
	uint64_t K = ashape[0], M = ashape[1], N = bshape[0], batch = 1;
	TCG_REQUIRE(ctx, bshape[1] == K, "tcg_matmul: invalid shapes have mismatch common dimension 0,1 (%llu vs %llu)",
		(unsigned long long) K, (unsigned long long) bshape[1]);
	for (int d = 2; d < 8; ++d)
	{
		TCG_REQUIRE(ctx, ashape[d] == bshape[d], "tcg_matmul: invalid shapes do not match for dimensions 2+ (dim %d)", d);
		batch *= ashape[d];
	}
	if (tcg_small_mode(ctx))
	{
		const uint64_t pair[2] = {0, 1};
		TCG_SMALL_RETURN(ctx, batch != 1 ? tcg_small_unsupported(ctx, "a batched matrix product") :
			tcg_small_contract(ctx, dtype, ashape, bshape, 1, pair, a, b, out));
	}
	return tcg_gemm(ctx, dtype, M, N, K, batch, a, K, M * K, 0, b, N, K * N, 0, out, N, M * N);
}

int tcg_contract (tcg_ctx* ctx, int dtype, const uint64_t ashape[8],
	const uint64_t bshape[8], int npairs, const uint64_t* pairs,
	const void* a, const void* b, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, ashape && bshape && pairs && a && b && out, "tcg_contract: NULL pointer");
	TCG_REQUIRE(ctx, npairs >= 1 && npairs <= 8, "tcg_contract: %d dimension pairs", npairs);
	bool acom[8] = {false}, bcom[8] = {false};
	uint64_t M = 1, N = 1, K = 1;
	// pairs sorted by the a-side dim: the order in which k is enumerated
	uint64_t pa[8], pb[8];
	for (int p = 0; p < npairs; ++p)
	{
		uint64_t ad = pairs[2 * p], bd = pairs[2 * p + 1];
		TCG_REQUIRE(ctx, ad < 8 && bd < 8, "tcg_contract: pair %d names a dim >= 8", p);
		TCG_REQUIRE(ctx, ashape[ad] == bshape[bd], "tcg_contract: invalid shapes do not match common dimensions (pair %d)", p);
		TCG_REQUIRE(ctx, !acom[ad] && !bcom[bd], "tcg_contract: contraction dimensions must be unique for each side");
		acom[ad] = bcom[bd] = true;
		int q = p;
		while (q > 0 && pa[q - 1] > ad) { pa[q] = pa[q - 1]; pb[q] = pb[q - 1]; --q; }
		pa[q] = ad;
		pb[q] = bd;
		K *= ashape[ad];
	}
	if (tcg_small_mode(ctx))
	{
		uint64_t sorted[16];
		for (int p = 0; p < npairs; ++p)
		{
			sorted[2 * p] = pa[p];
			sorted[2 * p + 1] = pb[p];
		}
		TCG_SMALL_RETURN(ctx, tcg_small_contract(ctx, dtype, ashape, bshape, npairs, sorted, a, b, out));
	}
	for (int d = 0; d < 8; ++d)
	{
		if (!acom[d]) { M *= ashape[d]; }
		if (!bcom[d]) { N *= bshape[d]; }
	}
	Operand oa = classify(ashape, acom), ob = classify(bshape, bcom);
	// b's contracted dims must be enumerated in the same order as a's
	bool same_order = true;
	uint64_t last = 0;
	bool have_last = false;
	for (int p = 0; p < npairs; ++p)
	{
		if (bshape[pb[p]] == 1) { continue; }
		if (have_last && pb[p] < last) { same_order = false; }
		last = pb[p];
		have_last = true;
	}
	const size_t esz = tcg_type_size(dtype);
	TCG_REQUIRE(ctx, esz != 0, "tcg_contract: unknown dtype %d", dtype);
	const void* A = a;
	const void* B = b;
	void* ta = nullptr;
	void* tb = nullptr;
	int rc = TCG_OK;
	int trans_a, trans_b;
	uint64_t lda, ldb;
	if (oa.direct)
	{
		// [contracted.., free..]: A(m,k) at k + m*K; else A(m,k) at m + k*M
		trans_a = oa.contracted_inner ? 0 : 1;
		lda = oa.contracted_inner ? K : M;
	}
	else
	{
		// repack to [contracted dims in pair order, free dims]
		uint64_t order[8];
		int n = 0;
		for (int p = 0; p < npairs; ++p) { order[n++] = pa[p]; }
		for (int d = 0; d < 8; ++d) { if (!acom[d]) { order[n++] = d; } }
		rc = tcg_alloc(ctx, esz * M * K, &ta);
		if (rc == TCG_OK) { rc = tcg_permute(ctx, dtype, ashape, order, a, ta); }
		A = ta;
		trans_a = 0;
		lda = K;
	}
	if (rc == TCG_OK)
	{
		if (ob.direct && same_order)
		{
			// [free.., contracted..]: B(k,n) at n + k*N; else B(k,n) at k + n*K
			trans_b = ob.contracted_inner ? 1 : 0;
			ldb = ob.contracted_inner ? K : N;
		}
		else
		{
			uint64_t order[8];
			int n = 0;
			for (int d = 0; d < 8; ++d) { if (!bcom[d]) { order[n++] = d; } }
			for (int p = 0; p < npairs; ++p) { order[n++] = pb[p]; }
			rc = tcg_alloc(ctx, esz * N * K, &tb);
			if (rc == TCG_OK) { rc = tcg_permute(ctx, dtype, bshape, order, b, tb); }
			B = tb;
			trans_b = 0;
			ldb = N;
		}
	}
	if (rc == TCG_OK)
	{
		rc = tcg_gemm(ctx, dtype, M, N, K, 1, A, lda, 0, trans_a, B, ldb, 0, trans_b, out, N, 0);
	}
	if (ta) { tcg_free(ctx, ta, esz * M * K); }
	if (tb) { tcg_free(ctx, tb, esz * N * K); }
	return rc;
}

int tcg_contract_sum (tcg_ctx* ctx, int dtype, const uint64_t ashape[8],
	const uint64_t bshape[8], int npairs, const uint64_t* pairs, int nterms,
	const void* const* a, const void* const* b, void* out)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, ashape && bshape && pairs && a && b && out, "tcg_contract_sum: NULL pointer");
	TCG_REQUIRE(ctx, nterms >= 1, "tcg_contract_sum: %d terms", nterms);
	TCG_REQUIRE(ctx, npairs >= 1 && npairs <= 8, "tcg_contract_sum: %d dimension pairs", npairs);
	for (int t = 0; t < nterms; ++t) { TCG_REQUIRE(ctx, a[t] && b[t], "tcg_contract_sum: operand of term %d is NULL", t); }
	if (tcg_small_mode(ctx)) { TCG_SMALL_RETURN(ctx, tcg_small_unsupported(ctx, "a sum of contractions")); }
	const size_t esz = tcg_type_size(dtype);
	TCG_REQUIRE(ctx, esz != 0, "tcg_contract_sum: unknown dtype %d", dtype);
	// the shape of every term as a matrix product (the rules of tcg_contract)
	bool acom[8] = {false}, bcom[8] = {false};
	uint64_t M = 1, N = 1, K = 1, pb_sorted[8], pa_sorted[8];
	for (int p = 0; p < npairs; ++p)
	{
		uint64_t ad = pairs[2 * p], bd = pairs[2 * p + 1];
		TCG_REQUIRE(ctx, ad < 8 && bd < 8, "tcg_contract_sum: pair %d names a dim >= 8", p);
		TCG_REQUIRE(ctx, ashape[ad] == bshape[bd], "tcg_contract_sum: invalid shapes do not match common dimensions (pair %d)", p);
		TCG_REQUIRE(ctx, !acom[ad] && !bcom[bd], "tcg_contract_sum: contraction dimensions must be unique for each side");
		acom[ad] = bcom[bd] = true;
		int q = p;
		while (q > 0 && pa_sorted[q - 1] > ad) { pa_sorted[q] = pa_sorted[q - 1]; pb_sorted[q] = pb_sorted[q - 1]; --q; }
		pa_sorted[q] = ad;
		pb_sorted[q] = bd;
		K *= ashape[ad];
	}
	for (int d = 0; d < 8; ++d)
	{
		if (!acom[d]) { M *= ashape[d]; }
		if (!bcom[d]) { N *= bshape[d]; }
	}
	if (M == 0 || N == 0) { return TCG_OK; }
	Operand oa = classify(ashape, acom), ob = classify(bshape, bcom);
	bool same_order = true, have_last = false;
	uint64_t last = 0;
	for (int p = 0; p < npairs; ++p)
	{
		if (bshape[pb_sorted[p]] == 1) { continue; }
		if (have_last && pb_sorted[p] < last) { same_order = false; }
		last = pb_sorted[p];
		have_last = true;
	}
	if (dtype == TCG_FLOAT && nterms > 1 && oa.direct && ob.direct && same_order)
	{
		// every term is a matrix in place: one product over the concatenated summed index
		int trans_a = oa.contracted_inner ? 0 : 1, trans_b = ob.contracted_inner ? 1 : 0;
		uint64_t lda = oa.contracted_inner ? K : M, ldb = ob.contracted_inner ? K : N;
		bool handled = false;
		int rc = tcg_gemm_f32_mfma_sum(ctx, M, N, K, (uint32_t) nterms, (const float* const*) a, lda, trans_a,
			(const float* const*) b, ldb, trans_b, (float*) out, N, &handled);
		if (rc != TCG_OK || handled) { return rc; }
	}
	// term by term, added up in term order: what the separate nodes compute
	int rc = tcg_contract(ctx, dtype, ashape, bshape, npairs, pairs, a[0], b[0], out);
	if (rc != TCG_OK || nterms == 1) { return rc; }
	void* term = nullptr;
	rc = tcg_alloc(ctx, esz * M * N, &term);
	for (int t = 1; t < nterms && rc == TCG_OK; ++t)
	{
		rc = tcg_contract(ctx, dtype, ashape, bshape, npairs, pairs, a[t], b[t], term);
		if (rc == TCG_OK) { rc = tcg_ew_binary(ctx, TCG_ADD, dtype, M * N, out, term, out); }
	}
	if (term) { tcg_free(ctx, term, esz * M * N); }
	return rc;
}

int tcg_gemm_terms (tcg_ctx* ctx, int dtype, uint64_t M, uint64_t N, uint64_t K, int nterms,
	const void* const* A, const uint64_t* lda, int trans_a,
	const void* const* B, const uint64_t* ldb, int trans_b,
	void* C, uint64_t ldc)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, A && B && lda && ldb && C, "tcg_gemm_terms: NULL pointer");
	TCG_REQUIRE(ctx, nterms >= 1, "tcg_gemm_terms: %d terms", nterms);
	TCG_REQUIRE(ctx, ldc >= N, "tcg_gemm_terms: ldc %llu < N %llu", (unsigned long long) ldc, (unsigned long long) N);
	for (int t = 0; t < nterms; ++t) { TCG_REQUIRE(ctx, A[t] && B[t], "tcg_gemm_terms: operand of term %d is NULL", t); }
	if (tcg_small_mode(ctx)) { TCG_SMALL_RETURN(ctx, tcg_small_unsupported(ctx, "a sum of matrix products")); }
	const size_t esz = tcg_type_size(dtype);
	TCG_REQUIRE(ctx, esz != 0, "tcg_gemm_terms: unknown dtype %d", dtype);
	if (M == 0 || N == 0) { return TCG_OK; }
	if (dtype == TCG_FLOAT && nterms > 1)
	{
		bool handled = false;
		int rc = tcg_gemm_f32_mfma_terms(ctx, M, N, K, (uint32_t) nterms, (const float* const*) A, lda, trans_a,
			(const float* const*) B, ldb, trans_b, (float*) C, ldc, &handled);
		if (rc != TCG_OK || handled) { return rc; }
	}
	// term by term, added up in term order
	int rc = tcg_gemm(ctx, dtype, M, N, K, 1, A[0], lda[0], 0, trans_a, B[0], ldb[0], 0, trans_b, C, ldc, 0);
	if (rc != TCG_OK || nterms == 1) { return rc; }
	TCG_REQUIRE(ctx, M < (1ull << 31) && N < (1ull << 31), "tcg_gemm_terms: too large");
	void* term = nullptr;
	rc = tcg_alloc(ctx, esz * M * N, &term);
	for (int t = 1; t < nterms && rc == TCG_OK; ++t)
	{
		rc = tcg_gemm(ctx, dtype, M, N, K, 1, A[t], lda[t], 0, trans_a, B[t], ldb[t], 0, trans_b, term, N, 0);
		if (rc != TCG_OK) { break; }
		const unsigned grid = tcg_grid(ctx, M * N, 256, 16);
		TCG_DISPATCH_ALL(ctx, dtype, (add_rows_k<T><<<grid, 256, 0, ctx->stream>>>((uint32_t) M, (uint32_t) N,
			(const T*) term, (T*) C, (int64_t) ldc)));
	}
	if (term) { tcg_free(ctx, term, esz * M * N); }
	if (rc != TCG_OK) { return rc; }
	TCG_LAUNCH_CHECK(ctx, "tcg_gemm_terms");
	return TCG_OK;
}

int tcg_gemm_terms_grid (tcg_ctx* ctx, int dtype, int mparts, const uint64_t* Mp, int nparts, const uint64_t* Np,
	uint64_t K, int nterms, const void* const* A, const uint64_t* lda, int trans_a,
	const void* const* B, const uint64_t* ldb, int trans_b, void* C, uint64_t ldc)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, Mp && Np && A && B && lda && ldb && C, "tcg_gemm_terms_grid: NULL pointer");
	TCG_REQUIRE(ctx, mparts >= 1 && nparts >= 1 && nterms >= 1, "tcg_gemm_terms_grid: %d x %d parts, %d terms", mparts, nparts, nterms);
	uint64_t N = 0;
	for (int j = 0; j < nparts; ++j) { N += Np[j]; }
	TCG_REQUIRE(ctx, ldc >= N, "tcg_gemm_terms_grid: ldc %llu < N %llu", (unsigned long long) ldc, (unsigned long long) N);
	for (int i = 0; i < mparts * nterms; ++i) { TCG_REQUIRE(ctx, A[i], "tcg_gemm_terms_grid: operand A[%d] is NULL", i); }
	for (int j = 0; j < nparts * nterms; ++j) { TCG_REQUIRE(ctx, B[j], "tcg_gemm_terms_grid: operand B[%d] is NULL", j); }
	if (tcg_small_mode(ctx)) { TCG_SMALL_RETURN(ctx, tcg_small_unsupported(ctx, "a sum of matrix products")); }
	TCG_REQUIRE(ctx, tcg_type_size(dtype) != 0, "tcg_gemm_terms_grid: unknown dtype %d", dtype);
	if (dtype == TCG_FLOAT)
	{
		bool handled = false;
		int rc = tcg_gemm_f32_mfma_grid(ctx, (uint32_t) mparts, Mp, (uint32_t) nparts, Np, K, (uint32_t) nterms,
			(const float* const*) A, lda, trans_a, (const float* const*) B, ldb, trans_b, (float*) C, ldc, &handled);
		if (rc != TCG_OK || handled) { return rc; }
	}
	// block by block
	const size_t esz = tcg_type_size(dtype);
	std::vector<uint64_t> la((size_t) nterms), lb((size_t) nterms);
	uint64_t m0 = 0;
	for (int i = 0; i < mparts; ++i)
	{
		uint64_t n0 = 0;
		for (int j = 0; j < nparts; ++j)
		{
			for (int t = 0; t < nterms; ++t)
			{
				la[t] = lda[i];
				lb[t] = ldb[j];
			}
			int rc = tcg_gemm_terms(ctx, dtype, Mp[i], Np[j], K, nterms, A + (size_t) i * nterms, la.data(), trans_a,
				B + (size_t) j * nterms, lb.data(), trans_b, (char*) C + esz * (m0 * ldc + n0), ldc);
			if (rc != TCG_OK) { return rc; }
			n0 += Np[j];
		}
		m0 += Mp[i];
	}
	return TCG_OK;
}

int tcg_gemm_terms_ranges (tcg_ctx* ctx, int dtype, uint64_t M, uint64_t N, uint64_t K, int nterms,
	const void* const* A, const uint64_t* lda, int trans_a,
	const void* const* B, const uint64_t* ldb, int trans_b,
	int nranges, void* ranges)
{
	if (!ctx) { return TCG_ERR_ARG; }
	TCG_REQUIRE(ctx, A && B && lda && ldb && ranges, "tcg_gemm_terms_ranges: NULL pointer");
	TCG_REQUIRE(ctx, nterms >= 1, "tcg_gemm_terms_ranges: %d terms", nterms);
	for (int t = 0; t < nterms; ++t) { TCG_REQUIRE(ctx, A[t] && B[t], "tcg_gemm_terms_ranges: operand of term %d is NULL", t); }
	if (tcg_small_mode(ctx)) { TCG_SMALL_RETURN(ctx, tcg_small_unsupported(ctx, "the K ranges of a matrix product")); }
	bool handled = false;
	if (dtype == TCG_FLOAT && nranges >= 2)
	{
		int rc = tcg_gemm_f32_mfma_ranges(ctx, M, N, K, (uint32_t) nterms, (const float* const*) A, lda, trans_a,
			(const float* const*) B, ldb, trans_b, (uint32_t) nranges, (float*) ranges, &handled);
		if (rc != TCG_OK) { return rc; }
	}
	if (!handled)
	{
		return tcg_fail(ctx, TCG_ERR_UNSUPPORTED,
			"tcg_gemm_terms_ranges: fp32 only, M, N >= 32, K a multiple of 16, 2..32 ranges of whole 16-column slabs, 16-byte aligned operands");
	}
	return TCG_OK;
}

} // extern "C"
