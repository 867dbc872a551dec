// fp32 GEMM on the matrix cores (v_mfma_f32_32x32x2_f32).
#include "tcg_internal.hpp"

int tcg_gemm_f32_mfma (tcg_ctx* ctx, uint64_t M, uint64_t N, uint64_t K, uint64_t batch,
	const float* A, uint64_t lda, uint64_t stride_a, int trans_a,
	const float* B, uint64_t ldb, uint64_t stride_b, int trans_b,
	float* C, uint64_t ldc, uint64_t stride_c, bool* handled)
{
	(void) ctx; (void) M; (void) N; (void) K; (void) batch; (void) A; (void) lda; (void) stride_a;
	(void) trans_a; (void) B; (void) ldb; (void) stride_b; (void) trans_b; (void) C; (void) ldc; (void) stride_c;
	*handled = false;
	return TCG_OK;
}
