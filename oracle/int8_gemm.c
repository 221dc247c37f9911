/*
 * C restatement of the integer contraction of the A8W8 GEMM.  TEST INFRASTRUCTURE ONLY
 * (loaded by tests and by bench.py's cpu_baseline leg; never by the flashnn_amd package).
 *
 *   acc[m,n] = sum_k (int32)a[m,k] * (int32)b[n,k]
 *
 * which is what the reference's kernel accumulates before its scale epilogue
 * (flashnn/triton_kernels/gemm_a8w8.py:135-150) and what quant_gemm.py:96-98 approximates
 * with an fp32 matmul.  Plain loops; OpenMP over rows of a.
 */
#include <stdint.h>

void fnn_oracle_int8_gemm(const int8_t* a, const int8_t* b, int32_t* acc, int64_t M,
                          int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        const int8_t* ar = a + m * lda;
        for (int64_t n = 0; n < N; ++n) {
            const int8_t* br = b + n * ldb;
            int32_t s = 0;
            for (int64_t k = 0; k < K; ++k) s += (int32_t)ar[k] * (int32_t)br[k];
            acc[m * ldc + n] = s;
        }
    }
}

/* out[m,n] = (float)acc * alpha_row[m] * alpha_col[n], the fp32 epilogue order of
 * flashnn/triton_kernels/gemm_a8w8.py:166-173 (before the cast to fp16/bf16). */
void fnn_oracle_a8w8_epilogue(const int32_t* acc, const float* alpha_row,
                              const float* alpha_col, float* out, int64_t M, int64_t N) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n)
            out[m * N + n] = ((float)acc[m * N + n] * alpha_row[m]) * alpha_col[n];
}
