/* Plain-C triple loops for the two GEMMs: an implementation that shares nothing with numpy's BLAS path.
 * TEST INFRASTRUCTURE ONLY (see gemm_oracle.py for the reference files each formula restates). Accumulates in
 * double so that it can arbitrate between fp32 evaluations.
 *
 *   oracle_gemm_bf16_tn   : c[i][j] = sum_t a[i][t] * b[j][t], a/b given as bf16 bit patterns
 *                           (contract of yan/jit_kernels/cute_gemm.py:21-38)
 *   oracle_gemm_fp8_nt    : c[i][j] = sum_kb sa[i][kb] * sb[j/128][kb] * sum_{t<128} A[i][128kb+t] * B[j][128kb+t]
 *                           (operands of yan/jit_kernels/gemm.py:23-30; scale granularity of
 *                            yan/include/gemm/fp8_gemm.cuh:48-61)
 *   oracle_gemm_float_nt  : c[i*ldc + j] = alpha * sum_t a[i + t*lda] * b[j + t*ldb] + beta * c[i*ldc + j] on raw
 *                           buffers, in the memory convention of yan/include/gemm/simple_gemm.cuh:210-214
 *                           (A and B with their row index contiguous, C row-major); beta == 0 ignores c's old values
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bf16_to_f32(uint16_t v) {
    uint32_t u = (uint32_t)v << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static float e4m3fn_to_f32(uint8_t v) {
    int e = (v >> 3) & 15, m = v & 7;
    float x;
    if ((v & 0x7f) == 0x7f) return NAN;
    x = e == 0 ? ldexpf((float)m / 8.0f, -6) : ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return (v & 0x80) ? -x : x;
}

void oracle_gemm_bf16_tn(int m, int n, int k, const uint16_t* a, const uint16_t* b, double* c) {
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            double acc = 0.0;
            for (int t = 0; t < k; ++t) acc += (double)bf16_to_f32(a[(size_t)i * k + t]) * bf16_to_f32(b[(size_t)j * k + t]);
            c[(size_t)i * n + j] = acc;
        }
}

/* sa element (i, kb) at sa[i * sa_stride_m + kb * sa_stride_k]; sb is [ceil(n/128)][k/128] row-major. */
void oracle_gemm_fp8_nt(int m, int n, int k, const uint8_t* a, const float* sa, long sa_stride_m, long sa_stride_k,
                        const uint8_t* b, const float* sb, double* c) {
    float table[256];
    int kblocks = k / 128;
    for (int v = 0; v < 256; ++v) table[v] = e4m3fn_to_f32((uint8_t)v);
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            double acc = 0.0;
            for (int kb = 0; kb < kblocks; ++kb) {
                double part = 0.0;
                for (int t = 0; t < 128; ++t)
                    part += (double)table[a[(size_t)i * k + kb * 128 + t]] * table[b[(size_t)j * k + kb * 128 + t]];
                acc += (double)sa[i * sa_stride_m + kb * sa_stride_k] * (double)sb[(size_t)(j / 128) * kblocks + kb] * part;
            }
            c[(size_t)i * n + j] = acc;
        }
}

void oracle_gemm_float_nt(int m, int n, int k, double alpha, const float* a, int lda, const float* b, int ldb,
                          double beta, const float* c_in, double* c_out, int ldc) {
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            double acc = 0.0;
            for (int t = 0; t < k; ++t) acc += (double)a[i + (size_t)t * lda] * (double)b[j + (size_t)t * ldb];
            c_out[(size_t)i * ldc + j] = alpha * acc + (beta != 0.0 ? beta * (double)c_in[(size_t)i * ldc + j] : 0.0);
        }
}
