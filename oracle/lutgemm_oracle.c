/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference LUT-GEMM arithmetic.
 *
 * This file is the checker for the HIP kernels.  It is compiled into oracle/_build/ and may be
 * loaded only by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py.
 * Nothing in the product package links, imports or falls back to it.
 *
 * Each function restates one reference kernel as plain loops over the same row-major operands and
 * the same padded table indexing:
 *   table entry (a, b) lives at a * lut_cols + b, lut_cols = 2^bits + 2
 *   (self_ops/src/approx_mult.h:17-18, self_ops/ops_py/approx_ops.py:70-77).
 *
 * Pinned by tests/test_oracle.py: brute-force numpy sums on small shapes, the exact-multiplier
 * table (reduces to integer matmul), STE tables (reduce to dense gC.B^T / A^T.gC), masked code 2^bits.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Forward: C[m,n] = sum_k lut[A[m,k]*lut_cols + B[k,n]], 32-bit unsigned wrap-around accumulate.
 * Follows self_ops/src/approx_gemm_forward.cu:183-207 (sum) and :219-227 (store). */
void oracle_lutgemm_forward(const uint8_t *A, const uint8_t *B, uint32_t *C, const uint16_t *lut,
                            int lut_cols, int M, int K, int N) {
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m) {
        uint32_t *crow = C + (size_t)m * N;
        for (int n = 0; n < N; ++n) crow[n] = 0u;
        for (int k = 0; k < K; ++k) {
            const uint16_t *lrow = lut + (size_t)A[(size_t)m * K + k] * lut_cols;
            const uint8_t *brow = B + (size_t)k * N;
            for (int n = 0; n < N; ++n) crow[n] += lrow[brow[n]];
        }
    }
}

/* Backward, reference order: fp32 accumulate, sequential over the reduction index, one fused
 * multiply-add per term, scaled by `factor` (1/16) once at the end.
 *   gA[m,k] = factor * sum_n gC[m,n] * (float)lutA[A[m,k]][B[k,n]]
 *       (self_ops/src/approx_gemm_backward.cu:213-227 accumulate, :235-241 scale)
 *   gB[k,n] = factor * sum_m (float)lutB[A[m,k]][B[k,n]] * gC[m,n]
 *       (self_ops/src/approx_gemm_backward.cu:447-461 accumulate, :469-475 scale) */
void oracle_lutgemm_backward_f32(const float *gC, const uint8_t *A, const uint8_t *B, float *gA,
                                 float *gB, const int16_t *lutA, const int16_t *lutB, int lut_cols,
                                 float factor, int M, int K, int N) {
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m) {
        for (int k = 0; k < K; ++k) {
            const int16_t *lrow = lutA + (size_t)A[(size_t)m * K + k] * lut_cols;
            float acc = 0.0f;
            for (int n = 0; n < N; ++n)
                acc = fmaf(gC[(size_t)m * N + n], (float)lrow[B[(size_t)k * N + n]], acc);
            gA[(size_t)m * K + k] = acc * factor;
        }
    }
#pragma omp parallel for schedule(static)
    for (int k = 0; k < K; ++k) {
        for (int n = 0; n < N; ++n) {
            const int b = B[(size_t)k * N + n];
            float acc = 0.0f;
            for (int m = 0; m < M; ++m)
                acc = fmaf((float)lutB[(size_t)A[(size_t)m * K + k] * lut_cols + b],
                           gC[(size_t)m * N + n], acc);
            gB[(size_t)k * N + n] = acc * factor;
        }
    }
}

/* Backward, exact sums in double (the judge of the 1e-5 tolerance); tables given as double so the
 * same routine serves int16x16 tables and unrounded fp32 slope tables.  Also returns sum |term|
 * per output (absA/absB may be NULL) for term-magnitude-relative error checks. */
void oracle_lutgemm_backward_f64(const float *gC, const uint8_t *A, const uint8_t *B, double *gA,
                                 double *gB, double *absA, double *absB, const double *lutA,
                                 const double *lutB, int lut_cols, double factor, int M, int K, int N) {
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m) {
        for (int k = 0; k < K; ++k) {
            const double *lrow = lutA + (size_t)A[(size_t)m * K + k] * lut_cols;
            double acc = 0.0, ab = 0.0;
            for (int n = 0; n < N; ++n) {
                double t = (double)gC[(size_t)m * N + n] * lrow[B[(size_t)k * N + n]];
                acc += t;
                ab += fabs(t);
            }
            gA[(size_t)m * K + k] = acc * factor;
            if (absA) absA[(size_t)m * K + k] = ab * factor;
        }
    }
#pragma omp parallel for schedule(static)
    for (int k = 0; k < K; ++k) {
        for (int n = 0; n < N; ++n) {
            const int b = B[(size_t)k * N + n];
            double acc = 0.0, ab = 0.0;
            for (int m = 0; m < M; ++m) {
                double t = lutB[(size_t)A[(size_t)m * K + k] * lut_cols + b] * (double)gC[(size_t)m * N + n];
                acc += t;
                ab += fabs(t);
            }
            gB[(size_t)k * N + n] = acc * factor;
            if (absB) absB[(size_t)k * N + n] = ab * factor;
        }
    }
}

/* gB alone, same float64 sums as oracle_lutgemm_backward_f64 (self_ops/src/approx_gemm_backward.cu:447-461
 * accumulate, :469-475 scale), walking A and gC row by row so that layers with hundreds of thousands of rows
 * finish in seconds: every thread owns a block of k and keeps its [k][n] sums; the order of the additions over m
 * is the reference's (m ascending).  Pinned by tests/test_oracle.py against oracle_lutgemm_backward_f64. */
void oracle_lutgemm_gradB_f64_rows(const float *gC, const uint8_t *A, const uint8_t *B, double *gB, double *absB,
                                   const double *lutB, int lut_cols, double factor, int M, int K, int N) {
    const int KB = 8;
#pragma omp parallel for schedule(dynamic, 1)
    for (int kb = 0; kb < K; kb += KB) {
        const int ke = kb + KB < K ? kb + KB : K;
        double *acc = (double *)calloc((size_t)2 * KB * N, sizeof(double));
        for (int m = 0; m < M; ++m) {
            const float *g = gC + (size_t)m * N;
            for (int k = kb; k < ke; ++k) {
                const double *lrow = lutB + (size_t)A[(size_t)m * K + k] * lut_cols;
                const uint8_t *brow = B + (size_t)k * N;
                double *s = acc + (size_t)2 * (k - kb) * N;
                for (int n = 0; n < N; ++n) {
                    const double t = lrow[brow[n]] * (double)g[n];
                    s[n] += t;
                    s[N + n] += fabs(t);
                }
            }
        }
        for (int k = kb; k < ke; ++k)
            for (int n = 0; n < N; ++n) {
                gB[(size_t)k * N + n] = acc[(size_t)2 * (k - kb) * N + n] * factor;
                if (absB) absB[(size_t)k * N + n] = acc[(size_t)2 * (k - kb) * N + N + n] * factor;
            }
        free(acc);
    }
}

/* Accurate fp32 GEMM C = A.B, sequential fp32 FMA over k
 * (self_ops/src/approx_gemm_forward.cu:456-470). */
void oracle_accgemm_forward_f32(const float *A, const float *B, float *C, int M, int K, int N) {
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m) {
        float *crow = C + (size_t)m * N;
        for (int n = 0; n < N; ++n) crow[n] = 0.0f;
        for (int k = 0; k < K; ++k) {
            const float a = A[(size_t)m * K + k];
            const float *brow = B + (size_t)k * N;
            for (int n = 0; n < N; ++n) crow[n] = fmaf(a, brow[n], crow[n]);
        }
    }
}
