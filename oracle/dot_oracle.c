/*
 * TEST INFRASTRUCTURE - not part of the product.  Only tests/, the smoke check
 * and bench.py's cpu_baseline leg may call this.
 *
 * CPU restatement of the reference contract behind Tensor.Dot and
 * Tensor.BatchMatrixMultiplication.  The reference holds no GEMM arithmetic of
 * its own: CpuTensor.Dot forwards to Intel MKL cblas_sgemm (mkl_rt, version not
 * pinned by the reference: Prod/Data/BlasServices.cs:44-45, README.md:22).  What
 * the reference does define, and what is restated here, is
 *   - how M, N, K and the leading dimensions follow from the operand shapes and
 *     transpose flags            (Prod/Data/BlasServices.cs:14-19),
 *   - the row-major meaning of the call      (BlasServices.cs:20, order 101),
 *   - the serial per-matrix loop of the batched form
 *                                (Prod/CPU/CpuTensor.cs:3018-3024).
 * The arithmetic itself is the published definition of SGEMM
 * (C <- alpha*op(A)*op(B) + beta*C; when beta == 0, C is not read), evaluated
 * with a double-precision accumulator and rounded once, so it sits inside the
 * rounding envelope of any fp32 summation order MKL may choose.
 */
#include <stddef.h>
#include <stdlib.h>

/* BlasServices.DotMkl, Prod/Data/BlasServices.cs:10-21 */
void oracle_dot(const float* A, int aH, int aW, int transposeA, const float* B, int bH, int bW, int transposeB,
                float* C, float alpha, float beta)
{
    const int M = transposeA ? aW : aH;   /* BlasServices.cs:14 */
    const int N = transposeB ? bH : bW;   /* :15 */
    const int K = transposeA ? aH : aW;   /* :16 */
    const int lda = aW, ldb = bW, ldc = N; /* :17-19 */
    (void)bH;
    if (M <= 0 || N <= 0) return;
#pragma omp parallel
    {
        /* one row of C at a time, accumulated in double; the loop order keeps the
         * innermost access to B contiguous for either transpose flag */
        double* acc = (double*)malloc(sizeof(double) * (size_t)N);
        int m;
#pragma omp for schedule(static)
        for (m = 0; m < M; ++m) {
            for (int n = 0; n < N; ++n) acc[n] = 0.0;
            if (!transposeB) {
                for (int k = 0; k < K; ++k) {
                    const double a = transposeA ? A[(size_t)k * lda + m] : A[(size_t)m * lda + k];
                    const float* brow = B + (size_t)k * ldb;
                    for (int n = 0; n < N; ++n) acc[n] += a * (double)brow[n];
                }
            } else {
                for (int n = 0; n < N; ++n) {
                    const float* brow = B + (size_t)n * ldb;
                    double s = 0.0;
                    for (int k = 0; k < K; ++k) {
                        const double a = transposeA ? A[(size_t)k * lda + m] : A[(size_t)m * lda + k];
                        s += a * (double)brow[k];
                    }
                    acc[n] = s;
                }
            }
            for (int n = 0; n < N; ++n) {
                double r = (double)alpha * acc[n];
                if (beta != 0.0f) r += (double)beta * (double)C[(size_t)m * ldc + n];
                C[(size_t)m * ldc + n] = (float)r;
            }
        }
        free(acc);
    }
}

/* CpuTensor.BatchMatrixMultiplication, Prod/CPU/CpuTensor.cs:3004-3025: a serial
 * loop of Dot over the matrices of three 3-D tensors; sub-tensor i starts at
 * i * MultDim0 (GetSubTensor -> Slice(Idx(i))). */
void oracle_bmm(const float* A, int aH, int aW, int transposeA, const float* B, int bH, int bW, int transposeB,
                float* C, int batch, float alpha, float beta)
{
    const int M = transposeA ? aW : aH;
    const int N = transposeB ? bH : bW;
    for (int i = 0; i < batch; ++i) {
        oracle_dot(A + (size_t)i * aH * aW, aH, aW, transposeA, B + (size_t)i * bH * bW, bH, bW, transposeB,
                   C + (size_t)i * M * N, alpha, beta);
    }
}

/* Column-major SGEMM as cuBLAS defines it (the reference's GPU call sites,
 * Prod/GPU/GpuTensor.cs:1192,1218, use this form).  Used to check that the
 * library's cuBLAS-shaped entry points honour lda/ldb/ldc and the op flags. */
void oracle_sgemm_colmajor(int transa, int transb, int m, int n, int k, float alpha, const float* A, int lda,
                           const float* B, int ldb, float beta, float* C, int ldc)
{
    int j;
#pragma omp parallel for schedule(static)
    for (j = 0; j < n; ++j) {
        for (int i = 0; i < m; ++i) {
            double s = 0.0;
            for (int l = 0; l < k; ++l) {
                const float a = transa ? A[(size_t)i * lda + l] : A[(size_t)l * lda + i];
                const float b = transb ? B[(size_t)l * ldb + j] : B[(size_t)j * ldb + l];
                s += (double)a * (double)b;
            }
            double r = (double)alpha * s;
            if (beta != 0.0f) r += (double)beta * (double)C[(size_t)j * ldc + i];
            C[(size_t)j * ldc + i] = (float)r;
        }
    }
}
