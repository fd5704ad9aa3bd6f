/*
 * CPU oracle for the Winograd F(2x2,3x3) forward path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic of the reference's two forward
 * ops so that the HIP kernels can be checked against it.  Nothing in the shipped
 * library links, loads or calls it: only the tests, the smoke check and the
 * benchmark's cpu_baseline leg do, and only as the checker / the CPU timing.
 *
 * Every function names the reference lines it follows (paths relative to the
 * reference checkout, xingyul/sparse-winograd-cnn):
 *   IT  = winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans_cuda.cu.cc
 *   ITO = winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans_op.cc
 *   CV  = winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_cuda.cu.cc
 *   CVO = winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_op.cc
 *   CVT = winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_test.py
 *   LIT = ResNet-18-var/winograd_imtrans.py
 *
 * How each function is pinned (the reference ships no golden vectors and cannot
 * be built here: it needs nvcc, cuBLAS and TensorFlow-1.x headers):
 *   oracle_imtrans_f32        matrix form B^T d B in float64 numpy, brute-force
 *                             tile gather, all-ones interior tile, linearity
 *   oracle_relu (relu flag)   elementwise definition max(t,0)
 *   oracle_gemm16_*           numpy float64 matmul
 *   oracle_output_transform   matrix form A^T p A in float64 numpy
 *   oracle_kernel_transform   matrix form G g G^T in float64 numpy
 *   whole path (nl=identity)  conv2d(x, g, stride 1, pad 1) from torch on the CPU,
 *                             the same relation the reference's own tests print
 *                             (CVT:177,187-204), plus a direct 3x3 loop nest
 *   The summation order inside cuBLAS is unspecified, so bitwise parity of the
 *   GEMM stage is unpinned by construction; it is held to a tolerance instead.
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

ORACLE_API int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

ORACLE_API void oracle_set_num_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* Tile counts: nH = (H+1)/2, nW = (W+1)/2 with pad 1 (ITO:46-47; IT:18-19 with pad=1). */
ORACLE_API int oracle_tiles(int extent) { return (extent + 1) / 2; }

/*
 * Input transform T = B^T d B over 4x4 tiles at stride 2, pad 1.
 * X  [B,H,W,C]  ->  TI [16,B,nH,nW,C].
 * Patch gather with zero fill outside the image: IT:22-23,44-92.
 * The 16 sums, each evaluated left to right in fp32: IT:112-127 (same text in CVT:58-73).
 * Store index i*(B*nH*nW*C) + b*nH*nW*C + (th*nW+tw)*C + c: IT:130-148.
 * relu != 0 applies the Winograd-domain ReLU that the layer wrapper applies on
 * the op's result (LIT:16-17): t > 0 ? t : 0.
 */
ORACLE_API void oracle_imtrans_f32(const float *X, float *TI, int B, int H, int W, int C, int relu)
{
    const int nH = (H + 1) / 2, nW = (W + 1) / 2;
    const size_t plane = (size_t)B * nH * nW * C;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b) {
        for (int th = 0; th < nH; ++th) {
            for (int tw = 0; tw < nW; ++tw) {
                const int y0 = 2 * th - 1, x0 = 2 * tw - 1;
                const float *src[16];
                for (int r = 0; r < 4; ++r)
                    for (int s = 0; s < 4; ++s) {
                        const int y = y0 + r, x = x0 + s;
                        src[4 * r + s] = (y > -1 && y < H && x > -1 && x < W)
                                             ? X + (((size_t)b * H + y) * W + x) * C
                                             : NULL;
                    }
                float *dst = TI + ((size_t)b * nH * nW + (size_t)th * nW + tw) * C;
                for (int c = 0; c < C; ++c) {
                    float d[16], t[16];
                    for (int j = 0; j < 16; ++j) d[j] = src[j] ? src[j][c] : 0.0f;
                    t[0]  = d[0] - d[2] - d[8] + d[10];
                    t[1]  = d[1] + d[2] - d[9] - d[10];
                    t[2]  = d[2] - d[1] + d[9] - d[10];
                    t[3]  = d[1] - d[3] - d[9] + d[11];
                    t[4]  = d[4] - d[6] + d[8] - d[10];
                    t[5]  = d[5] + d[6] + d[9] + d[10];
                    t[6]  = d[6] - d[5] - d[9] + d[10];
                    t[7]  = d[5] - d[7] + d[9] - d[11];
                    t[8]  = d[6] - d[4] + d[8] - d[10];
                    t[9]  = d[9] - d[6] - d[5] + d[10];
                    t[10] = d[5] - d[6] - d[9] + d[10];
                    t[11] = d[7] - d[5] + d[9] - d[11];
                    t[12] = d[4] - d[6] - d[12] + d[14];
                    t[13] = d[5] + d[6] - d[13] - d[14];
                    t[14] = d[6] - d[5] + d[13] - d[14];
                    t[15] = d[5] - d[7] - d[13] + d[15];
                    if (relu)
                        for (int i = 0; i < 16; ++i) t[i] = t[i] > 0.0f ? t[i] : 0.0f;
                    for (int i = 0; i < 16; ++i) dst[(size_t)i * plane + c] = t[i];
                }
            }
        }
    }
}

/*
 * The 16 per-position products P[i] (M x K, row-major) = TI[i] (M x C) . Wt[i] (C x K).
 * Reference: cublasSgemmBatched(N, N, m=K, n=M, k=C, A=Weight lda=K, B=Input ldb=C,
 * C=tmp ldc=K, batch 16) read as column-major, CV:80-85; operand bases i*M*C, i*K*C,
 * i*M*K from the `assign` kernel CV:55-61.  fp32 accumulation in ascending c.
 */
__attribute__((target_clones("arch=skylake-avx512", "arch=haswell", "default"), optimize("fp-contract=fast")))
static void gemm_rows_f32(const float *A, const float *Wt, float *P, long m0, long m1, int C, int K)
{
    for (long m = m0; m < m1; ++m) {
        float *p = P + (size_t)m * K;
        const float *a = A + (size_t)m * C;
        for (int k = 0; k < K; ++k) p[k] = 0.0f;
        for (int c = 0; c < C; ++c) {
            const float av = a[c];
            const float *w = Wt + (size_t)c * K;
            for (int k = 0; k < K; ++k) p[k] += av * w[k];
        }
    }
}

ORACLE_API void oracle_gemm16_f32(const float *TI, const float *Wt, float *P, long M, int C, int K)
{
    const long blk = 64;
    const long nblk = (M + blk - 1) / blk;
#pragma omp parallel for collapse(2) schedule(static)
    for (int i = 0; i < 16; ++i)
        for (long bi = 0; bi < nblk; ++bi) {
            const long m0 = bi * blk, m1 = (m0 + blk < M) ? m0 + blk : M;
            gemm_rows_f32(TI + (size_t)i * M * C, Wt + (size_t)i * C * K, P + (size_t)i * M * K, m0, m1, C, K);
        }
}

/* Same contraction with a float64 accumulator, rounded once to fp32: the error yardstick. */
ORACLE_API void oracle_gemm16_f64acc(const float *TI, const float *Wt, float *P, long M, int C, int K)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int i = 0; i < 16; ++i)
        for (long m = 0; m < M; ++m) {
            const float *a = TI + ((size_t)i * M + m) * C;
            const float *w = Wt + (size_t)i * C * K;
            float *p = P + ((size_t)i * M + m) * K;
            double acc[K];
            for (int k = 0; k < K; ++k) acc[k] = 0.0;
            for (int c = 0; c < C; ++c) {
                const double av = (double)a[c];
                for (int k = 0; k < K; ++k) acc[k] += av * (double)w[(size_t)c * K + k];
            }
            for (int k = 0; k < K; ++k) p[k] = (float)acc[k];
        }
}

/*
 * Output transform Y = A^T p A and 2x2 scatter.
 * P [16,B,nH,nW,K] -> Out [B,2nH,2nW,K] (never cropped: CVO:53).
 * Loads CV:22-37; the four 9-term sums, left to right, CV:39-46 (same text CVT:144-147);
 * scatter to (2th+dy, 2tw+dx) CV:48-51.
 */
ORACLE_API void oracle_output_transform_f32(const float *P, float *Out, int B, int nH, int nW, int K)
{
    const size_t plane = (size_t)B * nH * nW * K;
    const int H = 2 * nH, W = 2 * nW;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b)
        for (int th = 0; th < nH; ++th)
            for (int tw = 0; tw < nW; ++tw) {
                const float *src = P + (((size_t)b * nH + th) * nW + tw) * K;
                float *o00 = Out + (((size_t)b * H + 2 * th) * W + 2 * tw) * K;
                float *o01 = o00 + K;
                float *o10 = o00 + (size_t)W * K;
                float *o11 = o10 + K;
                for (int k = 0; k < K; ++k) {
                    float p[16];
                    for (int i = 0; i < 16; ++i) p[i] = src[(size_t)i * plane + k];
                    o00[k] = p[0] + p[1] + p[2] + p[4] + p[5] + p[6] + p[8] + p[9] + p[10];
                    o01[k] = p[1] - p[2] - p[3] + p[5] - p[6] - p[7] + p[9] - p[10] - p[11];
                    o10[k] = p[4] + p[5] + p[6] - p[8] - p[9] - p[10] - p[12] - p[13] - p[14];
                    o11[k] = p[5] - p[6] - p[7] - p[9] + p[10] + p[11] - p[13] + p[14] + p[15];
                }
            }
}

/*
 * The whole conv op: batched GEMM into a 16*M*K product buffer, then the output
 * transform (launcher order CV:65-93; shapes CVO:45-53).  `tmp` must hold 16*M*K
 * floats, M = B*nH*nW (CVO:57-59).  acc64 selects the float64-accumulated GEMM.
 */
ORACLE_API void oracle_conv_f32(const float *TI, const float *Wt, float *Out, float *tmp,
                                int C, int B, int nH, int nW, int K, int acc64)
{
    const long M = (long)B * nH * nW;
    if (acc64)
        oracle_gemm16_f64acc(TI, Wt, tmp, M, C, K);
    else
        oracle_gemm16_f32(TI, Wt, tmp, M, C, K);
    oracle_output_transform_f32(tmp, Out, B, nH, nW, K);
}

/*
 * Kernel transform U = G g G^T of a [3,3,C,K] (HWIO) kernel into [16,C,K], i = 4r+s.
 * Test-only helper in the reference: CVT:8-25.  Each term is divided before it is
 * summed, as there (CVT:13-20); divisions by 2 and 4 are exact in binary fp.
 */
ORACLE_API void oracle_kernel_transform_f32(const float *g, float *U, int C, int K)
{
    const size_t ck = (size_t)C * K;
    for (size_t e = 0; e < ck; ++e) {
        float q[9];
        for (int j = 0; j < 9; ++j) q[j] = g[(size_t)j * ck + e];
        float u[16];
        u[0]  = q[0];
        u[1]  = q[0] / 2 + q[1] / 2 + q[2] / 2;
        u[2]  = q[0] / 2 - q[1] / 2 + q[2] / 2;
        u[3]  = q[2];
        u[4]  = q[0] / 2 + q[3] / 2 + q[6] / 2;
        u[5]  = q[0] / 4 + q[1] / 4 + q[2] / 4 + q[3] / 4 + q[4] / 4 + q[5] / 4 + q[6] / 4 + q[7] / 4 + q[8] / 4;
        u[6]  = q[0] / 4 - q[1] / 4 + q[2] / 4 + q[3] / 4 - q[4] / 4 + q[5] / 4 + q[6] / 4 - q[7] / 4 + q[8] / 4;
        u[7]  = q[2] / 2 + q[5] / 2 + q[8] / 2;
        u[8]  = q[0] / 2 - q[3] / 2 + q[6] / 2;
        u[9]  = q[0] / 4 + q[1] / 4 + q[2] / 4 - q[3] / 4 - q[4] / 4 - q[5] / 4 + q[6] / 4 + q[7] / 4 + q[8] / 4;
        u[10] = q[0] / 4 - q[1] / 4 + q[2] / 4 - q[3] / 4 + q[4] / 4 - q[5] / 4 + q[6] / 4 - q[7] / 4 + q[8] / 4;
        u[11] = q[2] / 2 - q[5] / 2 + q[8] / 2;
        u[12] = q[6];
        u[13] = q[6] / 2 + q[7] / 2 + q[8] / 2;
        u[14] = q[6] / 2 - q[7] / 2 + q[8] / 2;
        u[15] = q[8];
        for (int i = 0; i < 16; ++i) U[(size_t)i * ck + e] = u[i];
    }
}
