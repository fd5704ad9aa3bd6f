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
 *   oracle_affine_f32         float64 x*s+t on inputs where that sum is exact, so that rounding
 *                             it once to fp32 is the fused result (and differs from mul-then-add)
 *   whole path (nl=identity)  conv2d(x, g, stride 1, pad 1) from torch on the CPU,
 *                             the same relation the reference's own tests print
 *                             (CVT:177,187-204), plus a direct 3x3 loop nest
 *   The summation order inside cuBLAS is unspecified, so bitwise parity of the
 *   GEMM stage is unpinned by construction; it is held to a tolerance instead.
 */
#include <math.h>
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

/* ---------------------------------------------------------------------------------------
 * Backward ops (CVG = winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_grad_cuda.cu.cc,
 * ITG = winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans_grad_cuda.cu.cc).
 * Pinned in tests/test_oracle_grad.py by the adjoint identities <f(x), g> == <x, f^T(g)>,
 * exact on integer inputs, against the forward functions above (which are pinned on their
 * own), and by float64 matrix forms.
 * ------------------------------------------------------------------------------------- */

/*
 * Gradient of the output transform: dP = A dY A^T per tile, [B,2nH,2nW,K] -> [16,B,nH,nW,K].
 * The 16 expressions of Grad_inverse_transform, CVG:22-43; store order CVG:46-64.
 */
ORACLE_API void oracle_output_transform_grad_f32(const float *dY, float *dP, int B, int nH, int nW, int K)
{
    const size_t plane = (size_t)B * nH * nW * K;
    const int H = 2 * nH, W = 2 * nW;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b)
        for (int th = 0; th < nH; ++th)
            for (int tw = 0; tw < nW; ++tw) {
                const float *g0 = dY + (((size_t)b * H + 2 * th) * W + 2 * tw) * K;
                const float *g1 = g0 + K, *g2 = g0 + (size_t)W * K, *g3 = g2 + K;
                float *dst = dP + (((size_t)b * nH + th) * nW + tw) * K;
                for (int k = 0; k < K; ++k) {
                    const float a = g0[k], bb = g1[k], c = g2[k], d = g3[k];
                    float p[16];
                    p[0] = a;          p[1] = a + bb;          p[2] = a - bb;          p[3] = -bb;
                    p[4] = a + c;      p[5] = a + bb + c + d;  p[6] = a - bb + c - d;  p[7] = -bb - d;
                    p[8] = a - c;      p[9] = a + bb - c - d;  p[10] = a - bb - c + d; p[11] = d - bb;
                    p[12] = -c;        p[13] = -c - d;         p[14] = d - c;          p[15] = d;
                    for (int i = 0; i < 16; ++i) dst[(size_t)i * plane + k] = p[i];
                }
            }
}

/*
 * Winograd2x2ConvGrad (launcher CVG:77-124): dP as above, then per position
 *   dTI[i] (M x C) = dP[i] (M x K) . W[i]^T      (cublasSgemmBatched T,N  CVG:103-108)
 *   dW[i]  (C x K) = TI[i]^T (C x M) . dP[i]     (cublasSgemmBatched N,T  CVG:115-120)
 * accumulated in float64.  tmp holds 16*M*K floats (conv_grad_op.cc:68-70).
 */
ORACLE_API void oracle_conv_grad_f32(const float *TI, const float *Wt, const float *dY, float *dTI, float *dW,
                                     float *tmp, int C, int B, int nH, int nW, int K)
{
    const long M = (long)B * nH * nW;
    oracle_output_transform_grad_f32(dY, tmp, B, nH, nW, K);
#pragma omp parallel for collapse(2) schedule(static)
    for (int i = 0; i < 16; ++i)
        for (long m = 0; m < M; ++m) {
            const float *dp = tmp + ((size_t)i * M + m) * K;
            float *o = dTI + ((size_t)i * M + m) * C;
            for (int c = 0; c < C; ++c) {
                const float *w = Wt + ((size_t)i * C + c) * K;
                double acc = 0.0;
                for (int k = 0; k < K; ++k) acc += (double)dp[k] * (double)w[k];
                o[c] = (float)acc;
            }
        }
#pragma omp parallel for collapse(2) schedule(static)
    for (int i = 0; i < 16; ++i)
        for (int c = 0; c < C; ++c) {
            double acc[K];
            for (int k = 0; k < K; ++k) acc[k] = 0.0;
            for (long m = 0; m < M; ++m) {
                const double a = (double)TI[((size_t)i * M + m) * C + c];
                const float *dp = tmp + ((size_t)i * M + m) * K;
                for (int k = 0; k < K; ++k) acc[k] += a * (double)dp[k];
            }
            for (int k = 0; k < K; ++k) dW[((size_t)i * C + c) * K + k] = (float)acc[k];
        }
}

/*
 * Per-channel affine map ahead of the transform: y = fmaf(x, scale[c], shift[c]) on every pixel of
 * X [B,H,W,C] (the padding the transform adds afterwards stays zero).  Restates the reference
 * model's BatchNorm-then-WinogradImTrans pairs at inference
 * (ResNet-18-var/imagenet-resnet-transWino-prune.py:117-118 ... :209-210) with the normalisation
 * reduced to scale = gamma/sqrt(var+eps), shift = beta - mean*scale.  fmaf rounds once.
 */
ORACLE_API void oracle_affine_f32(const float *X, const float *scale, const float *shift, float *Y, long pixels, int C)
{
#pragma omp parallel for schedule(static)
    for (long p = 0; p < pixels; ++p)
        for (int c = 0; c < C; ++c) Y[p * C + c] = fmaf(X[p * C + c], scale[c], shift[c]);
}


/*
 * Winograd2x2ImTransGrad: dX = sum over tiles of (B dT B^T) scattered back onto the 4x4 patch the
 * tile was gathered from (pixels outside the image drop out).  dT [16,B,nH,nW,C] -> dX [B,H,W,C].
 * The per-tile matrix follows OutputGradTransform ITG:39-62; the placement follows the gather of
 * Winograd2x2ImTransGradCompute ITG:98-114 (tile (h_col,w_col), patch offset (y+1-2h_col, x+1-2w_col)).
 * If `mask_src` is not NULL, dT is first multiplied by (mask_src > 0): the backward of the fused
 * Winograd-domain ReLU, mask_src being the forward op's (post-ReLU) output.
 * Unlike the reference, the incoming gradient is left untouched (ITG:124 overwrites it).
 */
ORACLE_API void oracle_imtrans_grad_f32(const float *dT, const float *mask_src, float *dX, int B, int H, int W, int C)
{
    const int nH = (H + 1) / 2, nW = (W + 1) / 2;
    const size_t plane = (size_t)B * nH * nW * C;
    memset(dX, 0, sizeof(float) * (size_t)B * H * W * C);
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; ++b) {
        double *acc = (double *)__builtin_malloc(sizeof(double) * (size_t)H * W * C);
        for (size_t e = 0; e < (size_t)H * W * C; ++e) acc[e] = 0.0;
        for (int th = 0; th < nH; ++th)
            for (int tw = 0; tw < nW; ++tw)
                for (int c = 0; c < C; ++c) {
                    const size_t off = (((size_t)b * nH + th) * nW + tw) * C + c;
                    double t[16], d[16];
                    for (int i = 0; i < 16; ++i) {
                        t[i] = (double)dT[(size_t)i * plane + off];
                        if (mask_src && !(mask_src[(size_t)i * plane + off] > 0.0f)) t[i] = 0.0;
                    }
                    d[0] = t[0];
                    d[1] = t[1] - t[2] + t[3];
                    d[2] = t[1] - t[0] + t[2];
                    d[3] = -t[3];
                    d[4] = t[4] - t[8] + t[12];
                    d[5] = t[5] - t[6] + t[7] - t[9] + t[10] - t[11] + t[13] - t[14] + t[15];
                    d[6] = t[5] - t[4] + t[6] + t[8] - t[9] - t[10] - t[12] + t[13] + t[14];
                    d[7] = t[11] - t[7] - t[15];
                    d[8] = t[4] - t[0] + t[8];
                    d[9] = t[2] - t[1] - t[3] + t[5] - t[6] + t[7] + t[9] - t[10] + t[11];
                    d[10] = t[0] - t[1] - t[2] - t[4] + t[5] + t[6] - t[8] + t[9] + t[10];
                    d[11] = t[3] - t[7] - t[11];
                    d[12] = -t[12];
                    d[13] = t[14] - t[13] - t[15];
                    d[14] = t[12] - t[13] - t[14];
                    d[15] = t[15];
                    for (int r = 0; r < 4; ++r)
                        for (int s = 0; s < 4; ++s) {
                            const int y = 2 * th - 1 + r, x = 2 * tw - 1 + s;
                            if (y > -1 && y < H && x > -1 && x < W) acc[((size_t)y * W + x) * C + c] += d[4 * r + s];
                        }
                }
        float *o = dX + (size_t)b * H * W * C;
        for (size_t e = 0; e < (size_t)H * W * C; ++e) o[e] = (float)acc[e];
        __builtin_free(acc);
    }
}
