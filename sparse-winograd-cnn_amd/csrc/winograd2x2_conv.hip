// Winograd F(2x2,3x3) convolution for gfx950: the 16 per-position GEMMs
// P_i [M,K] = TI_i [M,C] . W_i [C,K] on the matrix cores, with the output transform
// Y = A^T p A folded into the same kernel.
//
// Stands in for Winograd2x2ConvComputeLauncher of the reference
// (winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_cuda.cu.cc:65-93): the `assign`
// pointer-table kernel (:55-61), cublasSgemmBatched (:80-85) and the Output_transform
// kernel (:12-53) with its 16*M*K product buffer in between.
//
// A workgroup owns a BM x BN tile of the [M,K] plane and walks the 16 positions in
// ascending order.  For each position it accumulates P_i over C with fp32 MFMA, then
// adds +-P_i into four running tiles Y0..Y3.  Every one of the reference's 9-term sums
// (:39-46) lists its terms in ascending i, so this rolling accumulation reproduces
// their association exactly; only the order of the reduction over C (unspecified in
// cuBLAS) differs.  The products never reach memory.

#include "swc_common.h"

namespace swc {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// Signs of A^T (x) A^T: bit (4*i + j) set when +-P_i enters Y_j, j = 2*dy + dx.
// Row i = 4r+s contributes AT[dy][r]*AT[dx][s] with AT = [[1,1,1,0],[0,1,-1,-1]].
constexpr int kAT[2][4] = {{1, 1, 1, 0}, {0, 1, -1, -1}};
constexpr unsigned long long sign_mask(int want)
{
    unsigned long long m = 0;
    for (int i = 0; i < 16; ++i)
        for (int j = 0; j < 4; ++j)
            if (kAT[j / 2][i / 4] * kAT[j % 2][i % 4] == want) m |= 1ull << (4 * i + j);
    return m;
}
constexpr unsigned long long kPlus = sign_mask(1);
constexpr unsigned long long kMinus = sign_mask(-1);

// Round an fp32 value to the nearest bf16 (ties to even) and return it widened back to fp32.
__device__ __forceinline__ float round_bf16(float x)
{
    unsigned u = __float_as_uint(x);
    if ((u & 0x7f800000u) == 0x7f800000u) return x;  // inf / nan pass through
    u += 0x7fffu + ((u >> 16) & 1u);
    return __uint_as_float(u & 0xffff0000u);
}

template <int BM_, int BN_, int BK_, int WGM_, int WGN_>
struct ConvCfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_;
    static constexpr int NT = WGM * WGN * 64;      // threads per workgroup
    static constexpr int WM = BM / WGM, WN = BN / WGN;  // wave tile
    static constexpr int TM = WM / 32, TN = WN / 32;    // 32x32 MFMA tiles per wave
    static constexpr int LDA = BK + 4;  // row stride (floats): 4*odd keeps b128 row reads conflict-free
    static constexpr int LDB = BN + 4;
    static constexpr int NA = BM * BK / (4 * NT);  // float4 per thread per A tile
    static constexpr int NB = BK * BN / (4 * NT);
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile is made of 32x32 MFMA tiles");
    static_assert(BK % 8 == 0, "a k-step feeds 4 MFMAs from one b128 read per lane group");
    static_assert(BM * BK % (4 * NT) == 0 && BK * BN % (4 * NT) == 0, "tile loads divide evenly");
};

// VEC: C and K are multiples of 4 and all pointers 16-byte aligned (float4 global loads).
// BF16: both operands are rounded to bf16 on their way into LDS.
template <typename Cfg, bool VEC, bool BF16>
__global__ __launch_bounds__(Cfg::NT) void conv_f32_kernel(const float *__restrict__ TI, const float *__restrict__ Wt,
                                                           float *__restrict__ Out, size_t M, int C, int K, int nH,
                                                           int nW, unsigned tiles_n)
{
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, NT = Cfg::NT;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, LDA = Cfg::LDA, LDB = Cfg::LDB, NA = Cfg::NA, NB = Cfg::NB;

    __shared__ __attribute__((aligned(16))) float As[2][BM * LDA];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB];

    const unsigned lid = xcd_swizzle(blockIdx.x, gridDim.x);
    const size_t m0 = static_cast<size_t>(lid / tiles_n) * BM;
    const int n0 = static_cast<int>(lid % tiles_n) * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lg = lane >> 5;
    const int wm0 = (wave / Cfg::WGN) * Cfg::WM, wn0 = (wave % Cfg::WGN) * Cfg::WN;

    const int nkc = (C + BK - 1) / BK;
    const int steps = 16 * nkc;

    float4 ra[NA], rb[NB];

    auto load_global = [&](int s) {
        const int pos = s / nkc;
        const int c0 = (s - pos * nkc) * BK;
        const float *a_base = TI + static_cast<size_t>(pos) * M * C;
        const float *b_base = Wt + static_cast<size_t>(pos) * C * K;
#pragma unroll
        for (int q = 0; q < NA; ++q) {
            const int f = tid + q * NT;
            const int row = f / (BK / 4), c = c0 + (f % (BK / 4)) * 4;
            const size_t gm = m0 + row;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (gm < M) {
                const float *p = a_base + gm * C + c;
                if (VEC) {
                    if (c < C) v = *reinterpret_cast<const float4 *>(p);
                } else {
                    if (c + 0 < C) v.x = p[0];
                    if (c + 1 < C) v.y = p[1];
                    if (c + 2 < C) v.z = p[2];
                    if (c + 3 < C) v.w = p[3];
                }
            }
            ra[q] = v;
        }
#pragma unroll
        for (int q = 0; q < NB; ++q) {
            const int f = tid + q * NT;
            const int row = f / (BN / 4), n = n0 + (f % (BN / 4)) * 4;
            const int c = c0 + row;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (c < C) {
                const float *p = b_base + static_cast<size_t>(c) * K + n;
                if (VEC) {
                    if (n < K) v = *reinterpret_cast<const float4 *>(p);
                } else {
                    if (n + 0 < K) v.x = p[0];
                    if (n + 1 < K) v.y = p[1];
                    if (n + 2 < K) v.z = p[2];
                    if (n + 3 < K) v.w = p[3];
                }
            }
            rb[q] = v;
        }
    };

    auto store_lds = [&](int buf) {
#pragma unroll
        for (int q = 0; q < NA; ++q) {
            const int f = tid + q * NT;
            const int row = f / (BK / 4), c4 = f % (BK / 4);
            float4 v = ra[q];
            if (BF16) v = make_float4(round_bf16(v.x), round_bf16(v.y), round_bf16(v.z), round_bf16(v.w));
            *reinterpret_cast<float4 *>(&As[buf][row * LDA + c4 * 4]) = v;
        }
#pragma unroll
        for (int q = 0; q < NB; ++q) {
            const int f = tid + q * NT;
            const int row = f / (BN / 4), n4 = f % (BN / 4);
            float4 v = rb[q];
            if (BF16) v = make_float4(round_bf16(v.x), round_bf16(v.y), round_bf16(v.z), round_bf16(v.w));
            *reinterpret_cast<float4 *>(&Bs[buf][row * LDB + n4 * 4]) = v;
        }
    };

    floatx16 P[TM][TN];
    floatx16 Y[4][TM][TN];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                P[tm][tn][r] = 0.f;
#pragma unroll
                for (int j = 0; j < 4; ++j) Y[j][tm][tn][r] = 0.f;
            }
        }

    load_global(0);
    store_lds(0);
    __syncthreads();

    int kc = 0, pos = 0;
    for (int s = 0; s < steps; ++s) {
        const int buf = s & 1;
        if (s + 1 < steps) load_global(s + 1);

        const float *as = As[buf];
        const float *bs = Bs[buf];
#pragma unroll
        for (int kk = 0; kk < BK; kk += 8) {
            // Lane group lg feeds reduction indices kk+4*lg .. kk+4*lg+3, one per MFMA; the
            // order in which indices are reduced is free as long as A and B agree.
            float4 a[TM];
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
                a[tm] = *reinterpret_cast<const float4 *>(&as[(wm0 + tm * 32 + li) * LDA + kk + 4 * lg]);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                float b[TN];
#pragma unroll
                for (int tn = 0; tn < TN; ++tn) b[tn] = bs[(kk + 4 * lg + t) * LDB + wn0 + tn * 32 + li];
#pragma unroll
                for (int tm = 0; tm < TM; ++tm) {
                    const float av = t == 0 ? a[tm].x : t == 1 ? a[tm].y : t == 2 ? a[tm].z : a[tm].w;
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn)
                        P[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, b[tn], P[tm][tn], 0, 0, 0);
                }
            }
        }

        if (++kc == nkc) {
            // P_pos is complete: fold it into the running output tiles, ascending pos.
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int bit = 4 * pos + j;
                const bool plus = (kPlus >> bit) & 1ull, minus = (kMinus >> bit) & 1ull;
                if (plus) {
#pragma unroll
                    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                        for (int tn = 0; tn < TN; ++tn) Y[j][tm][tn] += P[tm][tn];
                } else if (minus) {
#pragma unroll
                    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                        for (int tn = 0; tn < TN; ++tn) Y[j][tm][tn] -= P[tm][tn];
                }
            }
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                    for (int r = 0; r < 16; ++r) P[tm][tn][r] = 0.f;
            kc = 0;
            ++pos;
        }

        if (s + 1 < steps) store_lds(buf ^ 1);
        __syncthreads();
    }

    // Scatter: tile row m = (b*nH + th)*nW + tw -> pixels (2th+dy, 2tw+dx) of image b
    // (winograd2x2_conv_cuda.cu.cc:48-51).  Accumulator register r of lane (lg, li) holds
    // row 8*(r/4) + 4*lg + r%4 and column li of a 32x32 tile.
    const size_t oW = 2 * static_cast<size_t>(nW);
    const size_t row_stride = oW * K;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const size_t gm = m0 + wm0 + tm * 32 + 8 * (r / 4) + 4 * lg + (r % 4);
            if (gm >= M) continue;
            const size_t tw = gm % nW;
            const size_t bt = gm / nW;  // b*nH + th
            float *o = Out + (bt * 2 * oW + 2 * tw) * K;
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) {
                const int col = n0 + wn0 + tn * 32 + li;
                if (col >= K) continue;
                o[col] = Y[0][tm][tn][r];
                o[K + col] = Y[1][tm][tn][r];
                o[row_stride + col] = Y[2][tm][tn][r];
                o[row_stride + K + col] = Y[3][tm][tn][r];
            }
        }
    }
}

template <typename Cfg, bool BF16>
int launch_conv(const float *TI, const float *Wt, float *Out, size_t M, int C, int K, int nH, int nW,
                hipStream_t stream)
{
    const size_t tiles_m = (M + Cfg::BM - 1) / Cfg::BM;
    const size_t tiles_n = (static_cast<size_t>(K) + Cfg::BN - 1) / Cfg::BN;
    if (tiles_m * tiles_n >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    const dim3 grid(static_cast<unsigned>(tiles_m * tiles_n)), block(Cfg::NT);
    const bool vec = (C % 4 == 0) && (K % 4 == 0) && aligned16(TI) && aligned16(Wt);
    if (vec)
        conv_f32_kernel<Cfg, true, BF16><<<grid, block, 0, stream>>>(TI, Wt, Out, M, C, K, nH, nW,
                                                                     static_cast<unsigned>(tiles_n));
    else
        conv_f32_kernel<Cfg, false, BF16><<<grid, block, 0, stream>>>(TI, Wt, Out, M, C, K, nH, nW,
                                                                      static_cast<unsigned>(tiles_n));
    return check_launch();
}

template <bool BF16>
int conv_entry(const float *Input, const float *Weight, float *Output, int C, int B, int nH, int nW, int K,
               int pad_h, int pad_w, swc_stream_t stream)
{
    if (Input == nullptr || Weight == nullptr || Output == nullptr) return SWC_ERR_NULL_POINTER;
    if (C <= 0 || B <= 0 || nH <= 0 || nW <= 0 || K <= 0) return SWC_ERR_BAD_DIMS;
    if (pad_h != 1 || pad_w != 1) return SWC_ERR_BAD_PAD;
    const size_t M = static_cast<size_t>(B) * nH * nW;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return launch_conv<ConvCfg<64, 64, 32, 2, 2>, BF16>(Input, Weight, Output, M, C, K, nH, nW, s);
}

}  // namespace
}  // namespace swc

extern "C" int swc_winograd2x2_conv(const float *Input, const float *Weight, float *Output, float *, const long long *,
                                    int C, int B, int nH, int nW, int K, int pad_h, int pad_w, swc_stream_t stream)
{
    return swc::conv_entry<false>(Input, Weight, Output, C, B, nH, nW, K, pad_h, pad_w, stream);
}

extern "C" int swc_winograd2x2_conv_bf16(const float *Input, const float *Weight, float *Output, float *,
                                         const long long *, int C, int B, int nH, int nW, int K, int pad_h, int pad_w,
                                         swc_stream_t stream)
{
    return swc::conv_entry<true>(Input, Weight, Output, C, B, nH, nW, K, pad_h, pad_w, stream);
}
