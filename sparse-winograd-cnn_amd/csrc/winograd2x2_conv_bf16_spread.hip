// Launches of the stored-tall kernel in its spread form (winograd2x2_conv_bf16_tall_kernel.h): the bf16-stored
// convolution for layers of 256 or 512 input channels with fewer 128-row x 64-column tiles than CUs.  Four workgroups
// per tile, one per row of the 4x4 position grid, write partial sums to a scratch buffer of the caller; a second
// kernel combines them, applies the epilogue and scatters the pixels.  A translation unit of its own: the
// instantiations take minutes to compile.  Part of what stands in for Winograd2x2ConvComputeLauncher
// (winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_cuda.cu.cc:65-93, whose tmp_data_buffer is such a scratch
// buffer, twice the size) when the transformed activations are held as bf16.
#include "winograd2x2_conv_bf16_tall_kernel.h"
#include "winograd2x2_conv_launch.h"

namespace swc {
namespace {

// Y(dy,dx) = sum_r a_dy[r] Z_r(dx), a_0 = (1,1,1,0), a_1 = (0,1,-1,-1) (the rows of the output transform,
// winograd2x2_conv_cuda.cu.cc:39-46), from the planes Part [4][2][M][K] a spread launch wrote, with the epilogue, to
// pixel (2th + dy, 2tw + dx) of the output (winograd2x2_conv_cuda.cu.cc:48-51).  One lane per tile row and four
// channels; K % 4 == 0, all pointers 16-byte aligned, M*K < 2^31.
__global__ __launch_bounds__(256) void spread_combine_kernel(const float *__restrict__ Part, float *__restrict__ Out, unsigned M,
                                                             int K, int nW, ConvEpilogue ep)
{
    const unsigned k4n = static_cast<unsigned>(K) / 4;
    const unsigned idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= M * k4n) return;
    const unsigned m = idx / k4n, k = (idx - m * k4n) * 4;
    const size_t plane = static_cast<size_t>(M) * K;
    const float *src = Part + static_cast<size_t>(m) * K + k;
    float4 z[4][2];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int dx = 0; dx < 2; ++dx) z[r][dx] = *reinterpret_cast<const float4 *>(src + (2 * r + dx) * plane);
    const unsigned bt = m / static_cast<unsigned>(nW), tw = m - bt * static_cast<unsigned>(nW);
    const size_t oW = 2 * static_cast<size_t>(nW), row_stride = oW * K;
    const size_t pix = (static_cast<size_t>(bt) * 2 * oW + 2 * tw) * K + k;
    float4 sc = {1.f, 1.f, 1.f, 1.f}, sh = {0.f, 0.f, 0.f, 0.f};
    if (ep.scale != nullptr) {
        sc = *reinterpret_cast<const float4 *>(ep.scale + k);
        sh = *reinterpret_cast<const float4 *>(ep.shift + k);
    }
#pragma unroll
    for (int dy = 0; dy < 2; ++dy)
#pragma unroll
        for (int dx = 0; dx < 2; ++dx) {
            float4 y;
            if (dy == 0) {
                y.x = z[0][dx].x + z[1][dx].x + z[2][dx].x;
                y.y = z[0][dx].y + z[1][dx].y + z[2][dx].y;
                y.z = z[0][dx].z + z[1][dx].z + z[2][dx].z;
                y.w = z[0][dx].w + z[1][dx].w + z[2][dx].w;
            } else {
                y.x = z[1][dx].x - z[2][dx].x - z[3][dx].x;
                y.y = z[1][dx].y - z[2][dx].y - z[3][dx].y;
                y.z = z[1][dx].z - z[2][dx].z - z[3][dx].z;
                y.w = z[1][dx].w - z[2][dx].w - z[3][dx].w;
            }
            const size_t at = pix + dy * row_stride + dx * static_cast<size_t>(K);
            if (ep.scale != nullptr) {
                y.x = __builtin_fmaf(y.x, sc.x, sh.x);
                y.y = __builtin_fmaf(y.y, sc.y, sh.y);
                y.z = __builtin_fmaf(y.z, sc.z, sh.z);
                y.w = __builtin_fmaf(y.w, sc.w, sh.w);
            }
            if (ep.residual != nullptr) {
                float4 q = *reinterpret_cast<const float4 *>(ep.residual + at);
                if (ep.residual_relu) {
                    q.x = q.x > 0.f ? q.x : 0.f;
                    q.y = q.y > 0.f ? q.y : 0.f;
                    q.z = q.z > 0.f ? q.z : 0.f;
                    q.w = q.w > 0.f ? q.w : 0.f;
                }
                y.x += q.x;
                y.y += q.y;
                y.z += q.z;
                y.w += q.w;
            }
            *reinterpret_cast<float4 *>(Out + at) = y;
        }
}

template <int NKC>
int launch_spread_as(const unsigned short *TI16, const unsigned short *Wt16, float *Out, float *Part, size_t M, int K, int nW,
                     const ConvEpilogue &ep, hipStream_t stream)
{
    using T = TallCfg<NKC, 2, false, true>;
    static_assert(2 * T::LDS_BYTES <= 160 * 1024, "two workgroups per CU");
    struct Tag {};
    const int st = raise_lds_limit<Tag>(reinterpret_cast<const void *>(conv_bf16_tall_kernel<T>), T::LDS_BYTES);
    if (st != SWC_OK) return st;
    const size_t tiles_m = (M + T::BM - 1) / T::BM, tiles_n = static_cast<size_t>(K) / T::BN;
    if (4 * tiles_m * tiles_n >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    conv_bf16_tall_kernel<T><<<dim3(static_cast<unsigned>(4 * tiles_m * tiles_n)), dim3(T::NT), T::LDS_BYTES, stream>>>(
        TI16, Wt16, Part, static_cast<unsigned>(M), K, nW, static_cast<unsigned>(tiles_n), static_cast<unsigned>(T::BM), ConvEpilogue());
    int rc = check_launch();
    if (rc != SWC_OK) return rc;
    const size_t lanes = M * (static_cast<size_t>(K) / 4);
    spread_combine_kernel<<<dim3(static_cast<unsigned>((lanes + 255) / 256)), dim3(256), 0, stream>>>(Part, Out, static_cast<unsigned>(M), K, nW, ep);
    return check_launch();
}

}  // namespace

bool bf16_spread_eligible(const void *TI16, const void *Wt16, const void *Out, const void *Part, size_t M, int C, int K,
                          const float *scale, const float *shift, const float *residual)
{
    return (C == 256 || C == 512) && bf16_tall_eligible(TI16, Wt16, M, C, K) && Part != nullptr && aligned16(Out) && aligned16(Part) &&
           aligned16(scale) && aligned16(shift) && aligned16(residual);
}

int launch_bf16_spread(const unsigned short *TI16, const unsigned short *Wt16, float *Out, float *Part, size_t M, int C, int K,
                       int nW, const float *scale, const float *shift, const float *residual, int residual_relu, hipStream_t stream)
{
    if (!bf16_spread_eligible(TI16, Wt16, Out, Part, M, C, K, scale, shift, residual)) return SWC_ERR_UNSUPPORTED;
    ConvEpilogue ep;
    ep.scale = scale;
    ep.shift = shift;
    ep.residual = residual;
    ep.residual_relu = residual_relu;
    return C == 256 ? launch_spread_as<4>(TI16, Wt16, Out, Part, M, K, nW, ep, stream)
                    : launch_spread_as<8>(TI16, Wt16, Out, Part, M, K, nW, ep, stream);
}

}  // namespace swc
