// Launches of the stored-tall kernel (winograd2x2_conv_bf16_tall_kernel.h), the bf16-stored convolution's form for
// layers of 64, 128, 256 or 512 input channels with enough 128-row x 64-column tiles to go round the CUs.  A translation
// unit of its own: its instantiations take minutes to compile.  Part of what stands in for
// Winograd2x2ConvComputeLauncher (winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_cuda.cu.cc:65-93) when the
// transformed activations are held as bf16.
#include "winograd2x2_conv_bf16_tall_kernel.h"
#include "winograd2x2_conv_launch.h"

namespace swc {
namespace {

template <int NKC, bool EPI>
int launch_tall_as(const unsigned short *TI16, const unsigned short *Wt16, float *Out, size_t M, int K, int nW,
                   size_t rows_per_wg, const ConvEpilogue &ep, hipStream_t stream)
{
    using T = TallCfg<NKC, 2, EPI>;
    static_assert(2 * T::LDS_BYTES <= 160 * 1024, "two workgroups per CU");
    struct Tag {};
    const int st = raise_lds_limit<Tag>(reinterpret_cast<const void *>(conv_bf16_tall_kernel<T>), T::LDS_BYTES);
    if (st != SWC_OK) return st;
    const size_t tiles_m = (M + rows_per_wg - 1) / rows_per_wg, tiles_n = static_cast<size_t>(K) / T::BN;
    if (tiles_m * tiles_n >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    conv_bf16_tall_kernel<T><<<dim3(static_cast<unsigned>(tiles_m * tiles_n)), dim3(T::NT), T::LDS_BYTES, stream>>>(
        TI16, Wt16, Out, static_cast<unsigned>(M), K, nW, static_cast<unsigned>(tiles_n), static_cast<unsigned>(rows_per_wg), ep);
    return check_launch();
}

}  // namespace

bool bf16_tall_eligible(const void *TI16, const void *Wt16, size_t M, int C, int K)
{
    return (C == 64 || C == 128 || C == 256 || C == 512) && K % 64 == 0 && aligned16(TI16) && aligned16(Wt16) && M < (1ull << 31) &&
           M * 16 * static_cast<size_t>(K) < (1ull << 31);
}

int launch_bf16_tall(const unsigned short *TI16, const unsigned short *Wt16, float *Out, size_t M, int C, int K, int nW,
                     size_t rows_per_wg, const float *scale, const float *shift, const float *residual, int residual_relu,
                     hipStream_t stream)
{
    if (!bf16_tall_eligible(TI16, Wt16, M, C, K) || rows_per_wg == 0 || rows_per_wg > 128) return SWC_ERR_UNSUPPORTED;
    ConvEpilogue ep;
    ep.scale = scale;
    ep.shift = shift;
    ep.residual = residual;
    ep.residual_relu = residual_relu;
    const bool epi = scale != nullptr || residual != nullptr;
    switch (C / 64) {
        case 1:
            return epi ? launch_tall_as<1, true>(TI16, Wt16, Out, M, K, nW, rows_per_wg, ep, stream)
                       : launch_tall_as<1, false>(TI16, Wt16, Out, M, K, nW, rows_per_wg, ep, stream);
        case 2:
            return epi ? launch_tall_as<2, true>(TI16, Wt16, Out, M, K, nW, rows_per_wg, ep, stream)
                       : launch_tall_as<2, false>(TI16, Wt16, Out, M, K, nW, rows_per_wg, ep, stream);
        case 4:
            return epi ? launch_tall_as<4, true>(TI16, Wt16, Out, M, K, nW, rows_per_wg, ep, stream)
                       : launch_tall_as<4, false>(TI16, Wt16, Out, M, K, nW, rows_per_wg, ep, stream);
        default:
            return epi ? launch_tall_as<8, true>(TI16, Wt16, Out, M, K, nW, rows_per_wg, ep, stream)
                       : launch_tall_as<8, false>(TI16, Wt16, Out, M, K, nW, rows_per_wg, ep, stream);
    }
}

}  // namespace swc
