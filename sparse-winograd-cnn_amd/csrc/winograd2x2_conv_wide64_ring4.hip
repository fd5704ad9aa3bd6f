// Launches of the wide48 kernel (winograd2x2_conv_wide_kernel.h) with 64-column workgroups and a 4-slot ring (the
// copies run three steps ahead; C % 128 == 0).  A translation unit of its own: its four instantiations take minutes
// to compile.  Part of what stands in for Winograd2x2ConvComputeLauncher
// (winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_cuda.cu.cc:65-93).
#include "winograd2x2_conv_wide_kernel.h"
#include "winograd2x2_conv_launch.h"

namespace swc {
namespace {

template <bool EXTRA, bool EPI>
int launch_wide64_ring4_as(const float *TI, const float *Wt, float *Out, size_t M, int C, int K, int nW, const WidePlan &plan,
                     const ConvEpilogue &ep, hipStream_t stream)
{
    using W = WideCfg<32, 1, EXTRA, 2, EPI, 4>;
    static_assert(2 * W::LAUNCH_LDS_BYTES <= 160 * 1024, "two workgroups per CU");
    struct Tag {};
    const int st = raise_lds_limit<Tag>(reinterpret_cast<const void *>(conv_wide48_kernel<W>), W::LAUNCH_LDS_BYTES);
    if (st != SWC_OK) return st;
    const unsigned tiles_n = static_cast<unsigned>(K / W::BN);
    conv_wide48_kernel<W><<<dim3(static_cast<unsigned>(plan.groups) * tiles_n), dim3(W::NT), W::LAUNCH_LDS_BYTES, stream>>>(
        TI, Wt, Out, static_cast<unsigned>(M), C, K, nW, tiles_n, static_cast<unsigned>(plan.rows_per_wg),
        static_cast<unsigned>(plan.main_rows), ep);
    return check_launch();
}

}  // namespace

int launch_wide48_n64_ring4(const float *TI, const float *Wt, float *Out, size_t M, int C, int K, int nW, const WidePlan &plan,
                      const float *scale, const float *shift, const float *residual, int residual_relu, hipStream_t stream)
{
    if (!plan.ok || plan.bn != 64 || C % 128 != 0 || !wide48_eligible(TI, Wt, M, C, K, 64)) return SWC_ERR_UNSUPPORTED;
    ConvEpilogue ep;
    ep.scale = scale;
    ep.shift = shift;
    ep.residual = residual;
    ep.residual_relu = residual_relu;
    const bool epi = scale != nullptr || residual != nullptr;
    if (plan.extra)
        return epi ? launch_wide64_ring4_as<true, true>(TI, Wt, Out, M, C, K, nW, plan, ep, stream)
                   : launch_wide64_ring4_as<true, false>(TI, Wt, Out, M, C, K, nW, plan, ep, stream);
    return epi ? launch_wide64_ring4_as<false, true>(TI, Wt, Out, M, C, K, nW, plan, ep, stream)
               : launch_wide64_ring4_as<false, false>(TI, Wt, Out, M, C, K, nW, plan, ep, stream);
}

}  // namespace swc
