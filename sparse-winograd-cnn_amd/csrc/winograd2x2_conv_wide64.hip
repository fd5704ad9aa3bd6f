// Launches of the wide48 kernel (winograd2x2_conv_wide_kernel.h) with 64-column workgroups (wave tile 48x16), for
// shapes where 128-column workgroups are too few to fill the device.  A translation unit of its own: its four
// instantiations take minutes to compile (the four with a 4-slot ring are in winograd2x2_conv_wide64_ring4.hip).  Part of what stands in for Winograd2x2ConvComputeLauncher
// (winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_cuda.cu.cc:65-93).
#include "winograd2x2_conv_wide_kernel.h"
#include "winograd2x2_conv_launch.h"

namespace swc {
namespace {

template <bool EXTRA, bool EPI>
int launch_wide64_as(const float *TI, const float *Wt, float *Out, size_t M, int C, int K, int nW, const WidePlan &plan,
                     const ConvEpilogue &ep, hipStream_t stream)
{
    using W = WideCfg<32, 1, EXTRA, 2, EPI>;
    static_assert(W::LAUNCH_LDS_BYTES <= 64 * 1024, "fits the default dynamic LDS limit");
    const unsigned tiles_n = static_cast<unsigned>(K / W::BN);
    conv_wide48_kernel<W><<<dim3(static_cast<unsigned>(plan.groups) * tiles_n), dim3(W::NT), W::LAUNCH_LDS_BYTES, stream>>>(
        TI, Wt, Out, static_cast<unsigned>(M), C, K, nW, tiles_n, static_cast<unsigned>(plan.rows_per_wg),
        static_cast<unsigned>(plan.main_rows), ep);
    return check_launch();
}

}  // namespace

int launch_wide48_n64(const float *TI, const float *Wt, float *Out, size_t M, int C, int K, int nW, const WidePlan &plan,
                      const float *scale, const float *shift, const float *residual, int residual_relu, hipStream_t stream)
{
    if (!plan.ok || plan.bn != 64 || !wide48_eligible(TI, Wt, M, C, K, 64)) return SWC_ERR_UNSUPPORTED;
    // With whole rounds of four steps per position the copies run three steps ahead (14x14x256 at batch 64 over
    // buffers that are not cache-resident: 65 us against 76).
    if (C % 128 == 0) return launch_wide48_n64_ring4(TI, Wt, Out, M, C, K, nW, plan, scale, shift, residual, residual_relu, stream);
    ConvEpilogue ep;
    ep.scale = scale;
    ep.shift = shift;
    ep.residual = residual;
    ep.residual_relu = residual_relu;
    const bool epi = scale != nullptr || residual != nullptr;
    if (plan.extra)
        return epi ? launch_wide64_as<true, true>(TI, Wt, Out, M, C, K, nW, plan, ep, stream)
                   : launch_wide64_as<true, false>(TI, Wt, Out, M, C, K, nW, plan, ep, stream);
    return epi ? launch_wide64_as<false, true>(TI, Wt, Out, M, C, K, nW, plan, ep, stream)
               : launch_wide64_as<false, false>(TI, Wt, Out, M, C, K, nW, plan, ep, stream);
}

}  // namespace swc
