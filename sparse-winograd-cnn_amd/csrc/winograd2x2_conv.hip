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

#include "winograd2x2_conv_kernel.h"
#include "winograd2x2_conv_bf16_kernel.h"
#include "winograd2x2_conv_launch.h"

namespace swc {
namespace {

// Synchronous kernel: any shape and alignment (register-staged tiles, guarded or descriptor loads).
template <typename Cfg, bool BF16>
int launch_sync(const float *TI, const float *Wt, float *Out, size_t M, int C, int K, int nH, int nW,
                const ConvEpilogue &ep, hipStream_t stream)
{
    const size_t tiles_m = (M + Cfg::BM - 1) / Cfg::BM;
    const size_t tiles_n = (static_cast<size_t>(K) + Cfg::BN - 1) / Cfg::BN;
    if (tiles_m * tiles_n >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    const dim3 grid(static_cast<unsigned>(tiles_m * tiles_n)), block(Cfg::NT);
    // The descriptor path addresses memory with 32-bit byte offsets and loads 16 bytes at a time.
    const bool fast = (C % 4 == 0) && (K % 4 == 0) && aligned16(TI) && aligned16(Wt) &&
                      static_cast<size_t>(C) * K < (1ull << 29) && static_cast<size_t>(Cfg::BM) * C < (1ull << 29);
    if (fast)
        conv_mfma_kernel<Cfg, true, BF16><<<grid, block, 0, stream>>>(TI, Wt, Out, M, C, K, nH, nW,
                                                                      static_cast<unsigned>(tiles_n), ep);
    else
        conv_mfma_kernel<Cfg, false, BF16><<<grid, block, 0, stream>>>(TI, Wt, Out, M, C, K, nH, nW,
                                                                       static_cast<unsigned>(tiles_n), ep);
    return check_launch();
}

// rows_per_wg <= Cfg::BM rows of the [M,K] plane go to each workgroup.
template <typename Cfg, int NSTAGE, bool BF16>
int launch_async(const float *TI, const float *Wt, float *Out, size_t M, int C, int K, int nH, int nW,
                 size_t rows_per_wg, const ConvEpilogue &ep, hipStream_t stream)
{
    constexpr int lds_bytes = async_lds_bytes<Cfg, NSTAGE>();
    static_assert(lds_bytes <= 160 * 1024, "a CU has 160 KiB of LDS");
    struct Tag {};
    const int st = raise_lds_limit<Tag>(reinterpret_cast<const void *>(conv_mfma_async_kernel<Cfg, NSTAGE, BF16>), lds_bytes);
    if (st != SWC_OK) return st;
    const size_t tiles_m = (M + rows_per_wg - 1) / rows_per_wg;
    const size_t tiles_n = (static_cast<size_t>(K) + Cfg::BN - 1) / Cfg::BN;
    if (tiles_m * tiles_n >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    const dim3 grid(static_cast<unsigned>(tiles_m * tiles_n)), block(Cfg::NT);
    conv_mfma_async_kernel<Cfg, NSTAGE, BF16><<<grid, block, lds_bytes, stream>>>(
        TI, Wt, Out, M, C, K, nH, nW, static_cast<unsigned>(tiles_n), static_cast<unsigned>(rows_per_wg), ep);
    return check_launch();
}

template <bool BF16>
int conv_entry(const float *Input, const float *Weight, float *Output, int C, int B, int nH, int nW, int K,
               int pad_h, int pad_w, const ConvEpilogue &ep, swc_stream_t stream)
{
    if (Input == nullptr || Weight == nullptr || Output == nullptr) return SWC_ERR_NULL_POINTER;
    if ((ep.scale == nullptr) != (ep.shift == nullptr)) return SWC_ERR_NULL_POINTER;
    if (C <= 0 || B <= 0 || nH <= 0 || nW <= 0 || K <= 0) return SWC_ERR_BAD_DIMS;
    if (pad_h != 1 || pad_w != 1) return SWC_ERR_BAD_PAD;
    const size_t M = static_cast<size_t>(B) * nH * nW;
    if (M >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // The bf16-operand variant has one tiling (ring32, 3-deep: its step is 8x shorter than the fp32 one and needs
    // two tiles in flight to cover the memory latency); fp32 picks among all of them.
    TilingChoice pick = {ring_eligible<Tile32>(Input, Weight, C, K, true) ? TILING_RING32 : TILING_SYNC, Tile32::BM};
    if (!BF16) pick = choose_tiling(Input, Weight, M, C, K, true, true);
    note_conv_kernel(tiling_name(pick.tiling));
    switch (pick.tiling) {
        case TILING_WIDE48:
        case TILING_WIDE48X64:
            return launch_wide48(Input, Weight, Output, M, C, K, nW, pick.wide, ep.scale, ep.shift, ep.residual, ep.residual_relu, s);
        case TILING_TALL16:
            return launch_async<Tall, 2, false>(Input, Weight, Output, M, C, K, nH, nW, pick.rows_per_wg, ep, s);
        case TILING_SHORT16:
            return launch_async<Short, 2, false>(Input, Weight, Output, M, C, K, nH, nW, pick.rows_per_wg, ep, s);
        case TILING_RING32:
            return launch_async<Tile32, BF16 ? 3 : 2, BF16>(Input, Weight, Output, M, C, K, nH, nW, Tile32::BM, ep, s);
        case TILING_RING16:
            return launch_async<Tile16, 3, false>(Input, Weight, Output, M, C, K, nH, nW, Tile16::BM, ep, s);
        default:
            return launch_sync<Tile32, BF16>(Input, Weight, Output, M, C, K, nH, nW, ep, s);
    }
}

}  // namespace
}  // namespace swc

extern "C" int swc_winograd2x2_conv(const float *Input, const float *Weight, float *Output, float *, const long long *,
                                    int C, int B, int nH, int nW, int K, int pad_h, int pad_w, swc_stream_t stream)
{
    return swc::conv_entry<false>(Input, Weight, Output, C, B, nH, nW, K, pad_h, pad_w, swc::ConvEpilogue(), stream);
}

extern "C" int swc_winograd2x2_conv_bf16(const float *Input, const float *Weight, float *Output, float *,
                                         const long long *, int C, int B, int nH, int nW, int K, int pad_h, int pad_w,
                                         swc_stream_t stream)
{
    return swc::conv_entry<true>(Input, Weight, Output, C, B, nH, nW, K, pad_h, pad_w, swc::ConvEpilogue(), stream);
}

extern "C" int swc_winograd2x2_conv_epilogue(const float *Input, const float *Weight, float *Output, const float *Scale,
                                             const float *Shift, const float *Residual, int residual_relu, int C, int B,
                                             int nH, int nW, int K, int pad_h, int pad_w, int precision,
                                             swc_stream_t stream)
{
    swc::ConvEpilogue ep;
    ep.scale = Scale;
    ep.shift = Shift;
    ep.residual = Residual;
    ep.residual_relu = residual_relu != 0;
    if (precision == 0) return swc::conv_entry<false>(Input, Weight, Output, C, B, nH, nW, K, pad_h, pad_w, ep, stream);
    if (precision == 1) return swc::conv_entry<true>(Input, Weight, Output, C, B, nH, nW, K, pad_h, pad_w, ep, stream);
    return SWC_ERR_BAD_DIMS;
}

extern "C" int swc_winograd2x2_weights_bf16(const float *Weight, unsigned short *Weight16t, int C, int K,
                                            swc_stream_t stream)
{
    using namespace swc;
    if (Weight == nullptr || Weight16t == nullptr) return SWC_ERR_NULL_POINTER;
    if (C <= 0 || K <= 0 || static_cast<size_t>(16) * C * K >= (1ull << 32)) return SWC_ERR_BAD_DIMS;
    const unsigned n = static_cast<unsigned>(16u * static_cast<size_t>(C) * K);
    weights_to_bf16_transposed_kernel<<<dim3((n + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        Weight, Weight16t, C, K, n);
    return check_launch();
}

namespace swc {
namespace {
template <typename Hb, int GROUPS = 1>
int launch_bf16_stored(const unsigned short *Input16, const unsigned short *Weight16t, float *Output, size_t M, int C,
                       int K, int nH, int nW, size_t rows_per_wg, size_t tiles_n, const ConvEpilogue &ep, hipStream_t s)
{
    const size_t tiles_m = (M + rows_per_wg - 1) / rows_per_wg;
    constexpr int lds_bytes = GROUPS * Hb::LDS_BYTES;
    static_assert(lds_bytes <= 160 * 1024, "a CU has 160 KiB of LDS");
    struct Tag {};
    const int st = raise_lds_limit<Tag>(reinterpret_cast<const void *>(conv_bf16_stored_kernel<Hb, GROUPS>), lds_bytes);
    if (st != SWC_OK) return st;
    conv_bf16_stored_kernel<Hb, GROUPS><<<dim3(static_cast<unsigned>(tiles_m * tiles_n)), dim3(64 * Hb::GW * GROUPS), lds_bytes, s>>>(
        Input16, Weight16t, Output, M, C, K, nH, nW, static_cast<unsigned>(tiles_n), static_cast<unsigned>(rows_per_wg), ep);
    return check_launch();
}
}  // namespace
}  // namespace swc

namespace swc {
namespace {
// Layers of 256 or 512 channels with so few 128-row x 64-column tiles that four workgroups per tile still find a CU
// each: with a scratch buffer the positions of a tile are dealt over four workgroups.  With 256 channels a workgroup's
// four positions are 16 steps only and the second kernel weighs twice as much: the form pays up to half as many
// workgroups (14x14x256 -> 256 at batch 16: 11.8 us against 14.8; at batch 32, 208 workgroups: 16.5 against 15.2;
// 7x7x512 -> 512 at batch 64, 256 workgroups: 18.5 against 23.9; at batch 128: 34.1 against 30.8).
bool bf16_spread_wanted(size_t M, int C, int K, size_t cus)
{
    if ((C != 256 && C != 512) || K % 64 != 0) return false;
    const size_t tall_n = static_cast<size_t>(K) / 64, tall_m = (M + 127) / 128;
    return 4 * tall_m * tall_n * static_cast<size_t>(512 / C) <= cus;
}
int conv_bf16in(const unsigned short *Input16, const unsigned short *Weight16t, float *Output, const float *Scale,
                const float *Shift, const float *Residual, int residual_relu, float *Workspace, size_t workspace_floats, int C,
                int B, int nH, int nW, int K, int pad_h, int pad_w, swc_stream_t stream);
}  // namespace
}  // namespace swc

extern "C" int swc_winograd2x2_conv_bf16in(const unsigned short *Input16, const unsigned short *Weight16t, float *Output,
                                           const float *Scale, const float *Shift, const float *Residual,
                                           int residual_relu, int C, int B, int nH, int nW, int K, int pad_h, int pad_w,
                                           swc_stream_t stream)
{
    return swc::conv_bf16in(Input16, Weight16t, Output, Scale, Shift, Residual, residual_relu, nullptr, 0, C, B, nH, nW, K, pad_h,
                            pad_w, stream);
}

extern "C" size_t swc_winograd2x2_conv_bf16in_workspace_floats(int C, int B, int nH, int nW, int K)
{
    using namespace swc;
    if (C <= 0 || B <= 0 || nH <= 0 || nW <= 0 || K <= 0) return 0;
    const size_t M = static_cast<size_t>(B) * nH * nW;
    if (M >= (1ull << 31) || M * 16 * static_cast<size_t>(K) >= (1ull << 31)) return 0;
    return bf16_spread_wanted(M, C, K, device_cus()) ? 8 * M * static_cast<size_t>(K) : 0;
}

extern "C" int swc_winograd2x2_conv_bf16in_ws(const unsigned short *Input16, const unsigned short *Weight16t, float *Output,
                                              const float *Scale, const float *Shift, const float *Residual,
                                              int residual_relu, float *Workspace, size_t workspace_floats, int C, int B,
                                              int nH, int nW, int K, int pad_h, int pad_w, swc_stream_t stream)
{
    return swc::conv_bf16in(Input16, Weight16t, Output, Scale, Shift, Residual, residual_relu, Workspace, workspace_floats, C, B, nH,
                            nW, K, pad_h, pad_w, stream);
}

namespace swc {
namespace {
int conv_bf16in(const unsigned short *Input16, const unsigned short *Weight16t, float *Output, const float *Scale,
                const float *Shift, const float *Residual, int residual_relu, float *Workspace, size_t workspace_floats, int C,
                int B, int nH, int nW, int K, int pad_h, int pad_w, swc_stream_t stream)
{
    if (Input16 == nullptr || Weight16t == nullptr || Output == nullptr) return SWC_ERR_NULL_POINTER;
    if ((Scale == nullptr) != (Shift == nullptr)) return SWC_ERR_NULL_POINTER;
    if (C <= 0 || B <= 0 || nH <= 0 || nW <= 0 || K <= 0) return SWC_ERR_BAD_DIMS;
    if (pad_h != 1 || pad_w != 1) return SWC_ERR_BAD_PAD;
    const size_t M = static_cast<size_t>(B) * nH * nW;
    if (M >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    using Deep = HbCfg<64, 4, 2>;   // 4-deep ring, up to two workgroups per CU
    using Wide = HbCfg<64, 3, 3>;   // 3-deep ring, up to three workgroups per CU
    using Split = HbCfg<64, 3, 2>;  // two groups of waves per workgroup, a 3-deep ring each
    using Quad = HbCfg<64, 3, 2, 32>;  // 32-row tiles, four groups of two waves per workgroup, a 3-deep ring each
    if (C % Deep::BK != 0 || !aligned16(Input16) || !aligned16(Weight16t) || static_cast<size_t>(HB_BM) * C >= (1ull << 30))
        return SWC_ERR_UNSUPPORTED;
    const size_t tiles_n = (static_cast<size_t>(K) + HB_BN - 1) / HB_BN;
    // Rows per workgroup: the workgroup count rounded up to a multiple of the CU count, as for the fp32
    // tilings (49 to 64 rows; conv2: 26.7 vs 28.8 us) -- unless the weights fill an L2 or more.  Every row group
    // walks all of the weights of its columns, and what does not stay in the XCD's L2 comes from the Infinity
    // Cache again for each of them: then the tallest tile (fewest row groups) and the deeper ring (a step more of
    // latency covered) win: 14x14 at batch 128, 512 -> 512: 96 us against 124 us, 256 -> 512: 57 against 66.
    const size_t cus = device_cus();
    const bool weights_beyond_l2 = static_cast<size_t>(16) * C * K * 2 >= device_l2_bytes();
    const size_t rows = weights_beyond_l2 ? static_cast<size_t>(HB_BM) : balanced_rows<HbStoreCfg>(M, tiles_n, cus);
    const size_t tiles_m = (M + rows - 1) / rows;
    if (tiles_m * tiles_n >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    ConvEpilogue ep;
    ep.scale = Scale;
    ep.shift = Shift;
    ep.residual = Residual;
    ep.residual_relu = residual_relu != 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // Layers of 64, 128, 256 or 512 channels with enough 128-row x 64-column tiles for three quarters of the CUs: the
    // tall tiles (twice the matrix work per byte through LDS, which bounds these layers: 14x14 at batch 128,
    // 512 -> 512 77 us against 100, 28x28, 128 -> 128 27 against 35; with a residual to add 35 against 58).  With more
    // tiles than CUs two workgroups share a CU and the rows are levelled over whole rounds of them.
    if (bf16_tall_eligible(Input16, Weight16t, M, C, K)) {
        const size_t tall_n = static_cast<size_t>(K) / 64, tall_m = (M + 127) / 128;
        if (tall_m * tall_n * 4 >= 3 * cus) {
            size_t tall_rows = 128;
            if (tall_m * tall_n > cus) {
                const size_t slots = 2 * cus, wgs = (tall_m * tall_n + slots - 1) / slots * slots;
                const size_t groups = wgs / tall_n > tall_m ? wgs / tall_n : tall_m;
                tall_rows = (M + groups - 1) / groups;
                if (tall_rows > 128) tall_rows = 128;
                if (tall_rows < 64) tall_rows = 64;
            }
            note_conv_kernel("stored-tall");
            return launch_bf16_tall(Input16, Weight16t, Output, M, C, K, nW, tall_rows, Scale, Shift, Residual, residual_relu != 0, s);
        }
    }
    // Far fewer tiles than that, 256 or 512 channels and a scratch buffer of the caller's: four workgroups per tile,
    // each a row of the position grid (7x7x512 at batch 64: 18.5 us, 23.9 without the buffer).
    if (Workspace != nullptr && bf16_spread_wanted(M, C, K, cus) && workspace_floats >= 8 * M * static_cast<size_t>(K) &&
        bf16_spread_eligible(Input16, Weight16t, Output, Workspace, M, C, K, Scale, Shift, Residual)) {
        note_conv_kernel("stored-spread");
        return launch_bf16_spread(Input16, Weight16t, Output, Workspace, M, C, K, nW, Scale, Shift, Residual, residual_relu != 0, s);
    }
    // A grid of full tiles that leaves every CU with one workgroup at most: the launch then lasts as long as one
    // workgroup's chain of steps, and splitting the 16 positions over two groups of waves halves the chain
    // (7x7x512 at batch 64: 30.7 us against 37.1; 14x14x256: 19.9 against 22.9).
    // Fewer tiles still, so that 32-row tiles also leave every CU with one workgroup at most, and long positions
    // (four steps or more): four groups of two waves, four positions each.  Such a launch is bound by what one CU
    // can copy into its LDS (about 40 bytes a clock), and twice the workgroups on twice the CUs move 1.5 times the
    // bytes in all: 7x7x512 at batch 64 23.8 us against 27.1.
    if ((M + 31) / 32 * tiles_n <= cus && C >= 4 * Quad::BK) {
        note_conv_kernel("stored-split4");
        return launch_bf16_stored<Quad, 4>(Input16, Weight16t, Output, M, C, K, nH, nW, 32, tiles_n, ep, s);
    }
    if ((M + HB_BM - 1) / HB_BM * tiles_n <= cus) {
        note_conv_kernel("stored-split");
        return launch_bf16_stored<Split, 2>(Input16, Weight16t, Output, M, C, K, nH, nW, HB_BM, tiles_n, ep, s);
    }
    // More resident workgroups hide more of each other's waits once there are enough of them to go round
    // (conv3: 18.7 vs 19.6 us); a grid that leaves CUs with one workgroup does better with the deeper
    // ring (conv4b: 30.8 vs 34.2 us).
    if (tiles_m * tiles_n > cus && !weights_beyond_l2) {
        note_conv_kernel("stored-ring3");
        return launch_bf16_stored<Wide>(Input16, Weight16t, Output, M, C, K, nH, nW, rows, tiles_n, ep, s);
    }
    note_conv_kernel("stored-ring4");
    return launch_bf16_stored<Deep>(Input16, Weight16t, Output, M, C, K, nH, nW, rows, tiles_n, ep, s);
}
}  // namespace
}  // namespace swc
