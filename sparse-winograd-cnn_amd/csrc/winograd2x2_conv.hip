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

// Asynchronous kernel (global -> LDS copies, NSTAGE-deep ring): needs whole BK chunks of
// channels, 16-byte granules and 32-bit byte offsets within a tile.
template <typename Cfg>
bool async_eligible(const float *TI, const float *Wt, int C, int K)
{
    return (C % Cfg::BK == 0) && (K % 4 == 0) && aligned16(TI) && aligned16(Wt) &&
           static_cast<size_t>(Cfg::BM) * C < (1ull << 29) && static_cast<size_t>(Cfg::BK) * K < (1ull << 29);
}

// rows_per_wg <= Cfg::BM rows of the [M,K] plane go to each workgroup.
template <typename Cfg, int NSTAGE, bool BF16>
int launch_async(const float *TI, const float *Wt, float *Out, size_t M, int C, int K, int nH, int nW,
                 size_t rows_per_wg, const ConvEpilogue &ep, hipStream_t stream)
{
    constexpr int lds_bytes = async_lds_bytes<Cfg, NSTAGE>();
    static_assert(lds_bytes <= 160 * 1024, "a CU has 160 KiB of LDS");
    if (lds_bytes > 64 * 1024) {
        // Above the default 64 KiB limit, which is raised once per kernel and device.
        constexpr int kMaxDevices = 64;
        static thread_local bool raised[kMaxDevices] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SWC_ERR_HIP;
        if (!raised[dev]) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(conv_mfma_async_kernel<Cfg, NSTAGE, BF16>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
            if (e != hipSuccess) return note_hip_error(e);
            raised[dev] = true;
        }
    }
    const size_t tiles_m = (M + rows_per_wg - 1) / rows_per_wg;
    const size_t tiles_n = (static_cast<size_t>(K) + Cfg::BN - 1) / Cfg::BN;
    if (tiles_m * tiles_n >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    const dim3 grid(static_cast<unsigned>(tiles_m * tiles_n)), block(Cfg::NT);
    conv_mfma_async_kernel<Cfg, NSTAGE, BF16><<<grid, block, lds_bytes, stream>>>(
        TI, Wt, Out, M, C, K, nH, nW, static_cast<unsigned>(tiles_n), static_cast<unsigned>(rows_per_wg), ep);
    return check_launch();
}

constexpr size_t kCUs = 256;  // MI355X

// Passes the chip makes over `wgs` workgroups of equal length: the busiest CU sets the time, so whole
// passes while the grid is small; with many short workgroups the tail evens out.
double passes(size_t wgs)
{
    return wgs <= 8 * kCUs ? static_cast<double>((wgs + kCUs - 1) / kCUs) : static_cast<double>(wgs) / kCUs + 0.5;
}

// Rows per workgroup that split M into as many equal row groups as fill whole passes of the chip, but
// never so few that one of the workgroup's 16-row MFMA tiles would hold no valid row at all (a
// workgroup computes all of its tiles whatever their content).
template <typename Cfg>
size_t balanced_rows(size_t M, size_t tiles_n)
{
    const size_t groups_min = (M + Cfg::BM - 1) / Cfg::BM;
    const size_t wgs = (groups_min * tiles_n + kCUs - 1) / kCUs * kCUs;
    size_t groups = wgs / tiles_n;
    if (groups < groups_min) groups = groups_min;
    size_t rows = (M + groups - 1) / groups;
    if (rows < static_cast<size_t>(Cfg::BM) - 15) rows = Cfg::BM - 15;
    return rows < static_cast<size_t>(Cfg::BM) ? rows : static_cast<size_t>(Cfg::BM);
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
    // 32x32 MFMAs, wave tile 32x32: the fewest LDS reads per MFMA; its results are bit-identical to
    // the synchronous kernel's.
    using Tile32 = ConvCfg<64, 64, 32, 2, 2>;
    using Tile16 = ConvCfg<64, 64, 16, 2, 2>;
    // 16x16 MFMAs, wave tile (16*TM)x16: row groups of any height up to 112 (Tall) or 32 (Short), so
    // that M can be dealt evenly over the 256 CUs where 64-row tiles leave CUs idle or a ragged tail.
    using Tall = ConvCfg<112, 64, 32, 1, 4, 2, 16>;
    using Short = ConvCfg<32, 64, 64, 1, 4, 3, 16>;
    if (!BF16) {
        // Cost = passes x MFMA work of a wave per pass (in 16x16 tiles), weighted by what each kernel
        // measured per unit of that work on MI355X relative to Tile32, over the ResNet-18 shapes at
        // batch 64 and 128: Tall 8 % more; Short 10 % more, 15 % more when its 64-channel steps are
        // fewer than two per position, but 3 % less while all of its workgroups are resident at once
        // (up to three per CU).
        const size_t tiles_n = (static_cast<size_t>(K) + 63) / 64;
        const bool ok32 = async_eligible<Tile32>(Input, Weight, C, K);
        const bool ok_tall = async_eligible<Tall>(Input, Weight, C, K);
        const bool ok_short = async_eligible<Short>(Input, Weight, C, K);
        // Tall levels its row groups over the CUs; Short does better with full 32-row groups (two whole MFMA
        // tiles) even where that leaves some CUs with one workgroup more (conv4a: 69 vs 73 us).
        const size_t rows_tall = balanced_rows<Tall>(M, tiles_n), rows_short = Short::BM;
        const size_t wgs_short = (M + rows_short - 1) / rows_short * tiles_n;
        const double w_short = C < 128 ? 1.15 : wgs_short <= 3 * kCUs ? 0.97 : 1.10;
        const double cost32 = ok32 ? passes((M + 63) / 64 * tiles_n) * 4.0 : 1e30;
        const double cost_tall = ok_tall ? passes((M + rows_tall - 1) / rows_tall * tiles_n) * 7.0 * 1.08 : 1e30;
        const double cost_short = ok_short ? passes(wgs_short) * 2.0 * w_short : 1e30;
        if (ok_tall && cost_tall < cost32 && cost_tall <= cost_short) {
            note_conv_kernel("tall16");
            return launch_async<Tall, 2, false>(Input, Weight, Output, M, C, K, nH, nW, rows_tall, ep, s);
        }
        if (ok_short && cost_short < cost32) {
            note_conv_kernel("short16");
            return launch_async<Short, 2, false>(Input, Weight, Output, M, C, K, nH, nW, rows_short, ep, s);
        }
    }
    // Ring depth: the fp32 step is long (16 MFMAs of 64 cycles per wave) and one tile in flight
    // covers the memory latency; the bf16 step is 8x shorter and needs two.
    if (async_eligible<Tile32>(Input, Weight, C, K)) {
        note_conv_kernel("ring32");
        return launch_async<Tile32, BF16 ? 3 : 2, BF16>(Input, Weight, Output, M, C, K, nH, nW, Tile32::BM, ep, s);
    }
    if (!BF16 && async_eligible<Tile16>(Input, Weight, C, K)) {
        note_conv_kernel("ring16");
        return launch_async<Tile16, 3, false>(Input, Weight, Output, M, C, K, nH, nW, Tile16::BM, ep, s);
    }
    note_conv_kernel("sync");
    return launch_sync<Tile32, BF16>(Input, Weight, Output, M, C, K, nH, nW, ep, s);
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
                                             const float *Shift, const float *Residual, int C, int B, int nH, int nW,
                                             int K, int pad_h, int pad_w, int precision, swc_stream_t stream)
{
    swc::ConvEpilogue ep;
    ep.scale = Scale;
    ep.shift = Shift;
    ep.residual = Residual;
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
template <typename Hb>
int launch_bf16_stored(const unsigned short *Input16, const unsigned short *Weight16t, float *Output, size_t M, int C,
                       int K, int nH, int nW, size_t rows_per_wg, size_t tiles_n, const ConvEpilogue &ep, hipStream_t s)
{
    const size_t tiles_m = (M + rows_per_wg - 1) / rows_per_wg;
    if (Hb::LDS_BYTES > 64 * 1024) {
        // Above the default 64 KiB limit, which is raised once per kernel and device.
        constexpr int kMaxDevices = 64;
        static thread_local bool raised[kMaxDevices] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SWC_ERR_HIP;
        if (!raised[dev]) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(conv_bf16_stored_kernel<Hb>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, Hb::LDS_BYTES);
            if (e != hipSuccess) return note_hip_error(e);
            raised[dev] = true;
        }
    }
    conv_bf16_stored_kernel<Hb><<<dim3(static_cast<unsigned>(tiles_m * tiles_n)), dim3(256), Hb::LDS_BYTES, s>>>(
        Input16, Weight16t, Output, M, C, K, nH, nW, static_cast<unsigned>(tiles_n), static_cast<unsigned>(rows_per_wg), ep);
    return check_launch();
}
}  // namespace
}  // namespace swc

extern "C" int swc_winograd2x2_conv_bf16in(const unsigned short *Input16, const unsigned short *Weight16t, float *Output,
                                           const float *Scale, const float *Shift, const float *Residual, int C, int B,
                                           int nH, int nW, int K, int pad_h, int pad_w, swc_stream_t stream)
{
    using namespace swc;
    if (Input16 == nullptr || Weight16t == nullptr || Output == nullptr) return SWC_ERR_NULL_POINTER;
    if ((Scale == nullptr) != (Shift == nullptr)) return SWC_ERR_NULL_POINTER;
    if (C <= 0 || B <= 0 || nH <= 0 || nW <= 0 || K <= 0) return SWC_ERR_BAD_DIMS;
    if (pad_h != 1 || pad_w != 1) return SWC_ERR_BAD_PAD;
    const size_t M = static_cast<size_t>(B) * nH * nW;
    if (M >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    using Deep = HbCfg<64, 4, 2>;   // 4-deep ring, up to two workgroups per CU
    using Wide = HbCfg<64, 3, 3>;   // 3-deep ring, up to three workgroups per CU
    if (C % Deep::BK != 0 || !aligned16(Input16) || !aligned16(Weight16t) || static_cast<size_t>(HB_BM) * C >= (1ull << 30))
        return SWC_ERR_UNSUPPORTED;
    const size_t tiles_n = (static_cast<size_t>(K) + HB_BN - 1) / HB_BN;
    // Rows per workgroup: the workgroup count rounded up to a multiple of the CU count, as for the fp32
    // tilings (49 to 64 rows; conv2: 26.7 vs 28.8 us).
    const size_t rows = balanced_rows<HbStoreCfg>(M, tiles_n);
    const size_t tiles_m = (M + rows - 1) / rows;
    if (tiles_m * tiles_n >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    ConvEpilogue ep;
    ep.scale = Scale;
    ep.shift = Shift;
    ep.residual = Residual;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // More resident workgroups hide more of each other's waits once there are enough of them to go round
    // (conv3: 18.7 vs 19.6 us); a grid that leaves CUs with one workgroup does better with the deeper
    // ring (conv4b: 30.8 vs 34.2 us).
    if (tiles_m * tiles_n > kCUs)
        return launch_bf16_stored<Wide>(Input16, Weight16t, Output, M, C, K, nH, nW, rows, tiles_n, ep, s);
    return launch_bf16_stored<Deep>(Input16, Weight16t, Output, M, C, K, nH, nW, rows, tiles_n, ep, s);
}
