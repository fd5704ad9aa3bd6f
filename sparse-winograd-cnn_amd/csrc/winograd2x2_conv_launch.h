// Host side of the ring kernels (winograd2x2_conv_kernel.h): which tiling a call gets, how its rows are dealt to
// the workgroups, and the launch itself.  Shared by the forward convolution (winograd2x2_conv.hip) and the data
// gradient of the backward pass (winograd2x2_grad.hip).
#pragma once

#include <string_view>

#include "winograd2x2_conv_kernel.h"

namespace swc {

// Compute units of the current device (256 on MI355X), read once per device and host thread.
inline size_t device_cus()
{
    constexpr int kMaxDevices = 64;
    static thread_local int cus[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    if (cus[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev] = n;
    }
    return static_cast<size_t>(cus[dev]);
}

// Bytes of one L2 (MI355X: 4 MiB per XCD, eight of them), read once per device and host thread.
inline size_t device_l2_bytes()
{
    constexpr int kMaxDevices = 64;
    static thread_local int l2[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 4u << 20;
    if (l2[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeL2CacheSize, dev) != hipSuccess || n <= 0) n = 4 << 20;
        l2[dev] = n;
    }
    return static_cast<size_t>(l2[dev]);
}

// How the wide48 kernel (winograd2x2_conv_wide_kernel.h) would cover M rows x N columns: `groups` row groups of
// rows_per_wg <= 48 rows cover main_rows; with `extra` the rows beyond are dealt out as 16x16 tiles, one per
// workgroup.  units: MFMA work of a wave per pass over the chip, in 16x16 tiles.
struct WidePlan {
    bool ok = false;
    bool extra = false;
    int bn = 128;   // columns per workgroup: 128 (wave tile 48x32) or 64 (48x16)
    size_t groups = 0, rows_per_wg = 0, main_rows = 0, wgs = 0;
    double units = 0;
};

// The kernel takes C in pairs of 32-channel steps, whole column groups of bn = 128 or 64, 16-byte granules, 32-bit
// byte offsets into the activations of one position and 31-bit ones into the output.
inline bool wide48_eligible(const void *A, const void *B, size_t M, int R, int N, int bn = 128)
{
    return R % 64 == 0 && N % bn == 0 && (reinterpret_cast<uintptr_t>(A) & 15u) == 0 && (reinterpret_cast<uintptr_t>(B) & 15u) == 0 &&
           M >= 48 && M * static_cast<size_t>(R) * 4 < (1ull << 32) && M * 16 * static_cast<size_t>(N) < (1ull << 31) &&
           static_cast<size_t>(R) * N * 16 * 4 < (1ull << 40);
}

// Either full 48-row groups in whole passes over the chip with the rest as extra tiles (6.25 units per pass with
// 128-column workgroups, 3.25 with 64-column ones), or the rows levelled over as many groups as fill whole passes
// (6 or 3 units), whichever makes fewer units in total.
inline WidePlan plan_wide48(size_t M, int N, size_t cus, int bn = 128)
{
    WidePlan best;
    best.bn = bn;
    const size_t tiles_n = static_cast<size_t>(N) / bn;
    const double unit = bn == 128 ? 6.0 : 3.0;
    const size_t xct = static_cast<size_t>(bn) / 16;   // extra tiles per left-over row tile and column group
    if (tiles_n == 0 || M < 48) return best;
    auto passes_of = [&](size_t wgs) { return static_cast<double>((wgs + cus - 1) / cus); };
    {   // levelled
        const size_t gmin = (M + 47) / 48;
        const size_t wgs = (gmin * tiles_n + cus - 1) / cus * cus;
        size_t groups = wgs / tiles_n > gmin ? wgs / tiles_n : gmin;
        const size_t rows = (M + groups - 1) / groups;
        groups = (M + rows - 1) / rows;
        best.ok = true;
        best.extra = false;
        best.groups = groups;
        best.rows_per_wg = rows;
        best.main_rows = M;
        best.wgs = groups * tiles_n;
        best.units = passes_of(best.wgs) * unit;
    }
    {   // full groups plus extra tiles
        const size_t gfull = M / 48;
        size_t groups = gfull * tiles_n / cus * cus / tiles_n;
        if (groups == 0) groups = gfull;
        const size_t main_rows = groups * 48;
        const size_t left_tiles = (M - main_rows + 15) / 16;
        if (left_tiles > 0 && left_tiles * xct <= groups) {
            const double units = passes_of(groups * tiles_n) * (unit + 0.25);
            if (units < best.units) {
                best.extra = true;
                best.groups = groups;
                best.rows_per_wg = 48;
                best.main_rows = main_rows;
                best.wgs = groups * tiles_n;
                best.units = units;
            }
        }
    }
    return best;
}

// Defined in winograd2x2_conv_bf16_tall.hip: the bf16-stored convolution over 128-row x 64-column tiles.
bool bf16_tall_eligible(const void *TI16, const void *Wt16, size_t M, int C, int K);
// The spread form of the same kernel (winograd2x2_conv_bf16_spread.hip): Part is a scratch buffer of 8*M*K floats.
bool bf16_spread_eligible(const void *TI16, const void *Wt16, const void *Out, const void *Part, size_t M, int C, int K,
                          const float *scale, const float *shift, const float *residual);
int launch_bf16_spread(const unsigned short *TI16, const unsigned short *Wt16, float *Out, float *Part, size_t M, int C, int K,
                       int nW, const float *scale, const float *shift, const float *residual, int residual_relu, hipStream_t stream);
int launch_bf16_tall(const unsigned short *TI16, const unsigned short *Wt16, float *Out, size_t M, int C, int K, int nW,
                     size_t rows_per_wg, const float *scale, const float *shift, const float *residual, int residual_relu,
                     hipStream_t stream);

// Defined in winograd2x2_conv_wide.hip (128-column workgroups) and winograd2x2_conv_wide64*.hip (64-column ones);
// launch_wide48 hands a plan with bn == 64 on to the second.
int launch_wide48_n64(const float *TI, const float *Wt, float *Out, size_t M, int C, int K, int nW, const WidePlan &plan,
                      const float *scale, const float *shift, const float *residual, int residual_relu, hipStream_t stream);
int launch_wide48_n64_ring4(const float *TI, const float *Wt, float *Out, size_t M, int C, int K, int nW, const WidePlan &plan,
                            const float *scale, const float *shift, const float *residual, int residual_relu,
                            hipStream_t stream);
int launch_wide48(const float *TI, const float *Wt, float *Out, size_t M, int C, int K, int nW, const WidePlan &plan,
                  const float *scale, const float *shift, const float *residual, int residual_relu, hipStream_t stream);

namespace {

// 32x32 MFMAs, wave tile 32x32: the fewest LDS reads per MFMA; its results are bit-identical to
// the synchronous kernel's.
using Tile32 = ConvCfg<64, 64, 32, 2, 2>;
using Tile16 = ConvCfg<64, 64, 16, 2, 2>;
// 16x16 MFMAs, wave tile (16*TM)x16: row groups of any height up to 112 (Tall) or 32 (Short), so
// that M can be dealt evenly over the CUs where 64-row tiles leave CUs idle or a ragged tail.
using Tall = ConvCfg<112, 64, 32, 1, 4, 2, 16>;
using Short = ConvCfg<32, 64, 64, 1, 4, 3, 16>;

enum Tiling { TILING_SYNC = 0, TILING_RING32, TILING_RING16, TILING_TALL16, TILING_SHORT16, TILING_WIDE48, TILING_WIDE48X64 };
inline const char *tiling_name(Tiling t)
{
    switch (t) {
        case TILING_RING32: return "ring32";
        case TILING_RING16: return "ring16";
        case TILING_TALL16: return "tall16";
        case TILING_SHORT16: return "short16";
        case TILING_WIDE48: return "wide48";
        case TILING_WIDE48X64: return "wide48x64";
        default: return "sync";
    }
}

// Passes the chip makes over `wgs` workgroups of equal length: the busiest CU sets the time, so whole
// passes while the grid is small; with many short workgroups the tail evens out.
inline double passes(size_t wgs, size_t cus)
{
    return wgs <= 8 * cus ? static_cast<double>((wgs + cus - 1) / cus) : static_cast<double>(wgs) / cus + 0.5;
}

// Rows per workgroup that split M into as many equal row groups as fill whole passes of the chip, but
// never so few that one of the workgroup's 16-row MFMA tiles would hold no valid row at all (a
// workgroup computes all of its tiles whatever their content).
template <typename Cfg>
size_t balanced_rows(size_t M, size_t tiles_n, size_t cus)
{
    const size_t groups_min = (M + Cfg::BM - 1) / Cfg::BM;
    const size_t wgs = (groups_min * tiles_n + cus - 1) / cus * cus;
    size_t groups = wgs / tiles_n;
    if (groups < groups_min) groups = groups_min;
    size_t rows = (M + groups - 1) / groups;
    if (rows < static_cast<size_t>(Cfg::BM) - 15) rows = Cfg::BM - 15;
    return rows < static_cast<size_t>(Cfg::BM) ? rows : static_cast<size_t>(Cfg::BM);
}

// A ring tiling takes whole BK chunks of the reduction range R, 16-byte granules and 32-bit byte offsets
// within a tile.  N: output columns (forward: they are the fast axis of the B operand and must come in fours).
template <typename Cfg>
bool ring_eligible(const void *A, const void *B, int R, int N, bool forward)
{
    return (R % Cfg::BK == 0) && (!forward || N % 4 == 0) && aligned16(A) && aligned16(B) &&
           static_cast<size_t>(Cfg::BM) * R < (1ull << 29) &&
           (forward ? static_cast<size_t>(Cfg::BK) * N : static_cast<size_t>(Cfg::BN) * R) < (1ull << 29);
}

struct TilingChoice {
    Tiling tiling;
    size_t rows_per_wg;
    WidePlan wide = WidePlan();  // TILING_WIDE48 only
};

// The tiling of a call with M rows, reduction length R and N output columns.  `ring16_ok`: the caller has a
// 16-index-step variant (the forward fp32 kernel only).
// Cost = passes x MFMA work of a wave per pass (in 16x16 tiles), weighted by what each kernel measured per
// unit of that work on MI355X relative to ring32 (`bench.py --workload sweep` times every tiling over the
// ResNet-18 shapes at batch 64 and 128 and a set of other shapes, and prints the choice made here against the
// best): tall16 8 % more with one workgroup per CU, 2 % less once a second one is resident (its waits
// then hide behind the other's MFMAs); short16 10 % more, 3 % less while all of its workgroups are resident at
// once (up to three per CU), and 2 % on top when a position is a single 64-index step.
inline TilingChoice choose_tiling(const void *A, const void *B, size_t M, int R, int N, bool forward, bool ring16_ok)
{
    const size_t cus = device_cus();
    const size_t tiles_n = (static_cast<size_t>(N) + 63) / 64;
    const bool ok32 = ring_eligible<Tile32>(A, B, R, N, forward);
    const bool ok16 = ring16_ok && ring_eligible<Tile16>(A, B, R, N, forward);
    const bool ok_tall = ring_eligible<Tall>(A, B, R, N, forward);
    const bool ok_short = ring_eligible<Short>(A, B, R, N, forward);
    // tall16 levels its row groups over the CUs; short16 does better with full 32-row groups (two whole MFMA
    // tiles) even where that leaves some CUs with one workgroup more (conv4a: 69 vs 73 us).
    const size_t rows_tall = balanced_rows<Tall>(M, tiles_n, cus), rows_short = Short::BM;
    // wide48 (forward only): 48-row x 128-column workgroups, left-over rows dealt out as extra tiles.
    const bool ok_wide = forward && wide48_eligible(A, B, M, R, N);
    const WidePlan wide = ok_wide ? plan_wide48(M, N, cus) : WidePlan();
    // the same with 64-column workgroups (wave tile 48x16: more LDS reads per MFMA, twice the workgroups)
    const bool ok_wide64 = forward && wide48_eligible(A, B, M, R, N, 64);
    const WidePlan wide64 = ok_wide64 ? plan_wide48(M, N, cus, 64) : WidePlan();
    if (const char *f = forced_conv_tiling()) {
        const std::string_view want(f);
        if (want == "wide48" && wide.ok) return {TILING_WIDE48, wide.rows_per_wg, wide};
        if (want == "wide48x64" && wide64.ok) return {TILING_WIDE48X64, wide64.rows_per_wg, wide64};
        if (want == "ring32" && ok32) return {TILING_RING32, Tile32::BM};
        if (want == "ring16" && ok16) return {TILING_RING16, Tile16::BM};
        if (want == "tall16" && ok_tall) return {TILING_TALL16, rows_tall};
        if (want == "short16" && ok_short) return {TILING_SHORT16, rows_short};
        return {TILING_SYNC, 64};
    }
    const size_t wgs_short = (M + rows_short - 1) / rows_short * tiles_n;
    const size_t wgs_tall = (M + rows_tall - 1) / rows_tall * tiles_n;
    const double w_tall = wgs_tall > cus ? 0.98 : 1.08;
    const double w_short = (wgs_short <= 3 * cus ? 0.97 : 1.10) * (R < 128 ? 1.02 : 1.0);
    const double cost32 = ok32 ? passes((M + 63) / 64 * tiles_n, cus) * 4.0 : 1e30;
    const double cost_tall = ok_tall ? passes(wgs_tall, cus) * 7.0 * w_tall : 1e30;
    const double cost_short = ok_short ? passes(wgs_short, cus) * 2.0 * w_short : 1e30;
    // wide48: a unit of its work measured 9 % more than ring32's with one workgroup per CU, 1 % more with two.
    const double cost_wide = wide.ok ? wide.units * (wide.wgs > cus ? 1.01 : 1.09) : 1e30;
    // 64-column workgroups: 12 % more per unit (14x14x256 at batch 64: 57 us against 70 for short16; 28x28x128: 56
    // against 54 for the 128-column workgroups).  With 64 channels a position is two steps, the ring has two slots
    // and the output transform's share grows: at 56x56x64, batch 64 (four workgroups per CU) the kernel alone is 4 %
    // faster than tall16 on cache-resident planes, but the transform + convolution pair, whose planes come from
    // HBM, is 4 % slower (110 us against 106); at batch 16 (one workgroup per CU) it wins both ways (20 us against
    // 22 for short16).  So below 128 channels only for a single pass, and never for less than a full pass.
    const double cost_wide64 =
        wide64.ok && (R >= 128 || wide64.wgs <= cus) && wide64.wgs >= cus ? wide64.units * 1.12 : 1e30;
    if (cost_wide64 < cost_wide && cost_wide64 < cost32 && cost_wide64 < cost_tall && cost_wide64 < cost_short)
        return {TILING_WIDE48X64, wide64.rows_per_wg, wide64};
    if (wide.ok && cost_wide < cost32 && cost_wide < cost_tall && cost_wide < cost_short) return {TILING_WIDE48, wide.rows_per_wg, wide};
    if (ok_tall && cost_tall < cost32 && cost_tall <= cost_short) return {TILING_TALL16, rows_tall};
    if (ok_short && cost_short < cost32) return {TILING_SHORT16, rows_short};
    if (ok32) return {TILING_RING32, Tile32::BM};
    if (ok16) return {TILING_RING16, Tile16::BM};
    return {TILING_SYNC, 64};
}

// Raises the dynamic-LDS limit of `kernel` above the default 64 KiB, once per kernel instance, device and thread.
template <typename Tag>
int raise_lds_limit(const void *kernel, int lds_bytes)
{
    if (lds_bytes <= 64 * 1024) return SWC_OK;
    constexpr int kMaxDevices = 64;
    static thread_local bool raised[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SWC_ERR_HIP;
    if (!raised[dev]) {
        const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (e != hipSuccess) return note_hip_error(e);
        raised[dev] = true;
    }
    return SWC_OK;
}

}  // namespace
}  // namespace swc
