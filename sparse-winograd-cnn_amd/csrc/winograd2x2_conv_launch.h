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

namespace {

// 32x32 MFMAs, wave tile 32x32: the fewest LDS reads per MFMA; its results are bit-identical to
// the synchronous kernel's.
using Tile32 = ConvCfg<64, 64, 32, 2, 2>;
using Tile16 = ConvCfg<64, 64, 16, 2, 2>;
// 16x16 MFMAs, wave tile (16*TM)x16: row groups of any height up to 112 (Tall) or 32 (Short), so
// that M can be dealt evenly over the CUs where 64-row tiles leave CUs idle or a ragged tail.
using Tall = ConvCfg<112, 64, 32, 1, 4, 2, 16>;
using Short = ConvCfg<32, 64, 64, 1, 4, 3, 16>;

enum Tiling { TILING_SYNC = 0, TILING_RING32, TILING_RING16, TILING_TALL16, TILING_SHORT16 };
inline const char *tiling_name(Tiling t)
{
    switch (t) {
        case TILING_RING32: return "ring32";
        case TILING_RING16: return "ring16";
        case TILING_TALL16: return "tall16";
        case TILING_SHORT16: return "short16";
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
    if (const char *f = forced_conv_tiling()) {
        const std::string_view want(f);
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
