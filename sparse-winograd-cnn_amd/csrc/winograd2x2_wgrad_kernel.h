// Weight gradient of the Winograd convolution for gfx950: dW_i [C,K] = TI_i^T [C,M] . dP_i [M,K]
// for the 16 positions, the second GEMM of Winograd2x2ConvGradComputeLauncher
// (winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_grad_cuda.cu.cc:115-120).
//
// The reduction runs over M (tens of thousands of rows) and the output is tiny (16*C*K), so the
// rows are split over workgroups: workgroup (split s, position i, tile tc, tile tk) reduces its
// share of the rows into a 64x64 tile of partial sums, and a second kernel adds the partials of
// every split in ascending s.  No atomics: results do not depend on scheduling.
//
// Both operands are stored with the reduction index as the slow axis ([m][c] and [m][k]), so both
// LDS tiles are [32 rows of m][64 floats] and both MFMA operands are read the same way: lane
// (li = l % 32, lg = l / 32) of MFMA t takes row 16*lg + t, column li of its wave's 32 columns.
#pragma once

#include "winograd2x2_conv_kernel.h"

namespace swc {
namespace {

constexpr int WG_BM = 64;      // tile rows (channels c)
constexpr int WG_BN = 64;      // tile columns (filters k)
constexpr int WG_BK = 32;      // rows of m per step
constexpr int WG_NSTAGE = 3;   // ring depth
// Rows 16..31 of a tile start WG_HALF_PAD floats later, which puts the two lane groups of an operand
// read on different banks.
constexpr int WG_HALF_PAD = 32;
constexpr int WG_TILE_FLOATS = WG_BK * 64 + WG_HALF_PAD;
constexpr int WG_STAGE_FLOATS = 2 * WG_TILE_FLOATS;
constexpr int WG_LDS_BYTES = WG_NSTAGE * WG_STAGE_FLOATS * 4;
constexpr int WG_COPIES = 4;   // wave-wide copies per thread and step: 2 of the TI tile, 2 of the dP tile

// grid.x = S * 16 * tiles_c * tiles_k.  Split s takes steps [s*steps_per_split, ...) of the
// steps_total = M/32 steps and writes its tile to Out + s*split_stride + i*C*K.
// Requires M % 32 == 0, C % 4 == 0, K % 4 == 0, 16-byte aligned TI and dP.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void wgrad_splitk_kernel(
    const float *__restrict__ TI, const float *__restrict__ dP, float *__restrict__ Out, size_t M, int C, int K,
    unsigned tiles_c, unsigned tiles_k, unsigned steps_per_split, unsigned steps_total, size_t split_stride)
{
    extern __shared__ __attribute__((aligned(1024))) float smem[];

    // Consecutive logical ids differ in tk first: the workgroups that read the same TI tile share an L2.
    unsigned id = xcd_swizzle(blockIdx.x, gridDim.x);
    const unsigned tk = id % tiles_k;
    id /= tiles_k;
    const unsigned tc = id % tiles_c;
    id /= tiles_c;
    const unsigned pos = id % 16, split = id / 16;
    const unsigned step0 = split * steps_per_split;
    const unsigned nsteps = steps_total - step0 < steps_per_split ? steps_total - step0 : steps_per_split;
    const int c0 = static_cast<int>(tc) * WG_BM, k0 = static_cast<int>(tk) * WG_BN;

    const int tid = threadIdx.x, lane = tid & 63;
    const unsigned wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lg = lane >> 5;
    const int wm0 = static_cast<int>(wave >> 1) * 32, wn0 = static_cast<int>(wave & 1) * 32;

    // ---- copies: wave-copy wl (0..7) of a tile covers rows 4*wl .. 4*wl+3 (1 KiB) -----------------
    const float *a_next = TI + (static_cast<size_t>(pos) * M + static_cast<size_t>(step0) * WG_BK) * C;
    const float *b_next = dP + (static_cast<size_t>(pos) * M + static_cast<size_t>(step0) * WG_BK) * K;
    unsigned a_voff[2], b_voff[2], t_lds[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const unsigned wl = wave * 2 + q;
        const unsigned row = 4 * wl + lane / 16, chunk = lane % 16;
        // columns beyond C (K) re-read the last valid 16 bytes; they only reach outputs that are never stored
        unsigned ca = c0 + 4 * chunk, cb = k0 + 4 * chunk;
        ca = ca + 4 <= static_cast<unsigned>(C) ? ca : static_cast<unsigned>(C) - 4;
        cb = cb + 4 <= static_cast<unsigned>(K) ? cb : static_cast<unsigned>(K) - 4;
        a_voff[q] = (row * static_cast<unsigned>(C) + ca) * 4u;
        b_voff[q] = (row * static_cast<unsigned>(K) + cb) * 4u;
        t_lds[q] = (wl * 256u + (wl >= 4 ? WG_HALF_PAD : 0)) * 4u;
    }
    const unsigned smem_base = lds_address(smem);
    unsigned steps_issued = 0, slot_next = 0;
    const size_t a_step = static_cast<size_t>(WG_BK) * C, b_step = static_cast<size_t>(WG_BK) * K;
    // Every thread issues exactly WG_COPIES copies per call, so that the outstanding-copy count means
    // the same in every wave; past the last step the last tile is copied again (never read).
    auto issue = [&]() __attribute__((always_inline)) {
        const unsigned dst = smem_base + slot_next * (WG_STAGE_FLOATS * 4);
#pragma unroll
        for (int q = 0; q < 2; ++q) async_copy16(a_next, a_voff[q], dst + t_lds[q]);
#pragma unroll
        for (int q = 0; q < 2; ++q) async_copy16(b_next, b_voff[q], dst + WG_TILE_FLOATS * 4 + t_lds[q]);
        ++steps_issued;
        if (steps_issued < nsteps) {
            a_next += a_step;
            b_next += b_step;
        }
        slot_next = slot_next + 1 == WG_NSTAGE ? 0 : slot_next + 1;
    };

    floatx16 acc[2] = {};
#pragma unroll
    for (int i = 0; i < WG_NSTAGE - 1; ++i) issue();

    const int a_off = lg * (16 * 64 + WG_HALF_PAD) + wm0 + li;
    const int b_off = WG_TILE_FLOATS + lg * (16 * 64 + WG_HALF_PAD) + wn0 + li;
    int st_cur = 0;
    for (unsigned st = 0; st < nsteps; ++st) {
        // Step st has landed once at most the copies of the WG_NSTAGE-2 steps after it are outstanding;
        // after the barrier everyone has also finished reading the slot that the next copies overwrite.
        wait_vmcnt<(WG_NSTAGE - 2) * WG_COPIES>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        issue();
        float a[16], b[16];
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            a[t] = smem[st_cur + a_off + t * 64];
            b[t] = smem[st_cur + b_off + t * 64];
        }
#pragma unroll
        for (int t = 0; t < 16; ++t) acc[t & 1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b[t], acc[t & 1], 0, 0, 0);
        st_cur = st_cur + WG_STAGE_FLOATS == WG_NSTAGE * WG_STAGE_FLOATS ? 0 : st_cur + WG_STAGE_FLOATS;
    }
    wait_vmcnt<0>();  // the surplus copies must land before the workgroup's LDS is handed on

    float *out = Out + split * split_stride + static_cast<size_t>(pos) * C * K;
    const int col = k0 + wn0 + li;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int row = c0 + wm0 + 8 * (r / 4) + 4 * lg + r % 4;
        if (row < C && col < K) out[static_cast<size_t>(row) * K + col] = acc[0][r] + acc[1][r];
    }
}

// dW = sum over splits, ascending, of the partial tiles.  One lane per 4 floats; the loads of eight splits are
// requested before the first of them is added.
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(const float *__restrict__ part, float *__restrict__ dW,
                                                           unsigned n4, unsigned splits, size_t split_stride)
{
    const unsigned idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= n4) return;
    const float4 *p = reinterpret_cast<const float4 *>(part) + idx;
    const size_t stride4 = split_stride / 4;
    float4 s = *p;
    unsigned q = 1;
    for (; q + 8 <= splits; q += 8) {
        float4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = p[(q + j) * stride4];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            s.x += v[j].x;
            s.y += v[j].y;
            s.z += v[j].z;
            s.w += v[j].w;
        }
    }
    for (; q < splits; ++q) {
        const float4 v = p[q * stride4];
        s.x += v.x;
        s.y += v.y;
        s.z += v.z;
        s.w += v.w;
    }
    reinterpret_cast<float4 *>(dW)[idx] = s;
}

}  // namespace
}  // namespace swc
