// Weight gradient of the Winograd convolution on 128x128 workgroup tiles (device code):
// dW_i [C,K] = TI_i^T [C,M] . dP_i [M,K] for the 16 positions, the second GEMM of the reference's backward pass
// (winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_grad_cuda.cu.cc:115-120), split along M over workgroups
// like wgrad_splitk_kernel (winograd2x2_wgrad_kernel.h), whose second kernel adds the partial tiles.
//
// Both operands are stored with the reduction index m as their slow axis, so an LDS tile is [BKM rows of m][128
// floats] as it lies in memory, and a lane's 16 bytes of a row are four *output* indices at one m.  With
// v_mfma_f32_16x16x4_f32 a lane (li = l % 16, lg = l / 16) supplies one value per operand: row (column) li of the
// tile at reduction index lg.  Tile t of a wave's 64 channels is therefore taken as the channels 4*li + t: one
// ds_read_b128 at (m = 4g + lg, channels 4*li ..) is the first operand of four tiles, one at (m, filters 4*li ..)
// the second operand of four tiles, and the sixteen MFMAs of a group of four m need two LDS reads.  A wave owns
// 64 channels x 64 filters (sixteen 16x16 tiles, interleaved by four in both directions), a workgroup of four
// waves 128 x 128.  In the accumulators register r of tile (t, u) is channel 4*(4*lg + r) + t, filter 4*li + u, so
// the four tiles u of one (t, r) are 16 consecutive bytes of a dW row.
#pragma once

#include "winograd2x2_conv_wide_kernel.h"

namespace swc {
namespace {

// BKM rows of m per step, a ring of NSTAGE slots, OCC waves per SIMD.
template <int BKM_, int NSTAGE_, int OCC_>
struct WgradWideCfg {
    static constexpr int BKM = BKM_, NSTAGE = NSTAGE_, OCC = OCC_, NT = 256, BC = 128, BKF = 128;
    static constexpr int NG = BKM / 4;                    // groups of four m (sixteen MFMAs per wave) per step
    static constexpr int TILE_BYTES = BKM * 128 * 4, STAGE_BYTES = 2 * TILE_BYTES, LDS_BYTES = NSTAGE * STAGE_BYTES;
    static constexpr int NCW = BKM / 8;                   // wave-wide copies (1 KiB = two rows) per wave, tile and step
    static constexpr int NCOPY = 2 * NCW;                 // copies per wave and step
    static_assert(BKM == 16 || BKM == 32, "two or four copies per wave and tile");
    static_assert(NSTAGE >= 3 && NCOPY <= NG, "one copy per group of MFMAs, all issued between two barriers");
    static_assert((NSTAGE - 2) * NCOPY < 64, "outstanding copies fit the counter");
    static_assert(LDS_BYTES <= 160 * 1024, "fits the CU");
};

// grid.x = S * 16 * tiles_c * tiles_k.  Split s takes steps [s*steps_per_split, ...) of the steps_total = M/BKM
// steps and writes its tile to Out + s*split_stride + pos*C*K.
// Requires M % BKM == 0, C % 128 == 0, K % 128 == 0, 16-byte aligned TI, dP and Out, BKM*max(C,K)*4 < 2^31.
template <typename G>
__global__ __launch_bounds__(G::NT) __attribute__((amdgpu_waves_per_eu(G::OCC, G::OCC))) void wgrad_wide_kernel(
    const float *__restrict__ TI, const float *__restrict__ dP, float *__restrict__ Out, size_t M, int C, int K,
    unsigned tiles_c, unsigned tiles_k, unsigned steps_per_split, unsigned steps_total, size_t split_stride)
{
    constexpr int BKM = G::BKM, NSTAGE = G::NSTAGE, NG = G::NG, NCW = G::NCW, NCOPY = G::NCOPY;
    constexpr int TILE_BYTES = G::TILE_BYTES, STAGE_BYTES = G::STAGE_BYTES;
    extern __shared__ __attribute__((aligned(1024))) unsigned char gsmem[];  // G::LDS_BYTES

    // Consecutive logical ids differ in tk first: the workgroups that read the same TI tile share an L2.
    unsigned id = xcd_swizzle(blockIdx.x, gridDim.x);
    const unsigned tk = id % tiles_k;
    id /= tiles_k;
    const unsigned tc = id % tiles_c;
    id /= tiles_c;
    const unsigned pos = id % 16, split = id / 16;
    const unsigned step0 = split * steps_per_split;
    const unsigned nsteps = steps_total - step0 < steps_per_split ? steps_total - step0 : steps_per_split;
    const unsigned c0 = tc * 128, k0 = tk * 128;

    const int tid = threadIdx.x, lane = tid & 63;
    const unsigned wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const unsigned wc = wave >> 1, wk = wave & 1;   // the wave's 64 channels and 64 filters within the tile

    // ---- copies: wave-copy j (0 .. BKM/2-1) of a tile covers its rows 2j, 2j+1; wave w issues j = w*NCW + q ----
    const float *a_next = TI + (static_cast<size_t>(pos) * M + static_cast<size_t>(step0) * BKM) * C + c0;
    const float *b_next = dP + (static_cast<size_t>(pos) * M + static_cast<size_t>(step0) * BKM) * K + k0;
    unsigned a_voff[NCW], b_voff[NCW];
#pragma unroll
    for (int q = 0; q < NCW; ++q) {
        const unsigned row = 2 * (wave * NCW + q) + lane / 32, chunk = lane % 32;
        a_voff[q] = (row * static_cast<unsigned>(C) + 4 * chunk) * 4u;
        b_voff[q] = (row * static_cast<unsigned>(K) + 4 * chunk) * 4u;
    }
    const unsigned smem_base = lds_address(gsmem);
    const unsigned copy_base = __builtin_amdgcn_readfirstlane(smem_base + wave * NCW * 1024u);
    const size_t a_step = static_cast<size_t>(BKM) * C, b_step = static_cast<size_t>(BKM) * K;
    unsigned steps_issued = 0;
    // The i-th copy (0 .. NCOPY-1) of the tiles of one step into ring slot SLOT; every wave issues all of them, so
    // the outstanding-copy count means the same in every wave.  Past the last step the last tiles are copied
    // again (never read).
    auto issue_copy = [&](auto slot_c, auto i_c) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_c)::value, I = decltype(i_c)::value;
        if constexpr (I < NCW)
            async_copy16_imm<SLOT * STAGE_BYTES + I * 1024>(a_next, a_voff[I], copy_base);
        else
            async_copy16_imm<SLOT * STAGE_BYTES + TILE_BYTES + (I - NCW) * 1024>(b_next, b_voff[I - NCW], copy_base);
        if constexpr (I == NCOPY - 1) {
            ++steps_issued;
            if (steps_issued < nsteps) {
                a_next += a_step;
                b_next += b_step;
            }
        }
    };

    // ---- operand reads: byte offsets within a slot; group g adds g*2048 (four rows) ----
    const unsigned a_rd = (lg * 128u + wc * 64u + li * 4u) * 4u;
    const unsigned b_rd = TILE_BYTES + (lg * 128u + wk * 64u + li * 4u) * 4u;
    floatx4 acc[4][4] = {};
    float4 fa[2], fb[2];
    auto read_group = [&](auto slot_c, auto g_c, auto buf_c) __attribute__((always_inline)) {
        constexpr int OFF = decltype(slot_c)::value * STAGE_BYTES + decltype(g_c)::value * 2048;
        constexpr int buf = decltype(buf_c)::value;
        fa[buf] = *reinterpret_cast<const float4 *>(gsmem + a_rd + OFF);
        fb[buf] = *reinterpret_cast<const float4 *>(gsmem + b_rd + OFF);
    };
    using I0 = std::integral_constant<int, 0>;

    // Prologue: the tiles of the first NSTAGE-1 steps and the first copy of the step after them are under way (the
    // state every step below starts from); the first tiles have landed and their first group is read.
    static_for<NSTAGE - 1>([&](auto s_c) { static_for<NCOPY>([&](auto i_c) { issue_copy(s_c, i_c); }); });
    issue_copy(std::integral_constant<int, NSTAGE - 1>{}, I0{});
    wait_vmcnt<(NSTAGE - 2) * NCOPY + 1>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_group(I0{}, I0{}, I0{});

    // One step on ring slot SLOT.  Group g multiplies what the group before it read and reads for the group after
    // it; the last group reads the first group of the next step from the next slot, so the wait for that slot's
    // copies and the workgroup's barrier sit at the end of the last group but one.  By then every wave has also
    // read all of this slot (the wait covers its LDS reads), which is what the copies issued from there on
    // overwrite: copy 0 of the step NSTAGE ahead in the last group, copies 1.. in the first groups of the next step.
    auto step = [&](auto slot_c) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_c)::value;
        constexpr int NEXT = (SLOT + 1) % NSTAGE, FREE = (SLOT + NSTAGE - 1) % NSTAGE;   // FREE: read in the step before
        static_for<NG>([&](auto g_c) {
            constexpr int g = decltype(g_c)::value;
            constexpr int cur = g & 1;
            if constexpr (g + 1 < NG)
                read_group(slot_c, std::integral_constant<int, g + 1>{}, std::integral_constant<int, cur ^ 1>{});
            else
                read_group(std::integral_constant<int, NEXT>{}, I0{}, I0{});
            if constexpr (g == NG - 1)
                issue_copy(slot_c, I0{});
            else if constexpr (g + 1 < NCOPY)
                issue_copy(std::integral_constant<int, FREE>{}, std::integral_constant<int, g + 1>{});
            __builtin_amdgcn_sched_barrier(0);
            const float4 a4 = fa[cur], b4 = fb[cur];
            const float av[4] = {a4.x, a4.y, a4.z, a4.w}, bv[4] = {b4.x, b4.y, b4.z, b4.w};
            static_for<16>([&](auto i_c) {
                constexpr int t = decltype(i_c)::value / 4, u = decltype(i_c)::value % 4;
                acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[t], bv[u], acc[t][u], 0, 0, 0);
            });
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (g == NG - 2) {
                // the next step's tiles have landed once only the copies of the steps after it are outstanding
                wait_vmcnt<(NSTAGE - 2) * NCOPY>();
                __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS reads of this slot are done
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            }
        });
    };
    static_assert(NG % 2 == 0, "the operand buffers alternate and a step starts on buffer 0");
    for (unsigned st = 0;;) {
        bool done = false;
        static_for<NSTAGE>([&](auto s_c) {
            if (!done) {
                step(s_c);
                done = ++st == nsteps;
            }
        });
        if (done) break;
    }
    wait_vmcnt<0>();  // the surplus copies must have landed before this workgroup's LDS can be handed on

    // ---- partial tile: register r of tile (t, u) is channel 4*(4*lg + r) + t, filter 4*li + u ----
    float *out = Out + split * split_stride + static_cast<size_t>(pos) * C * K +
                 static_cast<size_t>(c0 + wc * 64) * K + (k0 + wk * 64 + 4 * li);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float4 v = {acc[t][0][r], acc[t][1][r], acc[t][2][r], acc[t][3][r]};
            *reinterpret_cast<float4 *>(out + static_cast<size_t>(4 * (4 * lg + r) + t) * K) = v;
        }
}

}  // namespace
}  // namespace swc
