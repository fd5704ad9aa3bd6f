// Winograd convolution over bf16-stored operands for gfx950: the 16 GEMMs
// P_i [M,K] = TI_i [M,C] . W_i [C,K] with TI held in memory as bf16 [16,M,C] and the weights as
// bf16, transposed, [16,K,C]; fp32 accumulation, fp32 output transform and fp32 output, as in
// conv_mfma_async_kernel.  Same arithmetic as swc_winograd2x2_conv_bf16 (operands rounded to bf16,
// products exact in fp32), with the rounding done once by whoever wrote the operands instead of in
// this kernel's registers, and half the bytes to move: the path is HBM-bound.
//
// Both operands have the reduction index (channels) as their fast axis, so both LDS tiles are
// [64 rows][64 channels = 128 bytes = 8 chunks of 16 bytes] and an MFMA operand
// (v_mfma_f32_32x32x16_bf16: lane (li, lg) holds 8 consecutive channels 8*lg.. of row li) is one
// ds_read_b128 with no conversion.  Chunk c of row r is stored at slot c ^ ((r / 2) % 8): two 128-byte rows
// share 256 bytes of LDS, and with r % 8 rows r and r+8 of an operand read landed on the same banks (the
// counters showed every second LDS cycle as a bank conflict; none with r / 2).
#pragma once

#include "winograd2x2_conv_kernel.h"

namespace swc {
namespace {

constexpr int HB_BM = 64, HB_BN = 64;  // tile of the [M,K] plane; 4 waves, 2x2, 32x32 each
using HbStoreCfg = ConvCfg<HB_BM, HB_BN, 32, 2, 2>;

// BK channels per step (a tile row is BK*2 bytes = CH chunks of 16), NSTAGE ring slots, OCC waves per SIMD, BM
// rows per tile: 64 (four waves, 2x2) or 32 (two waves side by side).
template <int BK_, int NSTAGE_, int OCC_, int BM_ = HB_BM>
struct HbCfg {
    static constexpr int BK = BK_, NSTAGE = NSTAGE_, OCC = OCC_, BM = BM_;
    static constexpr int GW = BM / 16;                   // waves of a group: one per 32x32 part of the BM x 64 tile
    static constexpr int CH = BK / 8;                    // 16-byte chunks per tile row
    static constexpr int ROWS_PER_COPY = 64 / CH;        // rows one wave-wide copy (1 KiB) covers
    static constexpr int A_BYTES = BM * BK * 2;          // activation tile
    static constexpr int TILE_BYTES = 64 * BK * 2;       // weight tile
    static constexpr int PER_WAVE_A = A_BYTES / 1024 / GW, PER_WAVE = TILE_BYTES / 1024 / GW;  // copies per wave and step
    static constexpr int COPIES = PER_WAVE_A + PER_WAVE; // per thread and step
    static constexpr int STAGE_BYTES = A_BYTES + TILE_BYTES;
    static constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES;
    static constexpr int NMFMA = BK / 16;                // MFMAs per step and wave
    using Store = ConvCfg<BM, HB_BN, 32, BM / 32, 2>;
    static_assert(BK == 32 || BK == 64 || BK == 128, "a tile row is 4, 8 or 16 chunks");
    static_assert(BM == 64 || BM == 32, "four or two waves per group");
    static_assert(A_BYTES / 1024 % GW == 0 && TILE_BYTES / 1024 % GW == 0, "every wave issues the same number of copies");
    static_assert((NSTAGE - 2) * COPIES < 64, "vmcnt range");
};

// Requires C % BK == 0 and 16-byte aligned TI16 / Wt16.  M < 2^31.  grid.x = ceil(M / rows_per_wg) * tiles_n.
//
// GROUPS = 2 or 4: a workgroup is that many groups of waves that share the tile and split its 16 positions (0-7
// and 8-15, or four each), each group with its own ring; at the end the other groups hand their four partial
// output tiles to the first through LDS, which adds them to its own in ascending group order and stores.  For
// grids that leave a CU with one workgroup: the time of such a launch is one workgroup's chain of dependent
// steps (wait, barrier, copies, LDS reads, four MFMAs), and chains of a half or a quarter of the length run side by
// side on the same SIMDs.  The sum of the transform is then taken group by group instead of in one ascending
// chain.  Needs GROUPS*LDS_BYTES of LDS.
template <typename Cfg, int GROUPS = 1>
__global__ __launch_bounds__(64 * Cfg::GW * GROUPS) __attribute__((amdgpu_waves_per_eu(Cfg::OCC, Cfg::OCC))) void conv_bf16_stored_kernel(
    const unsigned short *__restrict__ TI16, const unsigned short *__restrict__ Wt16, float *__restrict__ Out, size_t M,
    int C, int K, int nH, int nW, unsigned tiles_n, unsigned rows_per_wg, ConvEpilogue ep)
{
    constexpr int BK = Cfg::BK, NSTAGE = Cfg::NSTAGE, CH = Cfg::CH, RPC = Cfg::ROWS_PER_COPY, PW = Cfg::PER_WAVE;
    constexpr int PWA = Cfg::PER_WAVE_A, GW = Cfg::GW;
    constexpr int ROW_BYTES = BK * 2;
    constexpr int RPL = ROW_BYTES >= 256 ? 1 : 256 / ROW_BYTES;  // tile rows per 256 bytes of LDS (one pass over its banks)
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem_b[];

    const unsigned lid = xcd_swizzle(blockIdx.x, gridDim.x);
    // A workgroup takes rows_per_wg <= BM rows (the launcher levels the load over the CUs with it).
    const size_t m0 = static_cast<size_t>(lid / tiles_n) * rows_per_wg;
    const int n0 = static_cast<int>(lid % tiles_n) * HB_BN;
    const unsigned rows_valid = static_cast<unsigned>(M - m0 < rows_per_wg ? M - m0 : rows_per_wg);
    const unsigned cols_valid = static_cast<unsigned>(K - n0 < HB_BN ? K - n0 : HB_BN);

    static_assert(GROUPS == 1 || GROUPS == 2 || GROUPS == 4, "one, two or four groups of waves");
    constexpr int NPOS = 16 / GROUPS;  // positions per group
    const int tid = threadIdx.x, lane = tid & 63;
    const unsigned wave_wg = __builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned group = wave_wg / GW, wave = wave_wg % GW;  // wave: index within the group
    const int li = lane & 31, lg = lane >> 5;
    const int wm0 = static_cast<int>(wave >> 1) * 32, wn0 = static_cast<int>(wave & 1) * 32;
    const int nkc = C / BK;
    unsigned char *const smem_g = smem_b + group * Cfg::LDS_BYTES;  // this group's ring

    // ---- copies: wave-copy wl of a tile covers its rows RPC*wl .. RPC*wl+RPC-1 (1 KiB) ------------------
    // Rows beyond the valid ones re-read the last valid row; they only reach outputs that are never stored.
    unsigned a_voff[PWA], b_voff[PW], ta_lds[PWA], tb_lds[PW];
#pragma unroll
    for (int q = 0; q < PWA; ++q) {
        const unsigned wl = wave * PWA + q;
        const unsigned row = RPC * wl + lane / CH, slot = lane % CH, chunk = slot ^ ((row / RPL) % CH);
        const unsigned ra = row < rows_valid ? row : rows_valid - 1;
        a_voff[q] = (ra * static_cast<unsigned>(C) + chunk * 8) * 2u;
        ta_lds[q] = wl * 1024u;
    }
#pragma unroll
    for (int q = 0; q < PW; ++q) {
        const unsigned wl = wave * PW + q;
        const unsigned row = RPC * wl + lane / CH, slot = lane % CH, chunk = slot ^ ((row / RPL) % CH);
        const unsigned rb = row < cols_valid ? row : cols_valid - 1;
        b_voff[q] = (rb * static_cast<unsigned>(C) + chunk * 8) * 2u;
        tb_lds[q] = Cfg::A_BYTES + wl * 1024u;
    }
    const unsigned smem_base = lds_address(smem_g);
    const size_t a_pos_stride = M * static_cast<size_t>(C), b_pos_stride = static_cast<size_t>(K) * C;
    // the group's first position: 0, or 8 for the second group
    const unsigned short *const a_first = TI16 + m0 * C + group * NPOS * a_pos_stride;
    const unsigned short *const b_first = Wt16 + static_cast<size_t>(n0) * C + group * NPOS * b_pos_stride;
    // The walk over the (position, channel chunk) steps, branch-free: a step advances both pointers by BK
    // channels, or by what takes them from a position's last chunk to the next position's first; after the
    // group's last step they return to its first position (the surplus copies are never read).
    const unsigned short *a_next = a_first, *b_next = b_first;
    const size_t a_jump = a_pos_stride - static_cast<size_t>(nkc - 1) * BK, b_jump = b_pos_stride - static_cast<size_t>(nkc - 1) * BK;
    int kc_left = nkc, steps_left = NPOS * nkc;
    unsigned dst_next = smem_base;
    // Every thread issues exactly Cfg::COPIES copies per call.
    auto issue = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < PWA; ++q) async_copy16(reinterpret_cast<const float *>(a_next), a_voff[q], dst_next + ta_lds[q]);
#pragma unroll
        for (int q = 0; q < PW; ++q) async_copy16(reinterpret_cast<const float *>(b_next), b_voff[q], dst_next + tb_lds[q]);
        const bool last_chunk = --kc_left == 0;
        kc_left = last_chunk ? nkc : kc_left;
        a_next += last_chunk ? a_jump : static_cast<size_t>(BK);
        b_next += last_chunk ? b_jump : static_cast<size_t>(BK);
        if (--steps_left == 0) {
            a_next = a_first;
            b_next = b_first;
        }
        dst_next = dst_next + Cfg::STAGE_BYTES == smem_base + Cfg::LDS_BYTES ? smem_base : dst_next + Cfg::STAGE_BYTES;
    };

    floatx16 Y[4][1][1];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) Y[j][0][0][r] = 0.f;

#pragma unroll
    for (int i = 0; i < NSTAGE - 1; ++i) issue();

    // byte offsets of this lane's operand chunks within a stage: MFMA h of a step takes chunk 2h + lg
    unsigned a_off[Cfg::NMFMA], b_off[Cfg::NMFMA];
#pragma unroll
    for (int h = 0; h < Cfg::NMFMA; ++h) {
        const unsigned ra = wm0 + li, rb = wn0 + li;
        a_off[h] = ra * ROW_BYTES + (((2 * h + lg) ^ ((ra / RPL) % CH)) * 16u);
        b_off[h] = Cfg::A_BYTES + rb * ROW_BYTES + (((2 * h + lg) ^ ((rb / RPL) % CH)) * 16u);
    }
    unsigned st_next = 0;  // byte offset of the ring slot whose operands are fetched next

    // The operands of a step are read from LDS one step ahead of the MFMAs that consume them, so that
    // the matrix work of step s runs while the reads of step s+1 (and the wait for its tiles) are in
    // flight: two register sets, F[s & 1].
    bf16x8 fa[2][Cfg::NMFMA], fb[2][Cfg::NMFMA];
    auto fetch = [&](int set) __attribute__((always_inline)) {
        // The tiles of the step to fetch have landed once at most the copies of the NSTAGE-2 steps
        // issued after it are outstanding; after the barrier every wave has also finished reading the
        // slot that the next copies overwrite (it was fetched one step earlier still).
        wait_vmcnt<(NSTAGE - 2) * Cfg::COPIES>();
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's own reads of the slot about to be refilled are done
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        issue();
#pragma unroll
        for (int h = 0; h < Cfg::NMFMA; ++h) {
            fa[set][h] = *reinterpret_cast<const bf16x8 *>(smem_g + st_next + a_off[h]);
            fb[set][h] = *reinterpret_cast<const bf16x8 *>(smem_g + st_next + b_off[h]);
        }
        st_next = st_next + Cfg::STAGE_BYTES == Cfg::LDS_BYTES ? 0 : st_next + Cfg::STAGE_BYTES;
    };
    fetch(0);

    auto positions = [&](auto first_tag) __attribute__((always_inline)) {
        static_for<NPOS>([&](auto pos_tag) {
            constexpr int pos = decltype(first_tag)::value + decltype(pos_tag)::value;
            floatx16 P = {};
            auto mfmas = [&](int set) __attribute__((always_inline)) {
    #pragma unroll
                for (int h = 0; h < Cfg::NMFMA; ++h) P = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][h], fb[set][h], P, 0, 0, 0);
            };
            // A position starts with its first step's operands in set 0.  Steps go in pairs so that the set
            // indices are compile-time constants (the sets must stay in registers); an odd last step moves
            // the prefetched set 1 into set 0.  Past the very last step the fetch reads the wrapped-around
            // copy, which is never used.
            int kc = 0;
    #pragma nounroll
            for (; kc + 1 < nkc; kc += 2) {
                fetch(1);
                mfmas(0);
                fetch(0);
                mfmas(1);
            }
            if (kc < nkc) {
                fetch(1);
                mfmas(0);
    #pragma unroll
                for (int h = 0; h < Cfg::NMFMA; ++h) {
                    fa[0][h] = fa[1][h];
                    fb[0][h] = fb[1][h];
                }
            }
            // fold P_pos into the running output tiles, ascending pos (winograd2x2_conv_cuda.cu.cc:39-46)
            constexpr unsigned long long plus = kPlus, minus = kMinus;
    #pragma unroll
            for (int j = 0; j < 4; ++j) {
                if ((plus >> (4 * pos + j)) & 1ull)
                    Y[j][0][0] += P;
                else if ((minus >> (4 * pos + j)) & 1ull)
                    Y[j][0][0] -= P;
                // pins the update here: otherwise the compiler defers all the adds to the end and keeps the
                // 16 product tiles alive instead of the 4 sums
                asm volatile("" : "+v"(Y[j][0][0]));
            }
        });
    };
    if constexpr (GROUPS == 1) {
        positions(std::integral_constant<int, 0>{});
    } else if constexpr (GROUPS == 2) {
        if (group == 0)
            positions(std::integral_constant<int, 0>{});
        else
            positions(std::integral_constant<int, 8>{});
    } else {
        if (group == 0)
            positions(std::integral_constant<int, 0>{});
        else if (group == 1)
            positions(std::integral_constant<int, 4>{});
        else if (group == 2)
            positions(std::integral_constant<int, 8>{});
        else
            positions(std::integral_constant<int, 12>{});
    }
    wait_vmcnt<0>();  // the surplus copies must land before the workgroup's LDS is handed on

    if constexpr (GROUPS > 1) {
        // The other groups' partial sums go through LDS, [group][j][register][thread of the group] (the rings are idle
        // by now), and are added to the first group's in ascending group order; the first group then stores alone.
        constexpr int TG = 64 * GW;  // threads of a group
        static_assert(GROUPS * Cfg::LDS_BYTES >= (GROUPS - 1) * 4 * 16 * TG * 4, "the rings hold the partial tiles");
        float *const xch = reinterpret_cast<float *>(smem_b);
        const int t = tid % TG;
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_s_barrier();  // every wave has finished reading its ring
        if (group != 0) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) xch[(((group - 1) * 4 + j) * 16 + r) * TG + t] = Y[j][0][0][r];
        }
        __syncthreads();
        if (group != 0) return;
#pragma unroll
        for (int g = 0; g < GROUPS - 1; ++g)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) Y[j][0][0][r] += xch[((g * 4 + j) * 16 + r) * TG + t];
    }
    store_output<typename Cfg::Store>(Y, Out, rows_valid, K, nW, m0, n0, wm0, wn0, li, lg, ep);
}

// W [16,C,K] fp32 -> Wt16 [16,K,C] bf16 (round to nearest even).  One lane per output element.
__global__ __launch_bounds__(256) void weights_to_bf16_transposed_kernel(const float *__restrict__ W,
                                                                         unsigned short *__restrict__ Wt16, int C, int K,
                                                                         unsigned n)
{
    const unsigned idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const unsigned c = idx % C, k = (idx / C) % K, pos = idx / (static_cast<unsigned>(C) * K);
    const float v = round_bf16(W[(static_cast<size_t>(pos) * C + c) * K + k]);
    Wt16[idx] = static_cast<unsigned short>(__float_as_uint(v) >> 16);
}

}  // namespace
}  // namespace swc
