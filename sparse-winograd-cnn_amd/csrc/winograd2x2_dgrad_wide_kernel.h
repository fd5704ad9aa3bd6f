// Data gradient of the Winograd convolution on 48-row x 128-column workgroups (device code):
// dTI_i [M,C] = dP_i [M,K] . W_i^T for the 16 positions i, the first GEMM of the reference's backward pass
// (winograd2x2_conv_grad_cuda.cu.cc:103-108), W [16,C,K] as the forward pass holds it.
//
// The tiling of the forward wide48 kernel (winograd2x2_conv_wide_kernel.h) without its output transform: a
// workgroup of four waves owns up to 48 rows x 128 columns of every plane and walks the 16 positions; each wave
// 48 x 32 = 3 x 2 tiles of v_mfma_f32_16x16x4_f32.  Both operands have the reduction index (K) as their fast axis,
// so both LDS tiles are rows of 32 floats (128 bytes, eight 16-byte chunks, chunk j of row r in slot j ^ (r % 8))
// and every MFMA operand group is one ds_read_b128.  A position's finished product tiles are stored while the next
// position's first step runs.  The ring has two slots, so a step's slot is a compile-time constant (steps come in
// pairs: K % 64 == 0); the copies a wave issues for a tile are 1 KiB apart in LDS and share one M0 value through
// the instruction's immediate offset, which moves source and destination alike.
//
// The 16 products are independent of each other here, so the rows that whole rounds of 48-row groups leave over
// are dealt out by position: one more workgroup per (left-over row group, column group, position), a sixteenth as
// long as the others and resident beside them (two workgroups fit a CU).
//
// The MFMA takes the weight tile as its first operand, so that a lane's four accumulator registers are four
// consecutive output columns of one row: a product tile is stored with one 16-byte store per lane.
#pragma once

#include "winograd2x2_conv_wide_kernel.h"

namespace swc {
namespace {

struct WideDgradCfg {
    static constexpr int BK = 32, TM = 3, TN = 2, NT = 256, BM = 48, BN = 128, CH = 8, OCC = 2;
    static constexpr int A_BYTES = BM * BK * 4, B_BYTES = BN * BK * 4, STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
    static constexpr int NA = 2, NB = 4, LPS = NA + NB;   // copies per wave and step (A: six wave-copies over three waves, the fourth repeats)
    static constexpr int NM = 4 * TM * TN;                // MFMAs per half step (one group of 16 reduction indices)
    static constexpr int TILE_STORES = TM * TN;           // store instructions of one position's product tiles per wave
};

template <int M0_IMM>
__device__ __forceinline__ void lds_copy_pair(unsigned v0, unsigned v1, const float *base, unsigned m0_base)
{
    asm volatile(
        "s_add_i32 m0, %3, %4\n\t"
        "s_nop 3\n\t"
        "global_load_lds_dwordx4 %0, %2\n\t"
        "global_load_lds_dwordx4 %1, %2 offset:1024"
        :
        : "v"(v0), "v"(v1), "s"(base), "s"(m0_base), "n"(M0_IMM)
        : "memory", "scc");
}
template <int M0_IMM>
__device__ __forceinline__ void lds_copy_quad(unsigned v0, unsigned v1, unsigned v2, unsigned v3, const float *base, unsigned m0_base)
{
    asm volatile(
        "s_add_i32 m0, %5, %6\n\t"
        "s_nop 3\n\t"
        "global_load_lds_dwordx4 %0, %4\n\t"
        "global_load_lds_dwordx4 %1, %4 offset:1024\n\t"
        "global_load_lds_dwordx4 %2, %4 offset:2048\n\t"
        "global_load_lds_dwordx4 %3, %4 offset:3072"
        :
        : "v"(v0), "v"(v1), "v"(v2), "v"(v3), "s"(base), "s"(m0_base), "n"(M0_IMM)
        : "memory", "scc");
}

// Requirements checked by the launcher: K % 64 == 0, C % 128 == 0, dP, W and dTI 16-byte aligned, M*max(C,K)*4 < 2^31.
// The first n_main = groups * (C / 128) workgroups walk all 16 positions of row group g (rows g*rows_per_wg ..,
// rows_per_wg <= 48; together main_rows = min(M, groups * rows_per_wg) rows).  The others take one position each of
// the 48-row groups from main_rows on: id - n_main = ((row group) * tiles_n + column group) * 16 + position.
__global__ __launch_bounds__(WideDgradCfg::NT) __attribute__((amdgpu_waves_per_eu(WideDgradCfg::OCC, WideDgradCfg::OCC))) void
conv_dgrad_wide_kernel(const float *__restrict__ dP, const float *__restrict__ Wt, float *__restrict__ dTI, unsigned M, int C, int K,
                       unsigned tiles_n, unsigned rows_per_wg, unsigned main_rows, unsigned n_main)
{
    using W = WideDgradCfg;
    constexpr int BK = W::BK, TM = W::TM, TN = W::TN, NA = W::NA, NB = W::NB, LPS = W::LPS, NM = W::NM;
    constexpr int A_BYTES = W::A_BYTES, STAGE_BYTES = W::STAGE_BYTES;
    extern __shared__ __attribute__((aligned(1024))) unsigned char dsmem[];  // W::LDS_BYTES

    const bool whole = blockIdx.x < n_main;   // walks all 16 positions
    const unsigned lid = whole ? xcd_swizzle(blockIdx.x, n_main) : blockIdx.x - n_main;
    const unsigned tile = whole ? lid : lid / 16;
    const unsigned pos0 = whole ? 0 : lid % 16;
    const unsigned m0 = whole ? (tile / tiles_n) * rows_per_wg : main_rows + (tile / tiles_n) * W::BM;
    const unsigned n0 = (tile % tiles_n) * W::BN;
    const unsigned rows_end = whole ? main_rows : M;
    const unsigned rows_cap = whole ? rows_per_wg : static_cast<unsigned>(W::BM);
    const unsigned rows_valid = rows_end - m0 < rows_cap ? rows_end - m0 : rows_cap;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const unsigned R = static_cast<unsigned>(K), N = static_cast<unsigned>(C);
    const int nkc = K / BK;

    // ---- copies ---------------------------------------------------------------------------------------------
    // Wave-copy wl of a tile covers its rows 8*wl .. 8*wl+7.  A: waves 0-2 take wave-copies 2w and 2w+1, wave 3
    // repeats wave 0's (every wave issues the same number, so that all count outstanding copies alike).
    // B: wave w takes 4w .. 4w+3.  Copy i of a run carries the immediate offset i*1024, so its per-lane offset is
    // biased by -(i*1024) against a tile pointer biased by +3072 the other way.
    constexpr unsigned kBias = 3072;
    const unsigned wa = wave < 3 ? wave : 0;
    unsigned a_voff[NA], b_voff[NB];
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        const unsigned row = 8 * (2 * wa + i) + lane / 8, chunk = (lane % 8) ^ (row % 8);
        const unsigned r = row < rows_valid ? row : rows_valid - 1;
        a_voff[i] = (r * R + chunk * 4) * 4u + kBias - i * 1024u;
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const unsigned row = 8 * (4 * wave + i) + lane / 8, chunk = (lane % 8) ^ (row % 8);
        b_voff[i] = (row * R + chunk * 4) * 4u + kBias - i * 1024u;   // row: output column n0 + row (C % 128 == 0: valid)
    }
    const unsigned smem_base = lds_address(dsmem);
    const unsigned a_m0 = smem_base + wa * 2048u, b_m0 = smem_base + A_BYTES + wave * 4096u;
    // Tile of (position p, chunk kc): A at dP + (p*M + m0)*K + kc*BK, B at W + (p*C + n0)*K + kc*BK.
    const float *const a_first =
        reinterpret_cast<const float *>(reinterpret_cast<const char *>(dP + (static_cast<size_t>(pos0) * M + m0) * R) - kBias);
    const float *const b_first =
        reinterpret_cast<const float *>(reinterpret_cast<const char *>(Wt + (static_cast<size_t>(pos0) * N + n0) * R) - kBias);
    const size_t a_jump = static_cast<size_t>(M) * R - static_cast<size_t>(nkc - 1) * BK;   // last chunk of a position -> first of the next
    const size_t b_jump = static_cast<size_t>(N) * R - static_cast<size_t>(nkc - 1) * BK;
    const float *a_next = a_first, *b_next = b_first;
    int kc_left = nkc, steps_left = (whole ? 16 : 1) * nkc;
    auto copies = [&](auto slot_tag) __attribute__((always_inline)) {
        constexpr int at = decltype(slot_tag)::value * STAGE_BYTES;
        lds_copy_pair<at>(a_voff[0], a_voff[1], a_next, a_m0);
        lds_copy_quad<at>(b_voff[0], b_voff[1], b_voff[2], b_voff[3], b_next, b_m0);
    };
    // After the last step the walk starts over: the surplus copies land in ring slots nobody reads any more.
    auto advance = [&]() __attribute__((always_inline)) {
        const bool last_chunk = --kc_left == 0;
        kc_left = last_chunk ? nkc : kc_left;
        a_next += last_chunk ? a_jump : static_cast<size_t>(BK);
        b_next += last_chunk ? b_jump : static_cast<size_t>(BK);
        if (--steps_left == 0) {
            a_next = a_first;
            b_next = b_first;
        }
    };

    // ---- MFMA operands: per group of 16 reduction indices lane group lg feeds indices 4*lg .. 4*lg+3, one per MFMA,
    // on both sides: one b128 read per 16-row (16-column) tile.  This lane's column of column tile tn is
    // 64*tn + 16*wave + li.
    unsigned a_lane[2], b_lane[2];
#pragma unroll
    for (int k8 = 0; k8 < 2; ++k8) {
        a_lane[k8] = (li * 8 + ((4 * k8 + lg) ^ (li % 8))) * 16u;
        b_lane[k8] = A_BYTES + ((16 * wave + li) * 8 + ((4 * k8 + lg) ^ (li % 8))) * 16u;
    }
    struct HalfFrag {
        float4 a[TM], b[TN];
    };
    auto read_half = [&](HalfFrag &F, auto slot_tag, int k8, int u) __attribute__((always_inline)) {  // unit u of TM + TN
        constexpr unsigned st = decltype(slot_tag)::value * STAGE_BYTES;
        if (u < TM)
            F.a[u] = *reinterpret_cast<const float4 *>(dsmem + a_lane[k8] + (st + u * 16 * 128));
        else
            F.b[u - TM] = *reinterpret_cast<const float4 *>(dsmem + b_lane[k8] + (st + (u - TM) * 64 * 128));
    };
    constexpr int NU = TM + TN;

    // ---- stores: plane p of dTI [16][M][C].  The weight tile is the MFMA's first operand, so register r of lane
    // (lg, li) holds column 4*lg + r of row li of a 16x16 tile: one 16-byte store per lane and tile.  A descriptor over
    // this workgroup's rows of the plane drops the rows that are not its own.
    unsigned out_voff[TM];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) out_voff[tm] = ((tm * 16 + li) * N + n0 + 16 * wave + 4 * lg) * 4u;
    float *const out_tile = dTI + (static_cast<size_t>(pos0) * M + m0) * N;
    const size_t out_plane = static_cast<size_t>(M) * N;
    const unsigned out_tile_bytes = rows_valid * N * 4u;

    floatx4 P[2][TM * TN];
    const floatx4 zero4 = {};
    auto store_tile = [&](int buf, int pos, int e) __attribute__((always_inline)) {
        const int tm = e / TN, tn = e % TN;
        const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(out_tile + pos * out_plane, out_tile_bytes);
        const floatx4 v = P[buf][e];
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(intx4, v), rsrc, out_voff[tm], tn * 256, 16 /* sc1: written through */);
    };

    using Slot0 = std::integral_constant<int, 0>;
    using Slot1 = std::integral_constant<int, 1>;
    copies(Slot0{});
    advance();
    copies(Slot1{});
    advance();
    wait_vmcnt<LPS>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    HalfFrag F1, F2;
#pragma unroll
    for (int u = 0; u < NU; ++u) read_half(F1, Slot0{}, 0, u);

    // One step of position pos on ring slot `slot`; first: its first step (the accumulators start from zero and the
    // stores of position pos-1 ride along in the first half, where the wait can count them).
    auto step = [&](auto pos_tag, auto first_tag, auto slot, auto other) __attribute__((always_inline)) {
        constexpr int pos = decltype(pos_tag)::value;
        constexpr bool first = decltype(first_tag)::value;
        constexpr bool stores = first && pos > 0;
        auto mfma_slot = [&](const HalfFrag &F, int i, bool from_zero) __attribute__((always_inline)) {
            const int tn = i % TN, tm = (i / TN) % TM, t = i / (TN * TM);
            const float4 a4 = F.a[tm], b4 = F.b[tn];
            const float av = t == 0 ? a4.x : t == 1 ? a4.y : t == 2 ? a4.z : a4.w;
            const float bv = t == 0 ? b4.x : t == 1 ? b4.y : t == 2 ? b4.z : b4.w;
            const int e = tm * TN + tn;
            P[pos & 1][e] = __builtin_amdgcn_mfma_f32_16x16x4f32(bv, av, from_zero ? zero4 : P[pos & 1][e], 0, 0, 0);
        };
        static_for<NM>([&](auto i_tag) __attribute__((always_inline)) {
            constexpr int i = decltype(i_tag)::value;
            mfma_slot(F1, i, first && i < TM * TN);
#pragma unroll
            for (int u = 0; u < NU; ++u)
                if (u * NM / NU == i) read_half(F2, slot, 1, u);
            if constexpr (stores) {
#pragma unroll
                for (int e = 0; e < TM * TN; ++e)
                    if (e * NM / (TM * TN) == i) store_tile((pos & 1) ^ 1, pos - 1, e);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        static_for<NM>([&](auto i_tag) __attribute__((always_inline)) {
            constexpr int i = decltype(i_tag)::value;
            mfma_slot(F2, i, false);
            if constexpr (i == 0) {
                // The next step's tile has landed once only what was issued after its copies is outstanding: this
                // step's product stores.  Memory operations complete in issue order.
                wait_vmcnt<(stores ? W::TILE_STORES : 0)>();
                __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS reads of this step are done
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            }
            if constexpr (i == 1) copies(slot);
#pragma unroll
            for (int u = 0; u < NU; ++u)
                if (2 + u * (NM - 2) / NU == i) read_half(F1, other, 0, u);
            __builtin_amdgcn_sched_barrier(0);
        });
        advance();
    };

    // Steps alternate between the two ring slots; a position has an even number of steps, so it starts on slot 0.
    auto position = [&](auto pos_tag) __attribute__((always_inline)) {
        step(pos_tag, std::true_type{}, Slot0{}, Slot1{});
        step(pos_tag, std::false_type{}, Slot1{}, Slot0{});
        for (int kc = 2; kc < nkc; kc += 2) {
            step(pos_tag, std::false_type{}, Slot0{}, Slot1{});
            step(pos_tag, std::false_type{}, Slot1{}, Slot0{});
        }
    };
    position(std::integral_constant<int, 0>{});   // relative to pos0
    if (whole) {
        static_for<15>([&](auto p_tag) { position(std::integral_constant<int, decltype(p_tag)::value + 1>{}); });
        wait_vmcnt<0>();  // the surplus copies must have landed before this workgroup's LDS can be handed on
#pragma unroll
        for (int e = 0; e < TM * TN; ++e) store_tile(1, 15, e);
    } else {
        wait_vmcnt<0>();
#pragma unroll
        for (int e = 0; e < TM * TN; ++e) store_tile(0, 0, e);
    }
}

}  // namespace
}  // namespace swc
