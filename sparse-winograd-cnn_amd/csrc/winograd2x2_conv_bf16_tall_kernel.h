// "stored-tall": the bf16-stored convolution for layers of 64, 128, 256 or 512 channels (device code).  Same contract as
// conv_bf16_stored_kernel (winograd2x2_conv_bf16_kernel.h): TI as bf16 [16,M,C], weights as bf16 [16,K,C], fp32
// accumulation, fp32 output transform and output.
//
// conv_bf16_stored_kernel is bound by instruction issue on those layers: per 64-channel step a wave issues four
// MFMAs (128 cycles of matrix work) among some sixty other instructions.  Here a workgroup of four waves owns
// 128 rows x 64 columns, each wave 64 x 32 = two v_mfma_f32_32x32x16_bf16 tiles, so a step is eight MFMAs per wave
// for the same number of copies per byte and three operand reads per two MFMAs; and what is not an MFMA is cut down:
//   * the channel count per position is a template parameter, so position, step and ring slot of every step are
//     compile-time constants: operand reads and copy destinations are a per-lane (per-wave) base plus an
//     immediate, with no address arithmetic in the loop;
//   * the output transform is taken as in the wide48 kernel (winograd2x2_conv_wide_kernel.h): sum/difference
//     pairs with partial sums continued by the MFMAs, 18 vector adds per element instead of 36, spread over the
//     steps of a position; three of the four output planes are stored before the last position.
// The ring has three slots (two tiles in flight: a step is far shorter than the memory latency).
#pragma once

#include "winograd2x2_conv_wide_kernel.h"

namespace swc {
namespace {

// Four (two) 16-byte-per-lane global -> LDS copies whose destinations are 1 KiB apart, with one M0 value: the
// immediate offset of the instruction moves source and destination alike, so copy i reads base + v_i + OFF + i*1024
// and writes LDS byte m0_base + M0_IMM + OFF + i*1024 + 16*lane.  base and m0_base must be wave-uniform.
template <int M0_IMM, int OFF>
__device__ __forceinline__ void lds_copy_run4(unsigned v0, unsigned v1, unsigned v2, unsigned v3, const char *base, unsigned m0_base)
{
    static_assert(OFF >= 0 && OFF + 3 * 1024 < 4096, "13-bit immediate offset");
    asm volatile(
        "s_add_i32 m0, %5, %6\n\t"
        "s_nop 3\n\t"
        "global_load_lds_dwordx4 %0, %4 offset:%7\n\t"
        "global_load_lds_dwordx4 %1, %4 offset:%8\n\t"
        "global_load_lds_dwordx4 %2, %4 offset:%9\n\t"
        "global_load_lds_dwordx4 %3, %4 offset:%10"
        :
        : "v"(v0), "v"(v1), "v"(v2), "v"(v3), "s"(base), "s"(m0_base), "n"(M0_IMM), "n"(OFF), "n"(OFF + 1024), "n"(OFF + 2048),
          "n"(OFF + 3072)
        : "memory", "scc");
}
template <int M0_IMM, int OFF>
__device__ __forceinline__ void lds_copy_run2(unsigned v0, unsigned v1, const char *base, unsigned m0_base)
{
    static_assert(OFF >= 0 && OFF + 1024 < 4096, "13-bit immediate offset");
    asm volatile(
        "s_add_i32 m0, %3, %4\n\t"
        "s_nop 3\n\t"
        "global_load_lds_dwordx4 %0, %2 offset:%5\n\t"
        "global_load_lds_dwordx4 %1, %2 offset:%6"
        :
        : "v"(v0), "v"(v1), "s"(base), "s"(m0_base), "n"(M0_IMM), "n"(OFF), "n"(OFF + 1024)
        : "memory", "scc");
}

// NKC 64-channel steps per position (C = 64*NKC), OCC waves per SIMD, EPI: scale/shift/residual in the stores.
// SPREAD: the 16 positions of a tile are dealt over four workgroups, one per row r of the 4x4 position grid; each
// writes the two partial sums Z_r(dx) = sum_s a_dx[s] P[r][s] of its tile as planes [r][dx][M][K] of a scratch buffer,
// and spread_combine_kernel takes Y(dy,dx) = sum_r a_dy[r] Z_r(dx) from there.  For layers with too few tiles for the
// CUs: a quarter of the bytes per workgroup through LDS, and every byte of the operands fetched by one XCD only.
template <int NKC_, int OCC_, bool EPI_, bool SPREAD_ = false>
struct TallCfg {
    static constexpr int NKC = NKC_, OCC = OCC_, NSTAGE = 3;
    static constexpr bool EPI = EPI_, EARLY = !EPI_, SPREAD = SPREAD_;
    static constexpr int NQ = SPREAD ? 4 : 16;           // positions a workgroup walks
    static_assert(!SPREAD || !EPI, "the epilogue of a spread launch is applied by the combining kernel");
    static constexpr int BM = 128, BN = 64, BK = 64, NT = 256, TM = 2;
    static constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2, STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int RING_BYTES = NSTAGE * STAGE_BYTES;
    static constexpr int RING_AT = 1024;                 // the ring starts behind the row offsets (BM * 4 bytes)
    static constexpr int LDS_BYTES = RING_AT + RING_BYTES;
    static constexpr int NA = A_BYTES / 1024 / 4, NB = B_BYTES / 1024 / 4, LPS = NA + NB;  // copies per wave and step
    static constexpr int PLANE_STORES = TM * 16;          // store instructions of one output plane per wave
    // A position that stores a plane does its vector work in its first steps and the stores in its last ones; a
    // position of a single step in the first half of the step and in the second.
    static constexpr int STORE_STEPS = NKC >= 2 ? NKC / 2 : 1;
    static constexpr int STORES_PER_STEP = PLANE_STORES / STORE_STEPS;
    static_assert(NKC == 1 || NKC == 2 || NKC == 4 || NKC == 8, "64, 128, 256 or 512 channels");
    static_assert(BM * 4 <= RING_AT && (NKC - 1) * 128 <= RING_AT, "the copies' M0 values stay non-negative");
    static_assert((NA - 1) * 1024 + (NKC - 1) * 128 < 4096, "immediate offsets of the copies");
    static_assert(LPS + STORES_PER_STEP < 64, "vmcnt range");
    static_assert(STORES_PER_STEP % 4 == 0, "stores go out in groups of four rows");
};

// Requirements checked by the launcher: C == 64*NKC, K % 64 == 0, TI16 and Wt16 16-byte aligned, M*C*2 < 2^32, the
// output below 2^31 bytes.  grid.x = ceil(M / rows_per_wg) * (K / 64), rows_per_wg <= 128; with SPREAD four times
// that (workgroup lid takes row lid / (grid.x / 4) of the position grid) and Out is the scratch buffer, 8*M*K floats.
template <typename T>
__global__ __launch_bounds__(T::NT) __attribute__((amdgpu_waves_per_eu(T::OCC, T::OCC))) void conv_bf16_tall_kernel(
    const unsigned short *__restrict__ TI16, const unsigned short *__restrict__ Wt16, float *__restrict__ Out, unsigned M,
    int K, int nW, unsigned tiles_n, unsigned rows_per_wg, ConvEpilogue ep)
{
    constexpr int NKC = T::NKC, NSTAGE = T::NSTAGE, TM = T::TM, LPS = T::LPS, NA = T::NA, NB = T::NB;
    constexpr int A_BYTES = T::A_BYTES, STAGE_BYTES = T::STAGE_BYTES, C = 64 * NKC;
    constexpr bool EPI = T::EPI;
    extern __shared__ __attribute__((aligned(1024))) unsigned char tsmem[];  // T::LDS_BYTES

    const unsigned lid_all = xcd_swizzle(blockIdx.x, gridDim.x);
    const unsigned tiles_all = T::SPREAD ? gridDim.x / 4 : gridDim.x;
    const unsigned grid_row = T::SPREAD ? lid_all / tiles_all : 0;  // r: this workgroup's positions are 4r .. 4r+3
    const unsigned lid = T::SPREAD ? lid_all % tiles_all : lid_all;
    const unsigned m0 = (lid / tiles_n) * rows_per_wg;
    const unsigned n0 = (lid % tiles_n) * T::BN;
    const unsigned rows_valid = M - m0 < rows_per_wg ? M - m0 : rows_per_wg;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lg = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- copies: wave-copy wl of a tile covers its rows 8*wl .. 8*wl+7 (1 KiB); chunk c (8 channels) of row r sits
    // in slot c ^ ((r/2) % 8).  Rows beyond the valid ones re-read the last valid row (never stored).
    // The immediate offset of a global->LDS load moves its source and its destination alike, so the copies of a
    // tile that a wave issues in a step (wave-copies wave*NA + i, 1 KiB apart in LDS) share one M0 value: copy i
    // carries the immediate i*1024 + kc*128, its per-lane offset is biased by -(i*1024) (against a tile pointer that
    // is biased the other way, so that it stays non-negative), and M0 by -(kc*128): the pointers move only from
    // position to position.
    constexpr unsigned kBias = (NA - 1) * 1024;
    unsigned a_voff[NA], b_voff[NB];
    const unsigned smem_base = lds_address(tsmem) + T::RING_AT;
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        const unsigned row = 8 * (wave * NA + i) + lane / 8, chunk = (lane % 8) ^ ((row / 2) % 8);
        const unsigned r = row < rows_valid ? row : rows_valid - 1;
        a_voff[i] = (r * static_cast<unsigned>(C) + chunk * 8) * 2u + kBias - i * 1024u;
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const unsigned row = 8 * (wave * NB + i) + lane / 8, chunk = (lane % 8) ^ ((row / 2) % 8);
        b_voff[i] = (row * static_cast<unsigned>(C) + chunk * 8) * 2u + kBias - i * 1024u;
    }
    const unsigned a_m0 = smem_base + wave * (NA * 1024u), b_m0 = smem_base + A_BYTES + wave * (NB * 1024u);
    const char *const a_base = reinterpret_cast<const char *>(TI16 + static_cast<size_t>(m0) * C) - kBias;
    const char *const b_base = reinterpret_cast<const char *>(Wt16 + static_cast<size_t>(n0) * C) - kBias;
    const size_t a_plane = static_cast<size_t>(M) * C * 2, b_plane = static_cast<size_t>(K) * C * 2;  // bytes
    const char *a_ptr = a_base, *b_ptr = b_base;  // tiles of the position whose copies are being issued
    auto scalar_ptr = [](const char *ptr) __attribute__((always_inline)) {
        const size_t b = reinterpret_cast<size_t>(ptr);
        const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(b));
        const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(b >> 32));
        return reinterpret_cast<const char *>((static_cast<size_t>(hi) << 32) | lo);
    };
    // The copies of global step si (position walked (si / NKC) % NQ, chunk si % NKC) into ring slot si % NSTAGE.
    // Past the last step the walk starts over: the surplus copies land in ring slots nobody reads any more.
    // A spread workgroup walks the columns of its grid row in the order of the walk's first row (1, 2, 0, 3).
    auto set_issue_position = [&](auto si_tag) __attribute__((always_inline)) {
        constexpr int si = decltype(si_tag)::value;
        if constexpr (si % NKC == 0) {
            constexpr size_t walked = kWidePos[(si / NKC) % T::NQ];
            const size_t pos = T::SPREAD ? 4 * grid_row + (walked & 3) : walked;
            a_ptr = scalar_ptr(a_base + pos * a_plane);
            b_ptr = scalar_ptr(b_base + pos * b_plane);
        }
    };
    auto copy_a = [&](auto si_tag) __attribute__((always_inline)) {
        constexpr int si = decltype(si_tag)::value, kc = si % NKC, at = (si % NSTAGE) * STAGE_BYTES;
        static_assert(NA == 4, "four copies of the activation tile per wave");
        lds_copy_run4<at - kc * 128, kc * 128>(a_voff[0], a_voff[1], a_voff[2], a_voff[3], a_ptr, a_m0);
    };
    auto copy_b = [&](auto si_tag) __attribute__((always_inline)) {
        constexpr int si = decltype(si_tag)::value, kc = si % NKC, at = (si % NSTAGE) * STAGE_BYTES;
        static_assert(NB == 2, "two copies of the weight tile per wave");
        lds_copy_run2<at - kc * 128, kc * 128>(b_voff[0], b_voff[1], b_ptr, b_m0);
    };

    // ---- MFMA operands: lane (li, lg) of group h (16 channels) holds channels 16*h + 8*lg .. +7 of its row: one
    // ds_read_b128 per 32-row tile.  The chunk's slot is (2h + lg) ^ ((row/2) % 8) = ((lg ^ (li/2) % 8)) ^ 2h.
    unsigned a_lane[4], b_lane[4];
#pragma unroll
    for (int h = 0; h < 4; ++h) {
        const unsigned slot = (2 * h + lg) ^ ((li / 2) % 8);
        a_lane[h] = T::RING_AT + (64 * wm + li) * 128u + slot * 16u;
        b_lane[h] = T::RING_AT + A_BYTES + (32 * wn + li) * 128u + slot * 16u;
    }
    struct Frag {
        bf16x8 a[TM], b;
    };
    auto read_group = [&](Frag &F, auto slot_tag, int h) __attribute__((always_inline)) {
        constexpr unsigned st = decltype(slot_tag)::value * STAGE_BYTES;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) F.a[tm] = *reinterpret_cast<const bf16x8 *>(tsmem + a_lane[h] + (st + tm * 32 * 128));
        F.b = *reinterpret_cast<const bf16x8 *>(tsmem + b_lane[h] + st);
    };

    // ---- output addressing: tile row m = (b*nH + th)*nW + tw -> pixel (2th + dy, 2tw + dx) of image b
    // (winograd2x2_conv_cuda.cu.cc:48-51).  The byte offset of every row's pixel (2th, 2tw), channel 0 (or out of
    // range, which the hardware drops, for rows that are not this workgroup's) is kept in LDS in front of the ring;
    // register r of lane (lg, li) holds row 8*(r/4) + 4*lg + r%4, column li of a 32x32 tile.
    const unsigned oW = 2u * static_cast<unsigned>(nW);
    const unsigned row_stride = oW * static_cast<unsigned>(K);  // floats
    const unsigned out_bytes = M * 4u * static_cast<unsigned>(K) * 4u;
    // spread: the two planes [grid_row][0..1][M][K] of the scratch buffer, rows addressed by tile row
    const unsigned part_plane_bytes = M * static_cast<unsigned>(K) * 4u;
    const __amdgpu_buffer_rsrc_t out_rsrc = T::SPREAD ? make_rsrc(Out + static_cast<size_t>(2 * grid_row) * M * K, 2 * part_plane_bytes)
                                                      : make_rsrc(Out, out_bytes);
    const __amdgpu_buffer_rsrc_t res_rsrc = make_rsrc(ep.residual, EPI && ep.residual != nullptr ? out_bytes : 0u);
    unsigned *const rowoff = reinterpret_cast<unsigned *>(tsmem);
    if (tid < T::BM) {
        const unsigned gm = m0 + tid;
        const unsigned bt = gm / static_cast<unsigned>(nW);
        const unsigned tw = gm - bt * static_cast<unsigned>(nW);
        if constexpr (T::SPREAD)
            rowoff[tid] = static_cast<unsigned>(tid) < rows_valid ? gm * static_cast<unsigned>(K) * 4u : kWideOutOfRange;
        else
            rowoff[tid] = static_cast<unsigned>(tid) < rows_valid ? (bt * 2u * oW + 2u * tw) * static_cast<unsigned>(K) * 4u : kWideOutOfRange;
    }
    const unsigned col = n0 + 32 * wn + li;
    const unsigned col_bytes = col * 4u;
    float sc = 1.f, sh = 0.f;
    if constexpr (EPI) {
        sc = ep.scale != nullptr ? ep.scale[col] : 1.f;
        sh = ep.shift != nullptr ? ep.shift[col] : 0.f;
    }
    const bool res_relu = EPI && ep.residual_relu != 0;
    auto plane_soff = [&](int j) { return ((j / 2) * row_stride + (j % 2) * static_cast<unsigned>(K)) * 4u; };

    floatx16 S[6][TM];
    const floatx16 zero16 = {};

    // Rows 4*v .. 4*v+3 of this lane in tile tm: their four pixel offsets.
    auto quarter_offsets = [&](int tm, int v) __attribute__((always_inline)) {
        return *reinterpret_cast<const uint4 *>(rowoff + 64 * wm + 32 * tm + 8 * v + 4 * lg);
    };
    // Store registers 4*v .. 4*v+3 of tile tm of plane j (q: residual values, EPI).
    auto store_quarter = [&](int j, int tm, int v, const float (&q)[4]) __attribute__((always_inline)) {
        const uint4 ro = quarter_offsets(tm, v);
        const unsigned soff = plane_soff(j);
        const unsigned off[4] = {ro.x, ro.y, ro.z, ro.w};
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float val = S[kWidePlaneSet[j]][tm][4 * v + r];
            if (kWidePlaneNeg[j]) val = -val;
            if constexpr (EPI) {
                val = __builtin_fmaf(val, sc, sh);
                float qq = q[r];
                if (res_relu) qq = qq > 0.f ? qq : 0.f;
                val += qq;
            }
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, val), out_rsrc, off[r] + col_bytes, soff, 16 /* sc1: written through */);
        }
    };
    auto load_residual_quarter = [&](int j, int tm, int v, float (&q)[4]) __attribute__((always_inline)) {
        const uint4 ro = quarter_offsets(tm, v);
        const unsigned soff = plane_soff(j);
        const unsigned off[4] = {ro.x, ro.y, ro.z, ro.w};
#pragma unroll
        for (int r = 0; r < 4; ++r)
            q[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(res_rsrc, off[r] + col_bytes, soff, 0));
    };
    const float no_residual[4] = {0.f, 0.f, 0.f, 0.f};

    // ---- prologue: fill the ring, wait for step 0, read its first two operand groups ---------------------------
    static_for<NSTAGE>([&](auto s_tag) {
        set_issue_position(s_tag);
        copy_a(s_tag);
        copy_b(s_tag);
    });
    wait_vmcnt<(NSTAGE - 1) * LPS>();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // the row offsets are written
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    Frag F[3];
    read_group(F[0], std::integral_constant<int, 0>{}, 0);
    read_group(F[1], std::integral_constant<int, 0>{}, 1);

    // Vector work of the q-th position in micro-units of four registers of one tile: unit u = (operation, tile,
    // quarter).  Kind 1: (x, y) <- (x + y, y - x); kind 2: x <- x + y (kWideOps).
    auto ride_unit = [&](auto q_tag, int u) __attribute__((always_inline)) {
        constexpr int q = decltype(q_tag)::value;
        const int o = u / (TM * 4), e = (u / 4) % TM, v = u % 4;
        const int kind = kWideOps[q][o][0], x = kWideOps[q][o][1], y = kWideOps[q][o][2];
#pragma unroll
        for (int r = 4 * v; r < 4 * v + 4; ++r) {
            if (kind == 1) {
                const float s = S[x][e][r] + S[y][e][r], d = S[y][e][r] - S[x][e][r];
                S[x][e][r] = s;
                S[y][e][r] = d;
            } else {
                S[x][e][r] += S[y][e][r];
            }
        }
        if (kind == 1)
            asm volatile("" : "+v"(S[x][e]), "+v"(S[y][e]));
        else
            asm volatile("" : "+v"(S[x][e]));
    };

    // One step: position q (in walking order), its kc-th 64-channel chunk.
    auto step = [&](auto q_tag, auto kc_tag) __attribute__((always_inline)) {
        constexpr int q = decltype(q_tag)::value, kc = decltype(kc_tag)::value;
        constexpr int s = q * NKC + kc;                         // global step index
        using Slot = std::integral_constant<int, s % NSTAGE>;   // this step's ring slot: the copies of step s+3 refill it
        using Next = std::integral_constant<int, (s + 1) % NSTAGE>;
        constexpr int dst = kWideDst[q];
        constexpr bool fresh = kc == 0 && kWideFresh[q];
        constexpr int store_plane = T::EARLY ? kWideStoreAt[q] : -1;
        constexpr int n_ops = (kWideOps[q][0][0] != 0) + (kWideOps[q][1][0] != 0);
        constexpr int n_units = n_ops * TM * 4;
        // MFMA slots of the position over which the vector work is spread: all of them, or those of the steps
        // before the ones that store (of the half step before the half that stores).
        constexpr bool one_step = NKC == 1;
        constexpr int ride_slots = store_plane < 0 ? NKC * 4 * TM : one_step ? 2 * TM : (NKC - T::STORE_STEPS) * 4 * TM;
        constexpr bool stores_here = store_plane >= 0 && kc >= NKC - T::STORE_STEPS;
        // Operations issued after the copies of the tile waited for (the next step's) and before the wait: the
        // copies of the step after it, and stores.  With several steps per position: those of the previous step and of
        // this one.  With one step per position a step stores in its second half: the last quarter of the step two back
        // (issued behind that step's copies), all of the previous step, half of this one.
        auto stores_at = [](int qq) constexpr { return T::EARLY && qq >= 0 && kWideStoreAt[qq >= 0 ? qq : 0] >= 0; };
        constexpr int prev_q = kc > 0 ? q : q - 1, prev_kc = kc > 0 ? kc - 1 : NKC - 1;
        constexpr bool stores_before = stores_at(prev_q) && prev_kc >= NKC - T::STORE_STEPS;
        constexpr int younger_stores =
            one_step ? (stores_at(q - 2) ? T::STORES_PER_STEP / 4 : 0) + (stores_at(q - 1) ? T::STORES_PER_STEP : 0) +
                           (stores_here ? T::STORES_PER_STEP / 2 : 0)
                     : (stores_before ? T::STORES_PER_STEP : 0) + (stores_here ? T::STORES_PER_STEP : 0);
        // The step's eight MFMAs, group h = i / 2, tile tm = i % 2; what else a wave has to issue goes between them.
        static_for<4 * TM>([&](auto i_tag) __attribute__((always_inline)) {
            constexpr int i = decltype(i_tag)::value, h = i / TM, tm = i % TM;
            constexpr int G = 4 * s + h;  // global operand-group index: its registers are F[G % 3]
            S[dst][tm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[G % 3].a[tm], F[G % 3].b, fresh && h == 0 ? zero16 : S[dst][tm], 0, 0, 0);
            constexpr int slot_in_pos = kc * 4 * TM + i;
#pragma unroll
            for (int u = 0; u < n_units; ++u)
                if (ride_slots > 0 && u * ride_slots / (n_units > 0 ? n_units : 1) == slot_in_pos) ride_unit(q_tag, u);
            if constexpr (stores_here && (one_step ? h >= 2 : h < 2)) {
                // this step's share of the plane's 8 quarters (TM tiles x 4), dealt over its first four slots (over
                // its last four when the position is this one step and the vector work fills the first four)
                constexpr int quarters_per_step = T::STORES_PER_STEP / 4;
                constexpr int first_quarter = (kc - (NKC - T::STORE_STEPS)) * quarters_per_step;
                constexpr int i_store = one_step ? i - 2 * TM : i;
#pragma unroll
                for (int w = 0; w < quarters_per_step; ++w)
                    if (w * 4 / quarters_per_step == i_store) {
                        const int qu = first_quarter + w;
                        store_quarter(store_plane, qu / 4, qu % 4, no_residual);
                    }
            }
            if constexpr (tm == TM - 1) {
                if constexpr (h == 2) {
                    // The next step's tile has landed once only what was issued after its copies is outstanding:
                    // the copies of the step after it and the stores of the previous step and of this one.
                    constexpr int n = LPS + younger_stores;
                    wait_vmcnt<(n < 63 ? n : 63)>();  // the counter's range; waiting for fewer outstanding operations is always safe
                    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS reads of this step are done
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                }
                // operands two groups ahead
                if constexpr (h < 2)
                    read_group(F[(G + 2) % 3], Slot{}, h + 2);
                else
                    read_group(F[(G + 2) % 3], Next{}, h - 2);
            }
            // this wave's copies of the tile NSTAGE steps ahead, behind the barrier
            if constexpr (i == 5) {
                set_issue_position(std::integral_constant<int, s + NSTAGE>{});
                copy_a(std::integral_constant<int, s + NSTAGE>{});
            }
            if constexpr (i == 6) copy_b(std::integral_constant<int, s + NSTAGE>{});
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    static_for<T::NQ>([&](auto q_tag) { static_for<NKC>([&](auto kc_tag) { step(q_tag, kc_tag); }); });

    // The surplus copies must have landed before this workgroup's LDS can be handed on.
    wait_vmcnt<0>();

    if constexpr (T::SPREAD) {
        // After the four positions of a grid row set 2 holds P[r][0] + P[r][1] + P[r][2] = Z_r(0) and set 1
        // P[r][2] + P[r][3] - P[r][1] = -Z_r(1) (kWideOps, q = 0 .. 3).
#pragma unroll
        for (int dx = 0; dx < 2; ++dx)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const uint4 ro = quarter_offsets(tm, v);
                    const unsigned off[4] = {ro.x, ro.y, ro.z, ro.w};
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float val = dx == 0 ? S[2][tm][4 * v + r] : -S[1][tm][4 * v + r];
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, val), out_rsrc, off[r] + col_bytes, dx * part_plane_bytes, 16);
                    }
                }
        return;
    }

    // What has not been stored yet: plane 3, or all four.  With a residual, the values of a plane are read in one
    // sweep before its stores and one plane ahead (loads and stores complete in issue order).
    constexpr int first_plane = T::EARLY ? 3 : 0;
    if constexpr (EPI) {
        float q[2][TM * 4][4];
#pragma unroll
        for (int i = 0; i < TM * 4; ++i) load_residual_quarter(first_plane, i / 4, i % 4, q[first_plane & 1][i]);
#pragma unroll
        for (int j = first_plane; j < 4; ++j) {
            if (j + 1 < 4) {
#pragma unroll
                for (int i = 0; i < TM * 4; ++i) load_residual_quarter(j + 1, i / 4, i % 4, q[(j + 1) & 1][i]);
            }
#pragma unroll
            for (int i = 0; i < TM * 4; ++i) store_quarter(j, i / 4, i % 4, q[j & 1][i]);
        }
    } else {
#pragma unroll
        for (int j = first_plane; j < 4; ++j)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int v = 0; v < 4; ++v) store_quarter(j, tm, v, no_residual);
    }
}

}  // namespace
}  // namespace swc
