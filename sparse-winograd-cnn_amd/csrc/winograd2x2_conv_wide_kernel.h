// "wide48": the fp32 ring kernel for shapes whose 16-row MFMA tiles do not divide evenly over the SIMDs
// with whole tiles per wave (device code; winograd2x2_conv.hip says what it replaces in the reference).
//
// A workgroup of four waves owns up to 48 rows x 128 columns of the [M,K] plane: each wave 48 x 32 = 3 x 2
// tiles of v_mfma_f32_16x16x4_f32, six tiles per SIMD.  What the row groups leave over (M - groups*48 rows,
// in 16-row tiles) is dealt out one 16x16 tile per workgroup and split four ways along the reduction index:
// every wave multiplies a quarter of each step's channels for that tile (two MFMAs on top of the 48 of its own
// tiles at 32 channels per step), and the four partial sums meet in LDS at the end.  At 28x28x128 -> 128, batch 64,
// that is 6.25 tile units per SIMD where whole tiles need 7.
//
// Output transform.  The 16 products P[r][s] (position 4r+s) enter the four outputs as
//   Y(dy,dx) = sum_r a_dy[r] sum_s a_dx[s] P[r][s],   a_0 = (1,1,1,0), a_1 = (0,1,-1,-1)
// (winograd2x2_conv_cuda.cu.cc:39-46).  Here they are taken in two stages, columns then rows, each as a
// sum/difference pair (x+y, y-x) of the two middle terms with the outer term accumulated onto it by the MFMAs
// themselves: a position either starts its accumulator from zero or continues on a partial sum that is already
// there.  18 vector adds per output element instead of the 36 of the term-by-term form; the association differs
// from the reference's left-to-right sums (its results agree to rounding, 1e-7 relative).  The positions are
// walked in the order this needs (kWidePos), and three of the four output planes are final before the last
// position and are stored while the matrix pipes are still busy.
#pragma once

#include "winograd2x2_conv_kernel.h"

namespace swc {
namespace {

// Position walked q-th, the register set its products accumulate into, and whether that set starts from zero.
// Sets: 0 = A, 1 = B, 2 = C, 3 = D, 4 = E, 5 = F.  Rows r are taken in the order 1, 2, 0, 3 and, within a row,
// s in the order 1, 2, 0, 3: T1 = P[r][1] and T2 = P[r][2] start from zero; (S, U) = (T1 + T2, T2 - T1);
// P[r][0] then accumulates onto a set to which S is added, P[r][3] onto U:
//   ZA_r = P[r][0] + P[r][1] + P[r][2],   NZB_r = P[r][2] + P[r][3] - P[r][1] = -(sum_s a_1[s] P[r][s]).
// The same pairing over the rows gives Y0 = ZA_0 + ZA_1 + ZA_2, -Y2 = ZA_2 + ZA_3 - ZA_1,
// -Y1 = NZB_0 + NZB_1 + NZB_2, Y3 = NZB_2 + NZB_3 - NZB_1.
constexpr int kWidePos[16] = {5, 6, 4, 7, 9, 10, 8, 11, 1, 2, 0, 3, 13, 14, 12, 15};
constexpr int kWideDst[16] = {0, 1, 2, 1, 0, 3, 4, 3, 0, 5, 2, 5, 0, 5, 4, 3};
constexpr bool kWideFresh[16] = {true, true, true, false, true, true, true, false,
                                 true, true, false, false, true, true, false, false};
// Vector work that rides on the first step of the q-th position (its operands were completed by earlier
// positions and none of them is the set that position accumulates into): up to two operations
// {kind, x, y}; kind 1: (x, y) <- (x + y, y - x); kind 2: x <- x + y.
constexpr int kWideOps[16][2][3] = {
    {{0, 0, 0}, {0, 0, 0}},  // q0   P11 -> A
    {{0, 0, 0}, {0, 0, 0}},  // q1   P12 -> B
    {{1, 0, 1}, {0, 0, 0}},  // q2   P10 -> C;        (A, B) = (S_1, U_1)
    {{2, 2, 0}, {0, 0, 0}},  // q3   P13 onto B;      C = ZA_1              (B ends as NZB_1)
    {{0, 0, 0}, {0, 0, 0}},  // q4   P21 -> A
    {{0, 0, 0}, {0, 0, 0}},  // q5   P22 -> D
    {{1, 0, 3}, {0, 0, 0}},  // q6   P20 -> E;        (A, D) = (S_2, U_2)
    {{2, 4, 0}, {0, 0, 0}},  // q7   P23 onto D;      E = ZA_2              (D ends as NZB_2)
    {{1, 2, 4}, {0, 0, 0}},  // q8   P01 -> A;        (C, E) = (ZA_1 + ZA_2, ZA_2 - ZA_1)
    {{1, 1, 3}, {0, 0, 0}},  // q9   P02 -> F;        (B, D) = (NZB_1 + NZB_2, NZB_2 - NZB_1)
    {{1, 0, 5}, {0, 0, 0}},  // q10  P00 onto C;      (A, F) = (S_0, U_0)
    {{2, 2, 0}, {0, 0, 0}},  // q11  P03 onto F;      C = Y0                (F ends as NZB_0)
    {{2, 1, 5}, {0, 0, 0}},  // q12  P31 -> A;        B = -Y1;              plane 0 (C) is stored
    {{0, 0, 0}, {0, 0, 0}},  // q13  P32 -> F;                              plane 1 (B) is stored
    {{1, 0, 5}, {2, 3, 5}},  // q14  P30 onto E;      (A, F) = (S_3, U_3);  D += U_3
    {{2, 4, 0}, {0, 0, 0}},  // q15  P33 onto D;      E = -Y2;              plane 2 (E) is stored; D ends as Y3
};
// Output plane j = 2*dy + dx stored in the first step of the q-th position (-1: none), the set that holds it
// and whether the set holds its negative.
constexpr int kWideStoreAt[16] = {-1, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1, 0, 1, -1, 2};
constexpr int kWidePlaneSet[4] = {2, 1, 4, 3};
constexpr bool kWidePlaneNeg[4] = {false, true, true, false};
constexpr unsigned long long wide_pos_packed()
{
    unsigned long long v = 0;
    for (int q = 0; q < 16; ++q) v |= static_cast<unsigned long long>(kWidePos[q]) << (4 * q);
    return v;
}

// BK channels per step; TN 16-column tiles per wave (the workgroup's tile is 48 rows x 64*TN columns);
// EXTRA: the workgroup also carries a 16x16 tile of the left-over rows; OCC waves per SIMD; EPI: the stores apply
// scale/shift and add a residual (ConvEpilogue).  The ring has NSTAGE slots: two, or four for grids of one workgroup
// per CU, where nothing else hides the latency of a tile that comes from HBM (the copies then run three steps
// ahead instead of one); a position's steps go round the slots a whole number of times, so C % (NSTAGE*BK) == 0.
template <int BK_, int TN_, bool EXTRA_, int OCC_, bool EPI_, int NSTAGE_ = 2>
struct WideCfg {
    static constexpr int BK = BK_, TN = TN_, OCC = OCC_, NSTAGE = NSTAGE_;
    static constexpr bool EXTRA = EXTRA_, EPI = EPI_;
    static constexpr int TM = 3, NT = 256, BM = 16 * TM, BN = 64 * TN;
    static constexpr int AROWS = BM + (EXTRA ? 16 : 0);   // rows of the A tile in LDS
    static constexpr int CH = BK / 4;                     // 16-byte chunks per A row
    static constexpr int A_BYTES = AROWS * BK * 4;
    static constexpr int NAW = AROWS * CH / 64, NBW = BK * BN / 256;  // wave-wide copies (1 KiB) per tile
    static constexpr int NA = (NAW + 3) / 4, NB = NBW / 4, LPS = NA + NB;
    static constexpr int RPC = 256 / BN;                  // B rows per copy
    static constexpr int B_BYTES = BK * BN * 4 + (BK / 4) * 64;  // 64 bytes after every 4 rows: lane groups read rows 4 apart
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES;
    // With two slots a tile is copied one step before its use: less than a trip to HBM takes.  The first step of a
    // position then also touches the next position's A tiles (one 4-byte global -> LDS load per wave into a landing
    // area behind the ring that nobody reads), so that their copies find the lines in L2.
    static constexpr bool TOUCH = NSTAGE == 2;
    static constexpr int TOUCH_BYTES = TOUCH ? 4 * 256 : 0;
    static constexpr int LAUNCH_LDS_BYTES = LDS_BYTES + TOUCH_BYTES;
    static constexpr int KS = BK / 16, KH = KS / 2;       // operand groups of 16 channels per step / per half
    static constexpr int NM = KH * 4 * TM * TN;           // MFMAs of a wave's own tiles per half step
    static constexpr int XK = BK / 4, XM = XK / 4;        // extra tile: channels and MFMAs per wave and step
    static constexpr int XCT = BN / 16;                   // extra tiles per left-over row tile and column group
    static constexpr int NTILE = TM * TN + (EXTRA ? 1 : 0);
    static constexpr int PLANE_OPS = TM * TN * 4;         // store instructions of one output plane
    static constexpr bool EARLY = !EPI;                   // planes are stored as they become final (a residual is read at the end instead)
    static_assert(BK == 32 || BK == 64, "a step is two or four operand groups");
    static_assert(NSTAGE == 2 || NSTAGE == 4, "two or four ring slots");
    static_assert(LAUNCH_LDS_BYTES <= 160 * 1024, "fits a CU");
    static_assert(!TOUCH || BK == 32, "a row of a step's A tile is one 128-byte line");
    static_assert(TN == 1 || TN == 2, "64 or 128 columns");
    static_assert(NBW % 4 == 0, "every wave issues the same number of B copies");
    static_assert(STAGE_BYTES % 256 == 0, "operand reads address a slot through their immediate offsets");
    static_assert(LDS_BYTES >= 4 * 4 * 4 * 64 * 4, "the ring holds the partial sums of the extra tile");
};

constexpr unsigned kWideOutOfRange = 0x80000000u;  // plus any scalar offset used here it stays below 2^32 and beyond every descriptor

// One 16-byte-per-lane global -> LDS copy like async_copy16, with the LDS address given as a scalar plus a
// compile-time constant (one instruction sets M0).
template <int LDS_IMM>
__device__ __forceinline__ void async_copy16_imm(const float *base, unsigned voff, unsigned lds_base)
{
    const size_t b = reinterpret_cast<size_t>(base);
    const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(b));
    const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(b >> 32));
    base = reinterpret_cast<const float *>((static_cast<size_t>(hi) << 32) | lo);
    lds_base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile(
        "s_add_i32 m0, %2, %3\n\t"
        "s_nop 3\n\t"
        "global_load_lds_dwordx4 %0, %1"
        :
        : "v"(voff), "s"(base), "s"(lds_base), "n"(LDS_IMM)
        : "memory", "scc");
}

// The same with 4 bytes per lane: what arrives is never read, the point is the lines it pulls into L2.
__device__ __forceinline__ void async_touch4(const float *base, unsigned voff, unsigned lds_addr)
{
    const size_t b = reinterpret_cast<size_t>(base);
    const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(b));
    const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(b >> 32));
    base = reinterpret_cast<const float *>((static_cast<size_t>(hi) << 32) | lo);
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    asm volatile(
        "s_mov_b32 m0, %2\n\t"
        "s_nop 3\n\t"
        "global_load_lds_dword %0, %1"
        :
        : "v"(voff), "s"(base), "s"(lds_addr)
        : "memory");
}

// Requirements checked by the launcher: C % (2*BK) == 0, K % BN == 0, TI and Wt 16-byte aligned, M*C*4 < 2^32,
// the output below 2^31 bytes.  grid.x = groups * tiles_n; the row groups cover main_rows = min(M, groups *
// rows_per_wg) rows, rows_per_wg <= 48; with EXTRA the rows from main_rows on are the left-over tiles, and row
// group g carries column tile g % XCT (within its columns) of left-over row tile g / XCT if that exists.
template <typename W>
__global__ __launch_bounds__(W::NT) __attribute__((amdgpu_waves_per_eu(W::OCC, W::OCC))) void conv_wide48_kernel(
    const float *__restrict__ TI, const float *__restrict__ Wt, float *__restrict__ Out, unsigned M, int C, int K, int nW,
    unsigned tiles_n, unsigned rows_per_wg, unsigned main_rows, ConvEpilogue ep)
{
    constexpr int BK = W::BK, TM = W::TM, TN = W::TN, BN = W::BN, CH = W::CH;
    constexpr int NA = W::NA, NB = W::NB, LPS = W::LPS, NAW = W::NAW, RPC = W::RPC;
    constexpr int A_BYTES = W::A_BYTES, STAGE_BYTES = W::STAGE_BYTES;
    constexpr int KS = W::KS, KH = W::KH, NM = W::NM, XM = W::XM, XK = W::XK, NTILE = W::NTILE;
    constexpr bool EXTRA = W::EXTRA, EPI = W::EPI;
    extern __shared__ __attribute__((aligned(1024))) unsigned char wsmem[];  // W::LAUNCH_LDS_BYTES

    const unsigned lid = xcd_swizzle(blockIdx.x, gridDim.x);
    const unsigned g = lid / tiles_n;
    const unsigned m0 = g * rows_per_wg;
    const int n0 = static_cast<int>(lid % tiles_n) * BN;
    const unsigned rows_valid = main_rows - m0 < rows_per_wg ? main_rows - m0 : rows_per_wg;
    // left-over tile of this workgroup
    const unsigned xt = g / W::XCT, xc = g % W::XCT;
    const bool has_extra = EXTRA && main_rows + 16 * xt < M;  // the same for the whole workgroup
    const unsigned xrow0 = has_extra ? main_rows + 16 * xt : m0;
    const unsigned xrows_valid = has_extra ? (M - xrow0 < 16 ? M - xrow0 : 16) : 1;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int R = C, N = K;
    // This lane's column of column tile tn, within the workgroup's columns: 64*tn + 16*wave + li.
    const int wcol = 16 * wave + li;

    // ---- copies ---------------------------------------------------------------------------------------
    // A tile: AROWS rows of CH 16-byte chunks, chunk j of row r in slot r*CH + (j ^ (r % CH)); the swizzle is
    // applied on the global side (a lane's LDS destination is fixed to base + 16*lane).  Rows beyond the valid
    // ones re-read the last valid row; what they produce is never stored.
    // B tile: BK rows of BN floats, RPC rows per copy, 64 bytes of padding after every 4 rows.
    unsigned a_voff[NA], b_voff[NB], c_lds[LPS];  // c_lds: LDS byte address of each copy within ring slot 0
    const unsigned smem_base = lds_address(wsmem);
#pragma unroll
    for (int q = 0; q < NA; ++q) {
        const unsigned wl = (q * 4 + wave) % NAW;
        const unsigned slot = wl * 64 + lane;
        const unsigned row = slot / CH;
        const unsigned chunk = (slot % CH) ^ (row % CH);
        unsigned grow;  // relative to m0
        if (row < static_cast<unsigned>(W::BM))
            grow = row < rows_valid ? row : rows_valid - 1;
        else
            grow = xrow0 - m0 + (row - W::BM < xrows_valid ? row - W::BM : xrows_valid - 1);
        a_voff[q] = (grow * static_cast<unsigned>(R) + chunk * 4) * 4u;
        c_lds[q] = smem_base + wl * 1024u;
    }
#pragma unroll
    for (int q = 0; q < NB; ++q) {
        const unsigned wl = q * 4 + wave;
        const unsigned slot = wl * 64 + lane;
        const unsigned krow = slot / (BN / 4);
        const unsigned n = n0 + (slot % (BN / 4)) * 4;
        b_voff[q] = (krow * static_cast<unsigned>(N) + n) * 4u;
        c_lds[NA + q] = smem_base + A_BYTES + wl * 1024u + (RPC * wl / 4) * 64u;
    }
    const int nkc = R / BK;

    // Copy issuer: running pointers to the tiles of the next step to fetch.  Position p: A at TI + (p*M + m0)*R,
    // B at Wt + p*R*N; a step advances A by BK floats and B by BK rows; at the end of a position both jump to the
    // position walked next.  After the last step the walk starts over (the surplus copies land in ring slots
    // nobody reads any more).
    const float *const a_base = TI + static_cast<size_t>(m0) * R;
    const size_t a_plane = static_cast<size_t>(M) * R, b_plane = static_cast<size_t>(R) * N;
    constexpr unsigned long long kPosPacked = wide_pos_packed();
    const float *a_next = a_base + kWidePos[0] * a_plane;
    const float *b_next = Wt + kWidePos[0] * b_plane;
    int kc_next = 0;
    unsigned q_next = 0;
    auto copy = [&](auto stage_tag, int i) __attribute__((always_inline)) {  // the i-th of this thread's LPS copies of a step
        constexpr int imm = decltype(stage_tag)::value * STAGE_BYTES;
        if (i < NA)
            async_copy16_imm<imm>(a_next, a_voff[i < NA ? i : 0], c_lds[i]);
        else
            async_copy16_imm<imm>(b_next, b_voff[i >= NA ? i - NA : 0], c_lds[i]);
    };
    auto advance = [&]() __attribute__((always_inline)) {
        a_next += BK;
        b_next += static_cast<size_t>(BK) * N;
        if (++kc_next == nkc) {
            kc_next = 0;
            q_next = (q_next + 1) & 15u;
            const size_t p = (kPosPacked >> (4 * q_next)) & 15u;
            a_next = a_base + p * a_plane;
            b_next = Wt + p * b_plane;
        }
    };

    // Lines touched ahead (W::TOUCH): the first step of a position touches the next position's A tiles of up to four
    // steps, wave w rows 16w .. 16w+15, one lane per 128-byte line.
    unsigned touch_voff = 0;
    const unsigned touch_lds = smem_base + W::LDS_BYTES + wave * 256u;
    if constexpr (W::TOUCH) {
        const unsigned row = 16u * wave + (lane & 15);
        unsigned grow;
        if (row < static_cast<unsigned>(W::BM))
            grow = row < rows_valid ? row : rows_valid - 1;
        else
            grow = has_extra ? xrow0 - m0 + (row - W::BM < xrows_valid ? row - W::BM : xrows_valid - 1) : rows_valid - 1;
        const unsigned line = static_cast<unsigned>(lane >> 4) < static_cast<unsigned>(nkc) ? lane >> 4 : nkc - 1;
        touch_voff = grow * static_cast<unsigned>(R) * 4u + line * 128u;
    }

    // ---- MFMA operands --------------------------------------------------------------------------------
    // Per group of 16 channels, lane group lg feeds channels 4*lg .. 4*lg+3, one per MFMA: A is one b128 read
    // per 16-row tile and group, B one float per MFMA and 16-column tile (read in pairs).  Every read is a
    // per-lane byte address plus a compile-time offset (ring slot, tile, group).
    struct HalfFrag {
        float4 a[KH][TM];
        float b[KH][4][TN];
    };
    // An LDS read addresses base register + 16-bit immediate: a ring of more than 64 KiB is read through two sets of
    // lane bases, one per half of the ring (NBANK == 2), so that slot, tile and group stay in the immediate.
    constexpr int NBANK = W::LDS_BYTES > 65536 ? 2 : 1, BANK_STAGES = W::NSTAGE / NBANK;
    unsigned a_lane[NBANK][KS];  // A: row li of tile 0, the lane's chunk of group k8
    unsigned b_lane[NBANK], xa_lane[NBANK], xb_lane[NBANK];
    // B row k sits at k*BN*4 + (k/4)*64 bytes; this lane's rows of group k8 are 16*k8 + 4*lg + t.
    // Extra tile: this wave's channels of a step are XK*wave + XM*lg + t, t < XM.
    const int x_ch = XK * wave + XM * lg;
#pragma unroll
    for (int bk = 0; bk < NBANK; ++bk) {
        const unsigned at = bk * BANK_STAGES * STAGE_BYTES;
#pragma unroll
        for (int k8 = 0; k8 < KS; ++k8) a_lane[bk][k8] = at + (li * CH + ((4 * k8 + lg) ^ (li % CH))) * 16u;
        b_lane[bk] = at + A_BYTES + 4u * lg * (BN * 4) + lg * 64u + wcol * 4u;
        xa_lane[bk] = at + (W::BM + li) * (BK * 4) + (((x_ch / 4) ^ (li % CH)) * 16u) + (x_ch % 4) * 4u;
        xb_lane[bk] = at + A_BYTES + x_ch * (BN * 4) + (x_ch / 4) * 64u + (xc * 16u + li) * 4u;
        if (bk > 0) {
            // kept in registers of their own (the compiler would otherwise fold them back into base + constant)
#pragma unroll
            for (int k8 = 0; k8 < KS; ++k8) asm volatile("" : "+v"(a_lane[bk][k8]));
            asm volatile("" : "+v"(b_lane[bk]), "+v"(xa_lane[bk]), "+v"(xb_lane[bk]));
        }
    }
    struct ExtraFrag {
        float a[XM], b[XM];
    };

    constexpr int NUB = 2 * TN, NU = KH * (TM + NUB);
    auto lds_f32 = [&](unsigned byte) __attribute__((always_inline)) { return *reinterpret_cast<const float *>(wsmem + byte); };
    auto read_unit = [&](HalfFrag &F, auto stage_tag, int h, int u) __attribute__((always_inline)) {
        constexpr int bank = decltype(stage_tag)::value / BANK_STAGES;
        constexpr unsigned st = (decltype(stage_tag)::value % BANK_STAGES) * STAGE_BYTES;
        const int k8l = u / (TM + NUB), v = u % (TM + NUB);
        const int k8 = h * KH + k8l;
        if (v < TM) {
            F.a[k8l][v] = *reinterpret_cast<const float4 *>(wsmem + a_lane[bank][k8] + (st + v * 16 * BK * 4));
        } else {
            const int tn = (v - TM) / 2, tp = (v - TM) % 2;
            const unsigned at = st + (16 * k8 + 2 * tp) * (BN * 4) + 4 * k8 * 64 + tn * 256;
            F.b[k8l][2 * tp][tn] = lds_f32(b_lane[bank] + at);
            F.b[k8l][2 * tp + 1][tn] = lds_f32(b_lane[bank] + at + BN * 4);
        }
    };
    constexpr int NXU = EXTRA ? 1 + XM / 2 : 0;
    auto read_extra = [&](ExtraFrag &X, auto stage_tag, int u) __attribute__((always_inline)) {
        constexpr int bank = decltype(stage_tag)::value / BANK_STAGES;
        constexpr unsigned st = (decltype(stage_tag)::value % BANK_STAGES) * STAGE_BYTES;
        if (u == 0) {
            if constexpr (XM == 2) {
                const float2 v = *reinterpret_cast<const float2 *>(wsmem + xa_lane[bank] + st);
                X.a[0] = v.x;
                X.a[1] = v.y;
            } else {
                const float4 v = *reinterpret_cast<const float4 *>(wsmem + xa_lane[bank] + st);
                X.a[0] = v.x;
                X.a[1] = v.y;
                X.a[2 % XM] = v.z;
                X.a[3 % XM] = v.w;
            }
        } else {
            const int t = 2 * (u - 1);
            X.b[t] = lds_f32(xb_lane[bank] + st + t * (BN * 4));
            X.b[t + 1] = lds_f32(xb_lane[bank] + st + (t + 1) * (BN * 4));
        }
    };

    // ---- output addressing ------------------------------------------------------------------------------
    // Tile row m = (b*nH + th)*nW + tw -> pixel (2th + dy, 2tw + dx) of image b (winograd2x2_conv_cuda.cu.cc:48-51).
    // Register r of lane (lg, li) holds row 4*lg + r, column li of a 16x16 tile.  A store is one buffer
    // instruction: per-lane byte offset of pixel (2th, 2tw) at this lane's column (or out of range, which the
    // hardware drops, for rows that are not this workgroup's), scalar offset for plane and column tile.
    const unsigned oW = 2u * static_cast<unsigned>(nW);
    const unsigned row_stride = oW * static_cast<unsigned>(K);  // floats
    const unsigned out_bytes = static_cast<unsigned>(M) * 4u * static_cast<unsigned>(K) * 4u;
    const __amdgpu_buffer_rsrc_t out_rsrc = make_rsrc(Out, out_bytes);
    const __amdgpu_buffer_rsrc_t res_rsrc = make_rsrc(ep.residual, EPI && ep.residual != nullptr ? out_bytes : 0u);
    auto pixel_offset = [&](unsigned gm, unsigned col) {  // bytes
        const unsigned bt = gm / static_cast<unsigned>(nW);
        const unsigned tw = gm - bt * static_cast<unsigned>(nW);
        return ((bt * 2u * oW + 2u * tw) * static_cast<unsigned>(K) + col) * 4u;
    };
    unsigned out_voff[TM][4];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const unsigned row = tm * 16 + 4 * lg + r;
            out_voff[tm][r] = row < rows_valid ? pixel_offset(m0 + row, n0 + wcol) : kWideOutOfRange;
        }
    float sc[TN], sh[TN];
    if constexpr (EPI) {
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const int col = n0 + 64 * tn + wcol;
            sc[tn] = ep.scale != nullptr ? ep.scale[col] : 1.f;
            sh[tn] = ep.shift != nullptr ? ep.shift[col] : 0.f;
        }
    }
    const bool res_relu = EPI && ep.residual_relu != 0;
    auto plane_soff = [&](int j) { return ((j / 2) * row_stride + (j % 2) * static_cast<unsigned>(K)) * 4u; };
    // value v of plane j (negated where the set holds the negative), with the epilogue applied
    auto finish_value = [&](float v, bool neg, float scale, float shift, float q) __attribute__((always_inline)) {
        if (neg) v = -v;
        if constexpr (EPI) {
            v = __builtin_fmaf(v, scale, shift);
            if (res_relu) q = q > 0.f ? q : 0.f;
            v += q;
        }
        return v;
    };

    floatx4 S[6][NTILE];
    const floatx4 zero4 = {};

    // Store tile e (= tm*TN + tn) of plane j from its set; q: the residual values to add (EPI).
    auto load_residual = [&](int j, int e, float (&q)[4]) __attribute__((always_inline)) {
        const int tm = e / TN, tn = e % TN;
        const unsigned soff = plane_soff(j) + tn * 256u;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            q[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(res_rsrc, out_voff[tm][r], soff, 0));
    };
    auto store_tile = [&](int j, int e, const float (&q)[4]) __attribute__((always_inline)) {
        const int tm = e / TN, tn = e % TN;
        const unsigned soff = plane_soff(j) + tn * 256u;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float v = finish_value(S[kWidePlaneSet[j]][e][r], kWidePlaneNeg[j], EPI ? sc[tn] : 1.f, EPI ? sh[tn] : 0.f, q[r]);
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), out_rsrc, out_voff[tm][r], soff, 16 /* sc1: written through */);
        }
    };
    const float no_residual[4] = {0.f, 0.f, 0.f, 0.f};

    using Stage0 = std::integral_constant<int, 0>;
    constexpr int NSTAGE = W::NSTAGE;
    // ---- prologue: fill the ring, wait for step 0, read its first half -------------------------------------
    static_for<NSTAGE>([&](auto s_tag) {
#pragma unroll
        for (int c = 0; c < LPS; ++c) copy(s_tag, c);
        advance();
    });
    wait_vmcnt<(NSTAGE - 1) * LPS>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    HalfFrag F1, F2;
    ExtraFrag FX;
#pragma unroll
    for (int u = 0; u < NU; ++u) read_unit(F1, Stage0{}, 0, u);

    // One step of the q-th position walked, on ring slot `stage`.  first: the position's first step (accumulators
    // start from zero where the schedule says so; the vector work and the stores of the schedule ride along).
    // after_first: the step before was the position's first (its line touch is still outstanding behind its copies).
    auto step = [&](auto q_tag, auto first_tag, auto stage_tag, auto after_first_tag) __attribute__((always_inline)) {
        constexpr int q = decltype(q_tag)::value;
        constexpr bool first = decltype(first_tag)::value;
        constexpr int NTOUCH = W::TOUCH && decltype(after_first_tag)::value ? 1 : 0;
        using Other = std::integral_constant<int, (decltype(stage_tag)::value + 1) % NSTAGE>;   // the next step's slot
        constexpr int dst = kWideDst[q];
        constexpr bool fresh = first && kWideFresh[q];
        constexpr int store_plane = first && W::EARLY ? kWideStoreAt[q] : -1;
        constexpr int n_ops = first ? (kWideOps[q][0][0] != 0) + (kWideOps[q][1][0] != 0) : 0;
        constexpr int n_ride = n_ops * NTILE;
        // Slots (MFMA indices 0 .. 2*NM-1 of the step) after which the ride units go: over the whole step, or
        // over the first quarter when the step also stores (the stores follow in the second quarter: all memory
        // operations other than the copies stay in the first half, where the waits can count them).
        constexpr int ride_span = store_plane >= 0 ? NM / 2 : 2 * NM;
        auto mfma_slot = [&](const HalfFrag &F, int i, bool from_zero) __attribute__((always_inline)) {
            const int tn = i % TN, tm = (i / TN) % TM, t = (i / (TN * TM)) % 4, k8l = i / (TN * TM * 4);
            const float4 a4 = F.a[k8l][tm];
            const float av = t == 0 ? a4.x : t == 1 ? a4.y : t == 2 ? a4.z : a4.w;
            const int e = tm * TN + tn;
            S[dst][e] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, F.b[k8l][t][tn], from_zero ? zero4 : S[dst][e], 0, 0, 0);
        };
        auto ride_unit = [&](int u) __attribute__((always_inline)) {
            const int o = u / NTILE, e = u % NTILE;
            const int kind = kWideOps[q][o][0], x = kWideOps[q][o][1], y = kWideOps[q][o][2];
            if (kind == 1) {
                const floatx4 s = S[x][e] + S[y][e], d = S[y][e] - S[x][e];
                S[x][e] = s;
                S[y][e] = d;
                asm volatile("" : "+v"(S[x][e]), "+v"(S[y][e]));
            } else {
                S[x][e] += S[y][e];
                asm volatile("" : "+v"(S[x][e]));
            }
        };
        auto ride_slot = [](int u) { return u * ride_span / (n_ride > 0 ? n_ride : 1); };
        auto store_slot = [](int e) { return NM / 2 + e * (NM / 2) / (TM * TN); };
        auto copy_slot = [](int c) { return 1 + c * (NM - 1) / LPS; };
        auto read_slot = [](int u) { return 1 + u * (NM - 1) / NU; };
        static_for<NM>([&](auto i_tag) __attribute__((always_inline)) {
            constexpr int i = decltype(i_tag)::value;
            mfma_slot(F1, i, fresh && i < TM * TN);
#pragma unroll
            for (int u = 0; u < NU; ++u)
                if (u * NM / NU == i) read_unit(F2, stage_tag, 1, u);
            if constexpr (EXTRA && i == NM / 2) {
                if (has_extra) {
#pragma unroll
                    for (int u = 0; u < NXU; ++u) read_extra(FX, stage_tag, u);
                }
            }
#pragma unroll
            for (int u = 0; u < n_ride; ++u)
                if (ride_slot(u) == i) ride_unit(u);
            if constexpr (store_plane >= 0) {
#pragma unroll
                for (int e = 0; e < TM * TN; ++e)
                    if (store_slot(e) == i) store_tile(store_plane, e, no_residual);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        static_for<NM>([&](auto i_tag) __attribute__((always_inline)) {
            constexpr int i = decltype(i_tag)::value;
            mfma_slot(F2, i, false);
            if (i == 0) {
                // The tile of the next step is complete once nothing but what was issued after its copies is
                // outstanding: the copies of the steps behind it in the ring, the line touch of the step before and
                // the stores (and residual loads) of this step's first half.  Memory operations complete in issue order.
                constexpr int mine = (NSTAGE - 2) * LPS + NTOUCH + (store_plane >= 0 ? W::PLANE_OPS : 0);
                wait_vmcnt<(mine < 63 ? mine : 63)>();
                __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS reads of this step are done
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            }
#pragma unroll
            for (int c = 0; c < LPS; ++c)
                if (copy_slot(c) == i) copy(stage_tag, c);
            if constexpr (W::TOUCH && first && i == NM - 1)  // behind the step's last copy
                async_touch4(a_base + kWidePos[(q + 1) & 15] * a_plane, touch_voff, touch_lds);
#pragma unroll
            for (int u = 0; u < NU; ++u)
                if (read_slot(u) == i) read_unit(F1, Other{}, 0, u);
#pragma unroll
            for (int u = 0; u < n_ride; ++u)
                if (ride_slot(u) == NM + i) ride_unit(u);
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (EXTRA) {
            if (has_extra) {
#pragma unroll
                for (int t = 0; t < XM; ++t)
                    S[dst][NTILE - 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(FX.a[t], FX.b[t], fresh && t == 0 ? zero4 : S[dst][NTILE - 1], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        advance();
    };

    // Steps go round the ring slots; a position has a multiple of NSTAGE steps, so it starts on slot 0.
    static_for<16>([&](auto q_tag) {
        step(q_tag, std::true_type{}, Stage0{}, std::false_type{});
        static_for<NSTAGE - 1>([&](auto s_tag) {
            step(q_tag, std::false_type{}, std::integral_constant<int, decltype(s_tag)::value + 1>{}, std::bool_constant<decltype(s_tag)::value == 0>{});
        });
        for (int kc = NSTAGE; kc < nkc; kc += NSTAGE)
            static_for<NSTAGE>([&](auto s_tag) { step(q_tag, std::false_type{}, s_tag, std::false_type{}); });
    });

    // The surplus copies must have landed before this workgroup's LDS can be handed on.
    wait_vmcnt<0>();

    // What has not been stored yet: plane 3, or all four.  With a residual, the values of a plane are read in one
    // sweep before its first store and one plane ahead (loads and stores complete in issue order, so a load issued
    // behind a store would wait for it).
    constexpr int first_plane = W::EARLY ? 3 : 0;
    if constexpr (EPI) {
        float q[2][TM * TN][4];
#pragma unroll
        for (int e = 0; e < TM * TN; ++e) load_residual(first_plane, e, q[first_plane & 1][e]);
#pragma unroll
        for (int j = first_plane; j < 4; ++j) {
            if (j + 1 < 4) {
#pragma unroll
                for (int e = 0; e < TM * TN; ++e) load_residual(j + 1, e, q[(j + 1) & 1][e]);
            }
#pragma unroll
            for (int e = 0; e < TM * TN; ++e) store_tile(j, e, q[j & 1][e]);
        }
    } else {
#pragma unroll
        for (int j = first_plane; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < TM * TN; ++e) store_tile(j, e, no_residual);
    }

    if constexpr (EXTRA) {
        if (has_extra) {
            // The four waves' partial sums of the extra tile meet in LDS, [plane][wave][register][lane] (the ring
            // is idle by now); wave j adds them in wave order and stores plane j.
            float *const xch = reinterpret_cast<float *>(wsmem);
            __builtin_amdgcn_s_waitcnt(0xc07f);
            __builtin_amdgcn_s_barrier();
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) xch[((j * 4 + wave) * 4 + r) * 64 + lane] = S[kWidePlaneSet[j]][NTILE - 1][r];
            __syncthreads();
            const int j = wave;
            const bool neg = j == 1 || j == 2;
            const int col = n0 + static_cast<int>(xc) * 16 + li;
            float xs = 1.f, xh = 0.f;
            if constexpr (EPI) {
                xs = ep.scale != nullptr ? ep.scale[col] : 1.f;
                xh = ep.shift != nullptr ? ep.shift[col] : 0.f;
            }
            const unsigned soff = plane_soff(j);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const unsigned row = 4 * lg + r;
                const unsigned voff = row < xrows_valid ? pixel_offset(xrow0 + row, col) : kWideOutOfRange;
                float v = xch[((j * 4 + 0) * 4 + r) * 64 + lane];
                v += xch[((j * 4 + 1) * 4 + r) * 64 + lane];
                v += xch[((j * 4 + 2) * 4 + r) * 64 + lane];
                v += xch[((j * 4 + 3) * 4 + r) * 64 + lane];
                float q = 0.f;
                if constexpr (EPI) q = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(res_rsrc, voff, soff, 0));
                v = finish_value(v, neg, xs, xh, q);
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), out_rsrc, voff, soff, 16);
            }
        }
    }
}

}  // namespace
}  // namespace swc
