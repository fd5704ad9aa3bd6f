// The fused GEMM + output-transform kernel of the Winograd convolution (device code).
// See winograd2x2_conv.hip for what it replaces in the reference.
#pragma once

#include <type_traits>

#include "swc_common.h"

namespace swc {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// Calls f(std::integral_constant<int, 0>{}) ... f(std::integral_constant<int, N-1>{}) in order: a loop
// whose index is a compile-time constant in every iteration.
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

// Signs of A^T (x) A^T: bit (4*i + j) set when +-P_i enters Y_j, j = 2*dy + dx.
// Row i = 4r+s contributes AT[dy][r]*AT[dx][s] with AT = [[1,1,1,0],[0,1,-1,-1]]
// (the sums at winograd2x2_conv_cuda.cu.cc:39-46).
constexpr int kAT[2][4] = {{1, 1, 1, 0}, {0, 1, -1, -1}};
constexpr unsigned long long sign_mask(int want)
{
    unsigned long long m = 0;
    for (int i = 0; i < 16; ++i)
        for (int j = 0; j < 4; ++j)
            if (kAT[j / 2][i / 4] * kAT[j % 2][i % 4] == want) m |= 1ull << (4 * i + j);
    return m;
}
constexpr unsigned long long kPlus = sign_mask(1);
constexpr unsigned long long kMinus = sign_mask(-1);

// Round an fp32 value to the nearest bf16 (ties to even) and return it widened back to fp32.
__device__ __forceinline__ float round_bf16(float x)
{
    unsigned u = __float_as_uint(x);
    if ((u & 0x7f800000u) == 0x7f800000u) return x;  // inf / nan pass through
    u += 0x7fffu + ((u >> 16) & 1u);
    return __uint_as_float(u & 0xffff0000u);
}

__device__ __forceinline__ float4 round_bf16(float4 v)
{
    return make_float4(round_bf16(v.x), round_bf16(v.y), round_bf16(v.z), round_bf16(v.w));
}

// Buffer descriptor over [base, base+bytes): loads through it return 0 beyond the end.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, unsigned bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, static_cast<int>(bytes), 0x00020000);
}

__device__ __forceinline__ float4 buffer_load_f4(__amdgpu_buffer_rsrc_t r, unsigned byte_offset)
{
    return __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(r, static_cast<int>(byte_offset), 0, 0));
}

constexpr unsigned kOutOfRange = 0xfffffff0u;  // a byte offset no descriptor here reaches

// MF selects the MFMA shape of the asynchronous kernel: 32 = v_mfma_f32_32x32x2_f32 (16 accumulator
// registers per tile), 16 = v_mfma_f32_16x16x4_f32 (4 registers per tile, 16-row granularity).
template <int BM_, int BN_, int BK_, int WGM_, int WGN_, int OCC_ = 2, int MF_ = 32, int BPAD_ = -1>
struct ConvCfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_, MF = MF_;
    static constexpr int OCC = OCC_;                     // waves per SIMD the register budget allows
    static constexpr int NT = WGM * WGN * 64;            // threads per workgroup
    static constexpr int WM = BM / WGM, WN = BN / WGN;   // wave tile
    static constexpr int TM = WM / MF, TN = WN / MF;     // MFMA tiles per wave
    static constexpr int LG = 64 / MF;                   // lane groups: each feeds 4 reduction indices per operand read
    static constexpr int KG = 4 * LG;                    // reduction indices per operand group (4 MFMAs)
    static constexpr int REGS = MF * MF / 64;            // accumulator registers per tile
    // Asynchronous kernel: floats of padding after every 4 rows (1 KiB) of the B tile in LDS.
    static constexpr int BPAD = BPAD_ >= 0 ? BPAD_ : (MF == 16 ? 16 : 0);
    static constexpr int LDA = BK + 4;  // synchronous kernel: row stride (floats), 4*odd keeps b128 row reads conflict-free
    static constexpr int LDB = BN + 4;
    static constexpr int NA = BM * BK / (4 * NT);        // synchronous kernel: float4 per thread per A tile
    static constexpr int NB = BK * BN / (4 * NT);
    static_assert(MF == 32 || MF == 16, "MFMA tile is 32x32 or 16x16");
    static_assert(WM % MF == 0 && WN % MF == 0, "wave tile is made of whole MFMA tiles");
    static_assert(BK % KG == 0, "a step is a whole number of operand groups");
};

template <typename Cfg>
using AccT = typename std::conditional<Cfg::MF == 32, floatx16, floatx4>::type;

// Optional per-element work folded into the output stores: out = fmaf(y, scale[k], shift[k]) + residual,
// or + max(residual, 0) with residual_relu (the `relu` that an identity shortcut applies to the unit's input,
// ResNet-18-var/imagenet-resnet-transWino-prune.py:135-143, without a pass of its own).
// scale and shift go together; either part may be absent (null).  All null: plain stores.
struct ConvEpilogue {
    const float *scale = nullptr;     // [K]
    const float *shift = nullptr;     // [K]
    const float *residual = nullptr;  // [B,2nH,2nW,K], the output's layout
    int residual_relu = 0;
};

// Output values are written once and not read again by the kernel that writes them.  A plain store leaves
// them as dirty lines in the XCD's L2 (up to 32 MB over the chip), which the write-back that ends every
// kernel then has to drain before the next kernel starts; a relaxed agent-scope store (sc1) is written
// through to the memory side as it is issued, so the kernel ends with nothing to drain (conv3: 2.9 us less
// per launch), and the values still reach the Infinity Cache for the kernel that reads them next (a
// nontemporal store saves the same drain but makes the consumer slower).
__device__ __forceinline__ void store_streaming(float *p, float v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Scatter of the four output tiles: tile row m = (b*nH + th)*nW + tw -> pixels (2th+dy, 2tw+dx)
// of image b (winograd2x2_conv_cuda.cu.cc:48-51).  Accumulator register r of lane (lg, li) holds
// column li and row 8*(r/4) + 4*lg + r%4 of a 32x32 tile, row 4*lg + r of a 16x16 tile.  Only the
// first rows_valid rows of the workgroup's tile are stored.  M < 2^31 (checked by the launcher),
// so tile-row arithmetic fits 32 bits.
template <typename Cfg>
__device__ __forceinline__ void store_output(const AccT<Cfg> (&Y)[4][Cfg::TM][Cfg::TN], float *__restrict__ Out,
                                             unsigned rows_valid, int K, int nW, size_t m0, int n0, int wm0, int wn0,
                                             int li, int lg, const ConvEpilogue ep = ConvEpilogue())
{
    constexpr int TM = Cfg::TM, TN = Cfg::TN, MF = Cfg::MF;
    const bool affine = ep.scale != nullptr, residual = ep.residual != nullptr;  // uniform over the grid
    const size_t oW = 2 * static_cast<size_t>(nW);
    const size_t row_stride = oW * K;
    const unsigned m032 = static_cast<unsigned>(m0);
    // fn(tm, r, tn, element offset of the tile's top-left pixel in this lane's column) for every valid value
    auto for_each_value = [&](auto fn) __attribute__((always_inline)) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
            for (int r = 0; r < Cfg::REGS; ++r) {
                const unsigned row = wm0 + tm * MF + (MF == 32 ? 8 * (r / 4) + 4 * lg + (r % 4) : 4 * lg + r);
                if (row >= rows_valid) continue;
                const unsigned gm = m032 + row;
                const unsigned bt = gm / static_cast<unsigned>(nW);  // b*nH + th
                const unsigned tw = gm - bt * static_cast<unsigned>(nW);
                const size_t pix = (static_cast<size_t>(bt) * 2 * oW + 2 * tw) * K;
#pragma unroll
                for (int tn = 0; tn < TN; ++tn) {
                    const int col = n0 + wn0 + tn * MF + li;
                    if (col >= K) continue;
                    fn(tm, r, tn, pix + col);
                }
            }
        }
    };
    auto finish = [&](int tm, int r, int tn, size_t at, float q0, float q1, float q2, float q3) __attribute__((always_inline)) {
        float y0 = Y[0][tm][tn][r], y1 = Y[1][tm][tn][r], y2 = Y[2][tm][tn][r], y3 = Y[3][tm][tn][r];
        if (affine) {
            const int col = n0 + wn0 + tn * MF + li;
            const float sc = ep.scale[col], sh = ep.shift[col];
            y0 = __builtin_fmaf(y0, sc, sh);
            y1 = __builtin_fmaf(y1, sc, sh);
            y2 = __builtin_fmaf(y2, sc, sh);
            y3 = __builtin_fmaf(y3, sc, sh);
        }
        float *o = Out + at;
        store_streaming(o, y0 + q0);
        store_streaming(o + K, y1 + q1);
        store_streaming(o + row_stride, y2 + q2);
        store_streaming(o + row_stride + K, y3 + q3);
    };
    if (!residual) {
        for_each_value([&](int tm, int r, int tn, size_t at) __attribute__((always_inline)) {
            float y0 = Y[0][tm][tn][r], y1 = Y[1][tm][tn][r], y2 = Y[2][tm][tn][r], y3 = Y[3][tm][tn][r];
            if (affine) {
                const int col = n0 + wn0 + tn * MF + li;
                const float sc = ep.scale[col], sh = ep.shift[col];
                y0 = __builtin_fmaf(y0, sc, sh);
                y1 = __builtin_fmaf(y1, sc, sh);
                y2 = __builtin_fmaf(y2, sc, sh);
                y3 = __builtin_fmaf(y3, sc, sh);
            }
            float *o = Out + at;
            store_streaming(o, y0);
            store_streaming(o + K, y1);
            store_streaming(o + row_stride, y2);
            store_streaming(o + row_stride + K, y3);
        });
        return;
    }
    // The residual is read in one sweep before the first store: loads and stores complete in issue
    // order, so a load issued behind a store also waits for that store, and interleaving them would
    // cost one memory round trip per group of values instead of one per tile.
    float q[4][TM][Cfg::REGS][TN];
    for_each_value([&](int tm, int r, int tn, size_t at) __attribute__((always_inline)) {
        const float *src = ep.residual + at;
        q[0][tm][r][tn] = src[0];
        q[1][tm][r][tn] = src[K];
        q[2][tm][r][tn] = src[row_stride];
        q[3][tm][r][tn] = src[row_stride + K];
    });
    if (ep.residual_relu) {  // uniform over the grid
        for_each_value([&](int tm, int r, int tn, size_t) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < 4; ++j) q[j][tm][r][tn] = q[j][tm][r][tn] > 0.f ? q[j][tm][r][tn] : 0.f;
        });
    }
    for_each_value([&](int tm, int r, int tn, size_t at) __attribute__((always_inline)) {
        finish(tm, r, tn, at, q[0][tm][r][tn], q[1][tm][r][tn], q[2][tm][r][tn], q[3][tm][r][tn]);
    });
}

// FAST: C and K are multiples of 4, TI and Wt 16-byte aligned, and a tile's rows fit 32-bit
//       byte offsets: global loads go through buffer descriptors, 16 bytes per lane, with the
//       ragged edges (rows beyond M, channels beyond C, columns beyond K) returned as zeros by
//       the descriptor's range check instead of by branches.
//       Otherwise: scalar, individually guarded loads (any C, K and alignment).
// BF16: both operands are rounded to bf16 on their way into LDS.
template <typename Cfg, bool FAST, bool BF16>
__global__ __launch_bounds__(Cfg::NT) __attribute__((amdgpu_waves_per_eu(Cfg::OCC, Cfg::OCC))) void conv_mfma_kernel(
    const float *__restrict__ TI, const float *__restrict__ Wt, float *__restrict__ Out, size_t M, int C, int K, int nH,
    int nW, unsigned tiles_n, ConvEpilogue ep)
{
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, NT = Cfg::NT;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, LDA = Cfg::LDA, LDB = Cfg::LDB, NA = Cfg::NA, NB = Cfg::NB;
    constexpr int KS = BK / 8;
    static_assert(Cfg::MF == 32, "the register-staged kernel is written for 32x32 MFMA tiles");
    static_assert(BM * BK % (4 * NT) == 0 && BK * BN % (4 * NT) == 0, "tile loads divide evenly");

    __shared__ __attribute__((aligned(16))) float As[2][BM * LDA];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB];

    const unsigned lid = xcd_swizzle(blockIdx.x, gridDim.x);
    const size_t m0 = static_cast<size_t>(lid / tiles_n) * BM;
    const int n0 = static_cast<int>(lid % tiles_n) * BN;
    const unsigned rows_valid = static_cast<unsigned>(M - m0 < BM ? M - m0 : BM);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lg = lane >> 5;
    const int wm0 = (wave / Cfg::WGN) * Cfg::WM, wn0 = (wave % Cfg::WGN) * Cfg::WN;

    // Per-thread constants of the tile loads: element f = tid + q*NT of a tile.
    unsigned a_voff[NA], b_voff[NB];  // byte offsets within the tile's descriptor (FAST)
    int a_cl[NA];                     // channel within the BK chunk
#pragma unroll
    for (int q = 0; q < NA; ++q) {
        const int f = tid + q * NT;
        a_cl[q] = (f % (BK / 4)) * 4;
        a_voff[q] = (static_cast<unsigned>(f / (BK / 4)) * C + a_cl[q]) * 4u;
    }
#pragma unroll
    for (int q = 0; q < NB; ++q) {
        const int f = tid + q * NT;
        const int n = n0 + (f % (BN / 4)) * 4;
        b_voff[q] = n < K ? (static_cast<unsigned>(f / (BN / 4)) * K + n) * 4u : kOutOfRange;
    }

    float4 ra[NA], rb[NB];

    // Fetch the tiles of (position pos, channels c0 .. c0+BK) into registers.
    auto load_global = [&](int pos, int c0) {
        if (FAST) {
            // Descriptors start at the tile's first element of this chunk and end with the tile's
            // last valid row (A) / the last channel row (B), so rows past either read as zero.
            const float *a_base = TI + (static_cast<size_t>(pos) * M + m0) * C + c0;
            const float *b_base = Wt + (static_cast<size_t>(pos) * C + c0) * K;
            const __amdgpu_buffer_rsrc_t ra_desc = make_rsrc(a_base, (rows_valid * static_cast<unsigned>(C) - c0) * 4u);
            const __amdgpu_buffer_rsrc_t rb_desc = make_rsrc(b_base, static_cast<unsigned>(C - c0) * K * 4u);
#pragma unroll
            for (int q = 0; q < NA; ++q)
                ra[q] = buffer_load_f4(ra_desc, c0 + a_cl[q] < C ? a_voff[q] : kOutOfRange);
#pragma unroll
            for (int q = 0; q < NB; ++q) rb[q] = buffer_load_f4(rb_desc, b_voff[q]);
        } else {
            const float *a_base = TI + static_cast<size_t>(pos) * M * C;
            const float *b_base = Wt + static_cast<size_t>(pos) * C * K;
#pragma unroll
            for (int q = 0; q < NA; ++q) {
                const int f = tid + q * NT;
                const int c = c0 + a_cl[q];
                const size_t gm = m0 + f / (BK / 4);
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (gm < M) {
                    const float *p = a_base + gm * C + c;
                    if (c + 0 < C) v.x = p[0];
                    if (c + 1 < C) v.y = p[1];
                    if (c + 2 < C) v.z = p[2];
                    if (c + 3 < C) v.w = p[3];
                }
                ra[q] = v;
            }
#pragma unroll
            for (int q = 0; q < NB; ++q) {
                const int f = tid + q * NT;
                const int n = n0 + (f % (BN / 4)) * 4;
                const int c = c0 + f / (BN / 4);
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (c < C) {
                    const float *p = b_base + static_cast<size_t>(c) * K + n;
                    if (n + 0 < K) v.x = p[0];
                    if (n + 1 < K) v.y = p[1];
                    if (n + 2 < K) v.z = p[2];
                    if (n + 3 < K) v.w = p[3];
                }
                rb[q] = v;
            }
        }
    };

    auto store_lds = [&](int buf) {
#pragma unroll
        for (int q = 0; q < NA; ++q) {
            const int f = tid + q * NT;
            *reinterpret_cast<float4 *>(&As[buf][(f / (BK / 4)) * LDA + (f % (BK / 4)) * 4]) =
                BF16 ? round_bf16(ra[q]) : ra[q];
        }
#pragma unroll
        for (int q = 0; q < NB; ++q) {
            const int f = tid + q * NT;
            *reinterpret_cast<float4 *>(&Bs[buf][(f / (BN / 4)) * LDB + (f % (BN / 4)) * 4]) =
                BF16 ? round_bf16(rb[q]) : rb[q];
        }
    };

    floatx16 Y[4][TM][TN];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r) Y[j][tm][tn][r] = 0.f;

    load_global(0, 0);
    store_lds(0);
    __syncthreads();

    // (position, channel chunk) of the next tile to fetch, and the LDS buffer being read.
    int npos = 0, nc0 = 0, buf = 0;

    // The position loop is fully unrolled so that the signs of the output transform are
    // compile-time constants; the loop over C stays a run-time loop.
#pragma unroll
    for (int pos = 0; pos < 16; ++pos) {
        floatx16 P[TM][TN];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r) P[tm][tn][r] = 0.f;

        for (int c0 = 0; c0 < C; c0 += BK) {
            nc0 += BK;
            if (nc0 >= C) {
                nc0 = 0;
                ++npos;
            }
            const bool more = npos < 16;
            if (more) load_global(npos, nc0);

            const float *as = As[buf];
            const float *bs = Bs[buf];
            // All LDS reads of the step are issued before its first MFMA so that their latency
            // overlaps the matrix pipeline.  Lane group lg feeds reduction indices
            // k8*8+4*lg .. +3, one per MFMA; the order in which indices are reduced is free as
            // long as A and B agree.
            float4 a[KS][TM];
            float b[KS][4][TN];
#pragma unroll
            for (int k8 = 0; k8 < KS; ++k8) {
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
                    a[k8][tm] = *reinterpret_cast<const float4 *>(&as[(wm0 + tm * 32 + li) * LDA + k8 * 8 + 4 * lg]);
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn)
                        b[k8][t][tn] = bs[(k8 * 8 + 4 * lg + t) * LDB + wn0 + tn * 32 + li];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int k8 = 0; k8 < KS; ++k8)
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int tm = 0; tm < TM; ++tm) {
                        const float av = t == 0 ? a[k8][tm].x : t == 1 ? a[k8][tm].y : t == 2 ? a[k8][tm].z : a[k8][tm].w;
#pragma unroll
                        for (int tn = 0; tn < TN; ++tn)
                            P[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, b[k8][t][tn], P[tm][tn], 0, 0, 0);
                    }
            __builtin_amdgcn_sched_barrier(0);

            if (more) store_lds(buf ^ 1);
            __syncthreads();
            buf ^= 1;
        }

        // P_pos is complete: fold it into the running output tiles, ascending pos.
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            constexpr unsigned long long plus = kPlus, minus = kMinus;
            const int bit = 4 * pos + j;
            if ((plus >> bit) & 1ull) {
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn) Y[j][tm][tn] += P[tm][tn];
            } else if ((minus >> bit) & 1ull) {
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn) Y[j][tm][tn] -= P[tm][tn];
            }
        }
        // Pin the updates here.  Y is not read again until the final stores, so without this the
        // compiler defers all the adds to the end and keeps the 16 product tiles alive instead
        // of the 4 running sums (4x the registers).
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < TN; ++tn) asm volatile("" : "+v"(Y[j][tm][tn]));
    }

    store_output<Cfg>(Y, Out, rows_valid, K, nW, m0, n0, wm0, wn0, li, lg, ep);
}

// ---------------------------------------------------------------------------------------------
// Asynchronous variant: tiles go from global memory straight into LDS (global_load_lds_dwordx4,
// 16 bytes per lane, no VGPR staging and no ds_write), NSTAGE tiles deep, so that the
// HBM/L2 latency of a tile is covered by the MFMA work of the NSTAGE-2 steps before it.
//
// Requirements checked by the launcher: C % BK == 0, K % 4 == 0, TI and Wt 16-byte aligned,
// tile offsets below 2^31 bytes.  Rows beyond M and columns beyond K are not zero-filled but
// clamped to the last valid row / column group: what they produce lands in accumulator rows
// and columns that are never stored.
//
// LDS layout of one stage (floats):
//   A: BM rows of BK/4 16-byte chunks; chunk j of row r sits in slot r*(BK/4) + (j ^ (r % (BK/4)))
//      so that the 8 lanes served together by one ds_read_b128 cycle (8 consecutive rows, same
//      chunk) fall into 8 different bank groups.  The swizzle is applied on the global side: a
//      lane always writes LDS slot (wave-uniform base + lane), and picks the global chunk that
//      belongs there.
//   B: BK rows of BN floats, unswizzled (a wavefront reads 32 consecutive floats of a row).
//
// The loads are inline assembly on purpose: the compiler's wait-count insertion would otherwise
// drain every outstanding load before each LDS read (it cannot tell the stages of the ring
// apart).  Their completion is tracked by hand with s_waitcnt vmcnt(n); loads return in order.
// ---------------------------------------------------------------------------------------------

__device__ __forceinline__ unsigned lds_address(const void *p)
{
    // generic -> LDS address space: the 32-bit value is the byte offset within the workgroup's LDS
    return static_cast<unsigned>(reinterpret_cast<size_t>((const __attribute__((address_space(3))) char *)p));
}

// One 16-byte-per-lane global -> LDS copy: lane l reads base + voff (bytes) and writes LDS byte
// address lds_base + 16*l.  lds_base must be wave-uniform.
__device__ __forceinline__ void async_copy16(const float *base, unsigned voff, unsigned lds_base)
{
    // The "s" constraints need values the compiler has in scalar registers; under register pressure
    // it sometimes computes uniform values on the vector unit, so pin them (a no-op when already scalar).
    // When it is not a no-op, the v_readfirstlane lands right in front of this statement, and a memory
    // instruction may read a scalar register only five cycles after a vector instruction wrote it; the
    // compiler cannot check that inside an assembly statement, so the statement keeps the distance itself
    // (s_mov + s_nop 3; one cycle of it is what the load needs behind the write of M0 anyway).
    const size_t b = reinterpret_cast<size_t>(base);
    const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(b));
    const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(b >> 32));
    base = reinterpret_cast<const float *>((static_cast<size_t>(hi) << 32) | lo);
    lds_base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile(
        "s_mov_b32 m0, %2\n\t"
        "s_nop 3\n\t"
        "global_load_lds_dwordx4 %0, %1"
        :
        : "v"(voff), "s"(base), "s"(lds_base)
        : "memory");  // m0 cannot be named as a clobber: the compiler treats it as reserved (-Winline-asm) and
                      // itself rewrites it immediately before each of its own instructions that read it
}

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding: vmcnt in bits 3:0
// and 15:14, expcnt 6:4, lgkmcnt 11:8).
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
    asm volatile("" ::: "memory");
}

// What the ring kernel does with the finished product tile P_i of a position:
//   RING_FORWARD: folds it into the four output tiles (Y_j +-= P_i) and stores Out [B,2nH,2nW,N] at the end; the B
//                 operand is Wt [16][R][N] (reduction index slow), as the forward weights are.
//   RING_DGRAD:   stores it as plane i of Out [16][M][N]; the B operand is Wt [16][N][R] (reduction index fast):
//                 with A = dP, R = K, N = C and Wt = W this is dTI_i = dP_i . W_i^T, the first GEMM of the
//                 reference's backward pass (winograd2x2_conv_grad_cuda.cu.cc:103-108).
enum RingMode { RING_FORWARD = 0, RING_DGRAD = 1 };

// Dynamic LDS the ring kernel needs at launch: NSTAGE ring slots of one A and one B tile (the forward B
// tile padded by 64 bytes per KiB with 16x16 MFMAs).  Above 64 KiB the launcher must first raise
// hipFuncAttributeMaxDynamicSharedMemorySize.
template <typename Cfg, int NSTAGE, int MODE = RING_FORWARD>
constexpr int async_lds_bytes()
{
    constexpr int nbw = Cfg::BK * Cfg::BN / 4 / 64, bpad = MODE == RING_FORWARD ? Cfg::BPAD : 0;
    return NSTAGE * (Cfg::BM * Cfg::BK + Cfg::BK * Cfg::BN + nbw * bpad) * 4;
}

// The ring kernel's body.  A [16][M][R] row-major (R = reduction length, a multiple of BK), the workgroup's tile
// starts at row m0, column n0 and owns rows_valid <= BM rows; wave tile at (wm0, wn0) within it; N = number of
// output columns.
// BF16 (forward only): the operands are rounded to bf16 (round-to-nearest-even, v_cvt_pk_bf16_f32) after they are
// read from LDS and multiplied with v_mfma_f32_32x32x16_bf16; accumulation, fold and stores stay fp32.
// NPOS: how many of the 16 positions (planes of TI, Wt and, in dgrad mode, Out) the call walks, starting at the
// planes the three pointers point to.  The forward fold needs all 16; the products of the data gradient are
// independent, so its launcher may deal groups of positions to different workgroups.
template <typename Cfg, int NSTAGE, bool BF16, int MODE, int NPOS = 16>
__device__ __forceinline__ void conv_ring_body(const float *__restrict__ TI, const float *__restrict__ Wt,
                                               float *__restrict__ Out, size_t M, int R, int N, int nW, const size_t m0,
                                               const int n0, const unsigned rows_valid, const int wm0, const int wn0,
                                               const ConvEpilogue ep)
{
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, NT = Cfg::NT, MF = Cfg::MF, LG = Cfg::LG, KG = Cfg::KG;
    constexpr int TM = Cfg::TM, TN = Cfg::TN;
    constexpr int KS = BK / KG, CH = BK / 4, NWAVES = NT / 64;
    constexpr bool DGRAD = MODE == RING_DGRAD;
    // Chunk j of tile row r sits at slot j ^ ((r >> SWZ) % CH).  With 32-row MFMA operands and rows of 128 (64) bytes,
    // two (four) rows share 256 bytes of LDS and rows r and r+8 (r+4) of an operand read would otherwise land on the same banks
    // (the counters showed every second LDS cycle of the data gradient as a bank conflict); the 16-row tilings
    // measure conflict-free as they are.
    constexpr int SWZ = MF != 32 ? 0 : BK == 16 ? 2 : BK == 32 ? 1 : 0;  // log2 of the tile rows per 256 bytes
    // Copies are wave-wide: 64 lanes x 16 bytes = 1 KiB.  NAW / NBW of them make an A / B tile; every
    // wave issues the same number (NA + NB) per step so that all waves count outstanding copies alike;
    // where the tile does not divide evenly the surplus copies repeat an earlier one (same bytes twice).
    constexpr int NAW = BM * CH / 64, NBW = BK * BN / 4 / 64;
    constexpr int NA = (NAW + NWAVES - 1) / NWAVES, NB = (NBW + NWAVES - 1) / NWAVES;
    // Forward B tile with 16x16 MFMAs: the four lane groups of an operand read hit rows 4 apart; 64 bytes of
    // padding after every copy (4 rows of 64 floats) put them on different banks.
    constexpr int BPAD = DGRAD ? 0 : Cfg::BPAD;  // floats
    static_assert(BPAD == 0 || BN == 64, "the padded B layout assumes one copy = 4 rows");
    constexpr int A_FLOATS = BM * BK, B_FLOATS = BK * BN + NBW * BPAD, STAGE_FLOATS = A_FLOATS + B_FLOATS;
    constexpr int LPS = NA + NB;  // copies per thread per step
    static_assert(NSTAGE >= 2, "a ring needs two slots");
    static_assert(KS % 2 == 0, "the MFMA chain of a step is split in two halves");
    static_assert(!BF16 || (KS == 4 && MF == 32 && !DGRAD), "the bf16 MFMA consumes 16 reduction indices: a half of a 32-index step");
    static_assert((CH & (CH - 1)) == 0, "swizzle needs a power-of-two chunk count");
    static_assert((BM * CH) % 64 == 0 && (BK * BN / 4) % 64 == 0, "tiles are whole wave-wide copies");
    static_assert((NSTAGE - 2) * LPS + (DGRAD ? TM * TN * Cfg::REGS : 0) < 64, "vmcnt range");
    static_assert(!DGRAD || NSTAGE <= 3, "the wait below allows for the stores of one earlier step");
    static_assert(NPOS == 16 || (DGRAD && NPOS >= 1 && 16 % NPOS == 0), "the output transform folds all 16 positions");

    static_assert(NSTAGE * STAGE_FLOATS * 4 == async_lds_bytes<Cfg, NSTAGE, MODE>(), "launcher and kernel agree on the LDS size");
    extern __shared__ __attribute__((aligned(1024))) float smem[];  // async_lds_bytes<Cfg, NSTAGE, MODE>() bytes

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int li = lane % MF, lg = lane / MF;

    // Per-thread byte offsets of the copies (constant over the whole kernel) and the
    // wave-uniform LDS byte offsets, relative to a stage, they land at.
    // A tile (and the B tile of RING_DGRAD): rows of BK/4 16-byte chunks; chunk j of row r sits in slot
    // r*(BK/4) + (j ^ (r % (BK/4))).
    unsigned a_voff[NA], b_voff[NB];
    unsigned a_lds[NA], b_lds[NB];  // wave-uniform byte offsets within a stage
    const unsigned wave_u = __builtin_amdgcn_readfirstlane(wave);
#pragma unroll
    for (int q = 0; q < NA; ++q) {
        const unsigned wl = (q * NWAVES + wave_u) % NAW;
        const unsigned slot = wl * 64 + lane;
        unsigned row = slot / CH;
        const unsigned chunk = (slot % CH) ^ ((row >> SWZ) % CH);
        row = row < rows_valid ? row : rows_valid - 1;
        a_voff[q] = (row * static_cast<unsigned>(R) + chunk * 4) * 4u;
        a_lds[q] = wl * 1024u;
    }
#pragma unroll
    for (int q = 0; q < NB; ++q) {
        const unsigned wl = (q * NWAVES + wave_u) % NBW;
        const unsigned slot = wl * 64 + lane;
        if (DGRAD) {   // B tile [BN columns][BK reduction indices], swizzled like A
            unsigned col = slot / CH;
            const unsigned chunk = (slot % CH) ^ ((col >> SWZ) % CH);
            col = n0 + col < static_cast<unsigned>(N) ? n0 + col : static_cast<unsigned>(N) - 1;
            b_voff[q] = (col * static_cast<unsigned>(R) + chunk * 4) * 4u;
            b_lds[q] = A_FLOATS * 4 + wl * 1024u;
        } else {       // B tile [BK reduction indices][BN columns]
            const unsigned krow = slot / (BN / 4);
            unsigned n = n0 + (slot % (BN / 4)) * 4;
            n = n + 4 <= static_cast<unsigned>(N) ? n : static_cast<unsigned>(N) - 4;
            b_voff[q] = (krow * static_cast<unsigned>(N) + n) * 4u;
            b_lds[q] = A_FLOATS * 4 + wl * (1024u + BPAD * 4);
        }
    }
    const unsigned smem_base = lds_address(smem);

    const int nkc = R / BK;
    using Acc = AccT<Cfg>;
    Acc Y[DGRAD ? 1 : 4][DGRAD ? 1 : TM][DGRAD ? 1 : TN];
    if constexpr (!DGRAD) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                    for (int r = 0; r < Cfg::REGS; ++r) Y[j][tm][tn][r] = 0.f;
    }

    // ---- copy issuer: running pointers to the tiles of the next step to fetch -------------
    // Tile of (pos, c0): A at TI + (pos*M + m0)*R + c0; B at Wt + (pos*R + c0)*N (forward) or
    // Wt + pos*N*R + c0 (dgrad; the column offset is in b_voff).  Consecutive steps advance A by BK floats, plus
    // (M-1)*R when the position wraps, and B by BK*N (forward) or by BK, plus (N-1)*R at the wrap (dgrad).
    const float *a_next = TI + m0 * R;
    const float *b_next = Wt;
    const size_t a_wrap = (M - 1) * static_cast<size_t>(R);
    const size_t b_inc = DGRAD ? static_cast<size_t>(BK) : static_cast<size_t>(BK) * N;
    const size_t b_wrap = DGRAD ? (static_cast<size_t>(N) - 1) * R : 0;
    int kc_next = 0, pos_next = 0;
    unsigned lds_next = smem_base;  // byte address of the next ring slot
    int slot_next = 0;
    auto copy = [&](int i) __attribute__((always_inline)) {  // the i-th of this thread's LPS copies of a step
        if (i < NA)
            async_copy16(a_next, a_voff[i < NA ? i : 0], lds_next + a_lds[i < NA ? i : 0]);
        else
            async_copy16(b_next, b_voff[i >= NA ? i - NA : 0], lds_next + b_lds[i >= NA ? i - NA : 0]);
    };
    // After the last step the issuer wraps around to the first tile again: the loop below
    // issues one step's copies per step unconditionally (so the outstanding-copy count is the
    // same at every wait), and the surplus copies at the end re-fetch valid memory into ring
    // slots nobody reads any more.
    auto advance = [&]() __attribute__((always_inline)) {
        a_next += BK;
        b_next += b_inc;
        if (++kc_next == nkc) {
            kc_next = 0;
            a_next += a_wrap;
            b_next += b_wrap;
            if (++pos_next == NPOS) {
                pos_next = 0;
                a_next = TI + m0 * R;
                b_next = Wt;
            }
        }
        lds_next += STAGE_FLOATS * 4;
        if (++slot_next == NSTAGE) {
            slot_next = 0;
            lds_next = smem_base;
        }
    };

    // ---- MFMA operands ---------------------------------------------------------------------
    // A step's reduction range BK is consumed in two halves of KH groups of KG indices (8 with
    // 32x32 MFMAs, 16 with 16x16).  Within a group, lane group lg feeds indices 4*lg .. 4*lg+3,
    // one per MFMA (the order in which indices are reduced is free as long as A and B agree), so
    // A comes as one b128 read per group and the forward B as 4 b32 reads, paired so that they merge into
    // ds_read2_b32; the dgrad B tile has the reduction index fast like A and is read the same way.
    constexpr int KH = KS / 2;
    struct HalfFrag {
        float4 a[KH][TM];
        float b[DGRAD ? 1 : KH][4][TN];
        float4 bq[DGRAD ? KH : 1][TN];
    };
    constexpr int NUB = DGRAD ? TN : 2 * TN;    // B read units per group: b128 reads, or b32 pairs
    constexpr int NU = KH * (TM + NUB);         // read units per half
    // MFMAs per half: fp32 32x32x2 reduces 2 indices each, bf16 32x32x16 all 16 of a half at once.
    constexpr int NM = BF16 ? TM * TN : KH * 4 * TM * TN;

    // Per-thread LDS offsets within a stage (A in 16-byte units, B in floats).
    int a_off[KS][TM];
#pragma unroll
    for (int k8 = 0; k8 < KS; ++k8)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            const int row = wm0 + tm * MF + li;
            a_off[k8][tm] = row * CH + ((LG * k8 + lg) ^ ((row >> SWZ) % CH));  // in 16-byte units
        }
    // Forward: B row k sits at k*BN floats plus BPAD per 4 rows; lane group lg reads rows 4*lg + t of a group.
    constexpr int BROW4 = 4 * BN + BPAD;
    const int b_off = A_FLOATS + lg * BROW4 + wn0 + li;
    int bq_off[DGRAD ? KS : 1][DGRAD ? TN : 1];  // dgrad: 16-byte units, relative to the B tile
    if constexpr (DGRAD) {
#pragma unroll
        for (int k8 = 0; k8 < KS; ++k8)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) {
                const int col = wn0 + tn * MF + li;
                bq_off[k8][tn] = A_FLOATS / 4 + col * CH + ((LG * k8 + lg) ^ ((col >> SWZ) % CH));
            }
    }

    // Read unit u of half h of the stage at float offset st into F.
    auto read_unit = [&](HalfFrag &F, int st, int h, int u) __attribute__((always_inline)) {
        const int k8l = u / (TM + NUB), v = u % (TM + NUB);
        const int k8 = h * KH + k8l;
        if (v < TM) {
            F.a[k8l][v] = reinterpret_cast<const float4 *>(smem)[st / 4 + a_off[k8][v]];
        } else if constexpr (DGRAD) {
            F.bq[k8l][v - TM] = reinterpret_cast<const float4 *>(smem)[st / 4 + bq_off[k8][v - TM]];
        } else {
            const int tn = (v - TM) / 2, tp = (v - TM) % 2;
            F.b[k8l][2 * tp][tn] = smem[st + b_off + k8 * LG * BROW4 + (2 * tp) * BN + tn * MF];
            F.b[k8l][2 * tp + 1][tn] = smem[st + b_off + k8 * LG * BROW4 + (2 * tp + 1) * BN + tn * MF];
        }
    };
    // ---- prologue: fill the ring, wait for step 0, read its first half ----------------------
#pragma unroll
    for (int i = 0; i < NSTAGE; ++i) {
#pragma unroll
        for (int c = 0; c < LPS; ++c) copy(c);
        advance();
    }
    wait_vmcnt<(NSTAGE - 1) * LPS>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    HalfFrag F1, F2;
#pragma unroll
    for (int u = 0; u < NU; ++u) read_unit(F1, 0, 0, u);

    // ---- main loop ----------------------------------------------------------------------------
    // A wave issues at most one instruction every four cycles and an MFMA occupies the matrix
    // pipe for 64 (32x32x2) or 32 (16x16x4) cycles, so everything that is not an MFMA is dealt out
    // between the MFMAs, a few instructions after each (sched_barrier pins the order):
    //   first half  (MFMAs on F1): the LDS reads of the step's second half F2;
    //   second half (MFMAs on F2): after the first MFMA, wait for the tile of step s+1 and
    //     barrier (everyone now holds step s entirely in registers, so its ring slot is free);
    //     then this thread's copies of step s+NSTAGE into that slot, one per MFMA, and the LDS
    //     reads of F1 of step s+1.
    //
    // What happens to a finished position (the fold into Y, up to 4*TM*TN vector adds, or the stores of
    // its product tiles) is dealt out the same way over the first step of the next position, which accumulates
    // into the other of two product buffers and starts its chains from a zero accumulator.
    int st_cur = 0;  // float offset of the ring slot of the current step
    Acc P[2][TM][TN];
    const Acc zero16 = {};

    // Forward.  Fold unit e of position `pos` (e = j*TM*TN + tm*TN + tn): Y_j +-= P.  The empty asm pins the
    // update here: Y is not read again until the final stores, so without it the compiler defers
    // all the adds to the end and keeps the 16 product tiles alive instead of the 4 sums.
    // Dgrad.  Unit e = tm*TN + tn: the product tile goes to plane `pos` of Out, written through (the gather
    // kernel that reads the planes next finds them in the Infinity Cache).  Register r of lane (lg, li) holds
    // row 4*lg + r, column li of a 16x16 tile; 8*(r/4) + 4*lg + r%4 of a 32x32 tile.
    constexpr int NE = DGRAD ? TM * TN : 4 * TM * TN;
    // dgrad: byte offset of this lane's first row and column within the workgroup's rows of a plane; what tile,
    // register and position add to it is the same for the whole wave, so a store is one instruction with a
    // scalar base and this offset, and whether a tile lies wholly inside the valid rows and columns is a scalar
    // test (only a ragged last tile takes per-lane predicates).
    const unsigned lane_off = (static_cast<unsigned>(wm0 + 4 * lg) * static_cast<unsigned>(N) + n0 + wn0 + li) * 4u;
    char *const out_tile = reinterpret_cast<char *>(DGRAD ? Out + m0 * N : Out);  // dgrad: this workgroup's first row in plane 0
    const unsigned rows_u = __builtin_amdgcn_readfirstlane(rows_valid);
    // dgrad: the product stores count on the same counter as the copies, and memory operations complete in the
    // order they were issued, so the wait for a tile must allow for the stores issued after its copies.  Their
    // number is known (REGS per tile) while every tile of the wave lies inside the valid rows and columns (`exact`);
    // a wave with a ragged tile waits for everything instead.
    const bool exact = DGRAD && static_cast<unsigned>(wm0 + TM * MF) <= rows_u && n0 + wn0 + TN * MF <= N;
    bool stores_behind = false;  // the previous step issued a position's product stores
    auto finish_unit = [&](const Acc (&Pp)[TM][TN], int pos, int e) __attribute__((always_inline)) {
        if constexpr (DGRAD) {
            const int tm = e / TN, tn = e % TN;
            const bool whole = static_cast<unsigned>(wm0 + tm * MF + MF) <= rows_u && n0 + wn0 + tn * MF + MF <= N;  // uniform
            char *const tile = out_tile + ((static_cast<size_t>(pos) * M + tm * MF) * N + tn * MF) * 4;
            const size_t row_bytes = static_cast<size_t>(N) * 4;
            if (whole) {
#pragma unroll
                for (int r = 0; r < Cfg::REGS; ++r) {
                    const int row_u = MF == 32 ? 8 * (r / 4) + (r % 4) : r;  // + tm*MF in tile, + 4*lg + wm0 in lane_off
                    store_streaming(reinterpret_cast<float *>(tile + row_u * row_bytes + lane_off), Pp[tm][tn][r]);
                }
            } else {
                const bool col_ok = n0 + wn0 + tn * MF + li < N;
#pragma unroll
                for (int r = 0; r < Cfg::REGS; ++r) {
                    const int row_u = MF == 32 ? 8 * (r / 4) + (r % 4) : r;
                    if (static_cast<unsigned>(wm0 + tm * MF + 4 * lg + row_u) < rows_valid && col_ok)
                        store_streaming(reinterpret_cast<float *>(tile + row_u * row_bytes + lane_off), Pp[tm][tn][r]);
                }
            }
        } else {
            constexpr unsigned long long plus = kPlus, minus = kMinus;
            const int j = e / (TM * TN), tm = (e / TN) % TM, tn = e % TN;
            const int bit = 4 * pos + j;
            if ((plus >> bit) & 1ull) {
                Y[j][tm][tn] += Pp[tm][tn];
                asm volatile("" : "+v"(Y[j][tm][tn]));
            } else if ((minus >> bit) & 1ull) {
                Y[j][tm][tn] -= Pp[tm][tn];
                asm volatile("" : "+v"(Y[j][tm][tn]));
            }
        }
    };
    // Slot (MFMA index 0 .. 2*NM-1 of the first step of the next position) after which unit e goes.
    auto finish_slot = [](int e) { return e * (2 * NM) / NE; };
    // dgrad: product stores of a position's first step that go out in its first half (before the wait for the
    // next tile) and in its second half (behind it).
    constexpr int NE1 = (NE * NM + 2 * NM - 1) / (2 * NM);  // units e with finish_slot(e) < NM
    constexpr int ST1 = DGRAD ? NE1 * Cfg::REGS : 0, ST2 = DGRAD ? (NE - NE1) * Cfg::REGS : 0;

    // One step.  first: the chains start from zero and the finish of position done_pos (held in
    // Pprev) rides along; otherwise done_pos is ignored.
    auto step = [&](Acc (&Pc)[TM][TN], const Acc (&Pprev)[TM][TN], auto first_tag, auto done_tag) __attribute__((always_inline)) {
        constexpr bool first = decltype(first_tag)::value;
        constexpr int done_pos = decltype(done_tag)::value;
        const int st_next = st_cur + STAGE_FLOATS == NSTAGE * STAGE_FLOATS ? 0 : st_cur + STAGE_FLOATS;
        auto mfma_slot = [&](const HalfFrag &F, int i, bool from_zero) __attribute__((always_inline)) {
            if constexpr (BF16) {
                // Lane group lg holds reduction indices {8*k8l + 4*lg + t}: 8 per half, the same
                // set on the A and the B side, which is all the MFMA needs.
                const int tn = i % TN, tm = i / TN;
                const float4 a0 = F.a[0][tm], a1 = F.a[1][tm];
                auto pk = [](float x, float y) { return __builtin_convertvector(floatx2{x, y}, bf16x2); };
                const bf16x2 p0 = pk(a0.x, a0.y), p1 = pk(a0.z, a0.w), p2 = pk(a1.x, a1.y), p3 = pk(a1.z, a1.w);
                const bf16x2 q0 = pk(F.b[0][0][tn], F.b[0][1][tn]), q1 = pk(F.b[0][2][tn], F.b[0][3][tn]);
                const bf16x2 q2 = pk(F.b[1][0][tn], F.b[1][1][tn]), q3 = pk(F.b[1][2][tn], F.b[1][3][tn]);
                const bf16x8 av = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
                const bf16x8 bv = {q0[0], q0[1], q1[0], q1[1], q2[0], q2[1], q3[0], q3[1]};
                Pc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, from_zero ? zero16 : Pc[tm][tn], 0, 0, 0);
            } else {
                const int tn = i % TN, tm = (i / TN) % TM, t = (i / (TN * TM)) % 4, k8l = i / (TN * TM * 4);
                const float4 a4 = F.a[k8l][tm];
                const float av = t == 0 ? a4.x : t == 1 ? a4.y : t == 2 ? a4.z : a4.w;
                float bv;
                if constexpr (DGRAD) {
                    const float4 b4 = F.bq[k8l][tn];
                    bv = t == 0 ? b4.x : t == 1 ? b4.y : t == 2 ? b4.z : b4.w;
                } else {
                    bv = F.b[k8l][t][tn];
                }
                if constexpr (MF == 32)
                    Pc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, from_zero ? zero16 : Pc[tm][tn], 0, 0, 0);
                else
                    Pc[tm][tn] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv, from_zero ? zero16 : Pc[tm][tn], 0, 0, 0);
            }
        };
        // Slots (MFMA indices of the second half) after which the copies and LDS reads go; all
        // behind the barrier that follows MFMA 0.
        auto copy_slot = [](int c) { return NM > 1 ? 1 + c * (NM - 1) / LPS : 0; };
        auto read_slot = [](int u) { return NM > 1 ? 1 + u * (NM - 1) / NU : 0; };
#pragma unroll
        for (int i = 0; i < NM; ++i) {
            mfma_slot(F1, i, first && i < TM * TN);
#pragma unroll
            for (int u = 0; u < NU; ++u)
                if (u * NM / NU == i) read_unit(F2, st_cur, 1, u);
            if (first && done_pos >= 0) {
#pragma unroll
                for (int e = 0; e < NE; ++e)
                    if (finish_slot(e) == i) finish_unit(Pprev, done_pos, e);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int i = 0; i < NM; ++i) {
            mfma_slot(F2, i, false);
            if (i == 0) {
                // The tile of the next step is complete once at most the copies of the NSTAGE-2
                // steps after it are outstanding.
                if constexpr (DGRAD) {
                    // Newer than the copies of the tile waited for: the copies of the NSTAGE-2 steps after it, the
                    // stores that went out with the previous step's copies (NSTAGE > 2), and this step's own so far.
                    constexpr int mine = first && done_pos >= 0 ? ST1 : 0;
                    if (!exact)
                        wait_vmcnt<0>();
                    else if (stores_behind && NSTAGE > 2)
                        wait_vmcnt<(NSTAGE - 2) * LPS + ST2 + mine>();
                    else
                        wait_vmcnt<(NSTAGE - 2) * LPS + mine>();
                } else {
                    wait_vmcnt<(NSTAGE - 2) * LPS>();
                }
                __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS reads of this step are done
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            }
#pragma unroll
            for (int c = 0; c < LPS; ++c)
                if (copy_slot(c) == i) copy(c);
#pragma unroll
            for (int u = 0; u < NU; ++u)
                if (read_slot(u) == i) read_unit(F1, st_next, 0, u);
            if (first && done_pos >= 0) {
#pragma unroll
                for (int e = 0; e < NE; ++e)
                    if (finish_slot(e) == NM + i) finish_unit(Pprev, done_pos, e);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        advance();
        st_cur = st_next;
        stores_behind = DGRAD && first && done_pos >= 0;
    };

    // The position loop is unrolled at compile time so that the signs of the output transform
    // are constants (a run-time loop over position pairs with branched folds measured 6 % slower).
    static_for<NPOS>([&](auto pos_tag) {
        constexpr int pos = decltype(pos_tag)::value;
        step(P[pos & 1], P[(pos & 1) ^ 1], std::true_type{}, std::integral_constant<int, pos - 1>{});
        for (int kc = 1; kc < nkc; ++kc)
            step(P[pos & 1], P[(pos & 1) ^ 1], std::false_type{}, std::integral_constant<int, -1>{});
    });
#pragma unroll
    for (int e = 0; e < NE; ++e) finish_unit(P[(NPOS - 1) & 1], NPOS - 1, e);

    // The surplus copies must have landed before this workgroup's LDS can be handed on.
    wait_vmcnt<0>();

    if constexpr (!DGRAD) store_output<Cfg>(Y, Out, rows_valid, N, nW, m0, n0, wm0, wn0, li, lg, ep);
}

// Forward: Out [B,2nH,2nW,K] from TI [16][M][C] and Wt [16][C][K].
// Requirements checked by the launcher: C % BK == 0, K % 4 == 0, TI and Wt 16-byte aligned,
// tile offsets below 2^31 bytes.  Rows beyond M and columns beyond K are not zero-filled but
// clamped to the last valid row / column group: what they produce lands in accumulator rows
// and columns that are never stored.
template <typename Cfg, int NSTAGE, bool BF16 = false>
__global__ __launch_bounds__(Cfg::NT) __attribute__((amdgpu_waves_per_eu(Cfg::OCC, Cfg::OCC))) void conv_mfma_async_kernel(
    const float *__restrict__ TI, const float *__restrict__ Wt, float *__restrict__ Out, size_t M, int C, int K, int nH,
    int nW, unsigned tiles_n, unsigned rows_per_wg, ConvEpilogue ep)
{
    const unsigned lid = xcd_swizzle(blockIdx.x, gridDim.x);
    // The workgroup's tile starts at row m0 and is BM rows tall, of which the first rows_valid are
    // its own (rows_per_wg <= BM lets the launcher split M evenly at 16-row granularity).
    const size_t m0 = static_cast<size_t>(lid / tiles_n) * rows_per_wg;
    const int n0 = static_cast<int>(lid % tiles_n) * Cfg::BN;
    const unsigned rows_valid = static_cast<unsigned>(M - m0 < rows_per_wg ? M - m0 : rows_per_wg);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the same for the whole wave: scalar
    const int wm0 = (wave / Cfg::WGN) * Cfg::WM, wn0 = (wave % Cfg::WGN) * Cfg::WN;
    conv_ring_body<Cfg, NSTAGE, BF16, RING_FORWARD>(TI, Wt, Out, M, C, K, nW, m0, n0, rows_valid, wm0, wn0, ep);
}

// Data gradient: dTI [16][M][C] from dP [16][M][K] and W [16][C][K]: dTI_i = dP_i . W_i^T.
// Requirements checked by the launcher: K % BK == 0 (the reduction), dP and W 16-byte aligned, tile offsets
// below 2^31 bytes.  Rows beyond M and columns beyond C are clamped on load and never stored.
// A workgroup owns one tile of NPOS consecutive planes: grid.x = (16 / NPOS) * tiles_m * tiles_n, the position
// group slowest, so that the workgroups running at the same time work on neighbouring rows of the same planes.
template <typename Cfg, int NSTAGE, int NPOS = 16>
__global__ __launch_bounds__(Cfg::NT) __attribute__((amdgpu_waves_per_eu(Cfg::OCC, Cfg::OCC))) void conv_dgrad_async_kernel(
    const float *__restrict__ dP, const float *__restrict__ Wt, float *__restrict__ dTI, size_t M, int C, int K,
    unsigned tiles_m, unsigned tiles_n, unsigned rows_per_wg)
{
    const unsigned lid = xcd_swizzle(blockIdx.x, gridDim.x);
    const unsigned per_group = tiles_m * tiles_n;
    const size_t pos0 = static_cast<size_t>(lid / per_group) * NPOS;
    const unsigned tile = lid % per_group;
    const size_t m0 = static_cast<size_t>(tile / tiles_n) * rows_per_wg;
    const int n0 = static_cast<int>(tile % tiles_n) * Cfg::BN;
    const unsigned rows_valid = static_cast<unsigned>(M - m0 < rows_per_wg ? M - m0 : rows_per_wg);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the same for the whole wave: scalar
    const int wm0 = (wave / Cfg::WGN) * Cfg::WM, wn0 = (wave % Cfg::WGN) * Cfg::WN;
    conv_ring_body<Cfg, NSTAGE, false, RING_DGRAD, NPOS>(dP + pos0 * M * K, Wt + pos0 * C * K, dTI + pos0 * M * C, M, K, C, 0,
                                                         m0, n0, rows_valid, wm0, wn0, ConvEpilogue());
}

}  // namespace
}  // namespace swc
