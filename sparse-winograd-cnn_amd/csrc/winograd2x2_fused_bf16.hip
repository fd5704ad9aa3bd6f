// Fused Winograd-ReLU convolution layer with bf16 GEMM operands for gfx950: input transform,
// Winograd-domain ReLU, the 16 per-position GEMMs and the output transform in one kernel, reading
// the fp32 NHWC input and the prepared bf16 weights [16,K,C] and writing the fp32 output.  Neither
// the transformed activations nor any bf16 copy of them reaches memory.
//
// Arithmetic: what swc_winograd2x2_imtrans_bf16out followed by swc_winograd2x2_conv_bf16in computes
// (fp32 transform in the reference's expression order, winograd2x2_imTrans_cuda.cu.cc:112-127, ReLU,
// one rounding to bf16, exact bf16 products accumulated in fp32, fp32 output transform in ascending
// position order, winograd2x2_conv_cuda.cu.cc:39-46), with the optional per-channel affine maps of
// swc_winograd2x2_imtrans_affine on the way in and of swc_winograd2x2_conv_epilogue on the way out.
//
// Structure, after relu_conv_fused_kernel: a workgroup (4 wavefronts, 2x2) owns 64 tiles x 64 output
// channels and walks the input channels 16 at a time (one v_mfma_f32_32x32x16_bf16 per position and
// chunk).  Its threads produce the chunk's transformed activations for all 16 positions into LDS as
// bf16 (thread = one tile row x 4 channels, float4 loads), the weight slices arrive by global -> LDS
// copies, and each wavefront keeps all 16 products as accumulators (256 registers), folding them
// into the four output tiles at the end.  With bf16 the matrix work is small; the kernel is bound by
// the producer's vector arithmetic and by the latency of its input loads, which are therefore
// requested two chunks ahead.

#include "winograd2x2_conv_kernel.h"

namespace swc {
namespace {

constexpr int GBM = 64, GBN = 64, GBK = 16;          // tiles x output channels x channels per chunk
constexpr int GA_BYTES = 16 * GBM * GBK * 2;          // transformed activations of a chunk, all positions: 32 KiB
constexpr int GB_BYTES = 16 * GBN * GBK * 2;          // weight slices of a chunk, all positions: 32 KiB
constexpr int GSTAGE_BYTES = GA_BYTES + GB_BYTES;
constexpr int GSMEM_BYTES = 2 * GSTAGE_BYTES;         // double buffered: 128 KiB
constexpr int GB_COPIES = GB_BYTES / 16 / 256;        // 16-byte copies per thread per chunk: 8

template <int I>
__device__ __forceinline__ float g_bt_d_b_one(const float (&d)[16])
{
    if (I == 0) return d[0] - d[2] - d[8] + d[10];
    if (I == 1) return d[1] + d[2] - d[9] - d[10];
    if (I == 2) return d[2] - d[1] + d[9] - d[10];
    if (I == 3) return d[1] - d[3] - d[9] + d[11];
    if (I == 4) return d[4] - d[6] + d[8] - d[10];
    if (I == 5) return d[5] + d[6] + d[9] + d[10];
    if (I == 6) return d[6] - d[5] - d[9] + d[10];
    if (I == 7) return d[5] - d[7] + d[9] - d[11];
    if (I == 8) return d[6] - d[4] + d[8] - d[10];
    if (I == 9) return d[9] - d[6] - d[5] + d[10];
    if (I == 10) return d[5] - d[6] - d[9] + d[10];
    if (I == 11) return d[7] - d[5] + d[9] - d[11];
    if (I == 12) return d[4] - d[6] - d[12] + d[14];
    if (I == 13) return d[5] + d[6] - d[13] - d[14];
    if (I == 14) return d[6] - d[5] + d[13] - d[14];
    return d[5] - d[7] - d[13] + d[15];
}

__device__ __forceinline__ unsigned g_pack_bf16(float lo, float hi)
{
    return __builtin_bit_cast(unsigned, __builtin_convertvector(floatx2{lo, hi}, bf16x2));  // v_cvt_pk_bf16_f32, RNE
}

// A 16-byte half h (8 channels) of row r of a [64 rows][32 bytes] LDS tile sits at slot h ^ ((r >> 3) & 1):
// the 16 lanes that one cycle of a ds_read_b128 serves then cover 256 distinct bytes.
__device__ __forceinline__ unsigned g_slot(unsigned row, unsigned half) { return half ^ ((row >> 3) & 1u); }

// Requires C % 16 == 0, 16-byte aligned X and Wt16, B*H*W*C < 2^30.  AFFINE: x -> fmaf(x, in_scale[c], in_shift[c])
// on pixels inside the image before the transform.
template <bool RELU, bool AFFINE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void relu_conv_fused_bf16_kernel(
    const float *__restrict__ X, const float *__restrict__ in_scale, const float *__restrict__ in_shift,
    const unsigned short *__restrict__ Wt16, float *__restrict__ Out, size_t M, int H, int W, int C, int K, int nH,
    int nW, unsigned tiles_n, ConvEpilogue ep)
{
    extern __shared__ __attribute__((aligned(1024))) unsigned char gsmem[];

    const unsigned lid = xcd_swizzle(blockIdx.x, gridDim.x);
    const size_t m0 = static_cast<size_t>(lid / tiles_n) * GBM;
    const int n0 = static_cast<int>(lid % tiles_n) * GBN;
    const unsigned cols_valid = static_cast<unsigned>(K - n0 < GBN ? K - n0 : GBN);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const unsigned wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lg = lane >> 5;
    const int wm0 = static_cast<int>(wave >> 1) * 32, wn0 = static_cast<int>(wave & 1) * 32;

    // ---- producer: this thread transforms channels 4*pq .. 4*pq+3 of the chunk for tile row pr ----
    const unsigned pr = tid >> 2, pq = tid & 3;
    unsigned pix_off[16];    // byte offset of the patch pixel's channel 4*pq in X; 0 where padded
    unsigned pix_valid = 0;  // bit j: pixel j of the 4x4 patch lies inside the image
    {
        size_t m = m0 + pr;
        if (m >= M) m = M - 1;  // rows beyond M recompute the last tile; never stored
        const unsigned tw = static_cast<unsigned>(m % nW);
        const unsigned bt = static_cast<unsigned>(m / nW);
        const unsigned th = bt % nH, b = bt / nH;
        const int y0 = 2 * static_cast<int>(th) - 1, x0 = 2 * static_cast<int>(tw) - 1;
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int y = y0 + r, x = x0 + s;
                const bool in = (y > -1) && (y < H) && (x > -1) && (x < W);  // winograd2x2_imTrans_cuda.cu.cc:46
                pix_off[4 * r + s] =
                    in ? static_cast<unsigned>(((static_cast<size_t>(b) * H + y) * W + x) * C + 4 * pq) * 4u : 0u;
                pix_valid |= in ? (1u << (4 * r + s)) : 0u;
            }
    }
    // byte offset of this thread's 8 output bytes within a position's [64][32 B] tile
    const unsigned a_wr_off = pr * 32u + g_slot(pr, pq >> 1) * 16u + (pq & 1u) * 8u;

    // ---- weight copies: wave-copy wc = 4*q + wave covers position wc/2, rows 32*(wc%2) .. +31 -------
    unsigned b_voff[GB_COPIES];
#pragma unroll
    for (int q = 0; q < GB_COPIES; ++q) {
        const unsigned wc = 4 * q + wave;
        const unsigned pos = wc >> 1, row = 32 * (wc & 1) + lane / 2;
        const unsigned half = g_slot(row, lane & 1);          // which 8 channels this lane's fixed slot must hold
        const unsigned kr = row < cols_valid ? row : cols_valid - 1;  // rows beyond K: clamped, never stored
        b_voff[q] = ((pos * static_cast<unsigned>(K) + n0 + kr) * static_cast<unsigned>(C) + half * 8) * 2u;
    }
    const unsigned smem_base = lds_address(gsmem);

    // ---- consumer offsets (bytes within a position's tile) ------------------------------------------
    const unsigned a_rd_off = (wm0 + li) * 32u + g_slot(wm0 + li, lg) * 16u;
    const unsigned b_rd_off = GA_BYTES + (wn0 + li) * 32u + g_slot(wn0 + li, lg) * 16u;

    floatx16 P[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) P[i][r] = 0.f;

    const int nchunks = C / GBK;

    float4 raw[2][16] = {};  // two chunks of input pixels in flight; indices are compile-time constants
    auto load_raw = [&](auto set_tag, int c0) __attribute__((always_inline)) {
        constexpr int set = decltype(set_tag)::value;
        const char *xc = reinterpret_cast<const char *>(X + c0);
#pragma unroll
        for (int j = 0; j < 16; ++j) raw[set][j] = *reinterpret_cast<const float4 *>(xc + pix_off[j]);
    };
    auto copy_b = [&](int c0, int stage) __attribute__((always_inline)) {
        const unsigned short *wc0 = Wt16 + c0;
        const unsigned dst = smem_base + stage * GSTAGE_BYTES + GA_BYTES + wave * 1024u;
#pragma unroll
        for (int q = 0; q < GB_COPIES; ++q)
            async_copy16(reinterpret_cast<const float *>(wc0), b_voff[q], dst + q * 4096);
    };
    // All 16 transformed values of the chunk held in raw[set] (4 channels each), as bf16, into `stage`;
    // two channels at a time, which keeps the live temporaries at 32 registers.
    auto produce = [&](auto set_tag, int c0, int stage) __attribute__((always_inline)) {
        constexpr int set = decltype(set_tag)::value;
        float sc[4] = {1.f, 1.f, 1.f, 1.f}, sh[4] = {0.f, 0.f, 0.f, 0.f};
        if (AFFINE) {
            const float4 s4 = *reinterpret_cast<const float4 *>(in_scale + c0 + 4 * pq);
            const float4 h4 = *reinterpret_cast<const float4 *>(in_shift + c0 + 4 * pq);
            sc[0] = s4.x, sc[1] = s4.y, sc[2] = s4.z, sc[3] = s4.w;
            sh[0] = h4.x, sh[1] = h4.y, sh[2] = h4.z, sh[3] = h4.w;
        }
        unsigned char *a_stage = gsmem + stage * GSTAGE_BYTES + a_wr_off;
#pragma unroll
        for (int pair = 0; pair < 2; ++pair) {
            float d0[16], d1[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const bool in = (pix_valid >> j) & 1u;
                const float4 v = raw[set][j];
                const float e0 = pair == 0 ? v.x : v.z, e1 = pair == 0 ? v.y : v.w;
                d0[j] = in ? (AFFINE ? __builtin_fmaf(e0, sc[2 * pair], sh[2 * pair]) : e0) : 0.f;
                d1[j] = in ? (AFFINE ? __builtin_fmaf(e1, sc[2 * pair + 1], sh[2 * pair + 1]) : e1) : 0.f;
            }
            static_for<16>([&](auto i_tag) {
                constexpr int I = decltype(i_tag)::value;
                float t0 = g_bt_d_b_one<I>(d0), t1 = g_bt_d_b_one<I>(d1);
                if (RELU) {
                    t0 = t0 > 0.f ? t0 : 0.f;
                    t1 = t1 > 0.f ? t1 : 0.f;
                }
                *reinterpret_cast<unsigned *>(a_stage + I * (GBM * 32) + pair * 4) = g_pack_bf16(t0, t1);
            });
            __builtin_amdgcn_sched_barrier(0);  // keeps the second pair's temporaries from overlapping the first's
        }
    };
    // The 16 MFMAs of a chunk, operands read one position ahead.
    auto consume = [&](int stage) __attribute__((always_inline)) {
        const unsigned char *st = gsmem + stage * GSTAGE_BYTES;
        bf16x8 a[2], b[2];
        a[0] = *reinterpret_cast<const bf16x8 *>(st + a_rd_off);
        b[0] = *reinterpret_cast<const bf16x8 *>(st + b_rd_off);
        static_for<16>([&](auto p_tag) {
            constexpr int p = decltype(p_tag)::value;
            if (p + 1 < 16) {
                a[(p + 1) & 1] = *reinterpret_cast<const bf16x8 *>(st + (p + 1) * (GBM * 32) + a_rd_off);
                b[(p + 1) & 1] = *reinterpret_cast<const bf16x8 *>(st + (p + 1) * (GBN * 32) + b_rd_off);
            }
            P[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[p & 1], b[p & 1], P[p], 0, 0, 0);
        });
    };

    // ---- prologue: chunk 0 produced into stage 0; the weights of chunks 0 and 1 and the pixels of
    //      chunks 1 (set 1) and 2 (set 0, after chunk 0 is produced) on their way --------------------
    copy_b(0, 0);
    load_raw(std::integral_constant<int, 0>{}, 0);
    if (nchunks > 1) load_raw(std::integral_constant<int, 1>{}, GBK);
    produce(std::integral_constant<int, 0>{}, 0, 0);
    if (nchunks > 1) copy_b(GBK, 1);
    if (nchunks > 2) load_raw(std::integral_constant<int, 0>{}, 2 * GBK);
    // Outstanding now, oldest first: [weights 0] [pixels 1] [weights 1] [pixels 2].  Stage 0 needs weights 0.
    wait_vmcnt<0>();
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    // ---- main loop: iteration `it` multiplies chunk `it` (stage it&1) and produces chunk it+1 from the
    //      pixel set (it+1)&1; after the barrier it requests the weights of chunk it+2 into the stage
    //      just vacated and then the pixels of chunk it+3 into the set just freed.  In that order the
    //      weights a barrier waits for are always older than the one chunk of pixel loads (16 per
    //      thread) that may still be in flight -----------------------------------------------------------
    auto iteration = [&](auto par_tag, int it) __attribute__((always_inline)) {
        constexpr int cur = decltype(par_tag)::value, nxt = cur ^ 1;
        consume(cur);
        if (it + 1 < nchunks) produce(std::integral_constant<int, nxt>{}, (it + 1) * GBK, nxt);
        // Stage `nxt` is complete once this thread's weight copies into it have landed and everyone has
        // written its rows; stage `cur` is free once everyone has read it.
        if (it + 2 < nchunks)
            wait_vmcnt<16>();  // the pixels of chunk it+2, requested after those weights, may stay in flight
        else
            wait_vmcnt<0>();
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (it + 2 < nchunks) copy_b((it + 2) * GBK, cur);
        if (it + 3 < nchunks) load_raw(std::integral_constant<int, nxt>{}, (it + 3) * GBK);
    };
    int it = 0;
    for (; it + 1 < nchunks; it += 2) {
        iteration(std::integral_constant<int, 0>{}, it);
        iteration(std::integral_constant<int, 1>{}, it + 1);
    }
    if (it < nchunks) iteration(std::integral_constant<int, 0>{}, it);
    wait_vmcnt<0>();

    // ---- fold the 16 products into the four output tiles, ascending position ------------------------
    floatx16 Y[4][1][1];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) Y[j][0][0][r] = 0.f;
    static_for<16>([&](auto i_tag) {
        constexpr int i = decltype(i_tag)::value;
        constexpr unsigned long long plus = kPlus, minus = kMinus;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if ((plus >> (4 * i + j)) & 1ull) Y[j][0][0] += P[i];
            else if ((minus >> (4 * i + j)) & 1ull) Y[j][0][0] -= P[i];
        }
    });
    using StoreCfg = ConvCfg<GBM, GBN, 32, 2, 2>;
    const unsigned rows_valid = static_cast<unsigned>(M - m0 < GBM ? M - m0 : GBM);
    store_output<StoreCfg>(Y, Out, rows_valid, K, nW, m0, n0, wm0, wn0, li, lg, ep);
}

}  // namespace
}  // namespace swc

extern "C" int swc_winograd2x2_relu_conv_bf16(const float *Input, const float *InScale, const float *InShift,
                                              const unsigned short *Weight16t, float *Output, const float *OutScale,
                                              const float *OutShift, const float *Residual, int C, int B, int H, int W,
                                              int K, int pad_h, int pad_w, int relu, swc_stream_t stream)
{
    using namespace swc;
    if (Input == nullptr || Weight16t == nullptr || Output == nullptr) return SWC_ERR_NULL_POINTER;
    if ((InScale == nullptr) != (InShift == nullptr) || (OutScale == nullptr) != (OutShift == nullptr))
        return SWC_ERR_NULL_POINTER;
    if (C <= 0 || B <= 0 || H <= 0 || W <= 0 || K <= 0) return SWC_ERR_BAD_DIMS;
    if (pad_h != 1 || pad_w != 1) return SWC_ERR_BAD_PAD;
    const int nH = (H + 1) / 2, nW = (W + 1) / 2;
    const size_t M = static_cast<size_t>(B) * nH * nW;
    if (M >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    // 16 channels per chunk read as float4, 16-byte weight copies, 32-bit byte offsets into the operands.
    const bool ok = (C % GBK == 0) && aligned16(Input) && aligned16(Weight16t) &&
                    (InScale == nullptr || (aligned16(InScale) && aligned16(InShift))) &&
                    static_cast<size_t>(B) * H * W * C < (1ull << 30) && static_cast<size_t>(16) * C * K < (1ull << 30);
    if (!ok) return SWC_ERR_UNSUPPORTED;
    const size_t tiles_m = (M + GBM - 1) / GBM, tiles_n = (static_cast<size_t>(K) + GBN - 1) / GBN;
    if (tiles_m * tiles_n >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid(static_cast<unsigned>(tiles_m * tiles_n)), block(256);
    ConvEpilogue ep;
    ep.scale = OutScale;
    ep.shift = OutShift;
    ep.residual = Residual;
    const int variant = (relu ? 1 : 0) + (InScale != nullptr ? 2 : 0);
    auto kern = variant == 0   ? relu_conv_fused_bf16_kernel<false, false>
                : variant == 1 ? relu_conv_fused_bf16_kernel<true, false>
                : variant == 2 ? relu_conv_fused_bf16_kernel<false, true>
                               : relu_conv_fused_bf16_kernel<true, true>;
    // 128 KiB of LDS is above the default 64 KiB limit, which is raised once per kernel and device.
    constexpr int kMaxDevices = 64;
    static thread_local bool raised[kMaxDevices][4] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SWC_ERR_HIP;
    if (!raised[dev][variant]) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, GSMEM_BYTES);
        if (e != hipSuccess) return note_hip_error(e);
        raised[dev][variant] = true;
    }
    kern<<<grid, block, GSMEM_BYTES, s>>>(Input, InScale, InShift, Weight16t, Output, M, H, W, C, K, nH, nW,
                                          static_cast<unsigned>(tiles_n), ep);
    return check_launch();
}
