// Fused Winograd-ReLU convolution layer for gfx950: input transform, Winograd-domain ReLU,
// the 16 per-position GEMMs and the output transform in one kernel.  The transformed activations
// (4x the input in size) never reach memory.
//
// Computes exactly what swc_winograd2x2_imtrans (relu) followed by swc_winograd2x2_conv computes,
// i.e. the layer pair WinogradImTrans(relu) -> WinogradConv of the reference model
// (ResNet-18-var/imagenet-resnet-transWino-prune.py:118-119), which there runs as
// Winograd2x2ImTransCompute, tf.nn.relu, cublasSgemmBatched and Output_transform with three
// full-size intermediates in between.
//
// Structure.  A workgroup (4 wavefronts) owns 64 tiles x 64 output channels and walks the input
// channels 8 at a time.  For a chunk of 8 channels it holds, in LDS, the transformed activations
// of its 64 tiles for all 16 positions (produced by its own threads from the NHWC input with the
// reference's left-to-right sums, so values and zero masks are bit-identical to the stand-alone
// transform) and the 16 weight slices [8 x 64] (copied global -> LDS directly).  Each wavefront
// accumulates its 32x32 tile of all 16 products P_0..P_15 at once, 256 accumulator registers, and
// folds them into the four output tiles only at the very end, in ascending position order (the
// association of winograd2x2_conv_cuda.cu.cc:39-46).  With the positions innermost there is one
// barrier per 64 MFMAs, 16 independent accumulation chains per wavefront, and the producer's
// arithmetic for the next chunk rides between the MFMAs of the current one.

#include "winograd2x2_conv_kernel.h"

namespace swc {
namespace {

constexpr int FBM = 64, FBN = 64, FBK = 8;                 // tiles x output channels x channels per chunk
constexpr int FA_FLOATS = 16 * FBM * FBK;                  // transformed activations of a chunk, all positions
constexpr int FB_FLOATS = 16 * FBK * FBN;                  // weight slices of a chunk, all positions
constexpr int FSTAGE_FLOATS = FA_FLOATS + FB_FLOATS;       // 64 KiB
constexpr int FSMEM_BYTES = 2 * FSTAGE_FLOATS * 4;         // double buffered: 128 KiB
constexpr int FB_COPIES = FB_FLOATS / 4 / 256;             // 16-byte copies per thread per chunk: 8

// The 16 sums of the input transform for one channel, each left to right
// (winograd2x2_imTrans_cuda.cu.cc:112-127); `I` selects which one.
template <int I>
__device__ __forceinline__ float bt_d_b_one(const float (&d)[16])
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

template <bool RELU>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void relu_conv_fused_kernel(
    const float *__restrict__ X, const float *__restrict__ Wt, float *__restrict__ Out, size_t M, int H, int W, int C,
    int K, int nH, int nW, unsigned tiles_n)
{
    extern __shared__ __attribute__((aligned(1024))) float smem[];

    const unsigned lid = xcd_swizzle(blockIdx.x, gridDim.x);
    const size_t m0 = static_cast<size_t>(lid / tiles_n) * FBM;
    const int n0 = static_cast<int>(lid % tiles_n) * FBN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lg = lane >> 5;
    const int wm0 = (wave >> 1) * 32, wn0 = (wave & 1) * 32;

    // ---- producer: this thread transforms 2 channels (pc, pc+1 of the chunk) of tile row pr ----
    const int pr = tid >> 2, pc = (tid & 3) * 2;
    unsigned pix_off[16];   // byte offset of the patch pixel's channel 0 (+pc) in X; 0 where padded
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
                pix_off[4 * r + s] = in ? static_cast<unsigned>(((static_cast<size_t>(b) * H + y) * W + x) * C + pc) * 4u : 0u;
                pix_valid |= in ? (1u << (4 * r + s)) : 0u;
            }
    }
    // where this thread's outputs go in a stage: row pr, 16-byte half (pc/4) swizzled by row bit 3 (rows r and r+8 of an operand read share banks otherwise)
    const int a_wr_off = pr * FBK + (((pc >> 2) ^ ((pr >> 3) & 1)) << 2) + (pc & 3);

    // ---- weight copies: 16-byte slot s = q*256 + tid of the chunk's [16][8][64] block ----------
    unsigned b_voff[FB_COPIES];
#pragma unroll
    for (int q = 0; q < FB_COPIES; ++q) {
        const unsigned s = q * 256 + tid;
        const unsigned pos = s / (FBK * FBN / 4), rem = s % (FBK * FBN / 4);
        const unsigned k = rem / (FBN / 4);
        unsigned n = n0 + (rem % (FBN / 4)) * 4;
        n = n + 4 <= static_cast<unsigned>(K) ? n : static_cast<unsigned>(K) - 4;  // columns beyond K: clamped, never stored
        b_voff[q] = ((pos * static_cast<unsigned>(C) + k) * K + n) * 4u;
    }
    const unsigned smem_base = lds_address(smem);
    const unsigned wave_lds = __builtin_amdgcn_readfirstlane(wave) * 1024u;

    // ---- consumer offsets (floats within a stage) -----------------------------------------------
    const int a_rd_off = (wm0 + li) * FBK + ((lg ^ (((wm0 + li) >> 3) & 1)) << 2);
    const int b_rd_off = FA_FLOATS + 4 * lg * FBN + wn0 + li;

    floatx16 P[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) P[i][r] = 0.f;

    const int nchunks = C / FBK;

    float2 raw[16];
    auto load_raw = [&](int c0) {
        const char *xc = reinterpret_cast<const char *>(X + c0);
#pragma unroll
        for (int j = 0; j < 16; ++j) raw[j] = *reinterpret_cast<const float2 *>(xc + pix_off[j]);
    };
    auto copy_b = [&](int c0, int stage) {
        const float *wc = Wt + static_cast<size_t>(c0) * K;
        const unsigned dst = smem_base + stage * (FSTAGE_FLOATS * 4) + FA_FLOATS * 4 + wave_lds;
#pragma unroll
        for (int q = 0; q < FB_COPIES; ++q) async_copy16(wc, b_voff[q], dst + q * 4096);
    };
    // Transformed value I of the chunk held in `raw`, both channels, written to plane I of `stage`.
    auto produce = [&](auto i_tag, int stage) {
        constexpr int I = decltype(i_tag)::value;
        float dx[16], dy[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const bool in = (pix_valid >> j) & 1u;
            dx[j] = in ? raw[j].x : 0.f;
            dy[j] = in ? raw[j].y : 0.f;
        }
        float tx = bt_d_b_one<I>(dx), ty = bt_d_b_one<I>(dy);
        if (RELU) {
            tx = tx > 0.f ? tx : 0.f;
            ty = ty > 0.f ? ty : 0.f;
        }
        *reinterpret_cast<float2 *>(&smem[stage * FSTAGE_FLOATS + I * (FBM * FBK) + a_wr_off]) = make_float2(tx, ty);
    };

    // ---- prologue: chunk 0 into stage 0, the weights of chunk 1 on their way -------------------
    copy_b(0, 0);
    load_raw(0);
    static_for<16>([&](auto i_tag) { produce(i_tag, 0); });
    if (nchunks > 1) {
        copy_b(FBK, 1);
        wait_vmcnt<FB_COPIES>();  // everything but chunk 1's copies
    } else {
        wait_vmcnt<0>();
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    // ---- main loop over channel chunks ------------------------------------------------------------
    // Timeline of iteration `it` (64 MFMAs per wavefront on stage it&1):
    //   start        the input pixels of chunk it+1 are requested (16 loads per thread);
    //   positions 0-7   MFMAs only (plus the LDS operand reads, one position pair ahead);
    //   positions 8-15  two of the producer's 16 outputs for chunk it+1 ride along per position:
    //                   the loads have had half an iteration to arrive;
    //   end          wait for the weight copies of chunk it+1 (issued an iteration ago), barrier,
    //                then request the weights of chunk it+2 into the stage just vacated.
    for (int it = 0; it < nchunks; ++it) {
        const int cur = it & 1, nxt = cur ^ 1;
        const float *st = smem + cur * FSTAGE_FLOATS;
        if (it + 1 < nchunks) load_raw((it + 1) * FBK);

        float4 a[2][2];
        float b[2][2][4];
        auto read_pair = [&](int buf, int p) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                a[buf][e] = *reinterpret_cast<const float4 *>(&st[(p + e) * (FBM * FBK) + a_rd_off]);
#pragma unroll
                for (int t = 0; t < 4; ++t) b[buf][e][t] = st[(p + e) * (FBK * FBN) + b_rd_off + t * FBN];
            }
        };
        read_pair(0, 0);
        static_for<8>([&](auto pp_tag) {
            constexpr int pp = decltype(pp_tag)::value;
            constexpr int buf = pp & 1;
            if (pp + 1 < 8) read_pair(buf ^ 1, 2 * (pp + 1));
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float4 a4 = a[buf][e];
                    const float av = t == 0 ? a4.x : t == 1 ? a4.y : t == 2 ? a4.z : a4.w;
                    P[2 * pp + e] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, b[buf][e][t], P[2 * pp + e], 0, 0, 0);
                }
                // On the last iteration this rewrites stage `nxt` from stale registers: nobody reads it.
                if (pp >= 4) {
                    if (t == 0) produce(std::integral_constant<int, (pp >= 4 ? 4 * (pp - 4) : 0) + 0>{}, nxt);
                    if (t == 1) produce(std::integral_constant<int, (pp >= 4 ? 4 * (pp - 4) : 0) + 1>{}, nxt);
                    if (t == 2) produce(std::integral_constant<int, (pp >= 4 ? 4 * (pp - 4) : 0) + 2>{}, nxt);
                    if (t == 3) produce(std::integral_constant<int, (pp >= 4 ? 4 * (pp - 4) : 0) + 3>{}, nxt);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        });

        // Stage `nxt` is complete once this thread's weight copies into it have landed and everyone
        // has written its transformed rows; stage `cur` is free once everyone has read it.
        wait_vmcnt<0>();
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (it + 2 < nchunks) copy_b((it + 2) * FBK, cur);
    }

    // ---- fold the 16 products into the four output tiles, ascending position -------------------
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
    using StoreCfg = ConvCfg<FBM, FBN, 32, 2, 2>;
    const unsigned rows_valid = static_cast<unsigned>(M - m0 < FBM ? M - m0 : FBM);
    store_output<StoreCfg>(Y, Out, rows_valid, K, nW, m0, n0, wm0, wn0, li, lg);
}

}  // namespace
}  // namespace swc

extern "C" int swc_winograd2x2_relu_conv(const float *Input, const float *Weight, float *Output, int C, int B, int H,
                                         int W, int K, int pad_h, int pad_w, int relu, swc_stream_t stream)
{
    using namespace swc;
    if (Input == nullptr || Weight == nullptr || Output == nullptr) return SWC_ERR_NULL_POINTER;
    if (C <= 0 || B <= 0 || H <= 0 || W <= 0 || K <= 0) return SWC_ERR_BAD_DIMS;
    if (pad_h != 1 || pad_w != 1) return SWC_ERR_BAD_PAD;
    const int nH = (H + 1) / 2, nW = (W + 1) / 2;
    const size_t M = static_cast<size_t>(B) * nH * nW;
    if (M >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    // 8 channels per chunk read as float2, 16-byte weight copies, 32-bit byte offsets into the input.
    const bool ok = (C % FBK == 0) && (K % 4 == 0) && aligned16(Weight) && ((reinterpret_cast<uintptr_t>(Input) & 7u) == 0) &&
                    static_cast<size_t>(B) * H * W * C < (1ull << 30) && static_cast<size_t>(16) * C * K < (1ull << 30);
    if (!ok) return SWC_ERR_UNSUPPORTED;
    const size_t tiles_m = (M + FBM - 1) / FBM, tiles_n = (static_cast<size_t>(K) + FBN - 1) / FBN;
    if (tiles_m * tiles_n >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid(static_cast<unsigned>(tiles_m * tiles_n)), block(256);
    // 128 KiB of LDS is above the default 64 KiB limit, which is raised once per kernel and device.
    auto kern = relu ? relu_conv_fused_kernel<true> : relu_conv_fused_kernel<false>;
    constexpr int kMaxDevices = 64;
    static thread_local bool raised[kMaxDevices][2] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SWC_ERR_HIP;
    if (!raised[dev][relu ? 1 : 0]) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, FSMEM_BYTES);
        if (e != hipSuccess) return note_hip_error(e);
        raised[dev][relu ? 1 : 0] = true;
    }
    kern<<<grid, block, FSMEM_BYTES, s>>>(Input, Weight, Output, M, H, W, C, K, nH, nW, static_cast<unsigned>(tiles_n));
    return check_launch();
}
