// Winograd F(2x2,3x3) input transform T = B^T d B with the Winograd-domain ReLU fused,
// for gfx950.  NHWC [B,H,W,C] -> [16,B,nH,nW,C], 4x4 tiles at stride 2, pad 1.
//
// Stands in for Winograd2x2ImTransCompute / Winograd2x2ImTransComputeLauncher of the
// reference (winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans_cuda.cu.cc:11-157)
// plus the tf.nn.relu its layer wrapper applies afterwards
// (ResNet-18-var/winograd_imtrans.py:16-17).
//
// The kernel is a pure stream: 4 bytes read and 64 bytes written per (tile, channel)
// with 48 adds, so HBM bandwidth bounds it.  Channels are the contiguous axis, a lane
// owns VEC consecutive channels and never needs another lane's data.


#include "swc_common.h"

namespace swc {
namespace {

// The 16 sums, each left to right in fp32, exactly as the reference writes them
// (winograd2x2_imTrans_cuda.cu.cc:112-127).  There are no multiplies, hence nothing
// for the compiler to contract, and fp adds are not reassociated without fast-math:
// results are bit-identical to the reference's.
__device__ __forceinline__ void bt_d_b(const float (&d)[16], float (&t)[16])
{
    t[0]  = d[0] - d[2] - d[8] + d[10];
    t[1]  = d[1] + d[2] - d[9] - d[10];
    t[2]  = d[2] - d[1] + d[9] - d[10];
    t[3]  = d[1] - d[3] - d[9] + d[11];
    t[4]  = d[4] - d[6] + d[8] - d[10];
    t[5]  = d[5] + d[6] + d[9] + d[10];
    t[6]  = d[6] - d[5] - d[9] + d[10];
    t[7]  = d[5] - d[7] + d[9] - d[11];
    t[8]  = d[6] - d[4] + d[8] - d[10];
    t[9]  = d[9] - d[6] - d[5] + d[10];
    t[10] = d[5] - d[6] - d[9] + d[10];
    t[11] = d[7] - d[5] + d[9] - d[11];
    t[12] = d[4] - d[6] - d[12] + d[14];
    t[13] = d[5] + d[6] - d[13] - d[14];
    t[14] = d[6] - d[5] + d[13] - d[14];
    t[15] = d[5] - d[7] - d[13] + d[15];
}

template <int VEC>
struct Vec;
template <>
struct Vec<1> {
    using type = float;
    static __device__ __forceinline__ float get(const float &v, int) { return v; }
    static __device__ __forceinline__ void set(float &v, int, float x) { v = x; }
    static __device__ __forceinline__ float zero() { return 0.0f; }
};
template <>
struct Vec<4> {
    using type = float4;
    static __device__ __forceinline__ float get(const float4 &v, int q)
    {
        return q == 0 ? v.x : q == 1 ? v.y : q == 2 ? v.z : v.w;
    }
    static __device__ __forceinline__ void set(float4 &v, int q, float x)
    {
        if (q == 0) v.x = x; else if (q == 1) v.y = x; else if (q == 2) v.z = x; else v.w = x;
    }
    static __device__ __forceinline__ float4 zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
};

// How the transformed planes are stored decides where the convolution that reads them next finds them.
// The planes are written once and read by a later kernel, never by this one.
//   fp32 planes up to 64 MiB: ordinary stores.  The planes stay in the 256 MB Infinity Cache and the
//     convolution reads them from there (7x7x512 at batch 64: the pair takes 84 us, 98 us when the planes are
//     streamed to HBM; 14x14x256: 79 vs 80 us, 52 vs 61 us with the bf16-operand convolution).
//   fp32 planes above 64 MiB: nontemporal stores, streamed past the caches.  With ordinary stores the kernel
//     is 45 % slower once its output is not already cache-resident (28x28x128 at batch 64, 103 MB of planes:
//     31 us against 21 us; every line it writes first evicts a dirty one), and the fp32 convolution, bound by
//     the matrix pipes, takes the same time either way (pair 86 us warm, 94 us cold with both).  The
//     bf16-operand convolution over fp32 planes is the one that loses: its pair takes 66 us streamed, 52 us
//     with ordinary stores.
//   bf16 planes up to 128 MiB: written through as they are issued (the agent-scope form of a store, sc1) but
//     still allocated in the Infinity Cache, because the bf16 convolution is bound by reading them (its step
//     is 25 % slower when they come from HBM); above that they cannot stay resident and are streamed.
// Two 8-byte agent-scope stores per float4 are not an option for fp32: 43 us instead of 21 us.
typedef float floatx4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void stream_store(float *p, float v) { __builtin_nontemporal_store(v, p); }
__device__ __forceinline__ void stream_store(float *p, const float4 &v)
{
    const floatx4_t t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<floatx4_t *>(p));
}
__device__ __forceinline__ void through_store(unsigned short *p, unsigned short v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void through_store(unsigned short *p, uint2 v)  // p is 8-byte aligned
{
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(p), (static_cast<unsigned long long>(v.y) << 32) | v.x,
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

typedef float floatx2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned pack_bf16(float lo, float hi)
{
    const bf16x2_t p = __builtin_convertvector(floatx2_t{lo, hi}, bf16x2_t);  // v_cvt_pk_bf16_f32, RNE
    return __builtin_bit_cast(unsigned, p);
}
typedef unsigned uintx2_t __attribute__((ext_vector_type(2)));
// OUT (the kernel's store mode): 0 = fp32 planes streamed, 3 = fp32 planes with ordinary stores,
// 1 = bf16 planes written through, 2 = bf16 planes streamed.
template <int OUT>
__device__ __forceinline__ void store_bf16(unsigned short *p, float v)
{
    const unsigned short h = static_cast<unsigned short>(pack_bf16(v, 0.f));
    if (OUT == 2)
        __builtin_nontemporal_store(h, p);
    else
        through_store(p, h);
}
template <int OUT>
__device__ __forceinline__ void store_bf16(unsigned short *p, const float4 &v)
{
    const uint2 h = make_uint2(pack_bf16(v.x, v.y), pack_bf16(v.z, v.w));
    if (OUT == 2) {
        const uintx2_t t = {h.x, h.y};
        __builtin_nontemporal_store(t, reinterpret_cast<uintx2_t *>(p));
    } else {
        through_store(p, h);
    }
}

template <int VEC, bool RELU>
__device__ __forceinline__ void transform_vec(const typename Vec<VEC>::type (&d)[16], typename Vec<VEC>::type (&t)[16])
{
#pragma unroll
    for (int q = 0; q < VEC; ++q) {
        float ds[16], ts[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) ds[j] = Vec<VEC>::get(d[j], q);
        bt_d_b(ds, ts);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float v = ts[i];
            if (RELU) v = v > 0.0f ? v : 0.0f;
            Vec<VEC>::set(t[i], q, v);
        }
    }
}

// One lane per (tile, channel vector).  Lanes are numbered along the flattened
// [M, C/VEC] plane of the output, so each of the 16 stores of a wavefront covers
// 64*VEC*4 contiguous bytes of one plane whatever C is; the 16 loads of a wavefront
// are contiguous per tile and overlap between neighbouring tiles in L1/L2.
//
// AFFINE: every pixel inside the image is first mapped to fma(x, scale[c], shift[c]) (an inference-mode
// batch normalisation folded into the load); the zero padding stays zero, as it does when the
// normalisation runs as its own pass before the transform.
template <int VEC, bool RELU, bool AFFINE, int OUT, typename Idx>
__global__ __launch_bounds__(256) void imtrans_direct_kernel(const float *__restrict__ X, float *__restrict__ TI,
                                                             const float *__restrict__ scale,
                                                             const float *__restrict__ shift, int H, int W, int C,
                                                             int nH, int nW, Idx items, size_t plane)
{
    using V = typename Vec<VEC>::type;
    // Consecutive logical blocks share input rows (the halo between tile rows, the overlap
    // between neighbouring tiles); keeping them on one XCD lets its L2 serve the re-reads
    // instead of every XCD fetching the same rows again.
    const Idx idx = static_cast<Idx>(xcd_swizzle(blockIdx.x, gridDim.x)) * 256 + threadIdx.x;
    if (idx >= items) return;
    const int CV = C / VEC;
    const int cv = static_cast<int>(idx % CV);
    Idx m = idx / CV;
    const int tw = static_cast<int>(m % nW);
    m /= nW;
    const int th = static_cast<int>(m % nH);
    const size_t b = static_cast<size_t>(m / nH);

    const int y0 = 2 * th - 1, x0 = 2 * tw - 1;
    const float *img = X + b * H * W * C + static_cast<size_t>(cv) * VEC;
    V d[16];
    V sc = Vec<VEC>::zero(), sh = Vec<VEC>::zero();
    if (AFFINE) {
        sc = *reinterpret_cast<const V *>(scale + static_cast<size_t>(cv) * VEC);
        sh = *reinterpret_cast<const V *>(shift + static_cast<size_t>(cv) * VEC);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int y = y0 + r;
        const bool yin = (y > -1) && (y < H);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int x = x0 + s;
            const bool in = yin && (x > -1) && (x < W);
            V v = Vec<VEC>::zero();
            if (in) {
                v = *reinterpret_cast<const V *>(img + (static_cast<size_t>(y) * W + x) * C);
                if (AFFINE) {
#pragma unroll
                    for (int q = 0; q < VEC; ++q)
                        Vec<VEC>::set(v, q, __builtin_fmaf(Vec<VEC>::get(v, q), Vec<VEC>::get(sc, q), Vec<VEC>::get(sh, q)));
                }
            }
            d[4 * r + s] = v;
        }
    }
    V t[16];
    transform_vec<VEC, RELU>(d, t);
    if (OUT == 1 || OUT == 2) {
        // the planes are stored as bf16 (round to nearest even): TI is then [16,B,nH,nW,C] of 2-byte elements
        unsigned short *dst16 = reinterpret_cast<unsigned short *>(TI) + static_cast<size_t>(idx) * VEC;
#pragma unroll
        for (int i = 0; i < 16; ++i) store_bf16<OUT>(dst16 + i * plane, t[i]);
        return;
    }
    float *dst = TI + static_cast<size_t>(idx) * VEC;
    if (OUT == 3) {
        V *dv = reinterpret_cast<V *>(dst);
#pragma unroll
        for (int i = 0; i < 16; ++i) dv[i * (plane / VEC)] = t[i];
        return;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) stream_store(dst + i * plane, t[i]);
}

template <int VEC, bool RELU, bool AFFINE, typename Idx>
int launch_direct(const float *X, const float *scale, const float *shift, float *TI, int B, int H, int W, int C, int nH,
                  int nW, bool bf16_out, hipStream_t stream)
{
    const size_t M = static_cast<size_t>(B) * nH * nW;
    const size_t items = M * (C / VEC);
    const size_t blocks = (items + 255) / 256;
    const dim3 grid(static_cast<unsigned>(blocks)), block(256);
    // Store mode by the size of the planes (see the store helpers above).
    if (bf16_out && 16 * M * C * 2 > (128ull << 20))
        imtrans_direct_kernel<VEC, RELU, AFFINE, 2, Idx><<<grid, block, 0, stream>>>(
            X, TI, scale, shift, H, W, C, nH, nW, static_cast<Idx>(items), M * C);
    else if (bf16_out)
        imtrans_direct_kernel<VEC, RELU, AFFINE, 1, Idx><<<grid, block, 0, stream>>>(
            X, TI, scale, shift, H, W, C, nH, nW, static_cast<Idx>(items), M * C);
    else if (16 * M * C * 4 <= (64ull << 20))
        imtrans_direct_kernel<VEC, RELU, AFFINE, 3, Idx><<<grid, block, 0, stream>>>(
            X, TI, scale, shift, H, W, C, nH, nW, static_cast<Idx>(items), M * C);
    else
        imtrans_direct_kernel<VEC, RELU, AFFINE, 0, Idx><<<grid, block, 0, stream>>>(
            X, TI, scale, shift, H, W, C, nH, nW, static_cast<Idx>(items), M * C);
    return check_launch();
}

template <bool AFFINE>
int imtrans_entry(const float *Input, const float *Scale, const float *Shift, float *TransIm, int C, int B, int H, int W,
                  int pad_h, int pad_w, int relu, bool bf16_out, swc_stream_t stream)
{
    if (Input == nullptr || TransIm == nullptr) return SWC_ERR_NULL_POINTER;
    if (AFFINE && (Scale == nullptr || Shift == nullptr)) return SWC_ERR_NULL_POINTER;
    if (C <= 0 || B <= 0 || H <= 0 || W <= 0) return SWC_ERR_BAD_DIMS;
    if (pad_h != 1 || pad_w != 1) return SWC_ERR_BAD_PAD;
    const int nH = (H + 1) / 2, nW = (W + 1) / 2;
    const size_t M = static_cast<size_t>(B) * nH * nW;
    // One lane per item, 256 per workgroup, grid.x below 2^31.
    if (M * C / 256 >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // a lane's 4 channels are 16 bytes of fp32 or 8 bytes of bf16
    const bool vec = (C % 4 == 0) && aligned16(Input) &&
                     (bf16_out ? (reinterpret_cast<uintptr_t>(TransIm) & 7u) == 0 : aligned16(TransIm)) &&
                     (!AFFINE || (aligned16(Scale) && aligned16(Shift)));
    const bool small = M * C < (1ull << 31);
#define SWC_DISPATCH(VEC, RELU)                                                                                    \
    (small ? launch_direct<VEC, RELU, AFFINE, unsigned>(Input, Scale, Shift, TransIm, B, H, W, C, nH, nW, bf16_out, s) \
           : launch_direct<VEC, RELU, AFFINE, unsigned long long>(Input, Scale, Shift, TransIm, B, H, W, C, nH, nW, bf16_out, s))
    if (vec) return relu ? SWC_DISPATCH(4, true) : SWC_DISPATCH(4, false);
    return relu ? SWC_DISPATCH(1, true) : SWC_DISPATCH(1, false);
#undef SWC_DISPATCH
}

}  // namespace
}  // namespace swc

extern "C" int swc_winograd2x2_imtrans(const float *Input, float *TransIm, int C, int B, int H, int W,
                                       int pad_h, int pad_w, int relu, swc_stream_t stream)
{
    return swc::imtrans_entry<false>(Input, nullptr, nullptr, TransIm, C, B, H, W, pad_h, pad_w, relu, false, stream);
}

extern "C" int swc_winograd2x2_imtrans_affine(const float *Input, const float *Scale, const float *Shift,
                                              float *TransIm, int C, int B, int H, int W, int pad_h, int pad_w,
                                              int relu, swc_stream_t stream)
{
    return swc::imtrans_entry<true>(Input, Scale, Shift, TransIm, C, B, H, W, pad_h, pad_w, relu, false, stream);
}

extern "C" int swc_winograd2x2_imtrans_bf16out(const float *Input, const float *Scale, const float *Shift,
                                               unsigned short *TransIm16, int C, int B, int H, int W, int pad_h,
                                               int pad_w, int relu, swc_stream_t stream)
{
    float *out = reinterpret_cast<float *>(TransIm16);
    if ((Scale == nullptr) != (Shift == nullptr)) return SWC_ERR_NULL_POINTER;
    if (Scale != nullptr)
        return swc::imtrans_entry<true>(Input, Scale, Shift, out, C, B, H, W, pad_h, pad_w, relu, true, stream);
    return swc::imtrans_entry<false>(Input, nullptr, nullptr, out, C, B, H, W, pad_h, pad_w, relu, true, stream);
}
