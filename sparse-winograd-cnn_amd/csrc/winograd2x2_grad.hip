// Backward of the two Winograd ops for gfx950.
//
// Stand in for Winograd2x2ConvGradComputeLauncher
// (winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_grad_cuda.cu.cc:77-124) and
// Winograd2x2ImTransGradComputeLauncher
// (winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans_grad_cuda.cu.cc:118-129).
//
// Conv grad keeps the reference's structure: dP = A dY A^T into the caller's 16*M*K temporary,
// then two batched GEMMs, both on this library's own MFMA kernels (the reference calls cublasSgemmBatched
// twice).  dTI = dP . W^T walks the 16 positions per workgroup like the forward kernel and stores each
// product plane as it is finished (conv_dgrad_async_kernel, winograd2x2_conv_kernel.h).  dW = TI^T . dP
// reduces over the tens of thousands of rows of M into a tiny output; it runs on the split-reduction kernel of
// winograd2x2_wgrad_kernel.h.  Shapes neither takes (odd channel counts, unaligned pointers) go to one
// plain tiled kernel.  ImTrans grad is one gather kernel: a lane
// produces the 2x2 input pixels its tile is centred on from the entries of B dT B^T that fall on
// them -- its own tile's and the up to 8 neighbouring tiles', handed over through LDS inside a
// workgroup's block of tiles -- optionally through the fused ReLU's mask; the incoming gradient is
// not modified (the reference transforms it in place first, :124).

#include <cstdio>
#include <mutex>

#include "swc_common.h"
#include "winograd2x2_conv_launch.h"
#include "winograd2x2_dgrad_wide_kernel.h"
#include "winograd2x2_wgrad_kernel.h"
#include "winograd2x2_wgrad_wide_kernel.h"

namespace swc {
namespace {

// ---- dP = A dY A^T (Grad_inverse_transform, winograd2x2_conv_grad_cuda.cu.cc:12-66) -------------
template <int VEC>
struct GVec;
template <>
struct GVec<1> {
    using type = float;
};
template <>
struct GVec<4> {
    using type = float4;
};
__device__ __forceinline__ float neg(float a) { return -a; }
__device__ __forceinline__ float4 neg(float4 a) { return make_float4(-a.x, -a.y, -a.z, -a.w); }
__device__ __forceinline__ float add(float a, float b) { return a + b; }
__device__ __forceinline__ float sub(float a, float b) { return a - b; }
__device__ __forceinline__ float4 add(float4 a, float4 b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }
__device__ __forceinline__ float4 sub(float4 a, float4 b) { return make_float4(a.x - b.x, a.y - b.y, a.z - b.z, a.w - b.w); }

// One lane per (tile, VEC output channels), numbered along the flattened [M, K/VEC] plane so that
// each of the 16 stores of a wavefront is contiguous in its plane.
template <int VEC>
__global__ __launch_bounds__(256) void output_transform_grad_kernel(const float *__restrict__ dY, float *__restrict__ dP,
                                                                    int nW, int K, unsigned items, size_t plane)
{
    using V = typename GVec<VEC>::type;
    const unsigned idx = xcd_swizzle(blockIdx.x, gridDim.x) * 256 + threadIdx.x;
    if (idx >= items) return;
    const unsigned KV = K / VEC;
    const unsigned kv = idx % KV, m = idx / KV;
    const unsigned tw = m % nW, bt = m / nW;  // bt = b*nH + th
    const size_t oW = 2 * static_cast<size_t>(nW);
    const float *g = dY + ((static_cast<size_t>(bt) * 2 * oW + 2 * tw) * K + static_cast<size_t>(kv) * VEC);
    const V a = *reinterpret_cast<const V *>(g), b = *reinterpret_cast<const V *>(g + K);
    const V c = *reinterpret_cast<const V *>(g + oW * K), d = *reinterpret_cast<const V *>(g + oW * K + K);
    V p[16];
    // the expressions of winograd2x2_conv_grad_cuda.cu.cc:28-43, left to right
    p[0] = a;                           p[1] = add(a, b);                   p[2] = sub(a, b);                   p[3] = neg(b);
    p[4] = add(a, c);                   p[5] = add(add(add(a, b), c), d);   p[6] = sub(add(sub(a, b), c), d);   p[7] = sub(neg(b), d);
    p[8] = sub(a, c);                   p[9] = sub(sub(add(a, b), c), d);   p[10] = add(sub(sub(a, b), c), d);  p[11] = sub(d, b);
    p[12] = neg(c);                     p[13] = sub(neg(c), d);             p[14] = sub(d, c);                  p[15] = d;
    float *dst = dP + static_cast<size_t>(idx) * VEC;
#pragma unroll
    for (int i = 0; i < 16; ++i) *reinterpret_cast<V *>(dst + i * plane) = p[i];
}


// ---- dX = col2im(B dT B^T) (+ ReLU mask) ----------------------------------------------------------
// Along one axis, pixel y lies in tile y/2 and in one neighbour; with patch offset r = y + 1 - 2*tile,
// (B dT B^T)[r][.] = sum_u BT[u][r] dT[u][.], BT = [[1,0,-1,0],[0,1,1,0],[0,-1,1,0],[0,1,0,-1]].
// A gather, one lane per (tile, VEC channels) producing the tile's four interior pixels
// (2th+a, 2tw+b), a, b in {0,1}.  Pixel (a,b) sits at patch offset (1+a, 1+b) of its own tile, at row
// 3 / 0 of the tile above / below (a = 0 / 1), at column 3 / 0 of the tile to the left / right
// (b = 0 / 1), and at a corner of the diagonal neighbour.  With
//   row(r)[v] = sum_u BT[u][r] dT[u][v]   (r=0: +u0   r=1: +u1 -u2 +u3   r=2: -u0 +u1 +u2   r=3: -u3)
// and the same combination over v for the column, the own tile needs all 16 planes once, each edge
// neighbour one row or column of 4 planes and each corner one plane: 36 loads for 4 pixels where the
// per-pixel form issues 64.
// Plane p of B^T d B from the 16 pixels of a patch, as the forward kernel evaluates it: the four
// terms of winograd2x2_imTrans_cuda.cu.cc:112-127 added left to right (only additions, so the value
// and its sign are those of the forward pass bit for bit).  ld(j) yields pixel j = 4r + s.
template <typename V, typename L>
__device__ __forceinline__ V plane_of_patch(int p, L ld)
{
    constexpr signed char term[16][4] = {{0, 2, 8, 10},  {1, 2, 9, 10},  {2, 1, 9, 10},   {1, 3, 9, 11},
                                         {4, 6, 8, 10},  {5, 6, 9, 10},  {6, 5, 9, 10},   {5, 7, 9, 11},
                                         {6, 4, 8, 10},  {9, 6, 5, 10},  {5, 6, 9, 10},   {7, 5, 9, 11},
                                         {4, 6, 12, 14}, {5, 6, 13, 14}, {6, 5, 13, 14},  {5, 7, 13, 15}};
    constexpr signed char sign[16][3] = {{-1, -1, 1}, {1, -1, -1}, {-1, 1, -1}, {-1, -1, 1},
                                         {-1, 1, -1}, {1, 1, 1},   {-1, -1, 1}, {-1, 1, -1},
                                         {-1, 1, -1}, {-1, -1, 1}, {-1, -1, 1}, {-1, 1, -1},
                                         {-1, -1, 1}, {1, -1, -1}, {-1, 1, -1}, {-1, -1, 1}};
    V t = ld(term[p][0]);
#pragma unroll
    for (int q = 0; q < 3; ++q) t = sign[p][q] > 0 ? add(t, ld(term[p][q + 1])) : sub(t, ld(term[p][q + 1]));
    return t;
}

// How the gradient is masked: not at all, by the sign of the forward result (mask_src = TI), or by
// the sign of the forward result recomputed from the forward input (mask_src = X [B,H,W,C], a
// quarter of TI's bytes).
enum { IG_NO_MASK = 0, IG_MASK_TI = 1, IG_MASK_INPUT = 2 };

// A workgroup takes a block of IG_TILES tiles of one image, rh rows by rw = 1 << rw_shift columns,
// and IG_LANES channel vectors of each.  Every lane loads its own tile's 16 planes once and leaves in
// LDS the 12 sums its neighbours need of them (two per edge, one per corner); a neighbour inside the
// block is read from there, one outside it from memory as above.  With every neighbour read from
// memory the kernel fetched 1.9 times the planes' size: the planes in flight exceed the L2 by far,
// so a second reader rarely hits.
constexpr int IG_LANES = 8;    // channel vectors per tile in a workgroup (128 contiguous bytes at VEC 4)
constexpr int IG_THREADS = 256;
constexpr int IG_TILES = IG_THREADS / IG_LANES;
// slots of the exchange: what a tile offers to the tile below, above, to the right, to the left
// (two sums each) and to its four diagonal neighbours
enum { IG_TO_BELOW = 0, IG_TO_ABOVE = 2, IG_TO_RIGHT = 4, IG_TO_LEFT = 6, IG_C33 = 8, IG_C30 = 9, IG_C03 = 10, IG_C00 = 11, IG_SLOTS = 12 };

// grid.x = cgroups * blocks_x * blocks_y * B
template <int VEC, int MASK>
__global__ __launch_bounds__(IG_THREADS) void imtrans_grad_tile_kernel(const float *__restrict__ dT,
                                                                       const float *__restrict__ mask_src,
                                                                       float *__restrict__ dX, int H, int W, int C, int nH,
                                                                       int nW, unsigned cgroups, unsigned blocks_x,
                                                                       unsigned blocks_y, int rw_shift, size_t plane)
{
    using V = typename GVec<VEC>::type;
    __shared__ V ex[IG_SLOTS][IG_THREADS];
    // consecutive logical ids are the channel groups of one block of tiles
    unsigned id = xcd_swizzle(blockIdx.x, gridDim.x);
    const unsigned cgroup = id % cgroups;
    id /= cgroups;
    const unsigned bxi = id % blocks_x;
    id /= blocks_x;
    const unsigned byi = id % blocks_y, b = id / blocks_y;
    const unsigned CV = C / VEC;
    const unsigned cv = cgroup * IG_LANES + threadIdx.x % IG_LANES;
    const int tl = threadIdx.x / IG_LANES;            // tile within the block
    const int rw = 1 << rw_shift, rh = IG_TILES >> rw_shift;
    const int ty = tl >> rw_shift, tx = tl & (rw - 1);
    const int th = static_cast<int>(byi) * rh + ty, tw = static_cast<int>(bxi) * rw + tx;
    const bool valid = th < nH && tw < nW && cv < CV;
    // pixel j = 4r + s of the patch of tile (th+dy, tw+dx) of the forward input, zero outside the image
    auto pixel = [&](int dy, int dx, int j) __attribute__((always_inline)) -> V {
        const int y = 2 * (th + dy) - 1 + j / 4, x = 2 * (tw + dx) - 1 + j % 4;
        V d = {};
        if (y >= 0 && y < H && x >= 0 && x < W)
            d = *reinterpret_cast<const V *>(mask_src + ((static_cast<size_t>(b) * H + y) * W + x) * C + static_cast<size_t>(cv) * VEC);
        return d;
    };
    // masked gradient of plane 4u+v at tile (th+dy, tw+dx)
    auto g = [&](int u, int v, int dy, int dx) __attribute__((always_inline)) -> V {
        const size_t off = static_cast<size_t>(4 * u + v) * plane +
                           ((static_cast<size_t>(b) * nH + (th + dy)) * nW + (tw + dx)) * C + static_cast<size_t>(cv) * VEC;
        V x = *reinterpret_cast<const V *>(dT + off);
        if (MASK != IG_NO_MASK) {
            const V t = MASK == IG_MASK_TI ? *reinterpret_cast<const V *>(mask_src + off)
                                           : plane_of_patch<V>(4 * u + v, [&](int j) __attribute__((always_inline)) { return pixel(dy, dx, j); });
            float *xp = reinterpret_cast<float *>(&x);
            const float *tp = reinterpret_cast<const float *>(&t);
#pragma unroll
            for (int q = 0; q < VEC; ++q) xp[q] = tp[q] > 0.f ? xp[q] : 0.f;
        }
        return x;
    };
    // combination over one axis: offset 1 -> +e1 -e2 +e3, offset 2 -> -e0 +e1 +e2
    auto mid = [](int a, V e0, V e1, V e2, V e3) __attribute__((always_inline)) -> V {
        return a == 0 ? add(sub(e1, e2), e3) : add(sub(e1, e0), e2);
    };
    V out[2][2];
    if (valid) {   // own tile: rows 1+a, then columns 1+b; and what the neighbours need of it
        V t[4][4];
        if (MASK == IG_MASK_INPUT) {
            // the own tile's patch is loaded once; bit p of keep[q] says whether plane p passed the ReLU
            unsigned keep[VEC] = {};
            {
                V d[16];
#pragma unroll
                for (int j = 0; j < 16; ++j) d[j] = pixel(0, 0, j);
#pragma unroll
                for (int p = 0; p < 16; ++p) {
                    const V tp = plane_of_patch<V>(p, [&](int j) __attribute__((always_inline)) { return d[j]; });
                    const float *tq = reinterpret_cast<const float *>(&tp);
#pragma unroll
                    for (int q = 0; q < VEC; ++q) keep[q] |= (tq[q] > 0.f ? 1u : 0u) << p;
                }
            }
#pragma unroll
            for (int p = 0; p < 16; ++p) {
                const size_t off = static_cast<size_t>(p) * plane +
                                   ((static_cast<size_t>(b) * nH + th) * nW + tw) * C + static_cast<size_t>(cv) * VEC;
                V x = *reinterpret_cast<const V *>(dT + off);
                float *xp = reinterpret_cast<float *>(&x);
#pragma unroll
                for (int q = 0; q < VEC; ++q) xp[q] = (keep[q] >> p) & 1u ? xp[q] : 0.f;
                t[p / 4][p % 4] = x;
            }
        } else {
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int v = 0; v < 4; ++v) t[u][v] = g(u, v, 0, 0);
        }
        V row[2][4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            row[0][v] = mid(0, t[0][v], t[1][v], t[2][v], t[3][v]);
            row[1][v] = mid(1, t[0][v], t[1][v], t[2][v], t[3][v]);
        }
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int bb = 0; bb < 2; ++bb) out[a][bb] = mid(bb, row[a][0], row[a][1], row[a][2], row[a][3]);
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            ex[IG_TO_BELOW + q][threadIdx.x] = mid(q, t[3][0], t[3][1], t[3][2], t[3][3]);
            ex[IG_TO_ABOVE + q][threadIdx.x] = mid(q, t[0][0], t[0][1], t[0][2], t[0][3]);
            ex[IG_TO_RIGHT + q][threadIdx.x] = mid(q, t[0][3], t[1][3], t[2][3], t[3][3]);
            ex[IG_TO_LEFT + q][threadIdx.x] = mid(q, t[0][0], t[1][0], t[2][0], t[3][0]);
        }
        ex[IG_C33][threadIdx.x] = t[3][3];
        ex[IG_C30][threadIdx.x] = t[3][0];
        ex[IG_C03][threadIdx.x] = t[0][3];
        ex[IG_C00][threadIdx.x] = t[0][0];
    }
    __syncthreads();
    if (!valid) return;

    const bool up = th > 0, down = th + 1 < nH, left = tw > 0, right = tw + 1 < nW;
    // the neighbour at (dy, dx) is lane threadIdx.x + nb(dy, dx) of this workgroup if its tile is in the block
    auto nb = [&](int dy, int dx) __attribute__((always_inline)) { return (dy * rw + dx) * IG_LANES; };
    auto inside = [&](int dy, int dx) __attribute__((always_inline)) {
        return ty + dy >= 0 && ty + dy < rh && tx + dx >= 0 && tx + dx < rw;
    };
    if (up) {      // row 3 of the tile above: -dT[3][v]
        V s0, s1;
        if (inside(-1, 0)) {
            s0 = ex[IG_TO_BELOW][threadIdx.x + nb(-1, 0)];
            s1 = ex[IG_TO_BELOW + 1][threadIdx.x + nb(-1, 0)];
        } else {
            const V e0 = g(3, 0, -1, 0), e1 = g(3, 1, -1, 0), e2 = g(3, 2, -1, 0), e3 = g(3, 3, -1, 0);
            s0 = mid(0, e0, e1, e2, e3);
            s1 = mid(1, e0, e1, e2, e3);
        }
        out[0][0] = sub(out[0][0], s0);
        out[0][1] = sub(out[0][1], s1);
    }
    if (down) {    // row 0 of the tile below: +dT[0][v]
        V s0, s1;
        if (inside(1, 0)) {
            s0 = ex[IG_TO_ABOVE][threadIdx.x + nb(1, 0)];
            s1 = ex[IG_TO_ABOVE + 1][threadIdx.x + nb(1, 0)];
        } else {
            const V e0 = g(0, 0, 1, 0), e1 = g(0, 1, 1, 0), e2 = g(0, 2, 1, 0), e3 = g(0, 3, 1, 0);
            s0 = mid(0, e0, e1, e2, e3);
            s1 = mid(1, e0, e1, e2, e3);
        }
        out[1][0] = add(out[1][0], s0);
        out[1][1] = add(out[1][1], s1);
    }
    if (left) {    // column 3 of the tile to the left: -dT[u][3]
        V s0, s1;
        if (inside(0, -1)) {
            s0 = ex[IG_TO_RIGHT][threadIdx.x + nb(0, -1)];
            s1 = ex[IG_TO_RIGHT + 1][threadIdx.x + nb(0, -1)];
        } else {
            const V e0 = g(0, 3, 0, -1), e1 = g(1, 3, 0, -1), e2 = g(2, 3, 0, -1), e3 = g(3, 3, 0, -1);
            s0 = mid(0, e0, e1, e2, e3);
            s1 = mid(1, e0, e1, e2, e3);
        }
        out[0][0] = sub(out[0][0], s0);
        out[1][0] = sub(out[1][0], s1);
    }
    if (right) {   // column 0 of the tile to the right: +dT[u][0]
        V s0, s1;
        if (inside(0, 1)) {
            s0 = ex[IG_TO_LEFT][threadIdx.x + nb(0, 1)];
            s1 = ex[IG_TO_LEFT + 1][threadIdx.x + nb(0, 1)];
        } else {
            const V e0 = g(0, 0, 0, 1), e1 = g(1, 0, 0, 1), e2 = g(2, 0, 0, 1), e3 = g(3, 0, 0, 1);
            s0 = mid(0, e0, e1, e2, e3);
            s1 = mid(1, e0, e1, e2, e3);
        }
        out[0][1] = add(out[0][1], s0);
        out[1][1] = add(out[1][1], s1);
    }
    // corners: (-1)(-1) dT[3][3], (-1)(+1) dT[3][0], (+1)(-1) dT[0][3], (+1)(+1) dT[0][0]
    if (up && left) out[0][0] = add(out[0][0], inside(-1, -1) ? ex[IG_C33][threadIdx.x + nb(-1, -1)] : g(3, 3, -1, -1));
    if (up && right) out[0][1] = sub(out[0][1], inside(-1, 1) ? ex[IG_C30][threadIdx.x + nb(-1, 1)] : g(3, 0, -1, 1));
    if (down && left) out[1][0] = sub(out[1][0], inside(1, -1) ? ex[IG_C03][threadIdx.x + nb(1, -1)] : g(0, 3, 1, -1));
    if (down && right) out[1][1] = add(out[1][1], inside(1, 1) ? ex[IG_C00][threadIdx.x + nb(1, 1)] : g(0, 0, 1, 1));
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int bb = 0; bb < 2; ++bb) {
            const int y = 2 * th + a, x = 2 * tw + bb;
            if (y < H && x < W)
                *reinterpret_cast<V *>(dX + ((static_cast<size_t>(b) * H + y) * W + x) * C + static_cast<size_t>(cv) * VEC) = out[a][bb];
        }
}

// ---- any shape, any alignment: Out_i [P x Q] = sum_r A_i(p, r) . B_i(r, q), i = 0..15 ---------------------
// Element (p, r) of A_i sits at A + i*a_batch + p*a_p + r*a_r (likewise B with b_r, b_q), so the same kernel
// serves dTI_i = dP_i . W_i^T and dW_i = TI_i^T . dP_i.  A 32x32 output tile per workgroup, 32 reduction
// indices per step through LDS, one fp32 fma per product: only the shapes the MFMA kernels do not take
// (C or K not a multiple of 4, M not a multiple of 32, unaligned pointers) come here.
__global__ __launch_bounds__(256) void gemm16_plain_kernel(const float *__restrict__ A, const float *__restrict__ Bm,
                                                           float *__restrict__ Out, int P, int Q, int Rn, size_t a_batch,
                                                           size_t a_p, size_t a_r, size_t b_batch, size_t b_r, size_t b_q,
                                                           unsigned tiles_q, unsigned tiles_p)
{
    __shared__ float As[32][33], Bs[32][33];
    unsigned id = blockIdx.x;
    const unsigned tq = id % tiles_q;
    id /= tiles_q;
    const unsigned tp = id % tiles_p, i = id / tiles_p;
    const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;  // ty = 0..7
    const float *a = A + i * a_batch, *b = Bm + i * b_batch;
    const int p0 = static_cast<int>(tp) * 32, q0 = static_cast<int>(tq) * 32;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int r0 = 0; r0 < Rn; r0 += 32) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int row = ty + 8 * k;  // tile row: p for A, r for B
            if (a_p == 1) {  // p is A's fast axis (dW: A = TI^T): the 32 lanes walk p so that a load is one 128-byte line
                const int pa = p0 + tx, ra = r0 + row;
                As[tx][row] = pa < P && ra < Rn ? a[pa + ra * a_r] : 0.f;
            } else {
                const int pa = p0 + row, ra = r0 + tx;
                As[row][tx] = pa < P && ra < Rn ? a[pa * a_p + ra * a_r] : 0.f;
            }
            const int rb = r0 + row, qb = q0 + tx;
            Bs[row][tx] = rb < Rn && qb < Q ? b[rb * b_r + qb * b_q] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 32; ++r) {
            const float bv = Bs[r][tx];
#pragma unroll
            for (int k = 0; k < 4; ++k) acc[k] = __builtin_fmaf(As[ty + 8 * k][r], bv, acc[k]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int p = p0 + ty + 8 * k, q = q0 + tx;
        if (p < P && q < Q) Out[(static_cast<size_t>(i) * P + p) * Q + q] = acc[k];
    }
}

int gemm16_plain(const float *A, const float *Bm, float *Out, size_t P, int Q, size_t Rn, size_t a_batch, size_t a_p,
                 size_t a_r, size_t b_batch, size_t b_r, size_t b_q, hipStream_t s)
{
    const size_t tiles_p = (P + 31) / 32, tiles_q = (static_cast<size_t>(Q) + 31) / 32;
    if (16 * tiles_p * tiles_q >= (1ull << 31) || P >= (1ull << 31) || Rn >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    gemm16_plain_kernel<<<dim3(static_cast<unsigned>(16 * tiles_p * tiles_q)), dim3(256), 0, s>>>(
        A, Bm, Out, static_cast<int>(P), Q, static_cast<int>(Rn), a_batch, a_p, a_r, b_batch, b_r, b_q,
        static_cast<unsigned>(tiles_q), static_cast<unsigned>(tiles_p));
    return check_launch();
}

// dTI [16][M][C] = dP [16][M][K] . W [16][C][K]^T on the ring kernel.  The 16 products are independent, so
// the grid is (pairs of positions) x (64x64 tiles): eight times the workgroups of the forward pass, each an
// eighth as long as one that walks all 16 positions, four resident per SIMD (the product accumulators are all the
// registers a wave needs here).  Short workgroups at different points of their loops overlap each other's
// waits and product stores, and the tile count no longer has to divide by the CU count.  Measured against
// the forward pass's tilings walking all 16 positions (us, dense operands): 28x28x128 at batch 64 67.7 (tall16
// 76.3), at batch 128 146.7 (152.5); 14x14x256 at batch 64 67.8 (short16 78.9); 56x56x64 87.9 (93.4);
// 7x7x512 77.1 (short16 95.6).  One, two or four positions per workgroup, two to four waves per SIMD and 128-row
// or 128-column tiles were within 5 % of this on some shapes and 10-20 % slower on others.
// SWC_ERR_UNSUPPORTED when the ring kernel does not take the shapes (K % 32, alignment, 32-bit offsets).
using DgradTile = ConvCfg<64, 64, 32, 2, 2, 4>;
constexpr int kDgradPositions = 2;

// dTI on 48-row x 128-column workgroups that walk all 16 positions (winograd2x2_dgrad_wide_kernel.h): 28x28x128 at
// batch 64 takes 6.125 tile units per SIMD this way where 64x64 tiles need 6.5 and leave a ragged last round.
// SWC_ERR_UNSUPPORTED when the shapes do not fit or too few workgroups would run.
int dgrad_wide(const float *dP, const float *W, float *dTI, size_t M, int C, int K, bool forced, hipStream_t s)
{
    if (K % 64 != 0 || C % 128 != 0 || !aligned16(dP) || !aligned16(W) || !aligned16(dTI) || M < 48 || M >= (1ull << 31) ||
        M * static_cast<size_t>(K > C ? K : C) * 4 >= (1ull << 31) || static_cast<size_t>(C) * K * 4 >= (1ull << 31))
        return SWC_ERR_UNSUPPORTED;
    const size_t cus = device_cus(), tiles_n = static_cast<size_t>(C) / 128;
    auto passes_of = [&](size_t wgs) { return static_cast<double>((wgs + cus - 1) / cus); };
    // levelled row groups in whole rounds of the chip
    const size_t gmin = (M + 47) / 48;
    size_t groups = (gmin * tiles_n + cus - 1) / cus * cus / tiles_n;
    if (groups < gmin) groups = gmin;
    size_t rows = (M + groups - 1) / groups;
    groups = (M + rows - 1) / rows;
    size_t main_rows = M, extra_wgs = 0;
    double units = passes_of(groups * tiles_n) * 6.0;
    // or full 48-row groups in whole rounds, the rest by position: workgroups of 6/16 of a unit each, resident beside
    // the others
    size_t g2 = (M / 48) * tiles_n / cus * cus / tiles_n;
    if (g2 == 0) g2 = M / 48;
    const size_t left_groups = (M - g2 * 48 + 47) / 48;
    const double units2 = passes_of(g2 * tiles_n) * 6.0 + passes_of(left_groups * tiles_n * 16) * 6.0 / 16.0;
    if (left_groups > 0 && units2 < units) {
        groups = g2;
        rows = 48;
        main_rows = g2 * 48;
        extra_wgs = left_groups * tiles_n * 16;
        units = units2;
    }
    // Against the 64x64-tile kernel (four of its workgroups to a SIMD, any number of tiles): worth it when the
    // rounds come out nearly full.
    const double ideal = static_cast<double>(M) * C / 256.0 / (4.0 * cus);  // tile units per SIMD with no rounding at all
    if (!forced && (units > 1.08 * ideal || groups * tiles_n < cus)) return SWC_ERR_UNSUPPORTED;
    using Wd = WideDgradCfg;
    static_assert(2 * Wd::LDS_BYTES <= 160 * 1024, "two workgroups per CU");
    const size_t n_main = groups * tiles_n;
    if (n_main + extra_wgs >= (1ull << 29)) return SWC_ERR_BAD_DIMS;
    conv_dgrad_wide_kernel<<<dim3(static_cast<unsigned>(n_main + extra_wgs)), dim3(Wd::NT), Wd::LDS_BYTES, s>>>(
        dP, W, dTI, static_cast<unsigned>(M), C, K, static_cast<unsigned>(tiles_n), static_cast<unsigned>(rows),
        static_cast<unsigned>(main_rows), static_cast<unsigned>(n_main));
    return check_launch();
}

int dgrad_own(const float *dP, const float *W, float *dTI, size_t M, int C, int K, hipStream_t s)
{
    // swc_winograd2x2_conv_force_tiling applies to the data gradient as well: "wide48" forces the wide kernel where
    // the shapes allow it, any other name the 64x64-tile kernel.
    const char *forced = forced_conv_tiling();
    const bool force_wide = forced != nullptr && std::string_view(forced) == "wide48";
    if (forced == nullptr || force_wide) {
        const int st = dgrad_wide(dP, W, dTI, M, C, K, force_wide, s);
        if (st != SWC_ERR_UNSUPPORTED) return st;
    }
    // 32-bit offsets: elements within a workgroup's rows of a plane, bytes within a position's weights
    if (static_cast<size_t>(DgradTile::BM) * C >= (1ull << 30) || static_cast<size_t>(C) * K >= (1ull << 30))
        return SWC_ERR_UNSUPPORTED;
    if (!ring_eligible<DgradTile>(dP, W, K, C, false)) return SWC_ERR_UNSUPPORTED;
    constexpr int kStages = 2;  // a third ring slot (stores waited for a step later) measured no faster
    constexpr int lds_bytes = async_lds_bytes<DgradTile, kStages, RING_DGRAD>();
    static_assert(lds_bytes <= 64 * 1024, "below the default dynamic LDS limit");
    const size_t tiles_m = (M + DgradTile::BM - 1) / DgradTile::BM;
    const size_t tiles_n = (static_cast<size_t>(C) + DgradTile::BN - 1) / DgradTile::BN;
    const size_t groups = 16 / kDgradPositions;
    if (groups * tiles_m * tiles_n >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    conv_dgrad_async_kernel<DgradTile, kStages, kDgradPositions>
        <<<dim3(static_cast<unsigned>(groups * tiles_m * tiles_n)), dim3(DgradTile::NT), lds_bytes, s>>>(
            dP, W, dTI, M, C, K, static_cast<unsigned>(tiles_m), static_cast<unsigned>(tiles_n),
            static_cast<unsigned>(DgradTile::BM));
    return check_launch();
}

// dW through the split-reduction kernel.  The partial tiles of the S row splits are parked in the
// dTI buffer, which the caller owns, which is at least S*16*C*K floats when S*K <= M, and which is
// only written (in full) by the dTI GEMM that runs afterwards.  Returns SWC_ERR_UNSUPPORTED when the
// shapes do not fit the kernel.
// dW on 128x128 tiles (wgrad_wide_kernel): one workgroup per CU in total, the rows split S ways.
using WgradWide = WgradWideCfg<16, 3, 2>;
int wgrad_wide(const float *TI, const float *dP, float *dW, float *scratch, size_t M, int C, int K, hipStream_t s)
{
    if (M % WgradWide::BKM != 0 || C % 128 != 0 || K % 128 != 0) return SWC_ERR_UNSUPPORTED;
    if (static_cast<size_t>(WgradWide::BKM) * C >= (1ull << 29) || static_cast<size_t>(WgradWide::BKM) * K >= (1ull << 29))
        return SWC_ERR_UNSUPPORTED;  // 32-bit byte offsets within a tile
    const size_t tiles_c = static_cast<size_t>(C) / 128, tiles_k = static_cast<size_t>(K) / 128;
    const size_t base = 16 * tiles_c * tiles_k;
    const size_t steps_total = M / WgradWide::BKM;
    const size_t cus = device_cus();
    size_t S = base >= cus ? 1 : (cus + base / 2) / base;
    if (S > M / K) S = M / K;   // the partial tiles are parked in the dTI buffer: S*16*C*K <= 16*M*C floats
    if (S > steps_total) S = steps_total;
    if (S < 1) S = 1;
    const size_t per = (steps_total + S - 1) / S;
    S = (steps_total + per - 1) / per;  // no empty split
    if (S * base >= (1ull << 31)) return SWC_ERR_UNSUPPORTED;
    const size_t nw = static_cast<size_t>(16) * C * K;
    wgrad_wide_kernel<WgradWide><<<dim3(static_cast<unsigned>(S * base)), dim3(WgradWide::NT), WgradWide::LDS_BYTES, s>>>(
        TI, dP, S == 1 ? dW : scratch, M, C, K, static_cast<unsigned>(tiles_c), static_cast<unsigned>(tiles_k),
        static_cast<unsigned>(per), static_cast<unsigned>(steps_total), nw);
    int st = check_launch();
    if (st != SWC_OK || S == 1) return st;
    const unsigned n4 = static_cast<unsigned>(nw / 4);
    wgrad_reduce_kernel<<<dim3((n4 + 255) / 256), dim3(256), 0, s>>>(scratch, dW, n4, static_cast<unsigned>(S), nw);
    return check_launch();
}

int wgrad_own(const float *TI, const float *dP, float *dW, float *scratch, size_t M, int C, int K, hipStream_t s)
{
    if (C % 4 != 0 || K % 4 != 0 || !aligned16(TI) || !aligned16(dP) || !aligned16(dW) || !aligned16(scratch))
        return SWC_ERR_UNSUPPORTED;
    // "wide48" forces the 128x128 tiles where the shapes allow them, any other forced tiling the 64x64 kernel
    const char *forced = forced_conv_tiling();
    if (forced == nullptr || std::string_view(forced) == "wide48") {
        const int st = wgrad_wide(TI, dP, dW, scratch, M, C, K, s);
        if (st != SWC_ERR_UNSUPPORTED) return st;
    }
    if (M % WG_BK != 0) return SWC_ERR_UNSUPPORTED;
    if (static_cast<size_t>(WG_BK) * C >= (1ull << 29) || static_cast<size_t>(WG_BK) * K >= (1ull << 29))
        return SWC_ERR_UNSUPPORTED;  // 32-bit byte offsets within a tile
    const size_t tiles_c = (static_cast<size_t>(C) + WG_BM - 1) / WG_BM, tiles_k = (static_cast<size_t>(K) + WG_BN - 1) / WG_BN;
    const size_t base = 16 * tiles_c * tiles_k;
    const size_t steps_total = M / WG_BK;
    // Two workgroups per CU measured best (conv3: 61 us with 512 workgroups, 65-70 with 256 or 768+).
    size_t S = base >= 512 ? 1 : (512 + base - 1) / base;
    if (S > M / K) S = M / K;
    if (S > steps_total) S = steps_total;
    if (S < 1) S = 1;
    const size_t per = (steps_total + S - 1) / S;
    S = (steps_total + per - 1) / per;  // no empty split
    if (S * base >= (1ull << 31)) return SWC_ERR_UNSUPPORTED;
    const size_t nw = static_cast<size_t>(16) * C * K;
    wgrad_splitk_kernel<<<dim3(static_cast<unsigned>(S * base)), dim3(256), WG_LDS_BYTES, s>>>(
        TI, dP, S == 1 ? dW : scratch, M, C, K, static_cast<unsigned>(tiles_c), static_cast<unsigned>(tiles_k),
        static_cast<unsigned>(per), static_cast<unsigned>(steps_total), nw);
    int st = check_launch();
    if (st != SWC_OK || S == 1) return st;
    const unsigned n4 = static_cast<unsigned>(nw / 4);
    wgrad_reduce_kernel<<<dim3((n4 + 255) / 256), dim3(256), 0, s>>>(scratch, dW, n4, static_cast<unsigned>(S), nw);
    return check_launch();
}

}  // namespace
}  // namespace swc

namespace swc {
namespace {

// The whole backward of the convolution; dP is the 16*M*K-float buffer that holds A dY A^T between the kernels.
int conv_grad_impl(const float *TInput, const float *Weight, const float *Output_grad, float *TInput_grad,
                   float *Weight_grad, float *dP, int C, int B, int H, int W, int K, int pad_h, int pad_w, hipStream_t s)
{
    if (TInput == nullptr || Weight == nullptr || Output_grad == nullptr || TInput_grad == nullptr ||
        Weight_grad == nullptr || dP == nullptr)
        return SWC_ERR_NULL_POINTER;
    if (C <= 0 || B <= 0 || H <= 0 || W <= 0 || K <= 0 || (H & 1) || (W & 1)) return SWC_ERR_BAD_DIMS;  // H = 2nH, W = 2nW
    if (pad_h != 1 || pad_w != 1) return SWC_ERR_BAD_PAD;
    const int nH = H / 2, nW = W / 2;
    // each factor is below 2^31, so B*nH fits 64 bits; the bound on it keeps the next product from wrapping
    const size_t bh = static_cast<size_t>(B) * nH;
    if (bh >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    const size_t M = bh * nW;
    if (M >= (1ull << 31) || M * K >= (1ull << 32) || M * C >= (1ull << 40)) return SWC_ERR_BAD_DIMS;

    const bool vec = (K % 4 == 0) && aligned16(Output_grad) && aligned16(dP);
    const unsigned items = static_cast<unsigned>(M * (vec ? K / 4 : K));
    const dim3 grid((items + 255) / 256), block(256);
    if (vec)
        output_transform_grad_kernel<4><<<grid, block, 0, s>>>(Output_grad, dP, nW, K, items, M * K);
    else
        output_transform_grad_kernel<1><<<grid, block, 0, s>>>(Output_grad, dP, nW, K, items, M * K);
    int st = check_launch();
    if (st != SWC_OK) return st;

    // dW first: its partial sums borrow the dTI buffer before the dTI GEMM fills it.
    st = wgrad_own(TInput, dP, Weight_grad, TInput_grad, M, C, K, s);
    if (st == SWC_ERR_UNSUPPORTED) {
        // Row-major dW[i] (C x K) = TI[i]^T (C x M) . dP[i] (M x K): the call at winograd2x2_conv_grad_cuda.cu.cc:115-120.
        st = gemm16_plain(TInput, dP, Weight_grad, static_cast<size_t>(C), K, M, M * C, 1, static_cast<size_t>(C), M * K,
                          static_cast<size_t>(K), 1, s);
    }
    if (st != SWC_OK) return st;
    // Row-major dTI[i] (M x C) = dP[i] (M x K) . W[i]^T (K x C): the call at winograd2x2_conv_grad_cuda.cu.cc:103-108.
    st = dgrad_own(dP, Weight, TInput_grad, M, C, K, s);
    if (st != SWC_ERR_UNSUPPORTED) return st;
    return gemm16_plain(dP, Weight, TInput_grad, M, C, static_cast<size_t>(K), M * K, static_cast<size_t>(K), 1,
                        static_cast<size_t>(C) * K, 1, static_cast<size_t>(K), s);
}

}  // namespace
}  // namespace swc

extern "C" int swc_winograd2x2_conv_grad(const float *TInput, const float *Weight, const float *Output_grad,
                                         float *TInput_grad, float *Weight_grad, float *tmp_data_buffer,
                                         long long *tmp_ptr_buffer, int C, int B, int H, int W, int K, int pad_h,
                                         int pad_w, swc_stream_t stream)
{
    (void)tmp_ptr_buffer;
    return swc::conv_grad_impl(TInput, Weight, Output_grad, TInput_grad, Weight_grad, tmp_data_buffer, C, B, H, W, K, pad_h,
                               pad_w, static_cast<hipStream_t>(stream));
}

// ---- the same backward pass for callers that cannot allocate ------------------------------------------------------
// The dP buffer lives in a fixed array in device memory (each GPU the library runs on holds its own copy until the
// process ends).  In host code the array's name stands for the symbol, not for a device address: the address on the
// current device comes from hipGetSymbolAddress, once per device, and only that pointer is handed to kernels.
namespace swc {
namespace {

constexpr size_t kStaticScratchFloats = SWC_CONV_GRAD_STATIC_MAX_FLOATS;
static __device__ __align__(256) float scratch[kStaticScratchFloats];

float *static_scratch(int *status)
{
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static float *ptrs[kMaxDevices] = {};
    int dev = 0;
    const hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        *status = e != hipSuccess ? note_hip_error(e) : SWC_ERR_HIP;
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(mu);
    if (ptrs[dev] == nullptr) {
        void *p = nullptr;
        const hipError_t es = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (es != hipSuccess || p == nullptr) {
            *status = es != hipSuccess ? note_hip_error(es) : SWC_ERR_HIP;
            return nullptr;
        }
        ptrs[dev] = static_cast<float *>(p);
    }
    *status = SWC_OK;
    return ptrs[dev];
}

}  // namespace
}  // namespace swc

extern "C" int swc_winograd2x2_conv_grad_static(const float *TInput, const float *Weight, const float *Output_grad,
                                                float *TInput_grad, float *Weight_grad, int C, int B, int H, int W, int K,
                                                int pad_h, int pad_w, swc_stream_t stream)
{
    if (C <= 0 || B <= 0 || H <= 0 || W <= 0 || K <= 0 || (H & 1) || (W & 1)) return SWC_ERR_BAD_DIMS;
    // dP holds 16*M*K floats, M = B*(H/2)*(W/2).  The products are bounded one factor at a time: a product of
    // four ints taken at once could wrap to a small value and slip past the limit.
    const size_t bh = static_cast<size_t>(B) * (H / 2);
    if (bh > swc::kStaticScratchFloats) return SWC_ERR_TOO_LARGE;
    const size_t M = bh * (W / 2);
    if (M > swc::kStaticScratchFloats || M * K > swc::kStaticScratchFloats / 16) return SWC_ERR_TOO_LARGE;
    int st = SWC_OK;
    float *dP = swc::static_scratch(&st);
    if (dP == nullptr) return st;
    return swc::conv_grad_impl(TInput, Weight, Output_grad, TInput_grad, Weight_grad, dP, C, B, H, W, K, pad_h, pad_w,
                               static_cast<hipStream_t>(stream));
}

namespace swc {
namespace {
// mask_mode: IG_NO_MASK (mask_source unused), IG_MASK_TI (mask_source = the forward result [16,B,nH,nW,C]) or
// IG_MASK_INPUT (mask_source = the forward input [B,H,W,C]).
int imtrans_grad_entry(const float *TransIm_grad, const float *relu_mask_source, int mask_mode, float *Input_grad, int C,
                       int B, int H, int W, int pad_h, int pad_w, swc_stream_t stream)
{
    if (TransIm_grad == nullptr || Input_grad == nullptr) return SWC_ERR_NULL_POINTER;
    if (C <= 0 || B <= 0 || H <= 0 || W <= 0) return SWC_ERR_BAD_DIMS;
    if (pad_h != 1 || pad_w != 1) return SWC_ERR_BAD_PAD;
    const int nH = (H + 1) / 2, nW = (W + 1) / 2;
    const size_t pixels = static_cast<size_t>(B) * H * W;
    if (pixels * C >= (1ull << 32)) return SWC_ERR_BAD_DIMS;
    const size_t plane = static_cast<size_t>(B) * nH * nW * C;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool vec = (C % 4 == 0) && aligned16(TransIm_grad) && aligned16(Input_grad) &&
                     (relu_mask_source == nullptr || aligned16(relu_mask_source));
    // one lane per (tile, channel vector): each writes the four pixels its tile is centred on
    const unsigned CV = static_cast<unsigned>(vec ? C / 4 : C);
    const unsigned cgroups = (CV + IG_LANES - 1) / IG_LANES;
    // Block shape: the one that reads the fewest planes.  A block of rh x rw tiles reads 16 planes per
    // tile and 4 per tile of its rim; lanes beyond the image's edge idle (weighted a quarter of a read).
    int rw_shift = 0;
    unsigned blocks_x = 0, blocks_y = 0;
    double best = 0;
    for (int sh = 0; (1 << sh) <= IG_TILES; ++sh) {
        const int rw = 1 << sh, rh = IG_TILES >> sh;
        const unsigned bx = (nW + rw - 1) / rw, by = (nH + rh - 1) / rh;
        const double blocks = static_cast<double>(bx) * by;
        const double cost = blocks * (2 * (rw < nW ? rw : nW) * (by > 1) + 2 * (rh < nH ? rh : nH) * (bx > 1)) * 4 +
                            (blocks * IG_TILES - static_cast<double>(nH) * nW) * 4;
        if (blocks_x == 0 || cost <= best) {  // ties go to the wider block
            best = cost;
            rw_shift = sh;
            blocks_x = bx;
            blocks_y = by;
        }
    }
    const size_t wgs = static_cast<size_t>(cgroups) * blocks_x * blocks_y * B;
    if (wgs >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    const dim3 grid(static_cast<unsigned>(wgs)), block(IG_THREADS);
#define SWC_LAUNCH(VEC, MASK)                                                                                   \
    imtrans_grad_tile_kernel<VEC, MASK><<<grid, block, 0, s>>>(TransIm_grad, relu_mask_source, Input_grad, H, W, C, \
                                                               nH, nW, cgroups, blocks_x, blocks_y, rw_shift, plane)
    if (vec) {
        if (mask_mode == IG_MASK_TI) SWC_LAUNCH(4, IG_MASK_TI);
        else if (mask_mode == IG_MASK_INPUT) SWC_LAUNCH(4, IG_MASK_INPUT);
        else SWC_LAUNCH(4, IG_NO_MASK);
    } else {
        if (mask_mode == IG_MASK_TI) SWC_LAUNCH(1, IG_MASK_TI);
        else if (mask_mode == IG_MASK_INPUT) SWC_LAUNCH(1, IG_MASK_INPUT);
        else SWC_LAUNCH(1, IG_NO_MASK);
    }
#undef SWC_LAUNCH
    return check_launch();
}
}  // namespace
}  // namespace swc

// Out [M][K] = Input [M][C] . Weight [K][C]^T: a 1x1 convolution over NHWC pixels.  It is one position of the data
// gradient's product with the roles renamed, so it runs on the same kernel, one plane per workgroup.
extern "C" int swc_winograd2x2_pointwise_conv(const float *Input, const float *Weight, float *Output, int C, long long M,
                                              int K, swc_stream_t stream)
{
    using namespace swc;
    if (Input == nullptr || Weight == nullptr || Output == nullptr) return SWC_ERR_NULL_POINTER;
    if (C <= 0 || K <= 0 || M <= 0 || M >= (1ll << 31)) return SWC_ERR_BAD_DIMS;
    // reduction over C in whole 32-index steps, 16-byte copies, 32-bit offsets within a tile's rows and the weights
    if (static_cast<size_t>(DgradTile::BM) * K >= (1ull << 30) || static_cast<size_t>(C) * K >= (1ull << 30) ||
        !ring_eligible<DgradTile>(Input, Weight, C, K, false))
        return SWC_ERR_UNSUPPORTED;
    constexpr int kStages = 2;
    constexpr int lds_bytes = async_lds_bytes<DgradTile, kStages, RING_DGRAD>();
    const size_t rows = static_cast<size_t>(M);
    const size_t tiles_m = (rows + DgradTile::BM - 1) / DgradTile::BM;
    const size_t tiles_n = (static_cast<size_t>(K) + DgradTile::BN - 1) / DgradTile::BN;
    if (tiles_m * tiles_n >= (1ull << 31)) return SWC_ERR_BAD_DIMS;
    conv_dgrad_async_kernel<DgradTile, kStages, 1>
        <<<dim3(static_cast<unsigned>(tiles_m * tiles_n)), dim3(DgradTile::NT), lds_bytes, static_cast<hipStream_t>(stream)>>>(
            Input, Weight, Output, rows, K, C, static_cast<unsigned>(tiles_m), static_cast<unsigned>(tiles_n),
            static_cast<unsigned>(DgradTile::BM));
    return check_launch();
}

extern "C" int swc_winograd2x2_imtrans_grad(const float *TransIm_grad, const float *relu_mask_source, float *Input_grad,
                                            int C, int B, int H, int W, int pad_h, int pad_w, swc_stream_t stream)
{
    return swc::imtrans_grad_entry(TransIm_grad, relu_mask_source, relu_mask_source ? swc::IG_MASK_TI : swc::IG_NO_MASK,
                                   Input_grad, C, B, H, W, pad_h, pad_w, stream);
}

extern "C" int swc_winograd2x2_imtrans_grad_relu_input(const float *TransIm_grad, const float *Input, float *Input_grad,
                                                       int C, int B, int H, int W, int pad_h, int pad_w,
                                                       swc_stream_t stream)
{
    if (Input == nullptr) return SWC_ERR_NULL_POINTER;
    return swc::imtrans_grad_entry(TransIm_grad, Input, swc::IG_MASK_INPUT, Input_grad, C, B, H, W, pad_h, pad_w, stream);
}


void Winograd2x2ConvGradComputeLauncher(const float *TInput, const float *Weight, const float *Output_grad,
                                        float *TInput_grad, float *Weight_grad, float *tmp_data_buffer,
                                        long long *tmp_ptr_buffer, int C, int B, int H, int W, int K, int pad_h, int pad_w)
{
    const int st = swc_winograd2x2_conv_grad(TInput, Weight, Output_grad, TInput_grad, Weight_grad, tmp_data_buffer,
                                             tmp_ptr_buffer, C, B, H, W, K, pad_h, pad_w, nullptr);
    if (st != SWC_OK) std::fprintf(stderr, "Winograd2x2ConvGradComputeLauncher: %s\n", swc_strerror(st));
}

void Winograd2x2ImTransGradComputeLauncher(const float *Output_grad, float *Input_grad, int C, int B, int H, int W,
                                           int pad_h, int pad_w)
{
    const int st = swc_winograd2x2_imtrans_grad(Output_grad, nullptr, Input_grad, C, B, H, W, pad_h, pad_w, nullptr);
    if (st != SWC_OK) std::fprintf(stderr, "Winograd2x2ImTransGradComputeLauncher: %s\n", swc_strerror(st));
}
