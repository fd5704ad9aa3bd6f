// Host op wrapper of Winograd2x2ConvGrad: what the reference's TensorFlow OpKernel does on the host
// (winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_grad_op.cc:36-78): the dimensions are read from the
// output gradient and the transformed input (:44-48), both results are shaped like the op's two inputs (:49-60),
// nH = (H+1)/2 (:62-63), the temporary holds 16*nH*nW*B*K floats (:66-67), the launcher runs with pad 1,1 (:74).
// Allocation stays with the caller's framework; the pointer table the reference also allocates (:69-71) is not
// needed.
#include "swc_common.h"

extern "C" int swc_winograd2x2_conv_grad_op_shape(int ti_rank, const int64_t *ti_dims, int w_rank, const int64_t *w_dims,
                                                  int g_rank, const int64_t *g_dims, int64_t ti_grad_dims[5],
                                                  int64_t w_grad_dims[3], int64_t *tmp_floats)
{
    if (ti_dims == nullptr || w_dims == nullptr || g_dims == nullptr || ti_grad_dims == nullptr || w_grad_dims == nullptr ||
        tmp_floats == nullptr)
        return SWC_ERR_NULL_POINTER;
    if (ti_rank != 5 || w_rank != 3 || g_rank != 4) return SWC_ERR_BAD_RANK;
    if (ti_dims[0] != 16 || w_dims[0] != 16) return SWC_ERR_BAD_RANK;
    for (int i = 1; i < 5; ++i)
        if (ti_dims[i] <= 0 || ti_dims[i] > INT32_MAX) return SWC_ERR_BAD_DIMS;
    for (int i = 1; i < 3; ++i)
        if (w_dims[i] <= 0 || w_dims[i] > INT32_MAX) return SWC_ERR_BAD_DIMS;
    for (int i = 0; i < 4; ++i)
        if (g_dims[i] <= 0 || g_dims[i] > INT32_MAX) return SWC_ERR_BAD_DIMS;
    // B, H, W, K come from the output gradient, C from the transformed input (:44-48); the forward op's output is
    // [B,2nH,2nW,K] (winograd2x2_conv_op.cc:53), so these must agree with the two inputs.
    const int64_t B = g_dims[0], H = g_dims[1], W = g_dims[2], K = g_dims[3], C = ti_dims[4];
    const int64_t nH = (H + 1) / 2, nW = (W + 1) / 2;
    if (ti_dims[1] != B || ti_dims[2] != nH || ti_dims[3] != nW || H != 2 * nH || W != 2 * nW) return SWC_ERR_BAD_DIMS;
    if (w_dims[1] != C || w_dims[2] != K) return SWC_ERR_BAD_DIMS;
    const int64_t M = B * nH * nW;  // each factor below 2^31: no overflow
    if (M >= (1ll << 31) || M > INT64_MAX / (16 * K)) return SWC_ERR_BAD_DIMS;
    for (int i = 0; i < 5; ++i) ti_grad_dims[i] = ti_dims[i];
    for (int i = 0; i < 3; ++i) w_grad_dims[i] = w_dims[i];
    *tmp_floats = 16 * M * K;
    return SWC_OK;
}

extern "C" int swc_winograd2x2_conv_grad_op_compute(const float *tinput, int ti_rank, const int64_t *ti_dims,
                                                    const float *weight, int w_rank, const int64_t *w_dims,
                                                    const float *output_grad, int g_rank, const int64_t *g_dims,
                                                    float *tinput_grad, float *weight_grad, float *tmp_data_buffer,
                                                    int64_t tmp_floats, swc_stream_t stream)
{
    int64_t ti_grad[5], w_grad[3], need = 0;
    const int st = swc_winograd2x2_conv_grad_op_shape(ti_rank, ti_dims, w_rank, w_dims, g_rank, g_dims, ti_grad, w_grad, &need);
    if (st != SWC_OK) return st;
    if (tmp_floats < need) return SWC_ERR_BAD_DIMS;
    return swc_winograd2x2_conv_grad(tinput, weight, output_grad, tinput_grad, weight_grad, tmp_data_buffer, nullptr,
                                     static_cast<int>(ti_dims[4]), static_cast<int>(g_dims[0]), static_cast<int>(g_dims[1]),
                                     static_cast<int>(g_dims[2]), static_cast<int>(g_dims[3]), 1, 1, stream);
}
