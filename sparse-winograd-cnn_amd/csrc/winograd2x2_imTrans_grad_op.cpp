// Host op wrapper of Winograd2x2ImTransGrad: what the reference's TensorFlow OpKernel does on the host
// (winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans_grad_op.cc:33-55): B, nH, nW, C are read from the
// gradient of the transformed input (:40-43), the result is [B, 2nH, 2nW, C] (:44-49), the launcher runs with
// pad 1,1 (:54).  The reference knows no other extent than H = 2nH; a forward input of odd extent (H = 2nH - 1)
// is accepted here when the caller says so through the result's dimensions.
#include "swc_common.h"

extern "C" int swc_winograd2x2_imtrans_grad_op_shape(int g_rank, const int64_t *g_dims, int64_t in_grad_dims[4])
{
    if (g_dims == nullptr || in_grad_dims == nullptr) return SWC_ERR_NULL_POINTER;
    if (g_rank != 5 || g_dims[0] != 16) return SWC_ERR_BAD_RANK;
    for (int i = 1; i < 5; ++i)
        if (g_dims[i] <= 0 || g_dims[i] > INT32_MAX) return SWC_ERR_BAD_DIMS;
    if (2 * g_dims[2] > INT32_MAX || 2 * g_dims[3] > INT32_MAX) return SWC_ERR_BAD_DIMS;
    in_grad_dims[0] = g_dims[1];      // B
    in_grad_dims[1] = 2 * g_dims[2];  // H = 2*nH (:44)
    in_grad_dims[2] = 2 * g_dims[3];  // W = 2*nW (:45)
    in_grad_dims[3] = g_dims[4];      // C
    return SWC_OK;
}

extern "C" int swc_winograd2x2_imtrans_grad_op_compute(const float *output_grad, int g_rank, const int64_t *g_dims,
                                                       const float *relu_output, const float *relu_input,
                                                       float *input_grad, int ig_rank, const int64_t *ig_dims,
                                                       swc_stream_t stream)
{
    int64_t want[4];
    const int st = swc_winograd2x2_imtrans_grad_op_shape(g_rank, g_dims, want);
    if (st != SWC_OK) return st;
    if (ig_dims == nullptr) return SWC_ERR_NULL_POINTER;
    if (ig_rank != 4) return SWC_ERR_BAD_RANK;
    if (relu_output != nullptr && relu_input != nullptr) return SWC_ERR_BAD_DIMS;  // one source for the mask
    // [B, H, W, C] with H in {2nH - 1, 2nH}: the extents that tile into nH x nW
    if (ig_dims[0] != want[0] || ig_dims[3] != want[3]) return SWC_ERR_BAD_DIMS;
    for (int i = 1; i < 3; ++i)
        if (ig_dims[i] != want[i] && ig_dims[i] != want[i] - 1) return SWC_ERR_BAD_DIMS;
    const int B = static_cast<int>(ig_dims[0]), H = static_cast<int>(ig_dims[1]), W = static_cast<int>(ig_dims[2]);
    const int C = static_cast<int>(ig_dims[3]);
    if (relu_input != nullptr)
        return swc_winograd2x2_imtrans_grad_relu_input(output_grad, relu_input, input_grad, C, B, H, W, 1, 1, stream);
    return swc_winograd2x2_imtrans_grad(output_grad, relu_output, input_grad, C, B, H, W, 1, 1, stream);
}
