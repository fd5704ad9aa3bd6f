// Host op wrapper of Winograd2x2Conv: what the reference's TensorFlow OpKernel does on the
// host (winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_op.cc:37-67) and its Python
// shape function (winograd2x2_conv.py:19-29).  The output allocation stays with the
// caller's framework; the two temporaries the reference allocates (:57-63) are not needed.
#include <cstdio>

#include "swc_common.h"

extern "C" int swc_winograd2x2_conv_op_shape(int in_rank, const int64_t *in_dims, int w_rank, const int64_t *w_dims,
                                             int64_t out_dims[4])
{
    if (in_dims == nullptr || w_dims == nullptr || out_dims == nullptr) return SWC_ERR_NULL_POINTER;
    if (in_rank != 5 || w_rank != 3) return SWC_ERR_BAD_RANK;  // with_rank(5) / with_rank(3), winograd2x2_conv.py:21-22
    if (in_dims[0] != 16 || w_dims[0] != 16) return SWC_ERR_BAD_RANK;
    for (int i = 1; i < 5; ++i)
        if (in_dims[i] <= 0 || in_dims[i] > INT32_MAX) return SWC_ERR_BAD_DIMS;
    for (int i = 1; i < 3; ++i)
        if (w_dims[i] <= 0 || w_dims[i] > INT32_MAX) return SWC_ERR_BAD_DIMS;
    if (w_dims[1] != in_dims[4]) return SWC_ERR_BAD_DIMS;  // C of the weights must be C of the input
    if (2 * in_dims[2] > INT32_MAX || 2 * in_dims[3] > INT32_MAX) return SWC_ERR_BAD_DIMS;
    out_dims[0] = in_dims[1];      // B
    out_dims[1] = 2 * in_dims[2];  // 2*nH, never cropped (winograd2x2_conv_op.cc:53)
    out_dims[2] = 2 * in_dims[3];  // 2*nW
    out_dims[3] = w_dims[2];       // K
    return SWC_OK;
}

extern "C" int swc_winograd2x2_conv_op_compute(const float *input, int in_rank, const int64_t *in_dims,
                                               const float *weight, int w_rank, const int64_t *w_dims, float *output,
                                               int out_rank, const int64_t *out_dims, int precision,
                                               swc_stream_t stream)
{
    int64_t want[4];
    const int st = swc_winograd2x2_conv_op_shape(in_rank, in_dims, w_rank, w_dims, want);
    if (st != SWC_OK) return st;
    if (out_dims == nullptr) return SWC_ERR_NULL_POINTER;
    if (out_rank != 4) return SWC_ERR_BAD_RANK;
    for (int i = 0; i < 4; ++i)
        if (out_dims[i] != want[i]) return SWC_ERR_BAD_DIMS;
    if (precision != 0 && precision != 1) return SWC_ERR_BAD_DIMS;
    // B, nH, nW, C, K read as at winograd2x2_conv_op.cc:45-49; pad 1,1 as at :66.
    const int B = static_cast<int>(in_dims[1]), nH = static_cast<int>(in_dims[2]), nW = static_cast<int>(in_dims[3]);
    const int C = static_cast<int>(in_dims[4]), K = static_cast<int>(w_dims[2]);
    return precision == 0
               ? swc_winograd2x2_conv(input, weight, output, nullptr, nullptr, C, B, nH, nW, K, 1, 1, stream)
               : swc_winograd2x2_conv_bf16(input, weight, output, nullptr, nullptr, C, B, nH, nW, K, 1, 1, stream);
}

void Winograd2x2ConvComputeLauncher(const float *Input, const float *Weight, float *Output, float *tmp_data_buffer,
                                    const long long *tmp_ptr_buffer, int C, int B, int nH, int nW, int K, int pad_h,
                                    int pad_w)
{
    const int st = swc_winograd2x2_conv(Input, Weight, Output, tmp_data_buffer, tmp_ptr_buffer, C, B, nH, nW, K, pad_h,
                                        pad_w, nullptr);
    if (st != SWC_OK) std::fprintf(stderr, "Winograd2x2ConvComputeLauncher: %s\n", swc_strerror(st));
}
