// Host op wrapper of Winograd2x2ImTrans: what the reference's TensorFlow OpKernel does on
// the host (winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans_op.cc:36-56) and
// its Python shape function (winograd2x2_imTrans.py:20-27), minus the tensor allocation,
// which stays with the caller's framework.
#include <cstdio>

#include "swc_common.h"

extern "C" int swc_winograd2x2_imtrans_op_shape(int in_rank, const int64_t *in_dims, int64_t out_dims[5])
{
    if (in_dims == nullptr || out_dims == nullptr) return SWC_ERR_NULL_POINTER;
    if (in_rank != 4) return SWC_ERR_BAD_RANK;  // shape.with_rank(4), winograd2x2_imTrans.py:22
    for (int i = 0; i < 4; ++i)
        if (in_dims[i] <= 0 || in_dims[i] > INT32_MAX) return SWC_ERR_BAD_DIMS;
    out_dims[0] = 16;
    out_dims[1] = in_dims[0];
    out_dims[2] = (in_dims[1] + 1) / 2;  // nH, winograd2x2_imTrans_op.cc:46
    out_dims[3] = (in_dims[2] + 1) / 2;  // nW, winograd2x2_imTrans_op.cc:47
    out_dims[4] = in_dims[3];
    return SWC_OK;
}

extern "C" int swc_winograd2x2_imtrans_op_compute(const float *input, int in_rank, const int64_t *in_dims,
                                                  float *output, int out_rank, const int64_t *out_dims, int relu,
                                                  swc_stream_t stream)
{
    int64_t want[5];
    const int st = swc_winograd2x2_imtrans_op_shape(in_rank, in_dims, want);
    if (st != SWC_OK) return st;
    if (out_dims == nullptr) return SWC_ERR_NULL_POINTER;
    if (out_rank != 5) return SWC_ERR_BAD_RANK;
    for (int i = 0; i < 5; ++i)
        if (out_dims[i] != want[i]) return SWC_ERR_BAD_DIMS;
    // B, H, W, C read as at winograd2x2_imTrans_op.cc:42-45; pad fixed to 1,1 as at :55.
    return swc_winograd2x2_imtrans(input, output, static_cast<int>(in_dims[3]), static_cast<int>(in_dims[0]),
                                   static_cast<int>(in_dims[1]), static_cast<int>(in_dims[2]), 1, 1, relu, stream);
}

void Winograd2x2ImTransComputeLauncher(const float *Input, float *TransIm, int C, int B, int H, int W, int pad_h,
                                       int pad_w)
{
    const int st = swc_winograd2x2_imtrans(Input, TransIm, C, B, H, W, pad_h, pad_w, 0, nullptr);
    if (st != SWC_OK) std::fprintf(stderr, "Winograd2x2ImTransComputeLauncher: %s\n", swc_strerror(st));
}
