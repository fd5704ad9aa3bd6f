"""Python binding of the Winograd2x2ImTrans op for PyTorch-ROCm tensors.

Mirrors winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans.py of the reference:
``winograd2x2_imTrans(I)`` (:13-14) with the shape rule of its RegisterShape function
(:20-27).  The gradient registration (:29-33) has no counterpart: forward only.
"""
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import swc_hip  # noqa: E402


def winograd2x2_imTrans_shape(shape):
    """[B,H,W,C] -> [16,B,(H+1)/2,(W+1)/2,C] (winograd2x2_imTrans.py:20-27), computed by the C++ host wrapper."""
    out = swc_hip.dims([0] * 5)
    swc_hip.check(swc_hip.lib().swc_winograd2x2_imtrans_op_shape(len(shape), swc_hip.dims(shape), out),
                  "winograd2x2_imTrans")
    return tuple(out)


def winograd2x2_imTrans(I, relu=False, out=None):
    """I: [B,H,W,C] float32 NHWC on the GPU -> [16,B,nH,nW,C].

    ``relu=True`` applies the Winograd-domain ReLU inside the same kernel (what
    ``nl(winograd2x2_imTrans(x))`` with ``nl=tf.nn.relu`` computes in
    ResNet-18-var/winograd_imtrans.py:16-17).  ``out`` may supply the result tensor.
    """
    I = swc_hip.require_cuda_f32(I, "I", 4)
    shape = winograd2x2_imTrans_shape(I.shape)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32, device=I.device)
    else:
        if tuple(out.shape) != shape or out.dtype != torch.float32 or out.device != I.device or not out.is_contiguous():
            raise ValueError("out must be a contiguous float32 tensor of shape %s on %s" % (shape, I.device))
    with torch.cuda.device(I.device):
        stream = torch.cuda.current_stream().cuda_stream
        st = swc_hip.lib().swc_winograd2x2_imtrans_op_compute(
            I.data_ptr(), 4, swc_hip.dims(I.shape), out.data_ptr(), 5, swc_hip.dims(out.shape), int(bool(relu)), stream)
    swc_hip.check(st, "winograd2x2_imTrans")
    return out
