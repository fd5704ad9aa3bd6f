"""Python binding of the Winograd2x2ImTrans op for PyTorch-ROCm tensors.

Mirrors winograd2x2_cublas/winograd2x2_imTrans/winograd2x2_imTrans.py of the reference:
``winograd2x2_imTrans(I)`` (:13-14) with the shape rule of its RegisterShape function
(:20-27), ``winograd2x2_imTrans_grad(grad)`` (:16-17), and the gradient registration (:29-33)
as a torch.autograd.Function.
"""
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import swc_hip  # noqa: E402


def winograd2x2_imTrans_shape(shape):
    """[B,H,W,C] -> [16,B,(H+1)/2,(W+1)/2,C] (winograd2x2_imTrans.py:20-27), computed by the C++ host wrapper."""
    return _plan(tuple(shape))[0]


# I.shape -> (output shape, and the two dimension arrays swc_winograd2x2_imtrans_op_compute takes): validated by the
# C++ host wrapper once per shape.
_PLANS = {}


def _plan(shape):
    plan = _PLANS.get(shape)
    if plan is None:
        out = swc_hip.dims([0] * 5)
        i_dims = swc_hip.dims(shape)
        swc_hip.check(swc_hip.lib().swc_winograd2x2_imtrans_op_shape(len(shape), i_dims, out), "winograd2x2_imTrans")
        o_shape = tuple(out)
        plan = (o_shape, i_dims, swc_hip.dims(o_shape))
        if len(_PLANS) >= 1024:
            _PLANS.clear()
        _PLANS[shape] = plan
    return plan


def _forward(I, relu, out, scale=None, shift=None, out_dtype=torch.float32):
    I = swc_hip.require_cuda_f32(I, "I", 4)
    shape, i_dims, o_dims = _plan(I.shape)
    if (scale is None) != (shift is None):
        raise ValueError("scale and shift go together")
    if scale is not None:
        scale = swc_hip.require_cuda_f32(scale, "scale", 1)
        shift = swc_hip.require_cuda_f32(shift, "shift", 1)
        if scale.shape[0] != I.shape[3] or shift.shape[0] != I.shape[3]:
            raise ValueError("scale and shift must have one entry per channel (%d)" % I.shape[3])
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("out_dtype must be torch.float32 or torch.bfloat16")
    if out is None:
        out = torch.empty(shape, dtype=out_dtype, device=I.device)
    else:
        if out.shape != shape or out.dtype != out_dtype or out.device != I.device or not out.is_contiguous():
            raise ValueError("out must be a contiguous %s tensor of shape %s on %s" % (out_dtype, shape, I.device))
    with swc_hip.on_device(I.device) as stream:
        if out_dtype == torch.bfloat16:
            B, H, W, C = I.shape
            st = swc_hip.lib().swc_winograd2x2_imtrans_bf16out(
                I.data_ptr(), None if scale is None else scale.data_ptr(), None if shift is None else shift.data_ptr(),
                out.data_ptr(), C, B, H, W, 1, 1, int(bool(relu)), stream)
        elif scale is not None:
            B, H, W, C = I.shape
            st = swc_hip.lib().swc_winograd2x2_imtrans_affine(
                I.data_ptr(), scale.data_ptr(), shift.data_ptr(), out.data_ptr(), C, B, H, W, 1, 1, int(bool(relu)),
                stream)
        else:
            st = swc_hip.lib().swc_winograd2x2_imtrans_op_compute(I.data_ptr(), 4, i_dims, out.data_ptr(), 5, o_dims,
                                                                  int(bool(relu)), stream)
    swc_hip.check(st, "winograd2x2_imTrans")
    return out


def winograd2x2_imTrans_grad(grad, H=None, W=None, relu_output=None, relu_input=None):
    """grad: [16,B,nH,nW,C] -> gradient w.r.t. the op's input, [B,H,W,C].

    As in the reference (winograd2x2_imTrans_grad_op.cc:44-45) H and W default to 2*nH, 2*nW.
    The gradient is taken through the fused ReLU when the forward pass's result (``relu_output``,
    computed with ``relu=True``) or its input (``relu_input`` [B,H,W,C]; the mask is recomputed from
    it, which reads a quarter of the bytes) is given.  ``grad`` is left untouched (the reference
    overwrites it).
    """
    grad = swc_hip.require_cuda_f32(grad, "grad", 5)
    if grad.shape[0] != 16:
        raise ValueError("grad must have shape [16,B,nH,nW,C]")
    _, B, nH, nW, C = grad.shape
    if relu_input is not None:
        if relu_output is not None:
            raise ValueError("give relu_output or relu_input, not both")
        relu_input = swc_hip.require_cuda_f32(relu_input, "relu_input", 4)
        if relu_input.shape[0] != B or relu_input.shape[3] != C:
            raise ValueError("relu_input must be the forward input [B,H,W,C]")
        H = relu_input.shape[1] if H is None else int(H)
        W = relu_input.shape[2] if W is None else int(W)
        if (H, W) != tuple(relu_input.shape[1:3]):
            raise ValueError("relu_input is %d x %d, not %d x %d" % (relu_input.shape[1], relu_input.shape[2], H, W))
    H = 2 * nH if H is None else int(H)
    W = 2 * nW if W is None else int(W)
    if (H + 1) // 2 != nH or (W + 1) // 2 != nW:
        raise ValueError("H, W = %d, %d do not tile into %d x %d" % (H, W, nH, nW))
    mask_ptr = None
    if relu_output is not None:
        relu_output = swc_hip.require_cuda_f32(relu_output, "relu_output", 5)
        if relu_output.shape != grad.shape:
            raise ValueError("relu_output must have grad's shape")
        mask_ptr = relu_output.data_ptr()
    out = torch.empty((B, H, W, C), dtype=torch.float32, device=grad.device)
    with swc_hip.on_device(grad.device) as stream:
        # the host op wrapper (winograd2x2_imTrans_grad_op.cc:33-55) checks the shapes against each other again
        st = swc_hip.lib().swc_winograd2x2_imtrans_grad_op_compute(
            grad.data_ptr(), 5, swc_hip.dims(grad.shape), mask_ptr, None if relu_input is None else relu_input.data_ptr(),
            out.data_ptr(), 4, swc_hip.dims(out.shape), stream)
    swc_hip.check(st, "winograd2x2_imTrans_grad")
    return out


class _ImTransFunction(torch.autograd.Function):
    """The RegisterGradient hook of the reference (winograd2x2_imTrans.py:29-33), with the fused ReLU."""

    @staticmethod
    def forward(ctx, I, relu):
        out = _forward(I, relu, None)
        ctx.hw = (I.shape[1], I.shape[2])
        ctx.relu = bool(relu)
        if relu:
            # the ReLU's mask is recomputed from the input in the backward pass: [B,H,W,C] kept, not [16,B,nH,nW,C]
            ctx.save_for_backward(I)
        return out

    @staticmethod
    def backward(ctx, grad):
        relu_input = ctx.saved_tensors[0] if ctx.relu else None
        return winograd2x2_imTrans_grad(grad.contiguous(), ctx.hw[0], ctx.hw[1], relu_input=relu_input), None


def winograd2x2_imTrans(I, relu=False, out=None, scale=None, shift=None, out_dtype=torch.float32):
    """I: [B,H,W,C] float32 NHWC on the GPU -> [16,B,nH,nW,C].

    ``scale``/``shift`` ([C] each, forward only): the transform of ``I*scale + shift`` (one fused
    multiply-add per pixel, zero padding left at zero) -- an inference-mode BatchNorm folded into the load.
    ``out_dtype=torch.bfloat16`` (forward only): the result is rounded to bf16 as it is stored, for
    ``winograd2x2_conv`` to read back at half the traffic.

    ``relu=True`` applies the Winograd-domain ReLU inside the same kernel (what
    ``nl(winograd2x2_imTrans(x))`` with ``nl=tf.nn.relu`` computes in
    ResNet-18-var/winograd_imtrans.py:16-17).  ``out`` may supply the result tensor (forward only: with an input that requires grad it raises).
    Differentiable: gradients flow through ``winograd2x2_imTrans_grad``.
    """
    needs_grad = isinstance(I, torch.Tensor) and I.requires_grad and torch.is_grad_enabled()
    if (scale is not None or out_dtype != torch.float32) and needs_grad:
        raise NotImplementedError("the scale/shift and bf16-output variants are forward only")
    if needs_grad:
        if out is not None:
            raise NotImplementedError("out= is forward only: the result written there would carry no gradient")
        return _ImTransFunction.apply(I, relu)
    return _forward(I, relu, out, scale, shift, out_dtype)
