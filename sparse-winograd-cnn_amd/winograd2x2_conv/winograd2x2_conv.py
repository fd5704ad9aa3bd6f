"""Python binding of the Winograd2x2Conv op for PyTorch-ROCm tensors.

Mirrors winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv.py of the reference:
``winograd2x2_conv(I, W)`` (:13-14) with the shape rule of its RegisterShape function
(:19-29), ``winograd2x2_conv_grad(i1, i2, grad)`` (:16-17), and the gradient registration
(:31-36) as a torch.autograd.Function.
"""
import ctypes
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import swc_hip  # noqa: E402

PRECISIONS = {"fp32": 0, "bf16": 1}


def winograd2x2_conv_shape(i_shape, w_shape):
    """I [16,B,nH,nW,C], W [16,C,K] -> [B,2nH,2nW,K] (winograd2x2_conv.py:19-29), computed by the C++ host wrapper."""
    return _plan(tuple(i_shape), tuple(w_shape))[0]


# (I.shape, W.shape) -> (output shape, and the three dimension arrays swc_winograd2x2_conv_op_compute takes): shapes
# are validated by the C++ host wrapper once; a layer that is called again with the same shapes pays one lookup.
_PLANS = {}


def _plan(i_shape, w_shape):
    key = (i_shape, w_shape)
    plan = _PLANS.get(key)
    if plan is None:
        out = swc_hip.dims([0] * 4)
        i_dims, w_dims = swc_hip.dims(i_shape), swc_hip.dims(w_shape)
        swc_hip.check(swc_hip.lib().swc_winograd2x2_conv_op_shape(len(i_shape), i_dims, len(w_shape), w_dims, out),
                      "winograd2x2_conv")
        shape = tuple(out)
        plan = (shape, i_dims, w_dims, swc_hip.dims(shape))
        if len(_PLANS) >= 1024:
            _PLANS.clear()
        _PLANS[key] = plan
    return plan


def _forward(I, W, precision, out, scale=None, shift=None, residual=None, residual_relu=False):
    if precision not in PRECISIONS:
        raise ValueError("precision must be one of %s" % sorted(PRECISIONS))
    I = swc_hip.require_cuda_f32(I, "I", 5)
    W = swc_hip.require_cuda_f32(W, "W", 3)
    if W.device != I.device:
        raise ValueError("I and W must be on the same device")
    shape, i_dims, w_dims, o_dims = _plan(I.shape, W.shape)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32, device=I.device)
    else:
        if out.shape != shape or out.dtype != torch.float32 or out.device != I.device or not out.is_contiguous():
            raise ValueError("out must be a contiguous float32 tensor of shape %s on %s" % (shape, I.device))
    if (scale is None) != (shift is None):
        raise ValueError("scale and shift go together")
    epilogue = scale is not None or residual is not None
    if scale is not None:
        scale = swc_hip.require_cuda_f32(scale, "scale", 1)
        shift = swc_hip.require_cuda_f32(shift, "shift", 1)
        if scale.shape[0] != shape[3] or shift.shape[0] != shape[3]:
            raise ValueError("scale and shift must have one entry per output channel (%d)" % shape[3])
    if residual is not None:
        residual = swc_hip.require_cuda_f32(residual, "residual", 4)
        if tuple(residual.shape) != shape:
            raise ValueError("residual must have the output's shape %s" % (shape,))
    with swc_hip.on_device(I.device) as stream:
        if epilogue:
            _, B, nH, nW, C = I.shape
            st = swc_hip.lib().swc_winograd2x2_conv_epilogue(
                I.data_ptr(), W.data_ptr(), out.data_ptr(), None if scale is None else scale.data_ptr(),
                None if shift is None else shift.data_ptr(), None if residual is None else residual.data_ptr(),
                int(bool(residual_relu)), C, B, nH, nW, shape[3], 1, 1, PRECISIONS[precision], stream)
        else:
            st = swc_hip.lib().swc_winograd2x2_conv_op_compute(
                I.data_ptr(), 5, i_dims, W.data_ptr(), 3, w_dims, out.data_ptr(), 4, o_dims, PRECISIONS[precision],
                stream)
    swc_hip.check(st, "winograd2x2_conv")
    return out


def winograd2x2_weights_bf16(W):
    """W [16,C,K] float32 -> [16,K,C] bfloat16 (round to nearest even, transposed): the weight layout
    ``winograd2x2_conv`` reads when its input is a bfloat16 tensor.  Prepare once per weight update."""
    W = swc_hip.require_cuda_f32(W, "W", 3)
    if W.shape[0] != 16:
        raise ValueError("W must have shape [16,C,K]")
    out = torch.empty((16, W.shape[2], W.shape[1]), dtype=torch.bfloat16, device=W.device)
    with swc_hip.on_device(W.device) as stream:
        st = swc_hip.lib().swc_winograd2x2_weights_bf16(W.data_ptr(), out.data_ptr(), W.shape[1], W.shape[2], stream)
    swc_hip.check(st, "winograd2x2_weights_bf16")
    return out


def _forward_bf16_stored(I, W, out, scale, shift, residual, residual_relu=False, workspace=True):
    """I [16,B,nH,nW,C] bfloat16; W [16,C,K] float32 or prepared [16,K,C] bfloat16."""
    I = swc_hip.require_cuda_f32(I, "I", 5, torch.bfloat16)
    if not isinstance(W, torch.Tensor) or W.dim() != 3:
        raise ValueError("W must be a rank-3 tensor")
    if W.dtype == torch.float32:
        W = winograd2x2_weights_bf16(W)
    W = swc_hip.require_cuda_f32(W, "W", 3, torch.bfloat16)
    _, B, nH, nW, C = I.shape
    if I.shape[0] != 16 or W.shape[0] != 16 or W.shape[2] != C or W.device != I.device:
        raise ValueError("I must be [16,B,nH,nW,C] and the prepared W [16,K,C] on the same device")
    K = W.shape[1]
    shape = (B, 2 * nH, 2 * nW, K)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32, device=I.device)
    elif out.shape != shape or out.dtype != torch.float32 or out.device != I.device or not out.is_contiguous():
        raise ValueError("out must be a contiguous float32 tensor of shape %s on %s" % (shape, I.device))
    if (scale is None) != (shift is None):
        raise ValueError("scale and shift go together")
    if scale is not None:
        scale = swc_hip.require_cuda_f32(scale, "scale", 1)
        shift = swc_hip.require_cuda_f32(shift, "shift", 1)
        if scale.shape[0] != K or shift.shape[0] != K:
            raise ValueError("scale and shift must have one entry per output channel (%d)" % K)
    if residual is not None:
        residual = swc_hip.require_cuda_f32(residual, "residual", 4)
        if tuple(residual.shape) != shape:
            raise ValueError("residual must have the output's shape %s" % (shape,))
    with swc_hip.on_device(I.device) as stream:
        L = swc_hip.lib()
        # the launcher's temporary, allocated per call as the reference's op does (winograd2x2_conv_op.cc:57-60);
        # most shapes need none
        tmp_floats = L.swc_winograd2x2_conv_bf16in_workspace_floats(C, B, nH, nW, K) if workspace else 0
        tmp = torch.empty(tmp_floats, dtype=torch.float32, device=I.device) if tmp_floats else None
        st = L.swc_winograd2x2_conv_bf16in_ws(
            I.data_ptr(), W.data_ptr(), out.data_ptr(), None if scale is None else scale.data_ptr(),
            None if shift is None else shift.data_ptr(), None if residual is None else residual.data_ptr(),
            int(bool(residual_relu)), None if tmp is None else tmp.data_ptr(), tmp_floats, C, B, nH, nW, K, 1, 1, stream)
    swc_hip.check(st, "winograd2x2_conv (bf16-stored operands)")
    return out


def winograd2x2_conv_grad_shape(i_shape, w_shape, g_shape):
    """(I.shape, W.shape, grad.shape) -> (dI shape, dW shape, floats of the launcher's temporary), by the host op
    wrapper (swc_winograd2x2_conv_grad_op_shape; winograd2x2_conv_grad_op.cc:44-67)."""
    ti_g, w_g, tmp = swc_hip.dims([0] * 5), swc_hip.dims([0] * 3), ctypes.c_int64(0)
    swc_hip.check(swc_hip.lib().swc_winograd2x2_conv_grad_op_shape(
        len(i_shape), swc_hip.dims(i_shape), len(w_shape), swc_hip.dims(w_shape), len(g_shape), swc_hip.dims(g_shape),
        ti_g, w_g, ctypes.byref(tmp)), "winograd2x2_conv_grad")
    return tuple(ti_g), tuple(w_g), int(tmp.value)


def winograd2x2_conv_grad(i1, i2, grad):
    """(I [16,B,nH,nW,C], W [16,C,K], grad [B,2nH,2nW,K]) -> (dI, dW), as the reference's
    winograd2x2_conv_grad (winograd2x2_conv.py:16-17).  fp32 throughout."""
    I = swc_hip.require_cuda_f32(i1, "i1", 5)
    W = swc_hip.require_cuda_f32(i2, "i2", 3)
    grad = swc_hip.require_cuda_f32(grad, "grad", 4)
    di_shape, dw_shape, tmp_floats = winograd2x2_conv_grad_shape(I.shape, W.shape, grad.shape)
    dI = torch.empty(di_shape, dtype=torch.float32, device=I.device)
    dW = torch.empty(dw_shape, dtype=torch.float32, device=I.device)
    tmp = torch.empty(tmp_floats, dtype=torch.float32, device=I.device)  # as winograd2x2_conv_grad_op.cc:66-67
    with swc_hip.on_device(I.device) as stream:
        st = swc_hip.lib().swc_winograd2x2_conv_grad_op_compute(
            I.data_ptr(), 5, swc_hip.dims(I.shape), W.data_ptr(), 3, swc_hip.dims(W.shape), grad.data_ptr(), 4,
            swc_hip.dims(grad.shape), dI.data_ptr(), dW.data_ptr(), tmp.data_ptr(), tmp_floats, stream)
    swc_hip.check(st, "winograd2x2_conv_grad")
    return dI, dW


class _ConvFunction(torch.autograd.Function):
    """The RegisterGradient hook of the reference (winograd2x2_conv.py:31-36).  The backward is fp32
    whatever the forward's GEMM precision was."""

    @staticmethod
    def forward(ctx, I, W, precision):
        ctx.save_for_backward(I, W)
        return _forward(I, W, precision, None)

    @staticmethod
    def backward(ctx, grad):
        I, W = ctx.saved_tensors
        dI, dW = winograd2x2_conv_grad(I, W, grad.contiguous())
        return dI, dW, None


def winograd2x2_conv(I, W, precision="fp32", out=None, scale=None, shift=None, residual=None, residual_relu=False,
                     workspace=True):
    """I: [16,B,nH,nW,C], W: [16,C,K], float32 on the GPU -> [B,2nH,2nW,K] (uncropped).

    A bfloat16 ``I`` (from ``winograd2x2_imTrans(..., out_dtype=torch.bfloat16)``) takes the bf16-stored
    kernel (forward only, needs C % 64 == 0); ``W`` is then float32 [16,C,K] (converted on every call) or the
    tensor ``winograd2x2_weights_bf16`` prepared from it.
    ``scale``/``shift`` ([K]) and ``residual`` ([B,2nH,2nW,K]), forward only: the result becomes
    ``conv*scale + shift + residual`` inside the kernel's stores (an inference BatchNorm and the
    residual add that follow the second convolution of a ResNet unit); with ``residual_relu=True`` it is
    ``... + relu(residual)`` (the identity shortcut of the reference model is ``relu(x)``).

    The bf16-stored kernel gets a temporary of the size its launcher asks for (most shapes: none), as the
    reference's op allocates its launcher's (winograd2x2_conv_op.cc:57-60); ``workspace=False`` calls it without.

    ``precision="bf16"`` rounds both GEMM operands to bf16 (fp32 accumulate).  Differentiable
    through ``winograd2x2_conv_grad`` when an input requires grad.
    """
    needs_grad = torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in (I, W))
    if isinstance(I, torch.Tensor) and I.dtype == torch.bfloat16:
        if needs_grad:
            raise NotImplementedError("the bf16-stored variant is forward only")
        return _forward_bf16_stored(I, W, out, scale, shift, residual, residual_relu, workspace)
    if residual_relu and residual is None:
        raise ValueError("residual_relu needs a residual")
    if (scale is not None or residual is not None) and needs_grad:
        raise NotImplementedError("the scale/shift/residual epilogue is forward only")
    if needs_grad:
        if out is not None:
            raise NotImplementedError("out= is forward only: the result written there would carry no gradient")
        return _ConvFunction.apply(I, W, precision)
    return _forward(I, W, precision, out, scale, shift, residual, residual_relu)


def winograd2x2_relu_conv(X, W, relu=True, out=None):
    """The layer pair in one kernel: ``winograd2x2_conv(relu(winograd2x2_imTrans(X)), W)``.

    X: [B,H,W,C] NHWC, W: [16,C,K], float32 on the GPU -> [B,2nH,2nW,K] (uncropped), fp32.  The
    [16,B,nH,nW,C] intermediate is never materialised.  Shapes the fused kernel does not cover
    (C % 8 != 0, K % 4 != 0, ...) run the two ops back to back instead.  Forward only.
    """
    import winograd2x2_imTrans.winograd2x2_imTrans as _it

    X = swc_hip.require_cuda_f32(X, "X", 4)
    W = swc_hip.require_cuda_f32(W, "W", 3)
    if W.device != X.device:
        raise ValueError("X and W must be on the same device")
    B, H, Wd, C = X.shape
    if W.shape[0] != 16 or W.shape[1] != C:
        raise ValueError("W must have shape [16,%d,K], got %s" % (C, tuple(W.shape)))
    K = W.shape[2]
    shape = (B, 2 * ((H + 1) // 2), 2 * ((Wd + 1) // 2), K)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32, device=X.device)
    elif tuple(out.shape) != shape or out.dtype != torch.float32 or out.device != X.device or not out.is_contiguous():
        raise ValueError("out must be a contiguous float32 tensor of shape %s on %s" % (shape, X.device))
    with torch.cuda.device(X.device):
        st = swc_hip.lib().swc_winograd2x2_relu_conv(X.data_ptr(), W.data_ptr(), out.data_ptr(), C, B, H, Wd, K, 1, 1,
                                                     int(bool(relu)), torch.cuda.current_stream().cuda_stream)
    if st == swc_hip.SWC_ERR_UNSUPPORTED:
        return _forward(_it.winograd2x2_imTrans(X, relu=relu), W, "fp32", out)
    swc_hip.check(st, "winograd2x2_relu_conv")
    return out


def winograd2x2_relu_conv_bf16(X, W, relu=True, out=None, in_affine=None, scale=None, shift=None, residual=None):
    """The layer pair in one kernel with bf16 GEMM operands: the values of
    ``winograd2x2_conv(winograd2x2_imTrans(X, relu, out_dtype=bfloat16), W16)``, the transformed
    activations never reaching memory.

    X: [B,H,W,C] float32 NHWC; W: float32 [16,C,K] (converted on every call) or the bfloat16 [16,K,C]
    tensor from ``winograd2x2_weights_bf16``.  ``in_affine=(scale, shift)`` ([C] each) maps the input as
    ``winograd2x2_imTrans(..., scale, shift)`` does; ``scale``/``shift`` ([K]) and ``residual`` act on the
    result as in ``winograd2x2_conv``.  Shapes the kernel does not cover (C % 16 != 0, ...) run the
    bf16-stored pair, or the fp32-stored pair with bf16 operands, instead.  Forward only.
    """
    import winograd2x2_imTrans.winograd2x2_imTrans as _it

    X = swc_hip.require_cuda_f32(X, "X", 4)
    W_in = W
    if isinstance(W, torch.Tensor) and W.dtype == torch.float32:
        W = winograd2x2_weights_bf16(W)
    W = swc_hip.require_cuda_f32(W, "W", 3, torch.bfloat16)
    B, H, Wd, C = X.shape
    if W.shape[0] != 16 or W.shape[2] != C or W.device != X.device:
        raise ValueError("the prepared W must have shape [16,K,%d] on X's device, got %s" % (C, tuple(W.shape)))
    K = W.shape[1]
    shape = (B, 2 * ((H + 1) // 2), 2 * ((Wd + 1) // 2), K)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32, device=X.device)
    elif tuple(out.shape) != shape or out.dtype != torch.float32 or out.device != X.device or not out.is_contiguous():
        raise ValueError("out must be a contiguous float32 tensor of shape %s on %s" % (shape, X.device))
    in_scale, in_shift = in_affine if in_affine is not None else (None, None)
    if (scale is None) != (shift is None) or (in_scale is None) != (in_shift is None):
        raise ValueError("scale and shift go together")
    checked = {}
    for name, t, n in (("in_scale", in_scale, C), ("in_shift", in_shift, C), ("scale", scale, K), ("shift", shift, K)):
        if t is not None:
            t = swc_hip.require_cuda_f32(t, name, 1)
            if t.shape[0] != n:
                raise ValueError("%s must have %d entries" % (name, n))
        checked[name] = t
    if residual is not None:
        residual = swc_hip.require_cuda_f32(residual, "residual", 4)
        if tuple(residual.shape) != shape:
            raise ValueError("residual must have the output's shape %s" % (shape,))
    ptr = lambda t: None if t is None else t.data_ptr()  # noqa: E731
    with torch.cuda.device(X.device):
        st = swc_hip.lib().swc_winograd2x2_relu_conv_bf16(
            X.data_ptr(), ptr(checked["in_scale"]), ptr(checked["in_shift"]), W.data_ptr(), out.data_ptr(),
            ptr(checked["scale"]), ptr(checked["shift"]), ptr(residual), C, B, H, Wd, K, 1, 1, int(bool(relu)),
            torch.cuda.current_stream().cuda_stream)
    if st == swc_hip.SWC_ERR_UNSUPPORTED:
        if C % 64 == 0:
            ti = _it.winograd2x2_imTrans(X, relu=relu, scale=checked["in_scale"], shift=checked["in_shift"],
                                         out_dtype=torch.bfloat16)
            return _forward_bf16_stored(ti, W, out, checked["scale"], checked["shift"], residual)
        if W_in.dtype != torch.float32:
            raise ValueError("this shape needs the float32 weights [16,C,K] (no bf16 kernel takes C = %d)" % C)
        ti = _it.winograd2x2_imTrans(X, relu=relu, scale=checked["in_scale"], shift=checked["in_shift"])
        return _forward(ti, W_in, "bf16", out, checked["scale"], checked["shift"], residual)
    swc_hip.check(st, "winograd2x2_relu_conv_bf16")
    return out
