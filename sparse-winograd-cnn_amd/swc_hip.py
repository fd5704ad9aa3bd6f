"""ctypes binding of libwinograd2x2_hip.so (the C ABI declared in include/winograd2x2.h).

There is no fallback: if the library has not been built, loading raises.
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libwinograd2x2_hip.so")
CSRC = os.path.join(_HERE, "csrc")

SWC_OK = 0
SWC_ERR_NULL_POINTER = -1
SWC_ERR_BAD_DIMS = -2
SWC_ERR_BAD_PAD = -3
SWC_ERR_HIP = -4
SWC_ERR_BAD_RANK = -5
SWC_ERR_UNSUPPORTED = -6
SWC_ERR_TOO_LARGE = -7

# Every symbol include/winograd2x2.h declares with C linkage.
C_SYMBOLS = (
    "swc_strerror", "swc_last_hip_error", "swc_version", "swc_winograd2x2_conv_last_kernel",
    "swc_winograd2x2_conv_force_tiling", "swc_winograd2x2_conv_grad_static",
    "swc_winograd2x2_imtrans", "swc_winograd2x2_imtrans_affine", "swc_winograd2x2_conv", "swc_winograd2x2_conv_bf16",
    "swc_winograd2x2_conv_epilogue",
    "swc_winograd2x2_imtrans_bf16out", "swc_winograd2x2_weights_bf16", "swc_winograd2x2_conv_bf16in",
    "swc_winograd2x2_conv_bf16in_ws", "swc_winograd2x2_conv_bf16in_workspace_floats",
    "swc_winograd2x2_relu_conv_bf16",
    "swc_winograd2x2_imtrans_op_shape", "swc_winograd2x2_imtrans_op_compute",
    "swc_winograd2x2_conv_op_shape", "swc_winograd2x2_conv_op_compute",
    "swc_winograd2x2_conv_grad_op_shape", "swc_winograd2x2_conv_grad_op_compute",
    "swc_winograd2x2_imtrans_grad_op_shape", "swc_winograd2x2_imtrans_grad_op_compute",
    "swc_winograd2x2_conv_grad", "swc_winograd2x2_imtrans_grad", "swc_winograd2x2_imtrans_grad_relu_input",
    "swc_winograd2x2_relu_conv", "swc_winograd2x2_pointwise_conv",
)
# The two C++-linkage launchers with the reference's exact signatures (Itanium mangling).
CXX_SYMBOLS = (
    "_Z33Winograd2x2ImTransComputeLauncherPKfPfiiiiii",
    "_Z30Winograd2x2ConvComputeLauncherPKfS0_PfS1_PKxiiiiiii",
    "_Z34Winograd2x2ConvGradComputeLauncherPKfS0_S0_PfS1_S1_Pxiiiiiii",
    "_Z37Winograd2x2ImTransGradComputeLauncherPKfPfiiiiii",
)

_lib = None


def build():
    """Compile the library for gfx950 with hipcc (works without a GPU)."""
    subprocess.check_call(["make", "-s", "-C", CSRC, "-j8"])
    return LIB_PATH


class SwcError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        msg = lib().swc_strerror(status).decode()
        if status == SWC_ERR_HIP:
            msg += " [hipError_t %d]" % lib().swc_last_hip_error()
        super().__init__("%s: %s (status %d)" % (where, msg, status))


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `make -C %s` (or __graft_entry__.build()); "
                "there is no CPU or PyTorch fallback for these ops" % (LIB_PATH, CSRC))
        L = ctypes.CDLL(LIB_PATH)
        vp, i32, fp = ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p
        i64p = ctypes.POINTER(ctypes.c_int64)
        L.swc_strerror.restype = ctypes.c_char_p
        L.swc_strerror.argtypes = [i32]
        L.swc_last_hip_error.restype = i32
        L.swc_last_hip_error.argtypes = []
        L.swc_version.restype = ctypes.c_char_p
        L.swc_version.argtypes = []
        L.swc_winograd2x2_conv_last_kernel.restype = ctypes.c_char_p
        L.swc_winograd2x2_conv_last_kernel.argtypes = []
        L.swc_winograd2x2_conv_force_tiling.restype = i32
        L.swc_winograd2x2_conv_force_tiling.argtypes = [ctypes.c_char_p]
        L.swc_winograd2x2_pointwise_conv.restype = i32
        L.swc_winograd2x2_pointwise_conv.argtypes = [fp] * 3 + [i32, ctypes.c_longlong, i32, vp]
        L.swc_winograd2x2_conv_grad_static.restype = i32
        L.swc_winograd2x2_conv_grad_static.argtypes = [fp] * 5 + [i32] * 7 + [vp]
        L.swc_winograd2x2_imtrans.restype = i32
        L.swc_winograd2x2_imtrans.argtypes = [fp, fp] + [i32] * 7 + [vp]
        L.swc_winograd2x2_imtrans_affine.restype = i32
        L.swc_winograd2x2_imtrans_affine.argtypes = [fp, fp, fp, fp] + [i32] * 7 + [vp]
        for f in (L.swc_winograd2x2_conv, L.swc_winograd2x2_conv_bf16):
            f.restype = i32
            f.argtypes = [fp, fp, fp, fp, vp] + [i32] * 7 + [vp]
        L.swc_winograd2x2_conv_epilogue.restype = i32
        L.swc_winograd2x2_conv_epilogue.argtypes = [fp] * 6 + [i32] * 9 + [vp]
        L.swc_winograd2x2_imtrans_bf16out.restype = i32
        L.swc_winograd2x2_imtrans_bf16out.argtypes = [fp, fp, fp, fp] + [i32] * 7 + [vp]
        L.swc_winograd2x2_weights_bf16.restype = i32
        L.swc_winograd2x2_weights_bf16.argtypes = [fp, fp, i32, i32, vp]
        L.swc_winograd2x2_conv_bf16in.restype = i32
        L.swc_winograd2x2_conv_bf16in.argtypes = [fp] * 6 + [i32] * 8 + [vp]
        L.swc_winograd2x2_conv_bf16in_ws.restype = i32
        L.swc_winograd2x2_conv_bf16in_ws.argtypes = [fp] * 6 + [i32, fp, ctypes.c_size_t] + [i32] * 7 + [vp]
        L.swc_winograd2x2_conv_bf16in_workspace_floats.restype = ctypes.c_size_t
        L.swc_winograd2x2_conv_bf16in_workspace_floats.argtypes = [i32] * 5
        L.swc_winograd2x2_relu_conv_bf16.restype = i32
        L.swc_winograd2x2_relu_conv_bf16.argtypes = [fp] * 8 + [i32] * 8 + [vp]
        L.swc_winograd2x2_imtrans_op_shape.restype = i32
        L.swc_winograd2x2_imtrans_op_shape.argtypes = [i32, i64p, i64p]
        L.swc_winograd2x2_imtrans_op_compute.restype = i32
        L.swc_winograd2x2_imtrans_op_compute.argtypes = [fp, i32, i64p, fp, i32, i64p, i32, vp]
        L.swc_winograd2x2_conv_op_shape.restype = i32
        L.swc_winograd2x2_conv_op_shape.argtypes = [i32, i64p, i32, i64p, i64p]
        L.swc_winograd2x2_conv_op_compute.restype = i32
        L.swc_winograd2x2_conv_op_compute.argtypes = [fp, i32, i64p, fp, i32, i64p, fp, i32, i64p, i32, vp]
        L.swc_winograd2x2_relu_conv.restype = i32
        L.swc_winograd2x2_relu_conv.argtypes = [fp] * 3 + [i32] * 8 + [vp]
        L.swc_winograd2x2_conv_grad_op_shape.restype = i32
        L.swc_winograd2x2_conv_grad_op_shape.argtypes = [i32, i64p, i32, i64p, i32, i64p, i64p, i64p, i64p]
        L.swc_winograd2x2_conv_grad_op_compute.restype = i32
        L.swc_winograd2x2_conv_grad_op_compute.argtypes = [fp, i32, i64p, fp, i32, i64p, fp, i32, i64p, fp, fp, fp,
                                                           ctypes.c_int64, vp]
        L.swc_winograd2x2_imtrans_grad_op_shape.restype = i32
        L.swc_winograd2x2_imtrans_grad_op_shape.argtypes = [i32, i64p, i64p]
        L.swc_winograd2x2_imtrans_grad_op_compute.restype = i32
        L.swc_winograd2x2_imtrans_grad_op_compute.argtypes = [fp, i32, i64p, fp, fp, fp, i32, i64p, vp]
        L.swc_winograd2x2_conv_grad.restype = i32
        L.swc_winograd2x2_conv_grad.argtypes = [fp] * 7 + [i32] * 7 + [vp]
        L.swc_winograd2x2_imtrans_grad.restype = i32
        L.swc_winograd2x2_imtrans_grad.argtypes = [fp] * 3 + [i32] * 6 + [vp]
        L.swc_winograd2x2_imtrans_grad_relu_input.restype = i32
        L.swc_winograd2x2_imtrans_grad_relu_input.argtypes = [fp] * 3 + [i32] * 6 + [vp]
        _lib = L
    return _lib


def dims(shape):
    return (ctypes.c_int64 * len(shape))(*[int(s) for s in shape])


class on_device(object):
    """``with on_device(dev) as stream:`` makes ``dev`` the current HIP device if it is not already (the
    usual case costs one query instead of a device switch and back) and yields the raw handle of
    PyTorch's current stream on it."""
    __slots__ = ("dev", "ctx")

    def __init__(self, dev):
        self.dev = dev
        self.ctx = None

    def __enter__(self):
        import torch

        idx = self.dev.index
        if idx is not None and idx != torch.cuda.current_device():
            self.ctx = torch.cuda.device(self.dev)
            self.ctx.__enter__()
        return torch.cuda.current_stream().cuda_stream

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False


def check(status, where):
    if status != SWC_OK:
        raise SwcError(status, where)


def require_cuda_f32(t, name, rank, dtype=None):
    """The checks a TensorFlow kernel registration did implicitly (float, DEVICE_GPU).
    ``dtype`` other than float32 is only used by the bf16-stored variant."""
    import torch

    dtype = torch.float32 if dtype is None else dtype
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a torch.Tensor, got %s" % (name, type(t).__name__))
    if t.dim() != rank:
        raise ValueError("%s must have rank %d, got shape %s" % (name, rank, tuple(t.shape)))
    if t.dtype != dtype:
        raise TypeError("%s must be %s, got %s" % (name, str(dtype).replace("torch.", ""), t.dtype))
    if not t.is_cuda:
        # The reference's CPU kernels print a message and exit(-1)
        # (winograd2x2_imTrans_op.cc:82-83, winograd2x2_conv_op.cc:89-90); here it is an error.
        raise RuntimeError("%s is on %s: these ops run on the GPU only (no CPU kernel exists)" % (name, t.device))
    return t.contiguous()
