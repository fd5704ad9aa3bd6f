"""Layer wrapper WinogradImTrans, after ResNet-18-var/winograd_imtrans.py:15-17."""
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import winograd2x2_imTrans.winograd2x2_imTrans  # noqa: E402

__all__ = ["WinogradImTrans", "identity"]


def identity(x):
    return x


_RELUS = (torch.relu, torch.nn.functional.relu)


def WinogradImTrans(x, nl=identity, affine=None, out_dtype=torch.float32):
    """``nl(winograd2x2_imTrans(x))`` as in the reference (winograd_imtrans.py:16-17).

    ``affine=(scale, shift)`` (forward only) transforms ``x*scale + shift`` instead of ``x``: the
    inference-mode BatchNorm that precedes every call in the reference model, folded into the kernel.
    ``out_dtype=torch.bfloat16`` (forward only) stores the result as bf16 for the bf16-stored convolution.

    ``nl`` may be a callable or the strings "identity"/"relu".  A ReLU (``torch.relu``,
    ``torch.nn.functional.relu``, an ``nn.ReLU`` module, or "relu") is fused into the
    transform kernel; any other callable is applied to the op's result.
    """
    op = winograd2x2_imTrans.winograd2x2_imTrans.winograd2x2_imTrans
    if affine is not None or out_dtype != torch.float32:
        scale, shift = affine if affine is not None else (None, None)
        base = op
        op = lambda t, relu=False: base(t, relu=relu, scale=scale, shift=shift, out_dtype=out_dtype)  # noqa: E731
    if nl is None or nl is identity or nl == "identity":
        return op(x)
    if nl == "relu" or isinstance(nl, torch.nn.ReLU) or any(nl is f for f in _RELUS):
        return op(x, relu=True)
    if not callable(nl):
        raise TypeError("nl must be callable, 'identity' or 'relu'")
    return nl(op(x))
