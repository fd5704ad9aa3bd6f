"""Layer wrapper WinogradConv, after ResNet-18-var/winograd_conv.py:15-28."""
import math
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import winograd2x2_conv.winograd2x2_conv  # noqa: E402

__all__ = ["WinogradConv"]


class WinogradConv(torch.nn.Module):
    """Holds the Winograd-domain weights W [16, in_channel, out_channel] and applies the op.

    Arguments follow ``WinogradConv(x, in_channel, out_channel, mask=None, W_init=None)``
    of the reference (winograd_conv.py:16), with ``x`` moved to ``forward``:

    * ``W_init``: callable filling a tensor in place, or a tensor/array of the weight's
      shape.  Default: the reference's ``variance_scaling_initializer(factor=2*9/32)``
      (:18-19): a normal truncated at two standard deviations with
      std = sqrt(1.3*factor/fan_in), fan_in = 16*in_channel as TensorFlow 1.x computes
      it for a rank-3 shape.
    * ``mask``: optional 0/1 array of the weight's shape; the reference multiplies it in on
      every step (:23-25).  Here W*mask is recomputed only while gradients are being recorded
      (so that they flow to W through the mask); otherwise the product is cached until W or
      mask is written to again (in place or replaced).

    W is a trainable parameter; gradients come from ``winograd2x2_conv_grad``.
    """

    def __init__(self, in_channel, out_channel, mask=None, W_init=None, precision="fp32", device=None):
        super().__init__()
        self.in_channel, self.out_channel, self.precision = int(in_channel), int(out_channel), precision
        W = torch.empty(16, self.in_channel, self.out_channel, dtype=torch.float32, device=device)
        if W_init is None:
            std = math.sqrt(1.3 * (2.0 * 9.0 / 32.0) / (16 * self.in_channel))
            torch.nn.init.trunc_normal_(W, mean=0.0, std=std, a=-2 * std, b=2 * std)
        elif callable(W_init):
            W_init(W)
        else:
            W.copy_(torch.as_tensor(W_init, dtype=torch.float32).reshape(W.shape))
        self.W = torch.nn.Parameter(W)
        if mask is not None:
            mask = torch.as_tensor(mask, dtype=torch.float32, device=W.device).reshape(W.shape).clone()
        self.register_buffer("mask", mask)
        self._masked = None
        self._bf16 = None

    def refresh(self):
        """Drop the cached W*mask and its bf16 copy.  Not needed after in-place updates of W or mask made on
        the tensors themselves or on ``detach()``ed views of them (optimizer steps, ``load_state_dict``,
        ``with torch.no_grad(): W.mul_(m)``): the caches are keyed on the tensors' version counters and storage,
        so those are noticed by themselves.  Needed after a write through ``.data`` (``layer.W.data.mul_(m)``,
        ``layer.W.data.copy_(w)``): a ``.data`` view carries a version counter of its own, so such a write leaves
        no trace on W."""
        self._masked = None
        self._bf16 = None

    def _weight_key(self):
        # In-place writes bump _version; a replaced or moved tensor changes data_ptr / device.
        w, m = self.W, self.mask
        return (w._version, w.data_ptr(), w.device, None if m is None else (m._version, m.data_ptr()))

    def bf16_weight(self):
        """W*mask as the [16,K,C] bfloat16 tensor the bf16-stored kernel reads; cached like masked_weight()."""
        key = self._weight_key()
        cached = self._bf16
        if cached is None or cached[0] != key:
            cached = (key, winograd2x2_conv.winograd2x2_conv.winograd2x2_weights_bf16(self.masked_weight()))
            self._bf16 = cached
        return cached[1]

    def masked_weight(self):
        """W*mask without autograd history, recomputed only when W or mask changed since the last call (a write
        through ``.data`` is not such a change: see refresh())."""
        if self.mask is None:
            return self.W.detach()   # shares W's version counter: a write to what is handed out is noticed
        key = self._weight_key()
        cached = self._masked
        if cached is None or cached[0] != key:
            cached = (key, (self.W.detach() * self.mask).contiguous())
            self._masked = cached
        return cached[1]

    def forward(self, x, affine=None, residual=None, residual_relu=False):
        """``affine=(scale, shift)`` and ``residual`` (forward only) are applied to the result inside
        the kernel: ``conv*scale + shift + residual`` (``+ relu(residual)`` with ``residual_relu``)."""
        if x.dtype == torch.bfloat16:      # bf16-stored activations: forward only
            w = self.bf16_weight()
        elif torch.is_grad_enabled() and self.W.requires_grad:
            w = self.W if self.mask is None else self.W * self.mask
        else:
            w = self.masked_weight()
        scale, shift = affine if affine is not None else (None, None)
        return winograd2x2_conv.winograd2x2_conv.winograd2x2_conv(x, w, precision=self.precision, scale=scale,
                                                                  shift=shift, residual=residual,
                                                                  residual_relu=residual_relu)
