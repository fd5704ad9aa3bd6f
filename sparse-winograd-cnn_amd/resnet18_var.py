"""Forward pass of the reference's ResNet-18 variant with its sixteen 3x3 convolutions routed
through the Winograd-ReLU ops (inference only).

Topology after ``Model._build_graph`` in ResNet-18-var/imagenet-resnet-transWino-prune.py:109-220:
conv1 7x7/2 (no BN, :113) -> pool 3/2 (:115); four stages of two residual units; every unit is
``BN -> WinogradImTrans(relu) -> WinogradConv -> BN -> WinogradImTrans(relu) -> WinogradConv -> BN``
(:117-123 ...), the first unit of a stage adds a 1x1 shortcut conv + BN (:126-129, :152-155, ...);
3/2 max-pools close stages 2 and 3 (:141,:166) but not stage 4 (pool4 is commented out, :191), so
stage 5 also runs at 14x14; ReLU, global average pool, (dropout: identity at inference), FC 1000
(:213-219).  Padding of the strided conv and the pools is TensorFlow's SAME (the extra pixel goes
after, not before).

Everything except the two Winograd ops is stock PyTorch.  Activations are kept NHWC in memory
(channels_last), so handing them to the ops and back costs no copies.  The BatchNorm in front of
each WinogradImTrans (inference statistics) is folded into the transform kernel as a per-channel
scale and shift, and the BatchNorm plus residual add behind each unit's second convolution into
that convolution's stores; ``fold_bn=False`` runs them as separate PyTorch passes instead.
"""
import os
import sys

import torch
import torch.nn.functional as F

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import swc_hip  # noqa: E402
from winograd_conv import WinogradConv  # noqa: E402
from winograd_imtrans import WinogradImTrans  # noqa: E402

# (unit name, C_in of the first conv, C_out, has 1x1 shortcut conv, max-pool after the unit)
UNITS = (
    ("2a", 64, 64, True, False), ("2b", 64, 64, False, True),
    ("3a", 64, 128, True, False), ("3b", 128, 128, False, True),
    ("4a", 128, 256, True, False), ("4b", 256, 256, False, False),
    ("5a", 256, 512, True, False), ("5b", 512, 512, False, False),
)


def winograd_layer_names():
    """The 16 weight names of the reference graph, in order (Winograd_W2a_2a ... Winograd_W5b_2b)."""
    return ["Winograd_W%s_2%s" % (u[0], ab) for u in UNITS for ab in "ab"]


def _same_pad(x, k, stride):
    """TensorFlow SAME padding for an NCHW tensor: total = max((ceil(n/s)-1)*s + k - n, 0), smaller half first."""
    pads = []
    for n in (x.shape[3], x.shape[2]):  # F.pad wants W first
        total = max((-(-n // stride) - 1) * stride + k - n, 0)
        pads += [total // 2, total - total // 2]
    return pads


def _max_pool_same(x):
    """3x3 stride-2 max-pool with TensorFlow SAME padding.  Where the padding falls entirely behind the
    data (even sizes) ``ceil_mode`` gives the same windows without a padded copy of the tensor."""
    pads = _same_pad(x, 3, 2)
    if pads[0] == 0 and pads[2] == 0:
        return F.max_pool2d(x, 3, 2, ceil_mode=True)
    return F.max_pool2d(F.pad(x, pads, value=float("-inf")), 3, 2)


def _bn_affine(bn):
    """Inference-mode BatchNorm2d as y = x*scale + shift; cached until a parameter or statistic changes."""
    tensors = (bn.weight, bn.bias, bn.running_mean, bn.running_var)
    key = tuple((t._version, t.data_ptr()) for t in tensors)
    cached = getattr(bn, "_swc_affine", None)
    if cached is None or cached[0] != key:
        scale = (bn.weight * torch.rsqrt(bn.running_var + bn.eps)).detach()
        cached = (key, scale.contiguous(), (bn.bias - bn.running_mean * scale).detach().contiguous())
        bn._swc_affine = cached
    return cached[1], cached[2]


def _conv_bn_folded(conv, bn):
    """A bias-free conv followed by an inference-mode BatchNorm as one conv: weights scaled per output
    channel, the shift as bias.  Cached until the weights or the BatchNorm change."""
    scale, shift = _bn_affine(bn)
    key = (conv.weight._version, conv.weight.data_ptr(), bn._swc_affine[0])
    cached = getattr(conv, "_swc_folded", None)
    if cached is None or cached[0] != key:
        cached = (key, (conv.weight * scale.view(-1, 1, 1, 1)).detach(), shift)
        conv._swc_folded = cached
    return cached[1], cached[2]


def _shortcut_folded(conv, bn, bn_out):
    """The 1x1 shortcut conv + its BatchNorm, for a branch whose last convolution applies ``bn_out`` and adds
    the shortcut in its stores: returns (W [Cout,Cin], scale, shift) such that
    ``branch*scale + shift + x_nhwc @ W.T == bn_out(branch) + bn(conv(x))``.  A 1x1 convolution over NHWC data is
    one matrix product, and its bias joins the shift the kernel adds anyway.  Cached like _conv_bn_folded."""
    w1, b1 = _conv_bn_folded(conv, bn)
    scale, shift = _bn_affine(bn_out)
    key = (conv._swc_folded[0], bn_out._swc_affine[0])
    cached = getattr(conv, "_swc_shortcut", None)
    if cached is None or cached[0] != key:
        cached = (key, w1.view(w1.shape[0], w1.shape[1]).contiguous(), scale, (shift + b1).contiguous())
        conv._swc_shortcut = cached
    return cached[1], cached[2], cached[3]


def pointwise_conv(x, w):
    """x [B,H,W,C] NHWC, w [K,C] -> [B,H,W,K]: a 1x1 convolution.  On the GPU it runs on the library's kernel
    (``swc_winograd2x2_pointwise_conv``) where that takes the shape (C % 32 == 0), else as a matrix product."""
    B, H, W, C = x.shape
    if x.is_cuda and x.dtype == torch.float32 and w.dtype == torch.float32 and x.is_contiguous() and w.is_contiguous():
        out = torch.empty((B, H, W, w.shape[0]), dtype=torch.float32, device=x.device)
        with swc_hip.on_device(x.device) as stream:
            st = swc_hip.lib().swc_winograd2x2_pointwise_conv(x.data_ptr(), w.data_ptr(), out.data_ptr(), C, B * H * W,
                                                              w.shape[0], stream)
        if st != swc_hip.SWC_ERR_UNSUPPORTED:
            swc_hip.check(st, "pointwise_conv")
            return out
    return torch.mm(x.reshape(-1, C), w.t()).view(B, H, W, w.shape[0])


def _to_nhwc(x):   # NCHW tensor in channels_last memory -> contiguous [B,H,W,C] view
    return x.permute(0, 2, 3, 1).contiguous()


def _to_nchw(y):   # contiguous [B,H,W,C] -> NCHW tensor in channels_last memory (a view)
    return y.permute(0, 3, 1, 2)


class WinogradUnit(torch.nn.Module):
    def __init__(self, name, c_in, c_out, shortcut, pool, masks, precision, fold_bn=True):
        super().__init__()
        self.name, self.pool, self.fold_bn = name, pool, fold_bn
        # "bf16": fp32 transformed activations, operands rounded inside the GEMM kernel;
        # "bf16_stored": the transformed activations themselves are kept in bf16 (needs fold_bn)
        self.ti_dtype = torch.bfloat16 if precision == "bf16_stored" else torch.float32
        precision = "bf16" if precision == "bf16_stored" else precision
        self.bn2a = torch.nn.BatchNorm2d(c_in)
        self.conv2a = WinogradConv(c_in, c_out, mask=masks.get("Winograd_W%s_2a/W" % name), precision=precision)
        self.bn2b = torch.nn.BatchNorm2d(c_out)
        self.conv2b = WinogradConv(c_out, c_out, mask=masks.get("Winograd_W%s_2b/W" % name), precision=precision)
        self.bn2c = torch.nn.BatchNorm2d(c_out)
        self.shortcut = shortcut
        if shortcut:
            self.bn_pre = torch.nn.BatchNorm2d(c_in) if name == "2a" else None  # BNReLU('res2a_1_relu') only in 2a
            self.conv1 = torch.nn.Conv2d(c_in, c_out, 1, bias=False)
            self.bn1 = torch.nn.BatchNorm2d(c_out)

    def branch(self, x, shortcut=None, out_affine=None, shortcut_relu=False):
        """The two Winograd layers.  With ``fold_bn`` the three BatchNorms and the residual add run inside
        the Winograd kernels (bn2a, bn2b in the transforms' loads; bn2c and ``+ shortcut`` in the second
        convolution's stores) and the result is already ``shortcut + branch``; ``shortcut`` is then NHWC and
        ``out_affine`` replaces bn2c's (scale, shift); ``shortcut_relu``: the kernel adds ``relu(shortcut)``."""
        if self.fold_bn:
            dt = self.ti_dtype
            h = self.conv2a(WinogradImTrans(_to_nhwc(x), torch.relu, affine=_bn_affine(self.bn2a), out_dtype=dt))
            h = self.conv2b(WinogradImTrans(h, torch.relu, affine=_bn_affine(self.bn2b), out_dtype=dt),
                            affine=out_affine if out_affine is not None else _bn_affine(self.bn2c), residual=shortcut,
                            residual_relu=shortcut_relu)
            return _to_nchw(h)
        h = _to_nchw(self.conv2a(WinogradImTrans(_to_nhwc(self.bn2a(x)), torch.relu)))
        h = _to_nchw(self.conv2b(WinogradImTrans(_to_nhwc(self.bn2b(h)), torch.relu)))
        return shortcut + self.bn2c(h)

    def forward(self, x):
        out_affine = None
        if self.shortcut:
            if self.bn_pre is not None and self.fold_bn:
                # BNReLU as x*scale + shift and an in-place ReLU: two elementwise passes instead of the library
                # BatchNorm's slower one plus a ReLU that allocates
                a, b = _bn_affine(self.bn_pre)
                s = torch.addcmul(b.view(1, -1, 1, 1), x, a.view(1, -1, 1, 1)).relu_()
            else:
                s = torch.relu(self.bn_pre(x)) if self.bn_pre is not None else torch.relu(x)
            if self.fold_bn:
                w1, scale, shift = _shortcut_folded(self.conv1, self.bn1, self.bn2c)
                sc = pointwise_conv(_to_nhwc(s), w1)
                out_affine = (scale, shift)
            else:
                sc = self.bn1(self.conv1(s))
        elif self.fold_bn:
            sc = _to_nhwc(x)   # the identity shortcut relu(x): its ReLU is applied where the kernel reads it
        else:
            sc = torch.relu(x)
        x = self.branch(x, sc, out_affine, shortcut_relu=self.fold_bn and not self.shortcut)
        if self.pool:
            x = _max_pool_same(x)
        return x


class ResNet18Var(torch.nn.Module):
    """``masks``: optional dict of 0/1 arrays keyed like the reference's pruning masks
    ('Winograd_W2a_2a/W', ...; prune_script.py:68-78).  ``precision``: 'fp32' or 'bf16' GEMM operands, or 'bf16_stored' (bf16 operands with
    the transformed activations also stored as bf16; needs ``fold_bn``)."""

    def __init__(self, masks=None, precision="fp32", num_classes=1000, fold_bn=True):
        super().__init__()
        masks = masks or {}
        self.conv1 = torch.nn.Conv2d(3, 64, 7, stride=2, bias=False)
        self.units = torch.nn.ModuleList(
            [WinogradUnit(n, ci, co, sc, pool, masks, precision, fold_bn) for n, ci, co, sc, pool in UNITS])
        self.linear = torch.nn.Linear(512, num_classes)
        self.eval()

    def winograd_convs(self):
        return [c for u in self.units for c in (u.conv2a, u.conv2b)]

    @torch.no_grad()
    def forward(self, image):
        """image: [B,H,W,3] float32 NHWC (already normalised) -> logits [B,num_classes]."""
        x = image.permute(0, 3, 1, 2)  # NCHW view over NHWC memory = channels_last
        x = self.conv1(F.pad(x, _same_pad(x, 7, 2)))
        x = _max_pool_same(x)
        x = x.contiguous(memory_format=torch.channels_last)
        for unit in self.units:
            x = unit(x)
        x = torch.relu(x).mean(dim=(2, 3))
        return self.linear(x)
