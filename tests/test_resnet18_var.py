"""The ResNet-18-var forward harness (benchmark config 5 topology) with its 16 convs through the ops."""
import numpy as np
import pytest
import torch

from helpers import rel_max


def test_topology_matches_reference_graph():
    # ResNet-18-var/imagenet-resnet-transWino-prune.py:117-212: names, channel pairs, 16 layers
    import resnet18_var
    model = resnet18_var.ResNet18Var()
    names = resnet18_var.winograd_layer_names()
    assert names[0] == "Winograd_W2a_2a" and names[-1] == "Winograd_W5b_2b" and len(names) == 16
    shapes = [tuple(c.W.shape) for c in model.winograd_convs()]
    want = [(64, 64)] * 4 + [(64, 128)] + [(128, 128)] * 3 + [(128, 256)] + [(256, 256)] * 3 + [(256, 512)] + [(512, 512)] * 3
    assert shapes == [(16, a, b) for a, b in want]
    assert [u.shortcut for u in model.units] == [True, False] * 4
    assert [u.pool for u in model.units] == [False, True, False, True, False, False, False, False]  # pool4 is commented out (:191)
    assert model.units[0].bn_pre is not None and model.units[2].bn_pre is None  # BNReLU only in res2a (:125)


def test_same_padding_rule():
    import resnet18_var
    x = torch.zeros(1, 1, 224, 224)
    assert resnet18_var._same_pad(x, 7, 2) == [2, 3, 2, 3]   # conv1: 224 -> 112
    assert resnet18_var._same_pad(torch.zeros(1, 1, 112, 112), 3, 2) == [0, 1, 0, 1]
    assert resnet18_var._same_pad(torch.zeros(1, 1, 7, 9), 3, 2) == [1, 1, 1, 1]


@pytest.mark.gpu
@pytest.mark.parametrize("precision,tol", [("fp32", 1e-3), ("bf16", 5e-2), ("bf16_stored", 5e-2)])
def test_forward_matches_oracle_path(oracle, precision, tol):
    # Same module, same weights: once on the GPU through the HIP ops, once on the CPU with the two
    # Winograd ops replaced by the oracle.
    import resnet18_var
    import winograd_conv
    torch.manual_seed(0)
    rng = np.random.default_rng(500)
    masks = {}
    for name, (_, ci, co, _, _) in zip(["%s_2a" % u[0] for u in resnet18_var.UNITS], resnet18_var.UNITS):
        w = rng.standard_normal((16, ci, co)).astype(np.float32)
        masks["Winograd_W%s/W" % name] = oracle.gen_prune_mask(w, 0.3)
    model = resnet18_var.ResNet18Var(masks=masks, precision=precision)
    for bn in [m for m in model.modules() if isinstance(m, torch.nn.BatchNorm2d)]:
        bn.running_mean.normal_(0, 0.1)
        bn.running_var.uniform_(0.5, 1.5)
        bn.weight.data.uniform_(0.5, 1.5)
        bn.bias.data.normal_(0, 0.1)
    image = torch.from_numpy(rng.standard_normal((2, 64, 64, 3)).astype(np.float32))

    def cpu_imtrans(x, nl=None, affine=None, out_dtype=torch.float32):
        x = x.numpy()
        if affine is not None:
            x = oracle.affine(x, affine[0].detach().numpy(), affine[1].detach().numpy())
        t = oracle.imtrans(x, relu=True)
        if out_dtype == torch.bfloat16:     # stored rounded; the CPU chain carries the rounded values as fp32
            t = oracle.round_bf16(t)
        return torch.from_numpy(t)

    def cpu_conv_forward(self, x, affine=None, residual=None):
        y = oracle.conv(x.numpy(), self.masked_weight().numpy(), acc64=True)
        if affine is not None:
            y = oracle.affine(y, affine[0].detach().numpy(), affine[1].detach().numpy())
        if residual is not None:
            y = y + residual.numpy()
        return torch.from_numpy(y)

    orig_imtrans, orig_forward = resnet18_var.WinogradImTrans, winograd_conv.WinogradConv.forward
    try:
        resnet18_var.WinogradImTrans = cpu_imtrans
        winograd_conv.WinogradConv.forward = cpu_conv_forward
        want = model(image).numpy()
    finally:
        resnet18_var.WinogradImTrans, winograd_conv.WinogradConv.forward = orig_imtrans, orig_forward

    dev = torch.device("cuda:0")
    model = model.to(dev)
    for c in model.winograd_convs():
        c.refresh()
    got = model(image.to(dev)).cpu().numpy()
    assert got.shape == want.shape == (2, 1000)
    assert np.isfinite(got).all()
    assert rel_max(got, want) <= tol
    # Folding the BatchNorm into the transform changes roundings only (one fma per pixel instead of
    # PyTorch's normalisation arithmetic).
    unfolded = resnet18_var.ResNet18Var(masks=masks, precision=precision, fold_bn=False)
    unfolded.load_state_dict(model.state_dict())
    unfolded = unfolded.to(dev)
    for c in unfolded.winograd_convs():
        c.refresh()
    assert rel_max(unfolded(image.to(dev)).cpu().numpy(), got) <= tol
