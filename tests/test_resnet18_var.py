"""The ResNet-18-var forward harness (benchmark config 5 topology) with its 16 convs through the ops."""
import numpy as np
import pytest
import torch

from helpers import expected_stored_launch, rel_max


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


PRECISIONS = [("fp32", 1e-3), ("bf16", 5e-2), ("bf16_stored", 5e-2)]


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(2, 7, 9, 64, 64), (1, 5, 5, 32, 40), (3, 14, 14, 128, 256), (1, 3, 3, 96, 20),
                                   (2, 4, 4, 48, 64)])
def test_pointwise_conv(shape):
    # The model's 1x1 shortcut convolutions (imagenet-resnet-transWino-prune.py:127,152,177,202) as a product over
    # NHWC pixels: against float64 numpy, exact on small integers; C = 48 is not taken by the kernel and falls back.
    import resnet18_var
    import swc_hip
    B, H, W, C, K = shape
    rng = np.random.default_rng(77)
    dev = torch.device("cuda:0")
    x = rng.standard_normal((B, H, W, C)).astype(np.float32)
    w = rng.standard_normal((K, C)).astype(np.float32)
    got = resnet18_var.pointwise_conv(torch.from_numpy(x).to(dev), torch.from_numpy(w).to(dev)).cpu().numpy()
    want = x.astype(np.float64).reshape(-1, C) @ w.astype(np.float64).T
    assert got.shape == (B, H, W, K)
    assert rel_max(got.reshape(-1, K), want) <= 1e-5
    xi = rng.integers(-4, 5, size=x.shape).astype(np.float32)
    wi = rng.integers(-4, 5, size=w.shape).astype(np.float32)
    goti = resnet18_var.pointwise_conv(torch.from_numpy(xi).to(dev), torch.from_numpy(wi).to(dev)).cpu().numpy()
    assert np.array_equal(goti.reshape(-1, K), xi.reshape(-1, C) @ wi.T)
    out = torch.empty(B * H * W * K, device=dev)
    st = swc_hip.lib().swc_winograd2x2_pointwise_conv(torch.from_numpy(x).to(dev).data_ptr(), torch.from_numpy(w).to(dev).data_ptr(),
                                                      out.data_ptr(), C, B * H * W, K, torch.cuda.current_stream().cuda_stream)
    assert st == (swc_hip.SWC_ERR_UNSUPPORTED if C % 32 else 0)


@pytest.mark.gpu
@pytest.mark.parametrize("precision,tol", PRECISIONS)
def test_forward_matches_oracle_path(oracle, precision, tol):
    _forward_against_oracle_path(oracle, precision, tol, batch=2, size=64, check_unfolded=True)


@pytest.mark.gpu
@pytest.mark.parametrize("precision,tol", PRECISIONS)
def test_forward_matches_oracle_path_at_224(oracle, precision, tol):
    # Benchmark config 5's image size: the 16 layers run at 56/28/14/14 as in
    # imagenet-resnet-transWino-prune.py:113-212 (the 64x64 case above runs them at 16/8/4/4).
    _forward_against_oracle_path(oracle, precision, tol, batch=2, size=224, check_unfolded=False)


def _forward_against_oracle_path(oracle, precision, tol, batch, size, check_unfolded):
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
    image = torch.from_numpy(rng.standard_normal((batch, size, size, 3)).astype(np.float32))

    def cpu_imtrans(x, nl=None, affine=None, out_dtype=torch.float32):
        x = x.numpy()
        if affine is not None:
            x = oracle.affine(x, affine[0].detach().numpy(), affine[1].detach().numpy())
        t = oracle.imtrans(x, relu=True)
        if out_dtype == torch.bfloat16:     # stored rounded; the CPU chain carries the rounded values as fp32
            t = oracle.round_bf16(t)
        return torch.from_numpy(t)

    def cpu_conv_forward(self, x, affine=None, residual=None, residual_relu=False):
        y = oracle.conv(x.numpy(), self.masked_weight().numpy(), acc64=True)
        if affine is not None:
            y = oracle.affine(y, affine[0].detach().numpy(), affine[1].detach().numpy())
        if residual is not None:
            y = y + (np.maximum(residual.numpy(), 0) if residual_relu else residual.numpy())
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
    assert got.shape == want.shape == (batch, 1000)
    assert np.isfinite(got).all()
    assert rel_max(got, want) <= tol
    if not check_unfolded:
        return
    # Folding the BatchNorm into the transform changes roundings only (one fma per pixel instead of
    # PyTorch's normalisation arithmetic).
    unfolded = resnet18_var.ResNet18Var(masks=masks, precision=precision, fold_bn=False)
    unfolded.load_state_dict(model.state_dict())
    unfolded = unfolded.to(dev)
    for c in unfolded.winograd_convs():
        c.refresh()
    assert rel_max(unfolded(image.to(dev)).cpu().numpy(), got) <= tol


# The distinct (H = W, C, K) of the 16 layers (imagenet-resnet-transWino-prune.py:117-211): 4x (56,64,64), (28,64,128),
# 3x (28,128,128), (14,128,256), 3x (14,256,256), (14,256,512), 3x (14,512,512).
LAYER_SHAPES = [(56, 64, 64), (28, 64, 128), (28, 128, 128), (14, 128, 256), (14, 256, 256), (14, 256, 512), (14, 512, 512)]


@pytest.mark.gpu
@pytest.mark.parametrize("precision", ["fp32", "bf16", "bf16_stored"])
@pytest.mark.parametrize("hw,C,K", LAYER_SHAPES)
def test_layers_at_batch_128(oracle, hw, C, K, precision):
    """Every layer shape of config 5 at its real batch (N = 128), so that the launcher makes the choice it
    makes in the benchmark: the transform is compared bit for bit and the convolution within tolerance with
    the oracle on the first and the last two images (tiles are independent, so a slice of the batch has the
    values it would have alone; the last images sit in the ragged final row groups)."""
    import swc_hip
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv
    from winograd2x2_imTrans.winograd2x2_imTrans import winograd2x2_imTrans
    dev = torch.device("cuda:0")
    N, k = 128, 2
    gen = torch.Generator(device=dev).manual_seed(hw * 1000 + C + K)
    x = torch.randn((N, hw, hw, C), device=dev, generator=gen)
    w = (np.random.default_rng(C * K).standard_normal((16, C, K)) * 0.05).astype(np.float32)
    oracle.gen_prune_mask(w, 0.2)
    w_gpu = torch.from_numpy(w).to(dev)
    stored = precision == "bf16_stored"
    ti = winograd2x2_imTrans(x, relu=True, out_dtype=torch.bfloat16 if stored else torch.float32)
    y = winograd2x2_conv(ti, w_gpu, precision="fp32" if stored else precision)
    kernel = swc_hip.lib().swc_winograd2x2_conv_last_kernel().decode()
    assert y.shape == (N, hw, hw, K)
    for sl in (slice(0, k), slice(N - k, N)):
        x_cpu = x[sl].cpu().numpy()
        ti_want = oracle.imtrans(x_cpu, relu=True)
        if stored:
            assert np.array_equal(ti[:, sl].view(torch.int16).cpu().numpy().view(np.uint16), oracle.bf16_bits(ti_want))
            ti_want, w_want = oracle.round_bf16(ti_want), oracle.round_bf16(w)
        else:
            assert np.array_equal(ti[:, sl].cpu().numpy(), ti_want)
            w_want = w
            if precision == "bf16":
                ti_want, w_want = oracle.round_bf16(ti_want), oracle.round_bf16(w)
        want = oracle.conv(ti_want, w_want, acc64=True)
        assert rel_max(y[sl].cpu().numpy(), want) <= 1e-4, (kernel, sl)
    if precision == "fp32":
        assert kernel != "sync", kernel   # every model shape runs on one of the copy-ring tilings
    if stored:
        # The launcher reads the CU count and the L2 size from the device; so does the expectation.
        props = torch.cuda.get_device_properties(dev)
        M = N * ((hw + 1) // 2) ** 2
        assert kernel in expected_stored_launch(M, C, K, props.multi_processor_count, props.L2_cache_size), kernel
