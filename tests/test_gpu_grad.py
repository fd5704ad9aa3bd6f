"""Parity of the backward ops (Winograd2x2ConvGrad, Winograd2x2ImTransGrad) against the CPU oracle.

Tolerances: gradients are sums of up to M (dW) or K (dTI) products in an order the GEMM library
chooses, so they are held to 1e-4 relative like the forward conv; on small integers every sum is
exact and the results must match bit for bit.
"""
import numpy as np
import pytest
import torch

from helpers import rel_max, tiles

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available()
    import swc_hip
    swc_hip.lib()
    return torch.device("cuda:0")


def gpu(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


@pytest.mark.parametrize("shape", [
    (2, 6, 6, 8), (2, 7, 5, 4), (1, 8, 4, 3), (1, 1, 1, 1), (4, 28, 28, 128), (2, 14, 14, 36),
    # several workgroup blocks of tiles along one axis, ragged at the far edge:
    (1, 9, 139, 8), (2, 141, 5, 4), (1, 37, 43, 12),
])
@pytest.mark.parametrize("masked", [False, True, "input"])
def test_imtrans_grad(oracle, dev, shape, masked):
    """masked: through the fused ReLU, with its mask read from the forward result (True) or recomputed
    from the forward input ("input"; must give the same bits)."""
    from winograd2x2_imTrans.winograd2x2_imTrans import winograd2x2_imTrans_grad
    B, H, W, C = shape
    rng = np.random.default_rng(31)
    x = rng.standard_normal(shape).astype(np.float32)
    if masked == "input":
        # values whose sums cancel exactly, so that entries of the transform sit at 0 (masked) and not near it
        x = rng.integers(-2, 3, size=shape).astype(np.float32)
    ti = oracle.imtrans(x, relu=True)
    kw = {}
    if masked is True:
        kw["relu_output"] = gpu(ti, dev)
    elif masked == "input":
        kw["relu_input"] = gpu(x, dev)
    g = rng.standard_normal(ti.shape).astype(np.float32)
    want = oracle.imtrans_grad(g, H, W, mask_src=ti if masked else None)
    got = winograd2x2_imTrans_grad(gpu(g, dev), H, W, **kw).cpu().numpy()
    assert got.shape == (B, H, W, C)
    assert rel_max(got, want) <= 1e-6
    gi = rng.integers(-4, 5, size=ti.shape).astype(np.float32)
    wanti = oracle.imtrans_grad(gi, H, W, mask_src=ti if masked else None)
    goti = winograd2x2_imTrans_grad(gpu(gi, dev), H, W, **kw).cpu().numpy()
    assert np.array_equal(goti, wanti)


def test_imtrans_grad_mask_from_input_matches_mask_from_output(dev):
    """On real-valued inputs the recomputed mask is the forward pass's own, bit for bit."""
    from winograd2x2_imTrans.winograd2x2_imTrans import winograd2x2_imTrans, winograd2x2_imTrans_grad
    torch.manual_seed(5)
    x = torch.randn(3, 13, 27, 20, device=dev)
    ti = winograd2x2_imTrans(x, relu=True)
    g = torch.randn_like(ti)
    a = winograd2x2_imTrans_grad(g, 13, 27, relu_output=ti)
    b = winograd2x2_imTrans_grad(g, relu_input=x)
    assert torch.equal(a, b)
    with pytest.raises(ValueError):
        winograd2x2_imTrans_grad(g, relu_output=ti, relu_input=x)
    with pytest.raises(ValueError):
        winograd2x2_imTrans_grad(g, relu_input=x[:, :12])


@pytest.mark.parametrize("shape", [
    (3, 3, 3, 32, 32), (2, 4, 4, 5, 7), (1, 1, 1, 1, 1), (2, 3, 5, 36, 100), (8, 14, 14, 128, 128),
    # M % 32 == 0 takes the split-reduction weight-gradient kernel:
    (2, 4, 4, 36, 100),   # one split, ragged channel and filter tiles
    (16, 4, 4, 36, 20),   # 8 splits of a single step each
    (6, 8, 8, 64, 72),    # 12 steps in 5 splits (3,3,3,3 -> per = 3, last split shorter)
])
def test_conv_grad(oracle, dev, shape):
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv_grad
    B, nH, nW, C, K = shape
    rng = np.random.default_rng(32)
    ti = np.maximum(rng.standard_normal((16, B, nH, nW, C)), 0).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    dy = rng.standard_normal((B, 2 * nH, 2 * nW, K)).astype(np.float32)
    dti_want, dw_want = oracle.conv_grad(ti, w, dy)
    dti, dw = winograd2x2_conv_grad(gpu(ti, dev), gpu(w, dev), gpu(dy, dev))
    assert rel_max(dti.cpu().numpy(), dti_want) <= TOL
    assert rel_max(dw.cpu().numpy(), dw_want) <= TOL
    if B * nH * nW <= 384:
        tii = rng.integers(-3, 4, size=ti.shape).astype(np.float32)
        wi = rng.integers(-3, 4, size=w.shape).astype(np.float32)
        dyi = rng.integers(-3, 4, size=dy.shape).astype(np.float32)
        a, b = winograd2x2_conv_grad(gpu(tii, dev), gpu(wi, dev), gpu(dyi, dev))
        aw, bw = oracle.conv_grad(tii, wi, dyi)
        assert np.array_equal(a.cpu().numpy(), aw) and np.array_equal(b.cpu().numpy(), bw)


@pytest.mark.parametrize("shape", [
    (8, 14, 14, 128, 128),   # levelled row groups
    (2, 20, 20, 128, 64),    # 16 full 48-row groups + 2 left-over row tiles: 256 (tile, position) products
    (2, 2, 197, 128, 64),    # the second left-over tile holds 4 rows
    (3, 5, 7, 256, 128),     # two column groups, one valid row per workgroup
    (32, 1, 193, 256, 64),   # two column groups, left-over rows
])
def test_conv_grad_data_gradient_on_wide_tiles(oracle, dev, shape):
    """dTI on the 48-row x 128-column kernel, forced on shapes below the size at which the launcher takes it by
    itself (swc_winograd2x2_conv_force_tiling("wide48") covers the data gradient as well)."""
    import swc_hip
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv_grad
    L = swc_hip.lib()
    B, nH, nW, C, K = shape
    rng = np.random.default_rng(34)
    ti = np.maximum(rng.standard_normal((16, B, nH, nW, C)), 0).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    dy = rng.standard_normal((B, 2 * nH, 2 * nW, K)).astype(np.float32)
    tii = rng.integers(-3, 4, size=ti.shape).astype(np.float32)
    wi = rng.integers(-3, 4, size=w.shape).astype(np.float32)
    dyi = rng.integers(-3, 4, size=dy.shape).astype(np.float32)
    assert L.swc_winograd2x2_conv_force_tiling(b"wide48") == 0
    try:
        dti, dw = winograd2x2_conv_grad(gpu(ti, dev), gpu(w, dev), gpu(dy, dev))
        a, b = winograd2x2_conv_grad(gpu(tii, dev), gpu(wi, dev), gpu(dyi, dev))
    finally:
        assert L.swc_winograd2x2_conv_force_tiling(None) == 0
    dti_want, dw_want = oracle.conv_grad(ti, w, dy)
    assert rel_max(dti.cpu().numpy(), dti_want) <= TOL
    assert rel_max(dw.cpu().numpy(), dw_want) <= TOL
    aw, bw = oracle.conv_grad(tii, wi, dyi)
    assert np.array_equal(a.cpu().numpy(), aw) and np.array_equal(b.cpu().numpy(), bw)
    # the same call with the 64x64-tile kernel forced gives the same values to rounding
    assert L.swc_winograd2x2_conv_force_tiling(b"ring32") == 0
    try:
        dti2, _ = winograd2x2_conv_grad(gpu(ti, dev), gpu(w, dev), gpu(dy, dev))
    finally:
        assert L.swc_winograd2x2_conv_force_tiling(None) == 0
    assert rel_max(dti2.cpu().numpy(), dti_want) <= TOL


@pytest.mark.parametrize("shape", [
    (1, 4, 4, 128, 128),     # M = 16: a single step, no split
    (2, 4, 6, 128, 128),     # M = 48: three steps, no split
    (4, 8, 9, 128, 128),     # M = 288: two splits of nine steps
    (2, 8, 17, 128, 256),    # M = 272 = 17 x 16: not a multiple of 32, two filter tiles
    (8, 8, 13, 256, 128),    # M = 832: six splits, the last one shorter, two channel tiles
])
def test_conv_grad_weight_gradient_on_wide_tiles(oracle, dev, shape):
    """dW on the 128x128-tile kernel (C and K multiples of 128, M a multiple of 16), taken by default and under
    "wide48"; any other forced tiling runs the 64x64-tile kernel or the plain GEMM on the same shapes."""
    import swc_hip
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv_grad
    L = swc_hip.lib()
    B, nH, nW, C, K = shape
    rng = np.random.default_rng(35)
    ti = np.maximum(rng.standard_normal((16, B, nH, nW, C)), 0).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    dy = rng.standard_normal((B, 2 * nH, 2 * nW, K)).astype(np.float32)
    tii = rng.integers(-3, 4, size=ti.shape).astype(np.float32)
    wi = rng.integers(-3, 4, size=w.shape).astype(np.float32)
    dyi = rng.integers(-3, 4, size=dy.shape).astype(np.float32)
    dti_want, dw_want = oracle.conv_grad(ti, w, dy)
    aw, bw = oracle.conv_grad(tii, wi, dyi)
    for forced in (None, b"wide48", b"ring32"):
        assert L.swc_winograd2x2_conv_force_tiling(forced) == 0
        try:
            dti, dw = winograd2x2_conv_grad(gpu(ti, dev), gpu(w, dev), gpu(dy, dev))
            a, b = winograd2x2_conv_grad(gpu(tii, dev), gpu(wi, dev), gpu(dyi, dev))
        finally:
            assert L.swc_winograd2x2_conv_force_tiling(None) == 0
        assert rel_max(dw.cpu().numpy(), dw_want) <= TOL, forced
        assert rel_max(dti.cpu().numpy(), dti_want) <= TOL, forced
        assert np.array_equal(b.cpu().numpy(), bw) and np.array_equal(a.cpu().numpy(), aw), forced


def test_autograd_through_the_layer(oracle, dev):
    # d/dx and d/dW of sum(g * WinogradConv(WinogradImTrans(x, relu))) against the oracle chain.
    from winograd_conv import WinogradConv
    from winograd_imtrans import WinogradImTrans
    rng = np.random.default_rng(33)
    B, H, W, C, K = 2, 8, 6, 16, 24
    x = rng.standard_normal((B, H, W, C)).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    mask = oracle.gen_prune_mask(w.copy(), 0.5)
    g = rng.standard_normal((B, 2 * tiles(H), 2 * tiles(W), K)).astype(np.float32)

    layer = WinogradConv(C, K, mask=mask, W_init=w).to(dev)
    xd = gpu(x, dev).requires_grad_(True)
    y = layer(WinogradImTrans(xd, torch.relu))
    (y * gpu(g, dev)).sum().backward()

    ti = oracle.imtrans(x, relu=True)
    dti, dw = oracle.conv_grad(ti, w * mask, g)
    dx = oracle.imtrans_grad(dti, H, W, mask_src=ti)
    assert rel_max(xd.grad.cpu().numpy(), dx) <= TOL
    assert rel_max(layer.W.grad.cpu().numpy(), dw * mask) <= TOL
    assert rel_max(y.detach().cpu().numpy(), oracle.conv(ti, w * mask, acc64=True)) <= TOL


def test_reference_linkage_grad_symbols(oracle, dev):
    # C++-linkage launchers with the reference's signatures (winograd2x2_conv_grad_op.cc:32,
    # winograd2x2_imTrans_grad_op.cc:29), null stream, caller-supplied temporaries.
    import ctypes

    import swc_hip
    raw = ctypes.CDLL(swc_hip.LIB_PATH)
    fcg = getattr(raw, swc_hip.CXX_SYMBOLS[2])
    fig = getattr(raw, swc_hip.CXX_SYMBOLS[3])
    fcg.restype = fig.restype = None
    fcg.argtypes = [ctypes.c_void_p] * 7 + [ctypes.c_int] * 7
    fig.argtypes = [ctypes.c_void_p] * 2 + [ctypes.c_int] * 6
    rng = np.random.default_rng(34)
    B, nH, nW, C, K = 2, 3, 4, 8, 12
    ti = rng.standard_normal((16, B, nH, nW, C)).astype(np.float32)
    w = rng.standard_normal((16, C, K)).astype(np.float32)
    dy = rng.standard_normal((B, 2 * nH, 2 * nW, K)).astype(np.float32)
    tid, wd, dyd = gpu(ti, dev), gpu(w, dev), gpu(dy, dev)
    dti, dw = torch.empty_like(tid), torch.empty_like(wd)
    tmp = torch.empty(16 * B * nH * nW * K, device=dev)
    ptrs = torch.empty(80, dtype=torch.int64, device=dev)
    dx = torch.empty(B, 2 * nH, 2 * nW, C, device=dev)
    torch.cuda.synchronize()
    fcg(tid.data_ptr(), wd.data_ptr(), dyd.data_ptr(), dti.data_ptr(), dw.data_ptr(), tmp.data_ptr(), ptrs.data_ptr(),
        C, B, 2 * nH, 2 * nW, K, 1, 1)
    fig(dti.data_ptr(), dx.data_ptr(), C, B, 2 * nH, 2 * nW, 1, 1)
    torch.cuda.synchronize()
    dti_want, dw_want = oracle.conv_grad(ti, w, dy)
    assert rel_max(dti.cpu().numpy(), dti_want) <= TOL and rel_max(dw.cpu().numpy(), dw_want) <= TOL
    assert rel_max(dx.cpu().numpy(), oracle.imtrans_grad(dti_want, 2 * nH, 2 * nW)) <= TOL


@pytest.mark.parametrize("shape", [
    (8, 14, 14, 128, 128),  # whole 64-row tiles except the last
    (5, 9, 11, 160, 96),    # M = 495: ragged last row tile; C = 160: the third column tile is half empty
    (3, 7, 7, 64, 64),      # two 32-index steps per position
    (63, 14, 14, 120, 128),  # C not a multiple of 16: ragged last column tile
    (2, 3, 3, 32, 32),      # one tile, one step per position
])
def test_data_gradient_on_the_ring_kernel(oracle, dev, shape):
    """dTI = dP . W^T at shapes the ring kernel takes (K % 32 == 0: pairs of positions dealt to workgroups of 64x64
    tiles), against the oracle; exact on small integers."""
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv_grad
    B, nH, nW, C, K = shape
    rng = np.random.default_rng(35)
    ti = np.maximum(rng.standard_normal((16, B, nH, nW, C)), 0).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    dy = rng.standard_normal((B, 2 * nH, 2 * nW, K)).astype(np.float32)
    dti_want, dw_want = oracle.conv_grad(ti, w, dy)
    dti, dw = winograd2x2_conv_grad(gpu(ti, dev), gpu(w, dev), gpu(dy, dev))
    assert rel_max(dti.cpu().numpy(), dti_want) <= TOL
    assert rel_max(dw.cpu().numpy(), dw_want) <= TOL
    tii = rng.integers(-3, 4, size=ti.shape).astype(np.float32)
    wi = rng.integers(-3, 4, size=w.shape).astype(np.float32)
    dyi = rng.integers(-3, 4, size=dy.shape).astype(np.float32)
    a, _ = winograd2x2_conv_grad(gpu(tii, dev), gpu(wi, dev), gpu(dyi, dev))
    assert np.array_equal(a.cpu().numpy(), oracle.conv_grad(tii, wi, dyi)[0])
