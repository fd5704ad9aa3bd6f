"""The fused layer kernel (transform + ReLU + 16 GEMMs + output transform) against the oracle and
against the two stand-alone ops it composes."""
import numpy as np
import pytest
import torch

from helpers import rel_l1, rel_max, tiles

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


SHAPES = [
    # B, H, W, C, K
    (3, 6, 6, 32, 32),      # the reference tests' shape
    (1, 16, 16, 64, 64),    # benchmark config 1
    (2, 7, 7, 8, 12),       # odd extent, one channel chunk, K below a tile
    (2, 5, 9, 24, 100),     # H != W, ragged K
    (1, 2, 2, 8, 4),        # a single tile
    (5, 18, 22, 40, 72),    # M = 495: ragged last workgroup
    (8, 28, 28, 128, 128),  # config 3 geometry
    (4, 14, 14, 256, 256),  # config 4a geometry
    (4, 7, 7, 512, 512),    # config 4b geometry (odd 7x7)
    (2, 56, 56, 64, 64),    # config 2 geometry
]


@pytest.mark.parametrize("relu", [True, False])
@pytest.mark.parametrize("shape", SHAPES)
def test_fused_matches_oracle_and_two_op_path(oracle, dev, shape, relu):
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv, winograd2x2_relu_conv
    from winograd2x2_imTrans.winograd2x2_imTrans import winograd2x2_imTrans
    import swc_hip
    B, H, W, C, K = shape
    rng = np.random.default_rng(41)
    x = rng.standard_normal((B, H, W, C)).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    if C * K >= 1024:
        oracle.gen_prune_mask(w, 0.2)
    xd, wd = gpu(x, dev), gpu(w, dev)
    out = torch.empty(B, 2 * tiles(H), 2 * tiles(W), K, device=dev)
    st = swc_hip.lib().swc_winograd2x2_relu_conv(xd.data_ptr(), wd.data_ptr(), out.data_ptr(), C, B, H, W, K, 1, 1,
                                                 int(relu), torch.cuda.current_stream().cuda_stream)
    assert st == 0, "these shapes are all eligible for the fused kernel"
    got = out.cpu().numpy()
    want = oracle.conv(oracle.imtrans(x, relu=relu), w, acc64=True)
    assert rel_max(got, want) <= TOL and rel_l1(got, want) <= TOL
    two = winograd2x2_conv(winograd2x2_imTrans(xd, relu=relu), wd).cpu().numpy()
    assert rel_max(got, two) <= TOL
    assert np.array_equal(winograd2x2_relu_conv(xd, wd, relu=relu).cpu().numpy(), got)


def test_fused_exact_on_integers(oracle, dev):
    # every product and sum exact in fp32: bit-for-bit equality pins the transform, operand
    # orientation, fold signs and scatter of the fused kernel
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_relu_conv
    rng = np.random.default_rng(42)
    for shape in [(2, 6, 6, 16, 20), (1, 7, 5, 8, 8), (3, 10, 10, 24, 64)]:
        B, H, W, C, K = shape
        x = rng.integers(-4, 5, size=(B, H, W, C)).astype(np.float32)
        w = rng.integers(-3, 4, size=(16, C, K)).astype(np.float32)
        got = winograd2x2_relu_conv(gpu(x, dev), gpu(w, dev)).cpu().numpy()
        assert np.array_equal(got, oracle.conv(oracle.imtrans(x, relu=True), w))


def test_fused_falls_back_on_unsupported_shapes(oracle, dev):
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_relu_conv
    import swc_hip
    rng = np.random.default_rng(43)
    x = rng.standard_normal((2, 6, 6, 5)).astype(np.float32)   # C % 8 != 0
    w = rng.standard_normal((16, 5, 7)).astype(np.float32)
    xd, wd = gpu(x, dev), gpu(w, dev)
    out = torch.empty(2, 6, 6, 7, device=dev)
    st = swc_hip.lib().swc_winograd2x2_relu_conv(xd.data_ptr(), wd.data_ptr(), out.data_ptr(), 5, 2, 6, 6, 7, 1, 1, 1, None)
    assert st == swc_hip.SWC_ERR_UNSUPPORTED
    got = winograd2x2_relu_conv(xd, wd).cpu().numpy()
    assert rel_max(got, oracle.conv(oracle.imtrans(x, relu=True), w, acc64=True)) <= TOL
