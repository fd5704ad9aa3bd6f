"""Seeded sweep of random small shapes through every op against the CPU oracle.

The hand-picked shapes of the other GPU tests aim at known boundaries (tile edges, vector widths,
kernel selection); this sweep draws shapes nobody picked: odd sizes, channel counts that are
multiples of 1, 4, 8 and 64, filter counts independent of them.  Bars as elsewhere: the input
transform and the ReLU mask bit-exact, the convolution and its gradients within 1e-4 of the
oracle's float64-accumulated result, everything bit-exact on small integers.
"""
import numpy as np
import pytest
import torch

from helpers import rel_max, tiles

pytestmark = pytest.mark.gpu
TOL = 1e-4
N_CASES = 24


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available()
    import swc_hip
    swc_hip.lib()
    return torch.device("cuda:0")


def gpu(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def draw_shape(rng):
    B = int(rng.integers(1, 5))
    H, W = int(rng.integers(1, 34)), int(rng.integers(1, 34))
    granule = int(rng.choice([1, 4, 8, 64]))
    C = granule * int(rng.integers(1, max(2, 160 // granule)))
    granule = int(rng.choice([1, 4, 8, 64]))
    K = granule * int(rng.integers(1, max(2, 160 // granule)))
    return B, H, W, C, K


@pytest.mark.parametrize("case", range(N_CASES))
def test_forward_and_backward_on_a_random_shape(oracle, dev, case):
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv, winograd2x2_conv_grad, winograd2x2_relu_conv
    from winograd2x2_imTrans.winograd2x2_imTrans import winograd2x2_imTrans, winograd2x2_imTrans_grad
    rng = np.random.default_rng(9000 + case)
    B, H, W, C, K = draw_shape(rng)
    nH, nW = tiles(H), tiles(W)
    print("case %d: B=%d H=%d W=%d C=%d K=%d" % (case, B, H, W, C, K), flush=True)
    x = rng.standard_normal((B, H, W, C)).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.1).astype(np.float32)

    # forward: transform (+ReLU) bit-exact, convolution within tolerance
    for relu in (False, True):
        ti_want = oracle.imtrans(x, relu=relu)
        ti_got = winograd2x2_imTrans(gpu(x, dev), relu=relu).cpu().numpy()
        assert ti_got.shape == (16, B, nH, nW, C)
        assert np.array_equal(ti_got, ti_want)
    y_want = oracle.conv(ti_want, w, acc64=True)
    ti_dev = gpu(ti_want, dev)
    y_got = winograd2x2_conv(ti_dev, gpu(w, dev)).cpu().numpy()
    assert y_got.shape == (B, 2 * nH, 2 * nW, K)
    assert rel_max(y_got, y_want) <= TOL
    # the whole layer in one kernel, where it takes the shape (else it falls back to the two ops)
    y_fused = winograd2x2_relu_conv(gpu(x, dev), gpu(w, dev), relu=True).cpu().numpy()
    assert rel_max(y_fused, y_want) <= TOL

    # backward
    dy = rng.standard_normal(y_want.shape).astype(np.float32)
    dti_want, dw_want = oracle.conv_grad(ti_want, w, dy)
    dti_got, dw_got = winograd2x2_conv_grad(ti_dev, gpu(w, dev), gpu(dy, dev))
    assert rel_max(dti_got.cpu().numpy(), dti_want) <= TOL
    assert rel_max(dw_got.cpu().numpy(), dw_want) <= TOL
    g = rng.standard_normal(ti_want.shape).astype(np.float32)
    dx_plain = winograd2x2_imTrans_grad(gpu(g, dev), H, W).cpu().numpy()
    assert rel_max(dx_plain, oracle.imtrans_grad(g, H, W)) <= 1e-6
    dx_want = oracle.imtrans_grad(g, H, W, mask_src=ti_want)
    dx_out = winograd2x2_imTrans_grad(gpu(g, dev), H, W, relu_output=ti_dev)
    dx_in = winograd2x2_imTrans_grad(gpu(g, dev), H, W, relu_input=gpu(x, dev))
    assert rel_max(dx_out.cpu().numpy(), dx_want) <= 1e-6
    assert torch.equal(dx_out, dx_in)

    # small integers: every sum is exact in fp32, so every op must match bit for bit
    xi = rng.integers(-3, 4, size=x.shape).astype(np.float32)
    wi = rng.integers(-2, 3, size=w.shape).astype(np.float32)
    ti_i = oracle.imtrans(xi, relu=True)
    assert np.array_equal(winograd2x2_imTrans(gpu(xi, dev), relu=True).cpu().numpy(), ti_i)
    yi = oracle.conv(ti_i, wi)
    assert np.array_equal(winograd2x2_conv(gpu(ti_i, dev), gpu(wi, dev)).cpu().numpy(), yi)
    dyi = rng.integers(-2, 3, size=yi.shape).astype(np.float32)
    dti_i, dw_i = oracle.conv_grad(ti_i, wi, dyi)
    got_dti, got_dw = winograd2x2_conv_grad(gpu(ti_i, dev), gpu(wi, dev), gpu(dyi, dev))
    assert np.array_equal(got_dti.cpu().numpy(), dti_i)
    assert np.array_equal(got_dw.cpu().numpy(), dw_i)
    dx_i = oracle.imtrans_grad(dti_i, H, W, mask_src=ti_i)
    assert np.array_equal(winograd2x2_imTrans_grad(got_dti, H, W, relu_input=gpu(xi, dev)).cpu().numpy(), dx_i)
