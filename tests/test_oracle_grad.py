"""Pins the oracle's backward functions.

The reference checks its gradient ops against tf.gradients of its TF-graph restatement and prints
a ratio (winograd2x2_conv_grad_test.py:197-227, winograd2x2_imTrans_grad_test.py:194-216); neither
can run here.  What fixes the backward of a linear map is the adjoint identity
<f(x), g> == <x, f^T(g)>, which is exact on small integers and fails for any wrong index, sign or
transposition, given the forward oracle (pinned on its own in tests/test_oracle.py).
"""
import numpy as np
import pytest

from helpers import AT, BT, tiles


def ints(rng, shape, lo=-4, hi=5):
    return rng.integers(lo, hi, size=shape).astype(np.float32)


def dot(a, b):
    return float(np.sum(a.astype(np.float64) * b.astype(np.float64)))


@pytest.mark.parametrize("B,H,W,C", [(2, 6, 6, 5), (1, 8, 4, 3), (2, 7, 5, 4), (1, 1, 1, 1), (1, 2, 3, 2)])
def test_imtrans_grad_is_the_adjoint(oracle, B, H, W, C):
    rng = np.random.default_rng(21)
    x = ints(rng, (B, H, W, C))
    g = ints(rng, (16, B, tiles(H), tiles(W), C))
    assert dot(oracle.imtrans(x), g) == dot(x, oracle.imtrans_grad(g, H, W))


def test_imtrans_grad_matrix_form_single_tile(oracle):
    # one interior tile: dd = B dT B^T placed on the patch
    rng = np.random.default_rng(22)
    g = np.zeros((16, 1, 3, 3, 2), dtype=np.float32)
    g[:, 0, 1, 1, :] = ints(rng, (16, 2))
    dx = oracle.imtrans_grad(g, 6, 6)
    for c in range(2):
        dd = BT.T @ g[:, 0, 1, 1, c].reshape(4, 4).astype(np.float64) @ BT
        want = np.zeros((6, 6))
        want[1:5, 1:5] = dd
        assert np.array_equal(dx[0, :, :, c], want)


def test_imtrans_grad_relu_mask(oracle):
    rng = np.random.default_rng(23)
    x = rng.standard_normal((2, 6, 6, 3)).astype(np.float32)
    g = ints(rng, (16, 2, 3, 3, 3))
    ti = oracle.imtrans(x, relu=True)
    assert np.array_equal(oracle.imtrans_grad(g, 6, 6, mask_src=ti), oracle.imtrans_grad(g * (ti > 0), 6, 6))


@pytest.mark.parametrize("B,nH,nW,K", [(2, 3, 3, 4), (1, 1, 2, 3)])
def test_output_transform_grad_is_the_adjoint_and_matrix_form(oracle, B, nH, nW, K):
    rng = np.random.default_rng(24)
    p = ints(rng, (16, B * nH * nW, K))
    dy = ints(rng, (B, 2 * nH, 2 * nW, K))
    dp = oracle.output_transform_grad(dy)
    assert dot(oracle.output_transform(p, B, nH, nW), dy) == dot(p, dp)
    tile = dy[0, 0:2, 0:2, 0].astype(np.float64)
    assert np.array_equal(dp[:, 0, 0], (AT.T @ tile @ AT).reshape(16))


@pytest.mark.parametrize("B,nH,nW,C,K", [(2, 3, 3, 5, 7), (1, 2, 2, 4, 4), (3, 1, 2, 6, 3)])
def test_conv_grad_adjoints(oracle, B, nH, nW, C, K):
    # C=5, K=7 is the reference test's shape (winograd2x2_conv_grad_test.py:160-163)
    rng = np.random.default_rng(25)
    ti, w = ints(rng, (16, B, nH, nW, C)), ints(rng, (16, C, K))
    dy = ints(rng, (B, 2 * nH, 2 * nW, K))
    dti, dw = oracle.conv_grad(ti, w, dy)
    y = oracle.conv(ti, w)
    # y is bilinear in (ti, w): <y, dy> == <ti, dti> == <w, dw>
    assert dot(y, dy) == dot(ti, dti) == dot(w, dw)
    # and the gradients are the adjoints of the two partial linear maps
    ti2, w2 = ints(rng, ti.shape), ints(rng, w.shape)
    assert dot(oracle.conv(ti2, w), dy) == dot(ti2, dti)
    assert dot(oracle.conv(ti, w2), dy) == dot(w2, dw)
    # float64 matmul form
    dp = oracle.output_transform_grad(dy).astype(np.float64)
    assert np.array_equal(dti.reshape(16, -1, C), np.matmul(dp, w.astype(np.float64).transpose(0, 2, 1)))
    assert np.array_equal(dw, np.matmul(ti.reshape(16, -1, C).astype(np.float64).transpose(0, 2, 1), dp))
