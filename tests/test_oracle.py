"""Pins the CPU oracle (oracle/winograd_oracle.c) before anything is checked against it.

The reference (xingyul/sparse-winograd-cnn) ships no golden vectors: its test scripts
draw unseeded inputs and print sum|a-b|/(sum|a|+sum|b|) against tf.nn.conv2d
(winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_test.py:164-204).  The oracle
is therefore pinned by what the mathematics fixes: float64 matrix forms written from
the textbook matrices, integer inputs on which fp32 is exact, closed forms, a direct
3x3 loop nest, and the same conv2d relation with torch's CPU conv2d as the library.
"""
import numpy as np
import pytest
import torch

from helpers import (direct_conv, imtrans_matrix, kernel_matrix, output_matrix, rel_l1, rel_max, tiles)

SHAPES = [
    (3, 6, 6, 32),    # the reference tests' own shape (winograd2x2_imTrans_test.py:160-164)
    (2, 7, 7, 5),     # odd extent, C not a multiple of 4 (C=5 as in winograd2x2_conv_grad_test.py:160-163)
    (1, 16, 16, 64),  # benchmark config 1
    (2, 5, 9, 3),     # H != W, both odd
    (1, 1, 1, 1),     # a single pixel: one tile, mostly padding
    (1, 2, 3, 7),
]


@pytest.mark.parametrize("shape", SHAPES)
def test_imtrans_exact_on_integers(oracle, shape):
    # Small integers: every fp32 partial sum is exact, so the 16 explicit sums must
    # equal B^T d B computed in float64 bit for bit, whatever their association.
    rng = np.random.default_rng(1)
    x = rng.integers(-8, 9, size=shape).astype(np.float32)
    got = oracle.imtrans(x)
    want = imtrans_matrix(x)
    assert got.shape == (16, shape[0], tiles(shape[1]), tiles(shape[2]), shape[3])
    assert np.array_equal(got.astype(np.float64), want)


@pytest.mark.parametrize("shape", SHAPES)
def test_imtrans_close_on_gaussians(oracle, shape):
    rng = np.random.default_rng(2)
    x = rng.standard_normal(shape).astype(np.float32)
    assert rel_max(oracle.imtrans(x), imtrans_matrix(x)) < 1e-6


def test_imtrans_all_ones_interior_tile(oracle):
    # For a constant patch only T5 = d5+d6+d9+d10 survives (=4); every other row/column
    # of B^T sums to zero.
    x = np.ones((1, 8, 8, 3), dtype=np.float32)
    t = oracle.imtrans(x)
    interior = t[:, 0, 1:3, 1:3, :]
    want = np.zeros(16)
    want[5] = 4
    assert np.array_equal(interior, np.broadcast_to(want[:, None, None, None], interior.shape))
    # top-left tile: row 0 and column 0 of the patch are padding
    corner = t[:, 0, 0, 0, 0]
    d = np.zeros((4, 4))
    d[1:, 1:] = 1
    from helpers import BT
    assert np.array_equal(corner, (BT @ d @ BT.T).reshape(16))


def test_imtrans_linearity(oracle):
    rng = np.random.default_rng(3)
    x = rng.integers(-4, 5, size=(2, 6, 5, 4)).astype(np.float32)
    y = rng.integers(-4, 5, size=(2, 6, 5, 4)).astype(np.float32)
    assert np.array_equal(oracle.imtrans(2 * x - 3 * y), 2 * oracle.imtrans(x) - 3 * oracle.imtrans(y))


# The order of the four terms of each sum, as the reference writes them
# (winograd2x2_imTrans_cuda.cu.cc:112-127): (patch index, sign) left to right.
TERMS = [
    [(0, 1), (2, -1), (8, -1), (10, 1)], [(1, 1), (2, 1), (9, -1), (10, -1)],
    [(2, 1), (1, -1), (9, 1), (10, -1)], [(1, 1), (3, -1), (9, -1), (11, 1)],
    [(4, 1), (6, -1), (8, 1), (10, -1)], [(5, 1), (6, 1), (9, 1), (10, 1)],
    [(6, 1), (5, -1), (9, -1), (10, 1)], [(5, 1), (7, -1), (9, 1), (11, -1)],
    [(6, 1), (4, -1), (8, 1), (10, -1)], [(9, 1), (6, -1), (5, -1), (10, 1)],
    [(5, 1), (6, -1), (9, -1), (10, 1)], [(7, 1), (5, -1), (9, 1), (11, -1)],
    [(4, 1), (6, -1), (12, -1), (14, 1)], [(5, 1), (6, 1), (13, -1), (14, -1)],
    [(6, 1), (5, -1), (13, 1), (14, -1)], [(5, 1), (7, -1), (13, -1), (15, 1)],
]


def test_imtrans_association_is_left_to_right(oracle):
    # Values that cancel catastrophically: any other association (e.g. the separable
    # (d0-d2)-(d8-d10)) rounds differently somewhere in 4096 random patches.
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((1, 4, 4, 4096)) * 10.0 ** rng.integers(-3, 4, size=(1, 4, 4, 4096))).astype(np.float32)
    # one full tile: a 4x4 image read through pad 1 gives tile (1,1) = rows 1..4 -> use 6x6 with the patch inside
    img = np.zeros((1, 6, 6, 4096), dtype=np.float32)
    img[:, 1:5, 1:5, :] = x
    t = oracle.imtrans(img)[:, 0, 1, 1, :]
    d = x.reshape(16, 4096)
    differs_from_separable = False
    for i, terms in enumerate(TERMS):
        acc = None
        for j, sgn in terms:
            v = d[j] if sgn > 0 else -d[j]
            acc = v.copy() if acc is None else (acc + v).astype(np.float32)
        assert np.array_equal(t[i], acc), i
    from helpers import BT
    sep = np.einsum("ur,rsc,vs->uvc", BT.astype(np.float32), x[0].astype(np.float32), BT.astype(np.float32)).reshape(16, -1)
    differs_from_separable = not np.array_equal(sep.astype(np.float32), t)
    assert differs_from_separable  # the inputs do discriminate between associations


def test_relu_is_elementwise_max_and_masks(oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 7, 6, 9)).astype(np.float32)
    t = oracle.imtrans(x)
    r = oracle.imtrans(x, relu=True)
    assert np.array_equal(r, np.maximum(t, 0))
    assert np.array_equal(r == 0, t <= 0)
    assert not np.signbit(r).any()  # no negative zeros leave the ReLU


@pytest.mark.parametrize("M,C,K", [(18, 32, 32), (7, 5, 7), (64, 64, 64), (1, 1, 1), (33, 130, 17)])
def test_gemm16_matches_float64_matmul(oracle, M, C, K):
    rng = np.random.default_rng(6)
    a = rng.standard_normal((16, M, C)).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    want = np.matmul(a.astype(np.float64), w.astype(np.float64))
    assert rel_max(oracle.gemm16(a, w), want) < 1e-5
    assert rel_max(oracle.gemm16(a, w, acc64=True), want) < 2e-7
    # integers: exact in both
    ai = rng.integers(-3, 4, size=(16, M, C)).astype(np.float32)
    wi = rng.integers(-3, 4, size=(16, C, K)).astype(np.float32)
    wanti = np.matmul(ai.astype(np.float64), wi.astype(np.float64))
    assert np.array_equal(oracle.gemm16(ai, wi), wanti)
    assert np.array_equal(oracle.gemm16(ai, wi, acc64=True), wanti)


@pytest.mark.parametrize("B,nH,nW,K", [(3, 3, 3, 32), (2, 4, 4, 7), (1, 1, 1, 1), (2, 3, 5, 6)])
def test_output_transform_exact_on_integers(oracle, B, nH, nW, K):
    rng = np.random.default_rng(7)
    p = rng.integers(-8, 9, size=(16, B * nH * nW, K)).astype(np.float32)
    got = oracle.output_transform(p, B, nH, nW)
    assert got.shape == (B, 2 * nH, 2 * nW, K)
    assert np.array_equal(got, output_matrix(p, B, nH, nW))
    pg = rng.standard_normal(p.shape).astype(np.float32)
    assert rel_max(oracle.output_transform(pg, B, nH, nW), output_matrix(pg, B, nH, nW)) < 1e-6


def test_kernel_transform_matches_GgGt(oracle):
    rng = np.random.default_rng(8)
    g = rng.integers(-8, 9, size=(3, 3, 5, 7)).astype(np.float32)  # /2 and /4 of small ints: exact
    assert np.array_equal(oracle.kernel_transform(g), kernel_matrix(g))
    g = rng.standard_normal((3, 3, 6, 4)).astype(np.float32)
    assert rel_max(oracle.kernel_transform(g), kernel_matrix(g)) < 1e-6


@pytest.mark.parametrize("B,H,W,C,K", [
    (3, 6, 6, 32, 32),   # winograd2x2_conv_test.py:158-162
    (2, 7, 7, 5, 7),     # odd size: crop [:, :H, :W] (winograd2x2_conv_test.py:152-153); C != K
    (1, 16, 16, 64, 64),  # benchmark config 1
    (2, 5, 8, 3, 9),
])
def test_whole_path_equals_conv2d(oracle, B, H, W, C, K):
    # winograd2x2_conv(winograd2x2_imTrans(x), G g G^T) == conv2d(x, g, SAME): the relation
    # the reference's tests print (winograd2x2_conv_test.py:177,187-204), torch on the CPU
    # standing in for tf.nn.conv2d.
    rng = np.random.default_rng(9)
    x = rng.standard_normal((B, H, W, C)).astype(np.float32)
    g = rng.standard_normal((3, 3, C, K)).astype(np.float32)
    y = oracle.conv(oracle.imtrans(x), oracle.kernel_transform(g), acc64=True)
    assert y.shape == (B, 2 * tiles(H), 2 * tiles(W), K)
    y = y[:, :H, :W, :]
    ref = torch.nn.functional.conv2d(
        torch.from_numpy(x).double().permute(0, 3, 1, 2),
        torch.from_numpy(g).double().permute(3, 2, 0, 1), padding=1).permute(0, 2, 3, 1).numpy()
    assert rel_max(y, ref) < 1e-5
    assert rel_l1(y, ref) < 1e-5
    assert rel_max(direct_conv(x, g), ref) < 1e-12
    y32 = oracle.conv(oracle.imtrans(x), oracle.kernel_transform(g), acc64=False)[:, :H, :W, :]
    assert rel_max(y32, ref) < 1e-4


def test_whole_path_integers_exact(oracle):
    rng = np.random.default_rng(10)
    x = rng.integers(-4, 5, size=(2, 6, 6, 8)).astype(np.float32)
    g = (4 * rng.integers(-4, 5, size=(3, 3, 8, 5))).astype(np.float32)  # multiples of 4: G g G^T stays integral
    y = oracle.conv(oracle.imtrans(x), oracle.kernel_transform(g))
    assert np.array_equal(y, direct_conv(x, g))


def test_gen_prune_mask_keeps_largest(oracle):
    # ResNet-18-var/prune_script.py:22-31
    rng = np.random.default_rng(11)
    w = rng.standard_normal((16, 8, 12)).astype(np.float32)
    w0 = w.copy()
    mask = oracle.gen_prune_mask(w, 0.3)
    keep = int(w0.size * 0.3)
    assert int(mask.sum()) == keep and mask.dtype == w0.dtype
    assert np.array_equal(w, w0 * mask)
    assert np.abs(w0[mask == 1]).min() >= np.abs(w0[mask == 0]).max()
    w1 = w0.copy()
    assert oracle.gen_prune_mask(w1, 0.0).all() and np.array_equal(w1, w0)  # rank[:-0] is empty: nothing pruned


def test_affine_is_a_single_rounding_fma(oracle):
    # x, s in [1,2) with full 24-bit significands make 48-bit products; t in [1,4) aligns within
    # two bits, so x*s+t is exact in float64 and rounding it once to fp32 is the fused result.
    rng = np.random.default_rng(77)
    C = 64
    x = (1 + rng.random((4, 5, 6, C))).astype(np.float32)
    s = (1 + rng.random(C)).astype(np.float32)
    t = (1 + 3 * rng.random(C)).astype(np.float32)
    exact = x.astype(np.float64) * s.astype(np.float64) + t.astype(np.float64)
    want = exact.astype(np.float32)
    got = oracle.affine(x, s, t)
    assert np.array_equal(got, want)
    # the check has teeth: multiply-then-add rounds twice and differs somewhere
    assert not np.array_equal((x * s).astype(np.float32) + t, want)
    # negative scale, zero shift, and the transform of the mapped image
    s2, t2 = -s, np.zeros_like(t)
    assert np.array_equal(oracle.affine(x, s2, t2), (-(x.astype(np.float64) * s)).astype(np.float32))
    assert np.array_equal(oracle.imtrans_affine(x, s, t, relu=True), oracle.imtrans(want, relu=True))


def test_round_bf16_is_nearest_even(oracle):
    import torch
    rng = np.random.default_rng(78)
    x = (rng.standard_normal(20000) * 10.0 ** rng.integers(-6, 7, 20000)).astype(np.float32)
    # exact ties: the 16 dropped bits are 0x8000, with the kept bit odd and even
    ties = np.array([0x3F808000, 0x3F818000, 0xBF808000, 0xBF818000, 0x00008000, 0x7F7E8000], dtype=np.uint32).view(np.float32)
    x = np.concatenate([x, ties, np.array([0.0, -0.0, 1.0, 3.0e38], dtype=np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()   # torch's CPU conversion rounds to nearest even
    got = oracle.round_bf16(x)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(oracle.bf16_bits(x), want.view(np.uint32) >> 16)
    assert np.array_equal(got[-10:-8].view(np.uint32), np.array([0x3F800000, 0x3F820000], dtype=np.uint32))
