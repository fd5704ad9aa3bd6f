"""Parity of the HIP path against the CPU oracle, through the C ABI, on a real MI355X.

Bars (from the build's north star): the input transform and its Winograd-domain ReLU zero
masks are bit-exact; the fp32 convolution is within 1e-4 relative error of the
float64-accumulated oracle, both as max|a-b|/max|b| and as the reference tests' own
sum|a-b|/(sum|a|+sum|b|) (winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_test.py:190,204).
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from helpers import direct_conv, rel_l1, rel_max, tiles

pytestmark = pytest.mark.gpu

TOL = 1e-4       # fp32 conv vs the oracle
TOL_BF16 = 3e-2  # bf16-operand conv vs the unrounded fp32 oracle

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the GPU"
    import swc_hip
    swc_hip.lib()  # raises if the HIP library is missing: no fallback exists
    return torch.device("cuda:0")


def ops():
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv
    from winograd2x2_imTrans.winograd2x2_imTrans import winograd2x2_imTrans
    return winograd2x2_imTrans, winograd2x2_conv


def gpu(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


IMTRANS_SHAPES = [
    (3, 6, 6, 32),      # winograd2x2_imTrans_test.py:160-164
    (2, 7, 7, 5),       # odd extent; C % 4 != 0 takes the scalar path
    (1, 16, 16, 64),    # benchmark config 1
    (2, 5, 9, 3),
    (1, 1, 1, 1),
    (1, 2, 3, 7),
    (2, 56, 56, 64),    # config 2 geometry, reduced batch
    (64, 28, 28, 128),  # config 3 in full
    (4, 14, 14, 256),   # config 4a geometry
    (4, 7, 7, 512),     # config 4b: odd 7x7 -> 4x4 tiles
    (1, 3, 3, 1028),    # C above the reference's 1024-thread block limit
]


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("shape", IMTRANS_SHAPES)
def test_imtrans_bit_exact(oracle, dev, shape, relu):
    imtrans, _ = ops()
    rng = np.random.default_rng(hash(shape) % 2 ** 31)
    x = rng.standard_normal(shape).astype(np.float32)
    want = oracle.imtrans(x, relu=relu)
    got = imtrans(gpu(x, dev), relu=relu).cpu().numpy()
    assert got.shape == want.shape
    assert np.array_equal(got == 0, want == 0), "zero mask differs"
    assert np.array_equal(got, want), "values differ"
    if relu:
        assert not np.signbit(got).any()


def test_imtrans_relu_mask_under_cancellation(oracle, dev):
    # Post-ReLU activations (half zeros) and wide dynamic range: many transformed values are
    # exact zeros or tiny residues of cancellation, where association decides the sign.
    imtrans, _ = ops()
    rng = np.random.default_rng(5)
    x = np.maximum(rng.standard_normal((8, 12, 12, 64)), 0) * 10.0 ** rng.integers(-3, 4, size=(8, 12, 12, 64))
    x = x.astype(np.float32)
    want = oracle.imtrans(x, relu=True)
    got = imtrans(gpu(x, dev), relu=True).cpu().numpy()
    assert np.array_equal(got == 0, want == 0)
    assert np.array_equal(got, want)
    assert 0.3 < float((want == 0).mean()) < 0.9


CONV_SHAPES = [
    # B, nH, nW, C, K
    (3, 3, 3, 32, 32),     # winograd2x2_conv_test.py:158-162
    (2, 4, 4, 5, 7),       # C=5, K=7 as in winograd2x2_conv_grad_test.py:160-163 (scalar-load path)
    (1, 8, 8, 64, 64),     # benchmark config 1
    (1, 1, 1, 1, 1),
    (2, 3, 5, 36, 100),    # ragged in M, C and K tiles
    (2, 14, 14, 64, 128),  # C != K as in Winograd_W3a_2a
    (8, 14, 14, 128, 128),  # config 3 geometry, reduced batch
    (8, 7, 7, 256, 256),   # config 4a
    (8, 4, 4, 512, 512),   # config 4b
    (1, 2, 2, 1028, 12),
    # shapes that steer the launcher onto each of its kernels and their ragged edges
    (2, 3, 5, 64, 100),    # copy-ring kernel, 32-channel steps: rows and columns beyond the last tile
    (1, 5, 7, 48, 20),     # copy-ring kernel, 16-channel steps (C % 32 != 0), K below one tile
    (3, 7, 7, 32, 64),     # a single 32-channel step per position
    (2, 3, 3, 96, 132),    # K = 2 tiles + 4 columns
    (1, 1, 1, 32, 4),      # one tile row, one column group
    (5, 9, 11, 160, 72),   # M = 495 (ragged last tile), C = 5 steps
    (8, 9, 9, 128, 72),    # short row groups (16x16 MFMAs), ragged rows and columns
    (63, 14, 14, 128, 120),  # tall row groups of 97 rows, last one 29; K = 2 tiles - 8 columns
    (32, 28, 28, 64, 64),  # tall row groups, one 64-channel reduction in two steps
]


def conv_inputs(shape, seed, density=1.0, relu=True):
    B, nH, nW, C, K = shape
    rng = np.random.default_rng(seed)
    ti = rng.standard_normal((16, B, nH, nW, C)).astype(np.float32)
    if relu:
        ti = np.maximum(ti, 0)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    if density < 1.0:
        import oracle as orc
        orc.gen_prune_mask(w, density)
    return ti, w


@pytest.mark.parametrize("shape", CONV_SHAPES)
def test_conv_fp32_matches_oracle(oracle, dev, shape):
    _, conv = ops()
    ti, w = conv_inputs(shape, 11, density=0.2 if shape[3] * shape[4] >= 1024 else 1.0)
    want = oracle.conv(ti, w, acc64=True)
    got = conv(gpu(ti, dev), gpu(w, dev)).cpu().numpy()
    assert got.shape == want.shape == (shape[0], 2 * shape[1], 2 * shape[2], shape[4])
    assert rel_max(got, want) <= TOL
    assert rel_l1(got, want) <= TOL


def test_conv_shapes_reach_every_kernel(dev):
    # The launcher picks a kernel from the shapes alone; the parity shapes above must cover all five.
    import swc_hip
    _, conv = ops()
    seen = set()
    # the last two: benchmark config 3, checked in full below, and config 4a's geometry (one 48-row x 64-column
    # workgroup per CU of an MI355X), checked in full in test_gpu_cfg4_full.py
    for shape in CONV_SHAPES + [(64, 14, 14, 128, 128), (64, 7, 7, 256, 256)]:
        B, nH, nW, C, K = shape
        conv(torch.zeros((16, B, nH, nW, C), device=dev), torch.zeros((16, C, K), device=dev))
        seen.add(swc_hip.lib().swc_winograd2x2_conv_last_kernel().decode())
    assert seen >= {"sync", "ring32", "ring16", "tall16", "short16", "wide48"}, seen
    if torch.cuda.get_device_properties(dev).multi_processor_count == 256:
        assert "wide48x64" in seen, seen


@pytest.mark.parametrize("tiling", ["ring32", "ring16", "tall16", "short16", "sync"])
@pytest.mark.parametrize("shape", [(8, 14, 14, 128, 128), (5, 9, 11, 192, 72), (63, 14, 14, 64, 120), (2, 3, 5, 64, 100)])
def test_conv_fp32_under_every_tiling(oracle, dev, shape, tiling):
    """The launcher's choice taken away (swc_winograd2x2_conv_force_tiling): every tiling must give the oracle's
    result on every shape it is eligible for, and the override must report what ran."""
    import swc_hip
    L = swc_hip.lib()
    _, conv = ops()
    ti, w = conv_inputs(shape, 14, density=0.2)
    want = oracle.conv(ti, w, acc64=True)
    assert L.swc_winograd2x2_conv_force_tiling(b"no-such-tiling") == swc_hip.SWC_ERR_UNSUPPORTED
    assert L.swc_winograd2x2_conv_force_tiling(tiling.encode()) == 0
    try:
        got = conv(gpu(ti, dev), gpu(w, dev)).cpu().numpy()
        assert L.swc_winograd2x2_conv_last_kernel().decode() == tiling   # all four shapes take every tiling
        assert rel_max(got, want) <= TOL and rel_l1(got, want) <= TOL
    finally:
        assert L.swc_winograd2x2_conv_force_tiling(None) == 0
    conv(gpu(ti, dev), gpu(w, dev))
    assert L.swc_winograd2x2_conv_last_kernel().decode() in ("ring32", "ring16", "tall16", "short16")


# wide48 takes C % 64 == 0 and K % 128 == 0.  The shapes cover its two ways of dealing out the rows: levelled row
# groups (down to one valid row per workgroup), and full 48-row groups with the rest as extra 16x16 tiles, whole and
# ragged, with one and with two column groups.
WIDE48_SHAPES = [
    (8, 14, 14, 128, 128),   # levelled: 13 rows per workgroup
    (3, 5, 7, 64, 128),      # levelled: M = 105 over 105 workgroups
    (2, 20, 20, 64, 128),    # 16 full groups + 2 extra tiles
    (2, 2, 197, 64, 128),    # 16 full groups + 20 rows: the second extra tile holds 4
    (32, 1, 193, 64, 256),   # two column groups: 128 full groups + 2 extra row tiles
    (8, 14, 14, 128, 256),   # two column groups, levelled
]


# The same kernel with 64-column workgroups ("wide48x64") takes K % 64 == 0.
WIDE48X64_SHAPES = [
    (8, 14, 14, 128, 64),    # one column group, levelled
    (3, 5, 7, 64, 192),      # three column groups, levelled: M = 105
    (2, 20, 20, 64, 64),     # 16 full groups + 2 extra row tiles of 4 tiles each
    (2, 2, 197, 128, 128),   # two column groups, the second extra row tile holds 4 rows
    (16, 7, 7, 256, 256),    # config 4a's geometry at a quarter of its batch
]


@pytest.mark.parametrize("shape,tiling", [(s, "wide48") for s in WIDE48_SHAPES] + [(s, "wide48x64") for s in WIDE48X64_SHAPES])
def test_conv_fp32_wide48(oracle, dev, shape, tiling):
    """The wide48 tilings forced on shapes below the size at which the launcher picks them by itself.  Their output
    transform is taken in another association than the reference's (sum/difference pairs, partial sums continued
    by the matrix pipes), so besides the tolerance check the integer check pins every sign and the scatter exactly."""
    import swc_hip
    L = swc_hip.lib()
    _, conv = ops()
    B, nH, nW, C, K = shape
    ti, w = conv_inputs(shape, 15, density=0.2)
    rng = np.random.default_rng(16)
    ti_int = rng.integers(-4, 5, size=(16, B, nH, nW, C)).astype(np.float32)
    w_int = rng.integers(-4, 5, size=(16, C, K)).astype(np.float32)
    scale = (0.5 + rng.random(K)).astype(np.float32) * rng.choice([-1, 1], K).astype(np.float32)
    shift = rng.standard_normal(K).astype(np.float32)
    res = rng.standard_normal((B, 2 * nH, 2 * nW, K)).astype(np.float32)
    assert L.swc_winograd2x2_conv_force_tiling(tiling.encode()) == 0
    try:
        got = conv(gpu(ti, dev), gpu(w, dev))
        assert L.swc_winograd2x2_conv_last_kernel().decode() == tiling
        got_int = conv(gpu(ti_int, dev), gpu(w_int, dev)).cpu().numpy()
        got_ep = conv(gpu(ti, dev), gpu(w, dev), scale=gpu(scale, dev), shift=gpu(shift, dev), residual=gpu(res, dev),
                      residual_relu=True).cpu().numpy()
        buf = gpu(res, dev)
        conv(gpu(ti, dev), gpu(w, dev), out=buf, residual=buf)   # residual aliasing the output
    finally:
        assert L.swc_winograd2x2_conv_force_tiling(None) == 0
    want = oracle.conv(ti, w, acc64=True)
    assert rel_max(got.cpu().numpy(), want) <= TOL and rel_l1(got.cpu().numpy(), want) <= TOL
    assert np.array_equal(got_int, oracle.conv(ti_int, w_int))
    # the epilogue's own arithmetic is exact against the oracle's on the kernel's plain output
    assert np.array_equal(got_ep, oracle.affine(got.cpu().numpy(), scale, shift) + np.maximum(res, 0))
    assert np.array_equal(buf.cpu().numpy(), got.cpu().numpy() + res)


@pytest.mark.parametrize("shape", [(3, 3, 3, 32, 32), (2, 4, 4, 5, 7), (2, 3, 5, 36, 100), (8, 9, 9, 128, 72),
                                   (63, 14, 14, 128, 120)])
def test_conv_fp32_exact_on_integers(oracle, dev, shape):
    # Small integers make every product and partial sum exact in fp32, whatever the
    # reduction order: the kernel must equal the oracle bit for bit, which pins operand
    # orientation, signs of the output transform and the 2x2 scatter.
    _, conv = ops()
    rng = np.random.default_rng(12)
    B, nH, nW, C, K = shape
    ti = rng.integers(-4, 5, size=(16, B, nH, nW, C)).astype(np.float32)
    w = rng.integers(-4, 5, size=(16, C, K)).astype(np.float32)
    assert np.array_equal(conv(gpu(ti, dev), gpu(w, dev)).cpu().numpy(), oracle.conv(ti, w))


def test_conv_full_config3(oracle, dev):
    # benchmark config 3 at full size: N=64, 28x28x128 -> 128, Winograd-domain ReLU on,
    # weights pruned to 20 % density.
    imtrans, conv = ops()
    rng = np.random.default_rng(300)
    x = rng.standard_normal((64, 28, 28, 128)).astype(np.float32)
    w = (np.random.default_rng(301).standard_normal((16, 128, 128)) * 0.05).astype(np.float32)
    oracle.gen_prune_mask(w, 0.2)
    ti_want = oracle.imtrans(x, relu=True)
    ti = imtrans(gpu(x, dev), relu=True)
    assert np.array_equal(ti.cpu().numpy(), ti_want)
    want = oracle.conv(ti_want, w, acc64=True)
    got = conv(ti, gpu(w, dev)).cpu().numpy()
    assert rel_max(got, want) <= TOL and rel_l1(got, want) <= TOL


@pytest.mark.parametrize("B,H,W,C,K", [(3, 6, 6, 32, 32), (2, 7, 7, 5, 7), (2, 28, 28, 128, 128), (2, 7, 9, 64, 96)])
def test_whole_path_equals_conv2d(dev, B, H, W, C, K):
    # winograd2x2_conv(winograd2x2_imTrans(x), G g G^T) == conv2d(x, g, SAME), the check the
    # reference's own test prints (winograd2x2_conv_test.py:177,187-204), odd sizes cropped
    # as its oracle does (:152-153).
    from winograd_weights import kernel_transform
    imtrans, conv = ops()
    rng = np.random.default_rng(13)
    x = rng.standard_normal((B, H, W, C)).astype(np.float32)
    g = rng.standard_normal((3, 3, C, K)).astype(np.float32)
    y = conv(imtrans(gpu(x, dev)), gpu(kernel_transform(g), dev)).cpu().numpy()
    assert y.shape == (B, 2 * tiles(H), 2 * tiles(W), K)
    ref = torch.nn.functional.conv2d(
        torch.from_numpy(x).double().permute(0, 3, 1, 2),
        torch.from_numpy(g).double().permute(3, 2, 0, 1), padding=1).permute(0, 2, 3, 1).numpy()
    assert rel_max(y[:, :H, :W, :], ref) <= TOL
    assert rel_l1(y[:, :H, :W, :], ref) <= TOL
    if B * H * W * C * K < 1 << 22:
        assert rel_max(direct_conv(x, g), ref) < 1e-12


@pytest.mark.parametrize("name", ["ref_b3_6x6_c32_k32", "odd_b2_7x7_c5_k7", "pruned_b2_10x6_c24_k40"])
def test_golden_fixtures(dev, name):
    imtrans, conv = ops()
    f = dict(np.load(os.path.join(HERE, "golden", name + ".npz")))
    x, w = gpu(f["x"], dev), gpu(f["w"], dev)
    ti, ti_relu = imtrans(x), imtrans(x, relu=True)
    assert np.array_equal(ti.cpu().numpy(), f["ti"])
    assert np.array_equal(ti_relu.cpu().numpy(), f["ti_relu"])
    for got, want in ((conv(ti, w), f["y"]), (conv(ti_relu, w), f["y_relu"])):
        assert rel_max(got.cpu().numpy(), want) <= TOL and rel_l1(got.cpu().numpy(), want) <= TOL


@pytest.mark.parametrize("shape", [(3, 3, 3, 32, 32), (2, 4, 4, 5, 7), (4, 14, 14, 128, 128)])
def test_conv_bf16_variant(oracle, dev, shape):
    # With both operands pre-rounded to bf16 the products are exact in fp32, so against an
    # oracle fed the same rounded operands only the accumulation order differs (<= 1e-4);
    # against the unrounded oracle the error is the bf16 rounding itself.
    _, conv = ops()
    ti, w = conv_inputs(shape, 14)
    got = conv(gpu(ti, dev), gpu(w, dev), precision="bf16").cpu().numpy()
    rnd = lambda a: torch.from_numpy(a).to(torch.bfloat16).to(torch.float32).numpy()  # noqa: E731
    assert rel_max(got, oracle.conv(rnd(ti), rnd(w), acc64=True)) <= TOL
    assert rel_max(got, oracle.conv(ti, w, acc64=True)) <= TOL_BF16


def test_full_size_properties(dev):
    # Size-independent checks at benchmark config 2 in full (N=64, 56x56x64 -> 64).
    imtrans, conv = ops()
    g = torch.Generator(device="cpu").manual_seed(200)
    x = torch.randn(64, 56, 56, 64, generator=g).clamp_(min=0).to(dev)
    w = (torch.randn(16, 64, 64, generator=g) * 0.05).to(dev)
    ti = imtrans(x, relu=True)
    # ReLU of the transform == clamp of the un-fused transform, exactly
    assert torch.equal(ti, imtrans(x).clamp_(min=0))
    # exact scaling by powers of two commutes with every add in both kernels
    assert torch.equal(imtrans(x * 4, relu=True), ti * 4)
    y = conv(ti, w)
    assert torch.equal(conv(ti, w * 0.5), y * 0.5)
    # images are independent: a batch slice gives the same rows
    assert torch.equal(conv(ti[:, 5:9].contiguous(), w), y[5:9])
    # positions are additive: zeroing all but position 5 leaves the A^T(x)A^T column of P5
    w5 = torch.zeros_like(w)
    w5[5] = w[5]
    p5 = (ti[5].reshape(-1, 64) @ w5[5]).reshape(64, 28, 28, 64)
    y5 = conv(ti, w5)
    for dy in (0, 1):
        for dx in (0, 1):  # position 5 is (r,s) = (1,1) and AT[dy][1]*AT[dx][1] = +1 for every (dy,dx)
            assert rel_max(y5[:, dy::2, dx::2, :].cpu().numpy(), p5.cpu().numpy()) <= TOL


def test_raw_c_abi_and_reference_linkage_symbols(oracle, dev):
    # Calls the launcher-level C entry points and the C++-linkage launchers that carry the
    # reference's exact signatures (winograd2x2_imTrans_op.cc:30, winograd2x2_conv_op.cc:31)
    # with raw device pointers.
    import swc_hip
    L = swc_hip.lib()
    rng = np.random.default_rng(15)
    B, H, W, C, K = 2, 6, 8, 16, 24
    nH, nW = tiles(H), tiles(W)
    x = rng.standard_normal((B, H, W, C)).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    xd, wd = gpu(x, dev), gpu(w, dev)
    want_ti = oracle.imtrans(x)
    want_y = oracle.conv(want_ti, w, acc64=True)

    side = torch.cuda.Stream(device=dev)
    ti = torch.empty(16, B, nH, nW, C, device=dev)
    y = torch.empty(B, 2 * nH, 2 * nW, K, device=dev)
    side.wait_stream(torch.cuda.current_stream())
    assert L.swc_winograd2x2_imtrans(xd.data_ptr(), ti.data_ptr(), C, B, H, W, 1, 1, 0, side.cuda_stream) == 0
    assert L.swc_winograd2x2_conv(ti.data_ptr(), wd.data_ptr(), y.data_ptr(), None, None, C, B, nH, nW, K, 1, 1,
                                  side.cuda_stream) == 0
    side.synchronize()
    assert np.array_equal(ti.cpu().numpy(), want_ti)
    assert rel_max(y.cpu().numpy(), want_y) <= TOL

    raw = ctypes.CDLL(swc_hip.LIB_PATH)
    fi = getattr(raw, swc_hip.CXX_SYMBOLS[0])
    fc = getattr(raw, swc_hip.CXX_SYMBOLS[1])
    fi.restype = fc.restype = None
    fi.argtypes = [ctypes.c_void_p] * 2 + [ctypes.c_int] * 6
    fc.argtypes = [ctypes.c_void_p] * 5 + [ctypes.c_int] * 7
    ti2 = torch.zeros_like(ti)
    y2 = torch.zeros_like(y)
    tmp = torch.empty(16 * B * nH * nW * K, device=dev)           # as winograd2x2_conv_op.cc:57-59
    ptrs = torch.empty(48, dtype=torch.int64, device=dev)         # as winograd2x2_conv_op.cc:61-63
    torch.cuda.synchronize()
    fi(xd.data_ptr(), ti2.data_ptr(), C, B, H, W, 1, 1)
    fc(ti2.data_ptr(), wd.data_ptr(), y2.data_ptr(), tmp.data_ptr(), ptrs.data_ptr(), C, B, nH, nW, K, 1, 1)
    torch.cuda.synchronize()
    assert np.array_equal(ti2.cpu().numpy(), want_ti)
    assert rel_max(y2.cpu().numpy(), want_y) <= TOL


def test_unaligned_views_take_the_scalar_path(oracle, dev):
    # A base pointer that is only 4-byte aligned must still give the right answer.
    imtrans, conv = ops()
    import swc_hip
    L = swc_hip.lib()
    rng = np.random.default_rng(16)
    B, H, W, C, K = 1, 4, 6, 8, 12
    nH, nW = tiles(H), tiles(W)
    x = rng.standard_normal((B, H, W, C)).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    xbuf = torch.zeros(x.size + 1, device=dev)
    xbuf[1:] = gpu(x.reshape(-1), dev)
    tibuf = torch.zeros(16 * B * nH * nW * C + 1, device=dev)
    wbuf = torch.zeros(w.size + 1, device=dev)
    wbuf[1:] = gpu(w.reshape(-1), dev)
    y = torch.empty(B, 2 * nH, 2 * nW, K, device=dev)
    s = torch.cuda.current_stream().cuda_stream
    assert L.swc_winograd2x2_imtrans(xbuf.data_ptr() + 4, tibuf.data_ptr() + 4, C, B, H, W, 1, 1, 1, s) == 0
    assert L.swc_winograd2x2_conv(tibuf.data_ptr() + 4, wbuf.data_ptr() + 4, y.data_ptr(), None, None,
                                  C, B, nH, nW, K, 1, 1, s) == 0
    torch.cuda.synchronize()
    want_ti = oracle.imtrans(x, relu=True)
    assert np.array_equal(tibuf[1:].cpu().numpy().reshape(want_ti.shape), want_ti)
    assert rel_max(y.cpu().numpy(), oracle.conv(want_ti, w, acc64=True)) <= TOL


def test_layer_wrappers_on_gpu(oracle, dev):
    from winograd_conv import WinogradConv
    from winograd_imtrans import WinogradImTrans
    rng = np.random.default_rng(17)
    x = rng.standard_normal((2, 8, 8, 16)).astype(np.float32)
    w = (rng.standard_normal((16, 16, 24)) * 0.05).astype(np.float32)
    mask = oracle.gen_prune_mask(w.copy(), 0.3)
    layer = WinogradConv(16, 24, mask=mask, W_init=w).to(dev)
    xd = gpu(x, dev)
    for nl in (torch.relu, "relu", torch.nn.ReLU()):
        assert np.array_equal(WinogradImTrans(xd, nl).cpu().numpy(), oracle.imtrans(x, relu=True))
    assert np.array_equal(WinogradImTrans(xd).cpu().numpy(), oracle.imtrans(x))
    assert np.array_equal(WinogradImTrans(xd, torch.tanh).cpu().numpy(),
                          torch.tanh(gpu(oracle.imtrans(x), dev)).cpu().numpy())
    y = layer(WinogradImTrans(xd, torch.relu)).detach().cpu().numpy()
    assert rel_max(y, oracle.conv(oracle.imtrans(x, relu=True), w * mask, acc64=True)) <= TOL


@pytest.mark.gpu
@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("shape", [(3, 6, 6, 32), (2, 7, 7, 5), (2, 5, 9, 3), (4, 28, 28, 128)])
def test_imtrans_affine_bit_exact(oracle, dev, shape, relu):
    # Folded inference BatchNorm: fmaf(x, scale, shift) inside the image, zeros outside, then the transform.
    imtrans, _ = ops()
    rng = np.random.default_rng(hash(shape) % 2 ** 31 + 1)
    x = rng.standard_normal(shape).astype(np.float32)
    scale = (0.5 + rng.random(shape[3])).astype(np.float32) * rng.choice([-1, 1], shape[3]).astype(np.float32)
    shift = rng.standard_normal(shape[3]).astype(np.float32)
    want = oracle.imtrans_affine(x, scale, shift, relu=relu)
    got = imtrans(gpu(x, dev), relu=relu, scale=gpu(scale, dev), shift=gpu(shift, dev)).cpu().numpy()
    assert np.array_equal(got == 0, want == 0), "zero mask differs"
    assert np.array_equal(got, want)
    # a non-zero shift must not leak into the padding: border tiles differ from transforming a padded-then-mapped image
    same = imtrans(gpu(oracle.affine(x, scale, shift), dev), relu=relu).cpu().numpy()
    assert np.array_equal(got, same)


def test_forward_pair_replays_in_a_hip_graph(dev):
    # The launchers allocate nothing and never synchronise, so imTrans + conv can be captured once and
    # replayed; every replay (with eager work and synchronisations in between) must equal the eager result.
    imtrans, conv = ops()
    g = torch.Generator(device="cpu").manual_seed(77)
    x = torch.randn(4, 14, 14, 64, generator=g).to(dev)
    w = (torch.randn(16, 64, 96, generator=g) * 0.05).to(dev)
    ti = torch.empty(16, 4, 7, 7, 64, device=dev)
    y = torch.empty(4, 14, 14, 96, device=dev)
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        conv(imtrans(x, relu=True, out=ti), w, out=y)   # warm-up outside the capture
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize(dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        conv(imtrans(x, relu=True, out=ti), w, out=y)
    for rep in range(4):
        x.copy_(torch.randn(4, 14, 14, 64, generator=g))
        y.zero_()
        graph.replay()
        torch.cuda.synchronize(dev)
        got = y.clone()
        want = conv(imtrans(x, relu=True), w)           # eager work between replays
        torch.cuda.synchronize(dev)
        assert torch.equal(got, want), rep


@pytest.mark.parametrize("shape", [(3, 3, 3, 32, 32), (2, 4, 4, 5, 7), (8, 9, 9, 128, 72), (16, 14, 14, 128, 128),
                                   (1, 5, 7, 48, 20)])
@pytest.mark.parametrize("parts", ["affine", "residual", "both", "both_relu"])
def test_conv_epilogue(oracle, dev, shape, parts):
    # Output = fmaf(conv, scale, shift) + residual (or + relu(residual)) inside the stores, on every kernel the
    # launcher picks.
    relu_res = parts == "both_relu"
    parts = "both" if relu_res else parts
    _, conv = ops()
    B, nH, nW, C, K = shape
    ti, w = conv_inputs(shape, 21)
    rng = np.random.default_rng(22)
    scale = (0.5 + rng.random(K)).astype(np.float32) * rng.choice([-1, 1], K).astype(np.float32)
    shift = rng.standard_normal(K).astype(np.float32)
    res = rng.standard_normal((B, 2 * nH, 2 * nW, K)).astype(np.float32)
    plain = conv(gpu(ti, dev), gpu(w, dev))
    kw, want = {}, plain.cpu().numpy()
    if parts in ("affine", "both"):
        kw.update(scale=gpu(scale, dev), shift=gpu(shift, dev))
        want = oracle.affine(want, scale, shift)
    if parts in ("residual", "both"):
        kw.update(residual=gpu(res, dev), residual_relu=relu_res)
        if relu_res:
            res = np.maximum(res, 0)
        want = want + res
    got = conv(gpu(ti, dev), gpu(w, dev), **kw).cpu().numpy()
    # same kernel, same accumulators: the epilogue arithmetic itself is exact against the oracle's
    assert np.array_equal(got, want)
    # and the whole thing against the float64-accumulated oracle
    full = oracle.conv(ti, w, acc64=True).astype(np.float64)
    if parts in ("affine", "both"):
        full = full * scale + shift
    if parts in ("residual", "both"):
        full = full + res
    assert rel_max(got, full) <= TOL
    # in place: residual aliasing the output
    if parts == "residual":
        buf = gpu(res, dev)
        conv(gpu(ti, dev), gpu(w, dev), out=buf, residual=buf)
        assert np.array_equal(buf.cpu().numpy(), want)


def test_channels_beyond_the_reference_block_limit(oracle, dev):
    # The reference launches one thread per channel (block = C, winograd2x2_imTrans_cuda.cu.cc:154) or per
    # filter (block = K, winograd2x2_conv_cuda.cu.cc:87), so it stops at 1024; these kernels do not.
    imtrans, conv = ops()
    rng = np.random.default_rng(41)
    x = rng.standard_normal((1, 4, 6, 2052)).astype(np.float32)
    assert np.array_equal(imtrans(gpu(x, dev), relu=True).cpu().numpy(), oracle.imtrans(x, relu=True))
    ti, w = conv_inputs((1, 2, 3, 64, 1100), 42)
    got = conv(gpu(ti, dev), gpu(w, dev)).cpu().numpy()
    assert rel_max(got, oracle.conv(ti, w, acc64=True)) <= TOL


def test_host_threads_on_their_own_streams(oracle, dev):
    # The launchers keep no shared mutable state: four host threads, each on its own stream with its own
    # tensors, must all get the result a single thread gets.
    import threading
    imtrans, conv = ops()
    shapes = [(2, 10, 10, 64, 64), (3, 6, 6, 32, 32), (2, 7, 9, 48, 20), (4, 14, 14, 128, 72)]
    inputs, wants, gots, errors = [], [], [None] * 4, []
    for i, (B, H, W, C, K) in enumerate(shapes):
        rng = np.random.default_rng(50 + i)
        x = rng.standard_normal((B, H, W, C)).astype(np.float32)
        w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
        inputs.append((gpu(x, dev), gpu(w, dev)))
        wants.append(oracle.conv(oracle.imtrans(x, relu=True), w, acc64=True))
    torch.cuda.synchronize(dev)

    def work(i):
        try:
            stream = torch.cuda.Stream(device=dev)
            with torch.cuda.stream(stream):
                for _ in range(20):
                    y = conv(imtrans(inputs[i][0], relu=True), inputs[i][1])
                stream.synchronize()
                gots[i] = y.cpu().numpy()
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for got, want in zip(gots, wants):
        assert rel_max(got, want) <= TOL


def test_imtrans_beyond_2_pow_31_elements_per_plane(dev):
    # M*C >= 2^31 switches the kernel to 64-bit lane indices.  The 137 GB result cannot be checked on the
    # host; sampled images must equal what the same op returns for them alone (32-bit path).
    imtrans, _ = ops()
    free, _total = torch.cuda.mem_get_info(dev)
    if free < 190e9:
        pytest.skip("needs 172 GB of free device memory")
    B, H, W, C = 21500, 56, 56, 128
    assert B * 28 * 28 * C >= 2 ** 31
    x = torch.empty(B, H, W, C, device=dev)
    for i in range(0, B, 500):
        x[i:i + 500].normal_()
    ti = imtrans(x, relu=True)
    for b in (0, 1, 7777, 13699, 13700, B - 1):   # 13699/13700 straddle the 2^31 boundary
        assert torch.equal(ti[:, b:b + 1], imtrans(x[b:b + 1].contiguous(), relu=True)), b
    del ti, x
    torch.cuda.empty_cache()
