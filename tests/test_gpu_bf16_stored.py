"""bf16-stored forward pair: imTrans writing bf16, the convolution reading bf16 activations and
prepared bf16 weights.  Through the C ABI (via the Python mirror), against the oracle."""
import numpy as np
import pytest
import torch

from helpers import expected_stored_launch, rel_max

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


def bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("shape", [(3, 6, 6, 32), (2, 7, 7, 5), (2, 5, 9, 3), (8, 28, 28, 128)])
def test_imtrans_bf16_output_is_the_rounded_fp32_transform(oracle, dev, shape, relu):
    from winograd2x2_imTrans.winograd2x2_imTrans import winograd2x2_imTrans
    rng = np.random.default_rng(61)
    x = rng.standard_normal(shape).astype(np.float32)
    want = oracle.bf16_bits(oracle.imtrans(x, relu=relu))
    got = winograd2x2_imTrans(gpu(x, dev), relu=relu, out_dtype=torch.bfloat16)
    assert got.dtype == torch.bfloat16
    assert np.array_equal(bits(got), want)
    # with the folded affine map
    scale = (0.5 + rng.random(shape[3])).astype(np.float32)
    shift = rng.standard_normal(shape[3]).astype(np.float32)
    want = oracle.bf16_bits(oracle.imtrans_affine(x, scale, shift, relu=relu))
    got = winograd2x2_imTrans(gpu(x, dev), relu=relu, scale=gpu(scale, dev), shift=gpu(shift, dev),
                              out_dtype=torch.bfloat16)
    assert np.array_equal(bits(got), want)


def test_weight_preparation(oracle, dev):
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_weights_bf16
    rng = np.random.default_rng(62)
    w = (rng.standard_normal((16, 24, 40)) * 0.05).astype(np.float32)
    got = winograd2x2_weights_bf16(gpu(w, dev))
    assert tuple(got.shape) == (16, 40, 24) and got.dtype == torch.bfloat16
    assert np.array_equal(bits(got), oracle.bf16_bits(w.transpose(0, 2, 1)))


@pytest.mark.parametrize("shape", [
    (3, 3, 3, 64, 32),      # one 64-channel step per position
    (2, 3, 5, 128, 100),    # ragged rows (M = 30) and columns (K = 100)
    (8, 14, 14, 128, 128),  # config 3 geometry, reduced batch
    (4, 7, 7, 256, 72),
    (1, 1, 1, 64, 4),
])
def test_conv_over_bf16_operands(oracle, dev, shape):
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv, winograd2x2_weights_bf16
    B, nH, nW, C, K = shape
    rng = np.random.default_rng(63)
    ti = np.maximum(rng.standard_normal((16, B, nH, nW, C)), 0).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    ti16, w16 = oracle.round_bf16(ti), oracle.round_bf16(w)
    want = oracle.conv(ti16, w16, acc64=True)          # products of bf16 values are exact in fp32
    ti_gpu = gpu(ti16, dev).to(torch.bfloat16)         # exact: the values are already bf16
    got = winograd2x2_conv(ti_gpu, gpu(w, dev)).cpu().numpy()
    assert got.shape == want.shape
    assert rel_max(got, want) <= TOL
    # prepared weights and the epilogue
    scale = (0.5 + rng.random(K)).astype(np.float32)
    shift = rng.standard_normal(K).astype(np.float32)
    res = rng.standard_normal(want.shape).astype(np.float32)
    got2 = winograd2x2_conv(ti_gpu, winograd2x2_weights_bf16(gpu(w, dev)), scale=gpu(scale, dev), shift=gpu(shift, dev),
                            residual=gpu(res, dev)).cpu().numpy()
    assert np.array_equal(got2, oracle.affine(got, scale, shift) + res)
    got3 = winograd2x2_conv(ti_gpu, winograd2x2_weights_bf16(gpu(w, dev)), scale=gpu(scale, dev), shift=gpu(shift, dev),
                            residual=gpu(res, dev), residual_relu=True).cpu().numpy()
    assert np.array_equal(got3, oracle.affine(got, scale, shift) + np.maximum(res, 0))
    # the same values as the kernel that rounds fp32 operands in its registers
    same = winograd2x2_conv(gpu(ti, dev), gpu(w, dev), precision="bf16").cpu().numpy()
    assert rel_max(got, same) <= TOL
    # which launch form ran: small grids split the positions over groups of waves, large ones take the tall tiles
    import swc_hip
    winograd2x2_conv(ti_gpu, gpu(w, dev))
    props = torch.cuda.get_device_properties(dev)
    want_launch = expected_stored_launch(B * nH * nW, C, K, props.multi_processor_count, props.L2_cache_size)
    assert swc_hip.lib().swc_winograd2x2_conv_last_kernel().decode() in want_launch


@pytest.mark.parametrize("shape", [
    (64, 4, 4, 512, 512),    # config 4b: 32 x 8 workgroups of 32 rows, eight steps per position
    (3, 5, 7, 256, 96),      # M = 105: the last row group holds 9 rows; the second column group 32 columns
    (1, 1, 1, 320, 4),       # one row, four columns, five steps per position
    (2, 9, 9, 1024, 192),    # sixteen steps per position
])
def test_stored_split4_kernel(oracle, dev, shape):
    """Small grids of long positions run `stored-split4` (32-row tiles, four groups of two waves, four positions
    each, partial sums added group by group): values against the oracle fed the same bf16 operands, exactly on
    integers, and the epilogue's arithmetic exactly."""
    import swc_hip
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv, winograd2x2_weights_bf16
    B, nH, nW, C, K = shape
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    if -(-B * nH * nW // 32) * -(-K // 64) > cus:
        pytest.skip("this device has too few CUs for the shape to take one 32-row tile per CU")
    rng = np.random.default_rng(68)
    ti = np.maximum(rng.standard_normal((16, B, nH, nW, C)), 0).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    ti16, w16 = oracle.round_bf16(ti), oracle.round_bf16(w)
    ti_gpu, w_gpu = gpu(ti16, dev).to(torch.bfloat16), winograd2x2_weights_bf16(gpu(w, dev))
    got = winograd2x2_conv(ti_gpu, w_gpu, workspace=False).cpu().numpy()
    assert swc_hip.lib().swc_winograd2x2_conv_last_kernel() == b"stored-split4"
    want = oracle.conv(ti16, w16, acc64=True)
    assert got.shape == want.shape
    assert rel_max(got, want) <= TOL
    ti_i = rng.integers(-3, 4, size=ti.shape).astype(np.float32)
    w_i = rng.integers(-3, 4, size=w.shape).astype(np.float32)
    got_i = winograd2x2_conv(gpu(ti_i, dev).to(torch.bfloat16), gpu(w_i, dev), workspace=False).cpu().numpy()
    assert np.array_equal(got_i, oracle.conv(ti_i, w_i))
    scale = (0.5 + rng.random(K)).astype(np.float32) * rng.choice([-1, 1], K).astype(np.float32)
    shift = rng.standard_normal(K).astype(np.float32)
    res = rng.standard_normal(want.shape).astype(np.float32)
    got2 = winograd2x2_conv(ti_gpu, w_gpu, scale=gpu(scale, dev), shift=gpu(shift, dev), residual=gpu(res, dev),
                            workspace=False).cpu().numpy()
    assert np.array_equal(got2, oracle.affine(got, scale, shift) + res)
    got3 = winograd2x2_conv(ti_gpu, w_gpu, residual=gpu(res, dev), residual_relu=True, workspace=False).cpu().numpy()
    assert np.array_equal(got3, got + np.maximum(res, 0))


@pytest.mark.parametrize("shape", [
    (64, 4, 4, 512, 512),    # config 4b: 8 x 8 tiles of 128 rows x 64 columns, four workgroups each
    (16, 7, 7, 256, 256),    # M = 784: the last row group holds 16 rows; four steps per position
    (3, 5, 7, 256, 128),     # M = 105: one ragged row group
    (1, 1, 1, 512, 64),      # one row
    (5, 9, 9, 512, 192),     # M = 405
])
def test_stored_spread_kernel(oracle, dev, shape):
    """Layers of 256 or 512 channels with too few 128-row x 64-column tiles for the chip, given a scratch buffer, run
    `stored-spread` (four workgroups per tile, one per row of the position grid; a second kernel combines their
    partial sums): values against the oracle fed the same bf16 operands, exactly on integers (every sign, the
    scatter), the epilogue's arithmetic exactly, and the entry point's fallback without a buffer."""
    import swc_hip
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv, winograd2x2_weights_bf16
    B, nH, nW, C, K = shape
    L = swc_hip.lib()
    M = B * nH * nW
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    if 4 * -(-M // 128) * (K // 64) * (512 // C) > cus:
        pytest.skip("this device has too few CUs for the shape to take the spread form")
    assert L.swc_winograd2x2_conv_bf16in_workspace_floats(C, B, nH, nW, K) == 8 * M * K
    rng = np.random.default_rng(69)
    ti = np.maximum(rng.standard_normal((16, B, nH, nW, C)), 0).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    ti16, w16 = oracle.round_bf16(ti), oracle.round_bf16(w)
    ti_gpu, w_gpu = gpu(ti16, dev).to(torch.bfloat16), winograd2x2_weights_bf16(gpu(w, dev))
    got = winograd2x2_conv(ti_gpu, w_gpu).cpu().numpy()
    assert L.swc_winograd2x2_conv_last_kernel() == b"stored-spread"
    want = oracle.conv(ti16, w16, acc64=True)
    assert got.shape == want.shape
    assert rel_max(got, want) <= TOL
    plain = winograd2x2_conv(ti_gpu, w_gpu, workspace=False).cpu().numpy()
    assert L.swc_winograd2x2_conv_last_kernel() != b"stored-spread"
    assert rel_max(got, plain) <= 1e-5
    ti_i = rng.integers(-3, 4, size=ti.shape).astype(np.float32)
    w_i = rng.integers(-3, 4, size=w.shape).astype(np.float32)
    got_i = winograd2x2_conv(gpu(ti_i, dev).to(torch.bfloat16), gpu(w_i, dev)).cpu().numpy()
    assert L.swc_winograd2x2_conv_last_kernel() == b"stored-spread"
    assert np.array_equal(got_i, oracle.conv(ti_i, w_i))
    scale = (0.5 + rng.random(K)).astype(np.float32) * rng.choice([-1, 1], K).astype(np.float32)
    shift = rng.standard_normal(K).astype(np.float32)
    res = rng.standard_normal(want.shape).astype(np.float32)
    got2 = winograd2x2_conv(ti_gpu, w_gpu, scale=gpu(scale, dev), shift=gpu(shift, dev), residual=gpu(res, dev)).cpu().numpy()
    assert np.array_equal(got2, oracle.affine(got, scale, shift) + res)
    got3 = winograd2x2_conv(ti_gpu, w_gpu, residual=gpu(res, dev), residual_relu=True).cpu().numpy()
    assert np.array_equal(got3, got + np.maximum(res, 0))
    # a buffer that is too small is not used
    y = torch.empty(B, 2 * nH, 2 * nW, K, device=dev)
    small = torch.empty(8 * M * K - 1, device=dev)
    st = L.swc_winograd2x2_conv_bf16in_ws(ti_gpu.data_ptr(), w_gpu.data_ptr(), y.data_ptr(), None, None, None, 0,
                                          small.data_ptr(), small.numel(), C, B, nH, nW, K, 1, 1,
                                          torch.cuda.current_stream().cuda_stream)
    assert st == 0 and L.swc_winograd2x2_conv_last_kernel() != b"stored-spread"
    assert np.array_equal(y.cpu().numpy(), plain)


@pytest.mark.parametrize("shape", [
    (6, 16, 16, 128, 1024),   # 12 x 16 tiles of 128 rows x 64 columns
    (25, 20, 20, 64, 256),    # 64 channels: a position is a single step (vector work and stores share it)
    (26, 31, 31, 64, 64),     # M = 24 986: levelled rows, one column group
    (3, 20, 25, 256, 1024),   # M = 1500: the last row group holds 92 rows
    (2, 16, 24, 512, 2048),   # 512 channels: eight steps per position
    (4, 25, 25, 128, 1024),   # more tiles than CUs: rows levelled over whole rounds (79 per workgroup on an MI355X)
])
def test_stored_tall_kernel(oracle, dev, shape):
    """Layers of 64, 128, 256 or 512 channels with enough tiles for the chip run `stored-tall` (128-row x 64-column
    workgroups, the output transform in the sum/difference association): values against the oracle fed the same
    bf16 operands, exactly on integers (every sign and the scatter), and the epilogue's arithmetic exactly."""
    import swc_hip
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv, winograd2x2_weights_bf16
    B, nH, nW, C, K = shape
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    if -(-B * nH * nW // 128) * (K // 64) * 4 < 3 * cus:
        pytest.skip("this device has too many CUs for the shape to take the tall tiles")
    rng = np.random.default_rng(67)
    ti = np.maximum(rng.standard_normal((16, B, nH, nW, C)), 0).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    ti16, w16 = oracle.round_bf16(ti), oracle.round_bf16(w)
    ti_gpu, w_gpu = gpu(ti16, dev).to(torch.bfloat16), winograd2x2_weights_bf16(gpu(w, dev))
    got = winograd2x2_conv(ti_gpu, w_gpu).cpu().numpy()
    assert swc_hip.lib().swc_winograd2x2_conv_last_kernel() == b"stored-tall"
    want = oracle.conv(ti16, w16, acc64=True)
    assert got.shape == want.shape
    assert rel_max(got, want) <= TOL
    # small integers: exact in bf16 and in every partial sum
    ti_i = rng.integers(-3, 4, size=ti.shape).astype(np.float32)
    w_i = rng.integers(-3, 4, size=w.shape).astype(np.float32)
    got_i = winograd2x2_conv(gpu(ti_i, dev).to(torch.bfloat16), gpu(w_i, dev)).cpu().numpy()
    assert np.array_equal(got_i, oracle.conv(ti_i, w_i))
    # the epilogue
    scale = (0.5 + rng.random(K)).astype(np.float32) * rng.choice([-1, 1], K).astype(np.float32)
    shift = rng.standard_normal(K).astype(np.float32)
    res = rng.standard_normal(want.shape).astype(np.float32)
    got2 = winograd2x2_conv(ti_gpu, w_gpu, scale=gpu(scale, dev), shift=gpu(shift, dev), residual=gpu(res, dev)).cpu().numpy()
    assert swc_hip.lib().swc_winograd2x2_conv_last_kernel() == b"stored-tall"
    assert np.array_equal(got2, oracle.affine(got, scale, shift) + res)
    got3 = winograd2x2_conv(ti_gpu, w_gpu, residual=gpu(res, dev), residual_relu=True).cpu().numpy()
    assert np.array_equal(got3, got + np.maximum(res, 0))
    buf = gpu(res, dev)
    winograd2x2_conv(ti_gpu, w_gpu, out=buf, residual=buf)      # residual aliasing the output
    assert np.array_equal(buf.cpu().numpy(), got + res)


def test_unsupported_channel_count_is_reported(dev):
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv
    import swc_hip
    ti = torch.zeros(16, 1, 2, 2, 48, device=dev, dtype=torch.bfloat16)
    with pytest.raises(swc_hip.SwcError, match="no kernel"):
        winograd2x2_conv(ti, torch.zeros(16, 48, 8, device=dev))


def test_whole_pair_against_fp32_path(oracle, dev):
    # config 3 in full: the bf16-stored pair against the fp64-accumulated oracle of the unrounded operands
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv
    from winograd2x2_imTrans.winograd2x2_imTrans import winograd2x2_imTrans
    rng = np.random.default_rng(64)
    x = rng.standard_normal((64, 28, 28, 128)).astype(np.float32)
    w = (rng.standard_normal((16, 128, 128)) * 0.05).astype(np.float32)
    y = winograd2x2_conv(winograd2x2_imTrans(gpu(x, dev), relu=True, out_dtype=torch.bfloat16), gpu(w, dev)).cpu().numpy()
    want = oracle.conv(oracle.imtrans(x, relu=True), w, acc64=True)
    assert rel_max(y, want) <= 1e-2
    exact = oracle.conv(oracle.round_bf16(oracle.imtrans(x, relu=True)), oracle.round_bf16(w), acc64=True)
    assert rel_max(y, exact) <= TOL


@pytest.mark.parametrize("shape", [
    (3, 6, 6, 16, 32),      # one 16-channel chunk
    (2, 7, 9, 32, 100),     # odd extent, ragged rows and columns, two chunks
    (2, 5, 5, 48, 20),      # three chunks (odd count)
    (8, 28, 28, 128, 128),  # config 3 geometry, reduced batch
    (4, 14, 14, 256, 72),
    (1, 2, 2, 64, 4),
])
@pytest.mark.parametrize("relu", [True, False])
def test_fused_bf16_layer(oracle, dev, shape, relu):
    # One kernel from the fp32 input to the fp32 output must give what the bf16-stored pair gives.
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_relu_conv_bf16, winograd2x2_weights_bf16
    B, H, W, C, K = shape
    rng = np.random.default_rng(65)
    x = rng.standard_normal((B, H, W, C)).astype(np.float32)
    w = (rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)
    ti16 = oracle.round_bf16(oracle.imtrans(x, relu=relu))
    want = oracle.conv(ti16, oracle.round_bf16(w), acc64=True)
    got = winograd2x2_relu_conv_bf16(gpu(x, dev), gpu(w, dev), relu=relu).cpu().numpy()
    assert got.shape == want.shape
    assert rel_max(got, want) <= TOL
    # folded input affine map and output epilogue, prepared weights
    s_in = (0.5 + rng.random(C)).astype(np.float32)
    t_in = rng.standard_normal(C).astype(np.float32)
    s_out = (0.5 + rng.random(K)).astype(np.float32)
    t_out = rng.standard_normal(K).astype(np.float32)
    res = rng.standard_normal(want.shape).astype(np.float32)
    ti16 = oracle.round_bf16(oracle.imtrans_affine(x, s_in, t_in, relu=relu))
    core = oracle.conv(ti16, oracle.round_bf16(w), acc64=True)
    want2 = core.astype(np.float64) * s_out + t_out + res
    got2 = winograd2x2_relu_conv_bf16(gpu(x, dev), winograd2x2_weights_bf16(gpu(w, dev)), relu=relu,
                                      in_affine=(gpu(s_in, dev), gpu(t_in, dev)), scale=gpu(s_out, dev),
                                      shift=gpu(t_out, dev), residual=gpu(res, dev)).cpu().numpy()
    assert rel_max(got2, want2) <= TOL


def test_fused_bf16_layer_falls_back(oracle, dev):
    # C = 40 is no multiple of 16: the wrapper runs the fp32-stored pair with bf16 operands (still HIP).
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_relu_conv_bf16
    rng = np.random.default_rng(66)
    x = rng.standard_normal((2, 6, 6, 40)).astype(np.float32)
    w = (rng.standard_normal((16, 40, 12)) * 0.05).astype(np.float32)
    want = oracle.conv(oracle.round_bf16(oracle.imtrans(x, relu=True)), oracle.round_bf16(w), acc64=True)
    got = winograd2x2_relu_conv_bf16(gpu(x, dev), gpu(w, dev)).cpu().numpy()
    assert rel_max(got, want) <= TOL
