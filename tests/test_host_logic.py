"""CPU-side checks: the C-ABI library loads and exports what include/winograd2x2.h declares,
the host op wrappers derive shapes and reject bad arguments as documented, and the Python
mirror of the reference's interface validates its inputs.  No kernel is launched here.
"""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import swc_hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "winograd2x2.h")).read()
    declared = set(re.findall(r"SWC_API\s+[\w\s\*]+?\b(swc_\w+|Winograd2x2\w+)\s*\(", header))
    assert set(swc_hip.C_SYMBOLS) == {d for d in declared if d.startswith("swc_")}
    assert {d for d in declared if d.startswith("Winograd2x2")} == {
        "Winograd2x2ImTransComputeLauncher", "Winograd2x2ConvComputeLauncher",
        "Winograd2x2ConvGradComputeLauncher", "Winograd2x2ImTransGradComputeLauncher"}
    L = ctypes.CDLL(swc_hip.LIB_PATH)
    for name in swc_hip.C_SYMBOLS + swc_hip.CXX_SYMBOLS:
        assert getattr(L, name) is not None, name
    assert swc_hip.lib().swc_version() == b"0.1"


def test_status_strings():
    L = swc_hip.lib()
    seen = {L.swc_strerror(s) for s in (0, -1, -2, -3, -4, -5)}
    assert len(seen) == 6 and L.swc_strerror(0) == b"ok"
    assert L.swc_strerror(-99) == b"unknown status"


@pytest.mark.parametrize("shape,want", [
    ((64, 28, 28, 128), (16, 64, 14, 14, 128)),
    ((3, 6, 6, 32), (16, 3, 3, 3, 32)),
    ((64, 7, 7, 512), (16, 64, 4, 4, 512)),   # odd extent rounds up: (H+1)/2
    ((2, 5, 9, 3), (16, 2, 3, 5, 3)),
    ((1, 1, 1, 1), (16, 1, 1, 1, 1)),
])
def test_imtrans_shape_rule(shape, want):
    from winograd2x2_imTrans.winograd2x2_imTrans import winograd2x2_imTrans_shape
    assert winograd2x2_imTrans_shape(shape) == want


@pytest.mark.parametrize("ishape,wshape,want", [
    ((16, 64, 14, 14, 128), (16, 128, 128), (64, 28, 28, 128)),
    ((16, 64, 4, 4, 512), (16, 512, 512), (64, 8, 8, 512)),   # never cropped back to 7x7
    ((16, 2, 4, 4, 5), (16, 5, 7), (2, 8, 8, 7)),
])
def test_conv_shape_rule(ishape, wshape, want):
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv_shape
    assert winograd2x2_conv_shape(ishape, wshape) == want


def test_shape_rules_reject_bad_input():
    L = swc_hip.lib()
    out = swc_hip.dims([0] * 5)
    assert L.swc_winograd2x2_imtrans_op_shape(3, swc_hip.dims((1, 2, 3)), out) == swc_hip.SWC_ERR_BAD_RANK
    assert L.swc_winograd2x2_imtrans_op_shape(4, swc_hip.dims((1, 0, 3, 4)), out) == swc_hip.SWC_ERR_BAD_DIMS
    assert L.swc_winograd2x2_imtrans_op_shape(4, swc_hip.dims((1, 2, 3, 2 ** 31)), out) == swc_hip.SWC_ERR_BAD_DIMS
    assert L.swc_winograd2x2_imtrans_op_shape(4, None, out) == swc_hip.SWC_ERR_NULL_POINTER
    o4 = swc_hip.dims([0] * 4)
    i5, w3 = swc_hip.dims((16, 2, 3, 3, 8)), swc_hip.dims((16, 8, 4))
    assert L.swc_winograd2x2_conv_op_shape(5, i5, 3, w3, o4) == 0
    assert L.swc_winograd2x2_conv_op_shape(4, i5, 3, w3, o4) == swc_hip.SWC_ERR_BAD_RANK
    assert L.swc_winograd2x2_conv_op_shape(5, i5, 2, w3, o4) == swc_hip.SWC_ERR_BAD_RANK
    assert L.swc_winograd2x2_conv_op_shape(5, swc_hip.dims((15, 2, 3, 3, 8)), 3, w3, o4) == swc_hip.SWC_ERR_BAD_RANK
    assert L.swc_winograd2x2_conv_op_shape(5, i5, 3, swc_hip.dims((16, 9, 4)), o4) == swc_hip.SWC_ERR_BAD_DIMS
    assert L.swc_winograd2x2_conv_op_shape(5, i5, 3, swc_hip.dims((16, 8, 0)), o4) == swc_hip.SWC_ERR_BAD_DIMS


def test_launchers_reject_bad_arguments_before_touching_the_gpu():
    L = swc_hip.lib()
    p = ctypes.c_void_p(4096)  # never dereferenced: every call below fails validation first
    assert L.swc_winograd2x2_imtrans(None, p, 4, 1, 4, 4, 1, 1, 0, None) == swc_hip.SWC_ERR_NULL_POINTER
    assert L.swc_winograd2x2_imtrans(p, None, 4, 1, 4, 4, 1, 1, 0, None) == swc_hip.SWC_ERR_NULL_POINTER
    assert L.swc_winograd2x2_imtrans(p, p, 0, 1, 4, 4, 1, 1, 0, None) == swc_hip.SWC_ERR_BAD_DIMS
    assert L.swc_winograd2x2_imtrans(p, p, 4, 1, -4, 4, 1, 1, 0, None) == swc_hip.SWC_ERR_BAD_DIMS
    assert L.swc_winograd2x2_imtrans(p, p, 4, 1, 4, 4, 0, 1, 0, None) == swc_hip.SWC_ERR_BAD_PAD
    assert L.swc_winograd2x2_imtrans(p, p, 4, 1, 4, 4, 1, 2, 0, None) == swc_hip.SWC_ERR_BAD_PAD
    for conv in (L.swc_winograd2x2_conv, L.swc_winograd2x2_conv_bf16):
        assert conv(None, p, p, None, None, 4, 1, 2, 2, 4, 1, 1, None) == swc_hip.SWC_ERR_NULL_POINTER
        assert conv(p, None, p, None, None, 4, 1, 2, 2, 4, 1, 1, None) == swc_hip.SWC_ERR_NULL_POINTER
        assert conv(p, p, None, None, None, 4, 1, 2, 2, 4, 1, 1, None) == swc_hip.SWC_ERR_NULL_POINTER
        assert conv(p, p, p, None, None, 4, 1, 2, 2, 0, 1, 1, None) == swc_hip.SWC_ERR_BAD_DIMS
        assert conv(p, p, p, None, None, 4, 1, 2, 2, 4, 1, 0, None) == swc_hip.SWC_ERR_BAD_PAD
    # gradient launchers
    assert L.swc_winograd2x2_conv_grad(p, p, p, p, p, None, None, 4, 1, 4, 4, 4, 1, 1, None) == swc_hip.SWC_ERR_NULL_POINTER
    assert L.swc_winograd2x2_conv_grad(p, p, p, p, p, p, None, 4, 1, 5, 4, 4, 1, 1, None) == swc_hip.SWC_ERR_BAD_DIMS  # H odd
    assert L.swc_winograd2x2_conv_grad(p, p, p, p, p, p, None, 4, 1, 4, 4, 4, 2, 1, None) == swc_hip.SWC_ERR_BAD_PAD
    assert L.swc_winograd2x2_imtrans_grad(None, None, p, 4, 1, 4, 4, 1, 1, None) == swc_hip.SWC_ERR_NULL_POINTER
    assert L.swc_winograd2x2_imtrans_grad(p, None, p, 4, 0, 4, 4, 1, 1, None) == swc_hip.SWC_ERR_BAD_DIMS
    assert L.swc_winograd2x2_imtrans_grad(p, None, p, 4, 1, 4, 4, 1, 0, None) == swc_hip.SWC_ERR_BAD_PAD
    # op level: an output of the wrong shape is refused
    i4, o5 = swc_hip.dims((1, 4, 4, 4)), swc_hip.dims((16, 1, 2, 2, 5))
    assert L.swc_winograd2x2_imtrans_op_compute(p, 4, i4, p, 5, o5, 0, None) == swc_hip.SWC_ERR_BAD_DIMS
    assert L.swc_winograd2x2_imtrans_op_compute(p, 4, i4, p, 4, o5, 0, None) == swc_hip.SWC_ERR_BAD_RANK
    i5, w3, o4 = swc_hip.dims((16, 1, 2, 2, 4)), swc_hip.dims((16, 4, 4)), swc_hip.dims((1, 4, 4, 4))
    assert L.swc_winograd2x2_conv_op_compute(p, 5, i5, p, 3, w3, p, 4, o4, 7, None) == swc_hip.SWC_ERR_BAD_DIMS
    assert L.swc_winograd2x2_conv_op_compute(p, 5, i5, p, 3, w3, p, 4, swc_hip.dims((1, 4, 4, 5)), 0, None) \
        == swc_hip.SWC_ERR_BAD_DIMS


def test_python_ops_refuse_cpu_tensors_and_wrong_types():
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv
    from winograd2x2_imTrans.winograd2x2_imTrans import winograd2x2_imTrans
    with pytest.raises(RuntimeError, match="GPU only"):
        winograd2x2_imTrans(torch.zeros(1, 4, 4, 4))
    with pytest.raises(ValueError, match="rank 4"):
        winograd2x2_imTrans(torch.zeros(4, 4, 4))
    with pytest.raises(TypeError, match="float32"):
        winograd2x2_imTrans(torch.zeros(1, 4, 4, 4, dtype=torch.float64))
    with pytest.raises(TypeError, match="torch.Tensor"):
        winograd2x2_imTrans(np.zeros((1, 4, 4, 4), dtype=np.float32))
    with pytest.raises(RuntimeError, match="GPU only"):
        winograd2x2_conv(torch.zeros(16, 1, 2, 2, 4), torch.zeros(16, 4, 4))
    with pytest.raises(ValueError, match="precision"):
        winograd2x2_conv(torch.zeros(16, 1, 2, 2, 4), torch.zeros(16, 4, 4), precision="fp8")


def test_layer_wrappers_signatures():
    import inspect

    from winograd_conv import WinogradConv
    from winograd_imtrans import WinogradImTrans, identity
    # ResNet-18-var/winograd_imtrans.py:16 and winograd_conv.py:16
    assert list(inspect.signature(WinogradImTrans).parameters)[:2] == ["x", "nl"]  # extras are keyword options
    assert inspect.signature(WinogradImTrans).parameters["nl"].default is identity
    assert list(inspect.signature(WinogradConv.__init__).parameters)[1:5] == ["in_channel", "out_channel", "mask", "W_init"]
    layer = WinogradConv(8, 12)
    assert tuple(layer.W.shape) == (16, 8, 12) and layer.W.requires_grad
    std = float(layer.W.std())
    assert 0 < std < np.sqrt(1.3 * (2 * 9 / 32) / (16 * 8))
    mask = np.zeros((16, 8, 12), dtype=np.float32)
    mask[:, ::2, :] = 1
    layer = WinogradConv(8, 12, mask=mask, W_init=lambda w: w.fill_(2.0))
    assert torch.equal(layer.masked_weight(), torch.from_numpy(mask) * 2.0)
    with pytest.raises(TypeError):
        WinogradImTrans(torch.zeros(1, 4, 4, 4), nl=3)


def test_masked_weight_cache_follows_weight_updates():
    """The cached W*mask must not outlive an in-place change of W or mask (optimizer step,
    load_state_dict), and an unmasked layer must hand out W itself."""
    from winograd_conv import WinogradConv
    mask = np.zeros((16, 4, 6), dtype=np.float32)
    mask[:, :, ::2] = 1
    m = torch.from_numpy(mask)
    layer = WinogradConv(4, 6, mask=mask, W_init=lambda w: w.fill_(2.0))
    first = layer.masked_weight()
    assert torch.equal(first, m * 2.0)
    assert layer.masked_weight() is first                      # unchanged weights: cache hit
    opt = torch.optim.SGD(layer.parameters(), lr=0.5)
    layer.W.grad = torch.ones_like(layer.W)
    opt.step()                                                 # W <- 1.5, in place
    assert torch.equal(layer.masked_weight(), m * 1.5)
    state = {k: v.clone() for k, v in layer.state_dict().items()}
    state["W"].fill_(-3.0)
    layer.load_state_dict(state)
    assert torch.equal(layer.masked_weight(), m * -3.0)
    with torch.no_grad():
        layer.mask.zero_()                                     # the mask changes too
    assert torch.count_nonzero(layer.masked_weight()) == 0
    plain = WinogradConv(4, 6)
    assert plain.masked_weight().data_ptr() == plain.W.data_ptr()
    k1 = plain._weight_key()
    assert plain._weight_key() == k1                           # stable key: the bf16 copy is reused
    with torch.no_grad():
        plain.W.mul_(2.0)
    assert plain._weight_key() != k1
    k2 = plain._weight_key()
    plain.masked_weight().mul_(0.5)                            # a write to what the layer hands out is noticed too
    assert plain._weight_key() != k2


def test_writes_through_dot_data_need_refresh():
    """A `.data` view has a version counter of its own: W*mask and the bf16 copy keep their old values after
    `layer.W.data.mul_()` until refresh() is called, as the docstrings of refresh() and masked_weight() say."""
    from winograd_conv import WinogradConv
    m = torch.ones(16, 4, 6)
    m[:, :, ::2] = 0
    layer = WinogradConv(4, 6, mask=m.numpy(), W_init=lambda w: w.fill_(2.0))
    assert torch.equal(layer.masked_weight(), m * 2.0)
    layer.W.data.mul_(3.0)
    assert torch.equal(layer.masked_weight(), m * 2.0)         # stale: nothing recorded the write
    layer.refresh()
    assert torch.equal(layer.masked_weight(), m * 6.0)
    layer.W.detach().mul_(0.5)                                 # the detach() view shares W's counter: noticed
    assert torch.equal(layer.masked_weight(), m * 3.0)


def test_weight_preparation_matches_oracle(oracle):
    from winograd_weights import gen_prune_mask, kernel_transform
    rng = np.random.default_rng(0)
    g = rng.standard_normal((3, 3, 6, 5)).astype(np.float32)
    assert np.allclose(kernel_transform(g), oracle.kernel_transform(g), rtol=0, atol=1e-6)
    w = rng.standard_normal((16, 6, 5)).astype(np.float32)
    w1, w2 = w.copy(), w.copy()
    assert np.array_equal(gen_prune_mask(w1, 0.2), oracle.gen_prune_mask(w2, 0.2))
    assert np.array_equal(w1, w2) and int((w1 != 0).sum()) == int(w.size * 0.2)


def test_gradient_op_shape_rules():
    """The host wrappers of the two gradient ops: winograd2x2_conv_grad_op.cc:44-67 (results shaped like the
    inputs, temporary of 16*nH*nW*B*K floats) and winograd2x2_imTrans_grad_op.cc:40-49 (H = 2nH)."""
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv_grad_shape
    L = swc_hip.lib()
    assert winograd2x2_conv_grad_shape((16, 64, 14, 14, 128), (16, 128, 128), (64, 28, 28, 128)) == (
        (16, 64, 14, 14, 128), (16, 128, 128), 16 * 14 * 14 * 64 * 128)
    assert winograd2x2_conv_grad_shape((16, 2, 4, 4, 5), (16, 5, 7), (2, 8, 8, 7)) == ((16, 2, 4, 4, 5), (16, 5, 7), 16 * 32 * 7)
    ti, w, g = swc_hip.dims((16, 2, 4, 4, 5)), swc_hip.dims((16, 5, 7)), swc_hip.dims((2, 8, 8, 7))
    o5, o3, tmp = swc_hip.dims([0] * 5), swc_hip.dims([0] * 3), ctypes.c_int64(0)
    ok = lambda *a: L.swc_winograd2x2_conv_grad_op_shape(*a, o5, o3, ctypes.byref(tmp))
    assert ok(5, ti, 3, w, 4, g) == 0
    assert ok(4, ti, 3, w, 4, g) == swc_hip.SWC_ERR_BAD_RANK
    assert ok(5, ti, 3, w, 3, g) == swc_hip.SWC_ERR_BAD_RANK
    assert ok(5, ti, 3, w, 4, swc_hip.dims((2, 7, 8, 7))) == swc_hip.SWC_ERR_BAD_DIMS      # the output is never cropped: H = 2nH
    assert ok(5, ti, 3, w, 4, swc_hip.dims((3, 8, 8, 7))) == swc_hip.SWC_ERR_BAD_DIMS      # B disagrees
    assert ok(5, ti, 3, swc_hip.dims((16, 5, 8)), 4, g) == swc_hip.SWC_ERR_BAD_DIMS        # K disagrees
    assert ok(5, ti, 3, swc_hip.dims((16, 6, 7)), 4, g) == swc_hip.SWC_ERR_BAD_DIMS        # C disagrees
    assert ok(5, None, 3, w, 4, g) == swc_hip.SWC_ERR_NULL_POINTER
    # compute: a temporary that is too small is refused before anything is launched
    p = ctypes.c_void_p(4096)
    assert L.swc_winograd2x2_conv_grad_op_compute(p, 5, ti, p, 3, w, p, 4, g, p, p, p, 16 * 32 * 7 - 1, None) == swc_hip.SWC_ERR_BAD_DIMS

    o4 = swc_hip.dims([0] * 4)
    assert L.swc_winograd2x2_imtrans_grad_op_shape(5, swc_hip.dims((16, 64, 4, 4, 512)), o4) == 0
    assert tuple(o4) == (64, 8, 8, 512)                                                        # 2nH, not the forward 7
    assert L.swc_winograd2x2_imtrans_grad_op_shape(4, swc_hip.dims((16, 64, 4, 4)), o4) == swc_hip.SWC_ERR_BAD_RANK
    assert L.swc_winograd2x2_imtrans_grad_op_shape(5, swc_hip.dims((15, 64, 4, 4, 512)), o4) == swc_hip.SWC_ERR_BAD_RANK
    assert L.swc_winograd2x2_imtrans_grad_op_shape(5, swc_hip.dims((16, 64, 0, 4, 512)), o4) == swc_hip.SWC_ERR_BAD_DIMS
    g5 = swc_hip.dims((16, 2, 4, 4, 8))
    bad = lambda ig, ro=None, ri=None: L.swc_winograd2x2_imtrans_grad_op_compute(p, 5, g5, ro, ri, p, 4, swc_hip.dims(ig), None)
    assert bad((2, 6, 8, 8)) == swc_hip.SWC_ERR_BAD_DIMS       # 6 does not tile into 4
    assert bad((2, 9, 8, 8)) == swc_hip.SWC_ERR_BAD_DIMS
    assert bad((2, 8, 8, 9)) == swc_hip.SWC_ERR_BAD_DIMS
    assert bad((2, 8, 8, 8), p, p) == swc_hip.SWC_ERR_BAD_DIMS  # two sources for the mask


def test_static_entry_bounds_its_size_one_factor_at_a_time():
    """16*B*(H/2)*(W/2)*K taken as one product of ints can wrap to a small number; the entry point must refuse such
    dimensions before it touches the GPU (the pointers here are never dereferenced)."""
    L = swc_hip.lib()
    p = ctypes.c_void_p(4096)
    big = 2 ** 31 - 2
    for dims in ((1, big, big, big, big), (1, 2 ** 16, 2 ** 17, 2 ** 17, 2 ** 16), (1, 2 ** 30, 4, 4, 2 ** 30),
                 (1, 2, 2, 2, 2 ** 21)):
        C, B, H, W, K = dims
        assert L.swc_winograd2x2_conv_grad_static(p, p, p, p, p, C, B, H, W, K, 1, 1, None) == swc_hip.SWC_ERR_TOO_LARGE, dims
        if dims[1] > 2:   # and the allocating entry refuses what no buffer could hold (the last case is valid there)
            assert L.swc_winograd2x2_conv_grad(p, p, p, p, p, p, None, C, B, H, W, K, 1, 1, None) == swc_hip.SWC_ERR_BAD_DIMS, dims
