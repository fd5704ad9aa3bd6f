"""The entry point that allocates nothing (swc_winograd2x2_conv_grad_static), through the C ABI: same results as
swc_winograd2x2_conv_grad, whose dP temporary it keeps in a fixed device array instead."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(L, dev, rng, B, nH, nW, C, K):
    M = B * nH * nW
    ti = torch.from_numpy(np.maximum(rng.standard_normal((16, B, nH, nW, C)), 0).astype(np.float32)).to(dev)
    w = torch.from_numpy((rng.standard_normal((16, C, K)) * 0.05).astype(np.float32)).to(dev)
    dy = torch.from_numpy(rng.standard_normal((B, 2 * nH, 2 * nW, K)).astype(np.float32)).to(dev)
    stream = torch.cuda.current_stream().cuda_stream
    out = []
    for static in (False, True):
        # the outputs start as NaN so that an element a kernel leaves unwritten cannot compare equal
        dti = torch.full((16, B, nH, nW, C), float("nan"), device=dev)
        dw = torch.full((16, C, K), float("nan"), device=dev)
        if static:
            st = L.swc_winograd2x2_conv_grad_static(ti.data_ptr(), w.data_ptr(), dy.data_ptr(), dti.data_ptr(), dw.data_ptr(),
                                                    C, B, 2 * nH, 2 * nW, K, 1, 1, stream)
        else:
            tmp = torch.empty(16 * M * K, device=dev)
            st = L.swc_winograd2x2_conv_grad(ti.data_ptr(), w.data_ptr(), dy.data_ptr(), dti.data_ptr(), dw.data_ptr(),
                                             tmp.data_ptr(), None, C, B, 2 * nH, 2 * nW, K, 1, 1, stream)
        assert st == 0, L.swc_strerror(st)
        torch.cuda.synchronize()
        out.append((dti.cpu().numpy(), dw.cpu().numpy()))
    return out


def test_static_scratch_entry_point_matches_the_allocating_one():
    import swc_hip
    L = swc_hip.lib()
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(77)
    # two calls in a row, the second with a smaller input: it must not see the first call's leftovers
    # the first one fills the array exactly: B*nH*nW*K = 1 048 576
    for shape in ((16, 16, 16, 64, 256), (8, 7, 7, 128, 64), (2, 3, 5, 36, 20)):
        (dti_a, dw_a), (dti_s, dw_s) = _both(L, dev, rng, *shape)
        assert np.isfinite(dti_a).all() and np.isfinite(dw_a).all()
        # same kernels on the same inputs: bit for bit
        assert np.array_equal(dti_s, dti_a) and np.array_equal(dw_s, dw_a), shape


def test_static_scratch_entry_point_rejects_what_does_not_fit():
    import swc_hip
    L = swc_hip.lib()
    dev = torch.device("cuda:0")
    one = torch.zeros(1, device=dev)
    p = one.data_ptr()
    # 16 * (64*14*14) * 128 floats of dP > 16 Mi floats: refused before anything is launched or dereferenced
    st = L.swc_winograd2x2_conv_grad_static(p, p, p, p, p, 128, 64, 28, 28, 128, 1, 1, None)
    assert st == swc_hip.SWC_ERR_TOO_LARGE
    assert b"scratch" in L.swc_strerror(st)
    assert L.swc_winograd2x2_conv_grad_static(p, p, p, p, p, 128, 64, 27, 28, 128, 1, 1, None) == swc_hip.SWC_ERR_BAD_DIMS
    # one float more than fits
    assert L.swc_winograd2x2_conv_grad_static(p, p, p, p, p, 64, 16, 32, 32, 257, 1, 1, None) == swc_hip.SWC_ERR_TOO_LARGE
