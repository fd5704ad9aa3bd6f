"""Benchmark config 4 at its full size: N=64, 14x14x256 -> 256 and 7x7x512 -> 512 (odd size, 4x4 tiles, compared
uncropped as [64,8,8,512]), Winograd-domain ReLU on, weights pruned to 10 % density, for the three precisions,
each against the oracle and with the kernel the launcher picks asserted."""
import numpy as np
import pytest
import torch

from helpers import expected_stored_launch, rel_l1, rel_max

pytestmark = pytest.mark.gpu
TOL = 1e-4


def gpu(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


@pytest.mark.parametrize("layer", [("4a", 14, 256, 256, 400), ("4b", 7, 512, 512, 410)])
def test_config4_full_size(oracle, layer):
    import swc_hip
    from winograd2x2_conv.winograd2x2_conv import winograd2x2_conv
    from winograd2x2_imTrans.winograd2x2_imTrans import winograd2x2_imTrans
    assert torch.cuda.is_available()
    dev = torch.device("cuda:0")
    L = swc_hip.lib()
    name, hw, C, K, seed = layer
    N = 64
    x = np.random.default_rng(seed).standard_normal((N, hw, hw, C)).astype(np.float32)
    w = (np.random.default_rng(seed + 1).standard_normal((16, C, K)) * 0.05).astype(np.float32)
    oracle.gen_prune_mask(w, 0.1)
    nT = (hw + 1) // 2
    M = N * nT * nT
    cus = torch.cuda.get_device_properties(dev).multi_processor_count

    ti_want = oracle.imtrans(x, relu=True)
    ti = winograd2x2_imTrans(gpu(x, dev), relu=True)
    assert tuple(ti.shape) == (16, N, nT, nT, C)
    assert np.array_equal(ti.cpu().numpy(), ti_want)

    # fp32
    want = oracle.conv(ti_want, w, acc64=True)
    got = winograd2x2_conv(ti, gpu(w, dev)).cpu().numpy()
    assert got.shape == want.shape == (N, 2 * nT, 2 * nT, K)
    assert rel_max(got, want) <= TOL and rel_l1(got, want) <= TOL
    if cus == 256:
        # the tiling follows from the CU count: on an MI355X 32-row groups fill the device at config 4b where 64-row
        # tiles leave CUs idle; at config 4a one 48-row x 64-column workgroup per CU does (64 of them carry one of the
        # 16 tiles of the 64 left-over rows)
        assert L.swc_winograd2x2_conv_last_kernel() == (b"wide48x64" if name == "4a" else b"short16")

    # bf16 operands, fp32 planes: against the oracle fed the same rounded operands
    want16 = oracle.conv(oracle.round_bf16(ti_want), oracle.round_bf16(w), acc64=True)
    got = winograd2x2_conv(ti, gpu(w, dev), precision="bf16").cpu().numpy()
    assert rel_max(got, want16) <= TOL and rel_l1(got, want16) <= TOL
    assert rel_max(got, want) <= 2e-2   # and the rounding itself stays small against the fp32 result

    # bf16-stored planes
    ti16 = winograd2x2_imTrans(gpu(x, dev), relu=True, out_dtype=torch.bfloat16)
    assert np.array_equal(ti16.view(torch.int16).cpu().numpy().view(np.uint16), oracle.bf16_bits(ti_want))
    got = winograd2x2_conv(ti16, gpu(w, dev)).cpu().numpy()
    assert rel_max(got, want16) <= TOL and rel_l1(got, want16) <= TOL
    # one tile per CU at most: the launcher splits the positions over two groups of waves (config 4a), or over four
    # on 32-row tiles where those fit the CUs as well (config 4b)
    props = torch.cuda.get_device_properties(dev)
    assert L.swc_winograd2x2_conv_last_kernel().decode() in expected_stored_launch(M, C, K, cus, props.L2_cache_size)
