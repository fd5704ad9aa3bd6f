"""The oracle must keep reproducing the committed golden fixtures bit for bit."""
import importlib.util
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
make_golden = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(make_golden)


def load(name):
    return dict(np.load(os.path.join(HERE, "golden", name + ".npz")))


@pytest.mark.parametrize("name", sorted(make_golden.CASES))
def test_oracle_reproduces_fixture(oracle, name):
    want = load(name)
    x, w = want["x"], want["w"]
    assert np.array_equal(oracle.imtrans(x), want["ti"])
    assert np.array_equal(oracle.imtrans(x, relu=True), want["ti_relu"])
    # the float64-accumulated GEMM rounds once per product, so it is reproducible bit for bit
    assert np.array_equal(oracle.conv(want["ti"], w, acc64=True), want["y"])
    assert np.array_equal(oracle.conv(want["ti_relu"], w, acc64=True), want["y_relu"])
    B, H, W, C, K, density, _ = make_golden.CASES[name]
    assert x.shape == (B, H, W, C) and w.shape == (16, C, K)
    if density < 1.0:
        assert int((w != 0).sum()) == int(w.size * density)
