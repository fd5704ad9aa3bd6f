"""MI355X-native Winograd-ReLU ops (forward): winograd2x2_imTrans and winograd2x2_conv.

The directory name is not a Python identifier; use it the way the reference's
``winograd2x2_cublas`` directory is used, by putting it on ``sys.path``/``PYTHONPATH``:

    import winograd2x2_imTrans.winograd2x2_imTrans
    import winograd2x2_conv.winograd2x2_conv
    from winograd_imtrans import WinogradImTrans
    from winograd_conv import WinogradConv

or ``importlib.import_module("sparse-winograd-cnn_amd")``, which does that for you.
"""
import os as _os
import sys as _sys

_HERE = _os.path.dirname(_os.path.abspath(__file__))
if _HERE not in _sys.path:
    _sys.path.insert(0, _HERE)
