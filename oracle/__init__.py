"""CPU oracle for the Winograd F(2x2,3x3) forward path.  TEST INFRASTRUCTURE ONLY.

ctypes bindings over ``oracle/liboracle.so`` (built from ``winograd_oracle.c`` by
``oracle/Makefile``) plus two tiny numpy restatements.  Imported only by the tests,
by the smoke check and by the benchmark's ``cpu_baseline`` leg; the shipped library
never touches it.

Reference lines followed are cited per function in ``winograd_oracle.c``.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

_F = ctypes.POINTER(ctypes.c_float)


def build(force=False):
    """Compile liboracle.so with gcc (no GPU needed)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.oracle_num_threads.restype = ctypes.c_int
        L.oracle_set_num_threads.argtypes = [ctypes.c_int]
        L.oracle_imtrans_f32.argtypes = [_F, _F] + [ctypes.c_int] * 5
        L.oracle_gemm16_f32.argtypes = [_F, _F, _F, ctypes.c_long, ctypes.c_int, ctypes.c_int]
        L.oracle_gemm16_f64acc.argtypes = [_F, _F, _F, ctypes.c_long, ctypes.c_int, ctypes.c_int]
        L.oracle_output_transform_f32.argtypes = [_F, _F] + [ctypes.c_int] * 4
        L.oracle_conv_f32.argtypes = [_F, _F, _F, _F] + [ctypes.c_int] * 6
        L.oracle_kernel_transform_f32.argtypes = [_F, _F, ctypes.c_int, ctypes.c_int]
        for f in (L.oracle_imtrans_f32, L.oracle_gemm16_f32, L.oracle_gemm16_f64acc,
                  L.oracle_output_transform_f32, L.oracle_conv_f32, L.oracle_kernel_transform_f32,
                  L.oracle_set_num_threads):
            f.restype = None
        _lib = L
    return _lib


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_F)


def num_threads():
    return int(lib().oracle_num_threads())


def set_num_threads(n):
    lib().oracle_set_num_threads(int(n))


def imtrans(x, relu=False):
    """x [B,H,W,C] fp32 -> [16,B,nH,nW,C] fp32."""
    x, xp = _f32(x)
    B, H, W, C = x.shape
    out = np.empty((16, B, (H + 1) // 2, (W + 1) // 2, C), dtype=np.float32)
    lib().oracle_imtrans_f32(xp, out.ctypes.data_as(_F), B, H, W, C, int(bool(relu)))
    return out


def affine(x, scale, shift):
    """x [...,C] -> fmaf(x, scale[c], shift[c]) elementwise, fp32 with a single rounding."""
    x, xp = _f32(x)
    scale, sp = _f32(scale)
    shift, hp = _f32(shift)
    C = x.shape[-1]
    assert scale.shape == (C,) and shift.shape == (C,)
    out = np.empty_like(x)
    L = lib()
    L.oracle_affine_f32.argtypes = [_F, _F, _F, _F, ctypes.c_long, ctypes.c_int]
    L.oracle_affine_f32.restype = None
    L.oracle_affine_f32(xp, sp, hp, out.ctypes.data_as(_F), x.size // C, C)
    return out


def imtrans_affine(x, scale, shift, relu=False):
    """Transform of the affinely mapped image (zero padding stays zero): imtrans(affine(x))."""
    return imtrans(affine(x, scale, shift), relu=relu)


def round_bf16(a):
    """fp32 -> nearest bf16 (ties to even), returned widened back to fp32.  Finite inputs only."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def bf16_bits(a):
    """The 16-bit patterns of round_bf16(a)."""
    return (round_bf16(a).view(np.uint32) >> 16).astype(np.uint16)


def gemm16(ti, w, acc64=False):
    """ti [16,M,C] (any leading tile dims), w [16,C,K] -> P [16,M,K] fp32."""
    ti, tp = _f32(ti)
    w, wp = _f32(w)
    C, K = int(w.shape[1]), int(w.shape[2])
    assert ti.shape[0] == 16 and w.shape[0] == 16 and ti.shape[-1] == C
    M = ti.size // (16 * C)
    out = np.empty((16, M, K), dtype=np.float32)
    fn = lib().oracle_gemm16_f64acc if acc64 else lib().oracle_gemm16_f32
    fn(tp, wp, out.ctypes.data_as(_F), M, C, K)
    return out


def output_transform(p, B, nH, nW):
    """p [16,B*nH*nW,K] -> [B,2nH,2nW,K] fp32."""
    p, pp = _f32(p)
    K = int(p.shape[-1])
    out = np.empty((B, 2 * nH, 2 * nW, K), dtype=np.float32)
    lib().oracle_output_transform_f32(pp, out.ctypes.data_as(_F), B, nH, nW, K)
    return out


def conv(ti, w, acc64=False):
    """ti [16,B,nH,nW,C], w [16,C,K] -> [B,2nH,2nW,K] fp32 (uncropped)."""
    ti, tp = _f32(ti)
    w, wp = _f32(w)
    _, B, nH, nW, C = ti.shape
    K = int(w.shape[2])
    assert w.shape == (16, C, K)
    tmp = np.empty(16 * B * nH * nW * K, dtype=np.float32)
    out = np.empty((B, 2 * nH, 2 * nW, K), dtype=np.float32)
    lib().oracle_conv_f32(tp, wp, out.ctypes.data_as(_F), tmp.ctypes.data_as(_F), C, B, nH, nW, K, int(bool(acc64)))
    return out


def kernel_transform(g):
    """g [3,3,C,K] (HWIO) -> U = G g G^T as [16,C,K] fp32."""
    g, gp = _f32(g)
    assert g.shape[:2] == (3, 3)
    C, K = int(g.shape[2]), int(g.shape[3])
    out = np.empty((16, C, K), dtype=np.float32)
    lib().oracle_kernel_transform_f32(gp, out.ctypes.data_as(_F), C, K)
    return out


def gen_prune_mask(mat, density):
    """Magnitude-pruning mask, restating ResNet-18-var/prune_script.py:22-31.

    Keeps the int(size*density) largest |w|, zeroes the rest of `mat` in place and
    returns the 0/1 mask in mat's dtype.  When int(size*density) == 0 the slice
    ``rank[:-0]`` is empty, so nothing is pruned (a quirk of the original kept here).
    """
    flat = mat.reshape(-1).copy()
    mask = np.ones_like(flat)
    rank = np.argsort(np.abs(flat), kind="stable")
    keep = int(rank.size * density)
    drop = rank[:-keep] if keep != 0 else rank[:0]
    flat[drop] = 0
    mask[drop] = 0
    np.copyto(mat, flat.reshape(mat.shape))
    return mask.reshape(mat.shape)


def _bind_grad():
    L = lib()
    if not hasattr(L, "_grad_bound"):
        L.oracle_output_transform_grad_f32.argtypes = [_F, _F] + [ctypes.c_int] * 4
        L.oracle_conv_grad_f32.argtypes = [_F, _F, _F, _F, _F, _F] + [ctypes.c_int] * 5
        L.oracle_imtrans_grad_f32.argtypes = [_F, _F, _F] + [ctypes.c_int] * 4
        for f in (L.oracle_output_transform_grad_f32, L.oracle_conv_grad_f32, L.oracle_imtrans_grad_f32):
            f.restype = None
        L._grad_bound = True
    return L


def output_transform_grad(dy):
    """dy [B,2nH,2nW,K] -> dP [16,B*nH*nW,K] (A dY A^T per tile)."""
    dy, dyp = _f32(dy)
    B, H, W, K = dy.shape
    nH, nW = H // 2, W // 2
    out = np.empty((16, B * nH * nW, K), dtype=np.float32)
    _bind_grad().oracle_output_transform_grad_f32(dyp, out.ctypes.data_as(_F), B, nH, nW, K)
    return out


def conv_grad(ti, w, dy):
    """Winograd2x2ConvGrad: (ti [16,B,nH,nW,C], w [16,C,K], dy [B,2nH,2nW,K]) -> (dti, dw)."""
    ti, tp = _f32(ti)
    w, wp = _f32(w)
    dy, dyp = _f32(dy)
    _, B, nH, nW, C = ti.shape
    K = int(w.shape[2])
    assert dy.shape == (B, 2 * nH, 2 * nW, K) and w.shape == (16, C, K)
    dti = np.empty_like(ti)
    dw = np.empty_like(w)
    tmp = np.empty(16 * B * nH * nW * K, dtype=np.float32)
    _bind_grad().oracle_conv_grad_f32(tp, wp, dyp, dti.ctypes.data_as(_F), dw.ctypes.data_as(_F),
                                     tmp.ctypes.data_as(_F), C, B, nH, nW, K)
    return dti, dw


def imtrans_grad(dt, H, W, mask_src=None):
    """Winograd2x2ImTransGrad: dt [16,B,nH,nW,C] -> dx [B,H,W,C]; mask_src (post-ReLU TI) applies the ReLU backward."""
    dt, dtp = _f32(dt)
    _, B, nH, nW, C = dt.shape
    assert nH == (H + 1) // 2 and nW == (W + 1) // 2
    mp = None
    if mask_src is not None:
        mask_src, mp = _f32(mask_src)
        assert mask_src.shape == dt.shape
    out = np.empty((B, H, W, C), dtype=np.float32)
    _bind_grad().oracle_imtrans_grad_f32(dtp, mp, out.ctypes.data_as(_F), B, H, W, C)
    return out
