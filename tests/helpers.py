"""Float64 matrix-form restatements and error metrics shared by the tests.

These are deliberately written from the textbook F(2x2,3x3) matrices, not from the
explicit sums the oracle and the kernels use, so that a wrong sign, index or
transposed operand in either shows up as a mismatch.
"""
import numpy as np

BT = np.array([[1, 0, -1, 0], [0, 1, 1, 0], [0, -1, 1, 0], [0, 1, 0, -1]], dtype=np.float64)
AT = np.array([[1, 1, 1, 0], [0, 1, -1, -1]], dtype=np.float64)
G = np.array([[1, 0, 0], [0.5, 0.5, 0.5], [0.5, -0.5, 0.5], [0, 0, 1]], dtype=np.float64)


def tiles(n):
    return (n + 1) // 2


def patches(x):
    """x [B,H,W,C] -> d [B,nH,nW,4,4,C]: 4x4 windows at stride 2, pad 1, zero filled."""
    B, H, W, C = x.shape
    nH, nW = tiles(H), tiles(W)
    xp = np.zeros((B, 2 * nH + 2, 2 * nW + 2, C), dtype=np.float64)
    xp[:, 1:H + 1, 1:W + 1, :] = x
    d = np.empty((B, nH, nW, 4, 4, C), dtype=np.float64)
    for r in range(4):
        for s in range(4):
            d[:, :, :, r, s, :] = xp[:, r:r + 2 * nH:2, s:s + 2 * nW:2, :]
    return d


def imtrans_matrix(x, relu=False):
    """T = B^T d B in float64 -> [16,B,nH,nW,C]."""
    d = patches(np.asarray(x, dtype=np.float64))
    t = np.einsum("ur,bhwrsc,vs->uvbhwc", BT, d, BT)
    t = t.reshape((16,) + t.shape[2:])
    return np.maximum(t, 0) if relu else t


def output_matrix(p, B, nH, nW):
    """Y = A^T p A in float64: p [16,B*nH*nW,K] -> [B,2nH,2nW,K]."""
    K = p.shape[-1]
    p = np.asarray(p, dtype=np.float64).reshape(4, 4, B, nH, nW, K)
    y = np.einsum("ur,rsbhwk,vs->bhuwvk", AT, p, AT)
    return y.reshape(B, 2 * nH, 2 * nW, K)


def kernel_matrix(g):
    """U = G g G^T in float64: g [3,3,C,K] -> [16,C,K]."""
    u = np.einsum("ur,rsck,vs->uvck", G, np.asarray(g, dtype=np.float64), G)
    return u.reshape((16,) + u.shape[2:])


def direct_conv(x, g):
    """Plain 3x3 cross-correlation, stride 1, pad 1, NHWC x HWIO, float64 loop nest."""
    x = np.asarray(x, dtype=np.float64)
    g = np.asarray(g, dtype=np.float64)
    B, H, W, C = x.shape
    K = g.shape[3]
    xp = np.zeros((B, H + 2, W + 2, C))
    xp[:, 1:-1, 1:-1, :] = x
    y = np.zeros((B, H, W, K))
    for r in range(3):
        for s in range(3):
            y += np.einsum("bhwc,ck->bhwk", xp[:, r:r + H, s:s + W, :], g[r, s])
    return y


def rel_max(a, b):
    """max|a-b| / max|b|."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    den = np.max(np.abs(b))
    return float(np.max(np.abs(a - b)) / (den if den > 0 else 1.0))


def rel_l1(a, b):
    """The reference tests' printed figure: sum|a-b| / (sum|a| + sum|b|)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    den = np.sum(np.abs(a)) + np.sum(np.abs(b))
    return float(np.sum(np.abs(a - b)) / (den if den > 0 else 1.0))


def expected_stored_launch(M, C, K, cus, l2_bytes, workspace=True):
    """The launch form swc_winograd2x2_conv_bf16in_ws (swc_winograd2x2_conv_bf16in with workspace=False) picks for
    tile rows M, channels C, filters K on a device with `cus` compute units and L2s of `l2_bytes` (the rules of
    its launcher, restated), as a one-element tuple."""
    ceil = lambda a, b: -(-a // b)
    if C in (64, 128, 256, 512) and K % 64 == 0 and ceil(M, 128) * (K // 64) * 4 >= 3 * cus:
        return ("stored-tall",)
    if workspace and C in (256, 512) and K % 64 == 0 and 4 * ceil(M, 128) * (K // 64) * (512 // C) <= cus:
        return ("stored-spread",)
    if ceil(M, 32) * ceil(K, 64) <= cus and C >= 256:
        return ("stored-split4",)
    if ceil(M, 64) * ceil(K, 64) <= cus:
        return ("stored-split",)
    return ("stored-ring4",) if 16 * C * K * 2 >= l2_bytes else ("stored-ring3",)
