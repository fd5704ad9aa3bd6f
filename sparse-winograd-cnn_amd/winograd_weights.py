"""Weight preparation for the Winograd-domain convolution (host side, numpy).

* ``kernel_transform``: U = G g G^T of a spatial [3,3,C,K] kernel into the [16,C,K]
  layout the conv op consumes.  The reference only has this in its test scripts
  (winograd2x2_cublas/winograd2x2_conv/winograd2x2_conv_test.py:8-25); it trains the
  [16,C,K] weights directly.
* ``gen_prune_mask``: magnitude pruning of Winograd-domain weights, after
  ResNet-18-var/prune_script.py:22-31.
"""
import numpy as np

_G = np.array([[1, 0, 0], [0.5, 0.5, 0.5], [0.5, -0.5, 0.5], [0, 0, 1]])


def kernel_transform(kernel):
    """kernel [3,3,C,K] (HWIO) -> [16,C,K] with position i = 4*r + s."""
    g = np.asarray(kernel)
    if g.ndim != 4 or g.shape[:2] != (3, 3):
        raise ValueError("kernel must have shape [3,3,C,K], got %s" % (g.shape,))
    u = np.einsum("ur,rsck,vs->uvck", _G, g.astype(np.float64), _G)
    return u.reshape((16,) + g.shape[2:]).astype(g.dtype if g.dtype.kind == "f" else np.float32)


def gen_prune_mask(mat, density):
    """Keep the int(mat.size*density) largest-magnitude entries of ``mat``; zero the rest in place.

    Returns the 0/1 mask in mat's dtype and shape.  As in the original, a count of zero
    prunes nothing (``rank[:-0]`` is an empty slice).
    """
    flat = mat.reshape(-1).copy()
    rank = np.argsort(np.abs(flat))
    keep = int(rank.size * density)
    mask = np.ones_like(flat)
    if keep != 0:
        drop = rank[:-keep]
        flat[drop] = 0
        mask[drop] = 0
    np.copyto(mat, flat.reshape(mat.shape))
    return mask.reshape(mat.shape)
