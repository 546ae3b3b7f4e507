"""float64 restatement of GeometricH1Loss (makani/utils/losses.py:268-360) on the oracle transform.
TEST INFRASTRUCTURE ONLY.

Pinned by: the transform pins of oracle.sht; Parseval on a Legendre-Gauss grid (the L2 part of a band-limited field
equals its quadrature integral, tests/test_oracle_pins.py); the closed form for a single harmonic Y_l^m, whose loss is
alpha + (1 - alpha) sqrt(l (l + 1)) times its amplitude.
"""
import numpy as np

from .sht import ShtTables, sht_forward


def degree_power(c):
    """|c_l0|^2 + 2 sum_{m>0} |c_lm|^2 over the last axis (losses.py:301-303)."""
    p = c.real ** 2 + c.imag ** 2
    return p[..., :, 0] + 2.0 * p[..., :, 1:].sum(axis=-1)


class GeometricH1Loss:
    def __init__(self, img_shape, size_average=False, reduction=True, absolute=False, squared=False, alpha=0.5, grid="equiangular"):
        self.t = ShtTables(img_shape[0], img_shape[1], None, None, grid)
        self.size_average, self.reduction, self.absolute, self.squared, self.alpha = size_average, reduction, absolute, squared, alpha
        l = np.arange(self.t.lmax, dtype=np.float64)
        self.h1 = l * (l + 1)

    def norms(self, x):
        n = x.shape[0]
        p = degree_power(sht_forward(np.asarray(x, dtype=np.float64), self.t))
        l2 = p.reshape(n, -1).sum(axis=-1)
        h1 = (p * self.h1).reshape(n, -1).sum(axis=-1)
        if not self.squared:
            return self.alpha * np.sqrt(l2) + (1 - self.alpha) * np.sqrt(h1)
        return self.alpha * l2 + (1 - self.alpha) * h1

    def __call__(self, prd, tar, mask=None):
        prd, tar = np.asarray(prd, dtype=np.float64), np.asarray(tar, dtype=np.float64)
        if self.absolute:
            v = self.norms(prd - tar)
            if self.reduction:
                return v.mean() if self.size_average else v.sum()
            return v
        v = self.norms(prd - tar) / self.norms(tar)
        if mask is not None:
            v = v * np.asarray(mask, dtype=np.float64)
        if self.reduction:
            if self.size_average:
                return v.mean() if mask is None else v.sum() / np.asarray(mask, dtype=np.float64).sum()
            return v.sum()
        return v
