"""Real spherical harmonic transform pair (oracle; numpy, float64 by default).

Restates the forward/inverse of torch-harmonics' RealSHT / InverseRealSHT as Makani
uses them (makani/models/common/spectral_convolution.py:131,133,141;
makani/models/networks/sfnonet.py:596,598,616):

  forward : X = 2 pi * rfft(x, axis=-1, norm="forward")[..., :mmax]
            c[..., l, m] = sum_k X[..., k, m] * weights[m, l, k],
            weights[m, l, k] = Pbar_l^m(cos theta_k) * w_k
  inverse : X[..., k, m] = sum_l c[..., l, m] * pct[m, l, k]
            x = irfft(X, n=nlon, axis=-1, norm="forward")   (C2R: Im of the m=0 and
            Nyquist bins is dropped, bins >= mmax are zero)
"""
import numpy as np

from .quadrature import grid_nodes, default_lmax
from .legendre import legpoly


class ShtTables:
    """Grid, quadrature weights and both Legendre tables for one transform size."""

    def __init__(self, nlat, nlon, lmax=None, mmax=None, grid="lobatto", norm="ortho", csphase=True):
        self.nlat, self.nlon, self.grid, self.norm, self.csphase = nlat, nlon, grid, norm, csphase
        self.theta, self.quad_w = grid_nodes(nlat, grid)
        self.lmax = lmax or default_lmax(nlat, grid)
        self.mmax = mmax or nlon // 2 + 1
        self._weights = None
        self._pct = None

    @property
    def weights(self):
        """Analysis table [m, l, k] (Legendre * quadrature weight)."""
        if self._weights is None:
            p = legpoly(self.mmax, self.lmax, self.theta, norm=self.norm, inverse=False, csphase=self.csphase)
            self._weights = p * self.quad_w[None, None, :]
        return self._weights

    @property
    def pct(self):
        """Synthesis table [m, l, k]."""
        if self._pct is None:
            self._pct = legpoly(self.mmax, self.lmax, self.theta, norm=self.norm, inverse=True, csphase=self.csphase)
        return self._pct


def rfft_lon(x, mmax):
    """Longitude stage of the forward transform: 2 pi/nlon * sum_n x e^{-i m phi_n}, m < mmax."""
    X = 2.0 * np.pi * np.fft.rfft(x, axis=-1, norm="forward")
    return X[..., :mmax]


def irfft_lon(X, nlon):
    """Longitude stage of the inverse: unnormalised C2R inverse DFT, zero-padded to nlon//2+1."""
    return np.fft.irfft(X, n=nlon, axis=-1, norm="forward")


def legendre_analysis(X, weights):
    """c[..., l, m] = sum_k X[..., k, m] weights[m, l, k] (per-order real contraction on Re and Im)."""
    # matmul over m: (m, l, k) @ (..., m, k, 1)
    Xm = np.moveaxis(X, -1, -2)                                # (..., m, k)
    c = np.einsum("mlk,...mk->...lm", weights, Xm, optimize=True)
    return c


def legendre_synthesis(c, pct):
    """X[..., k, m] = sum_l c[..., l, m] pct[m, l, k]."""
    return np.einsum("mlk,...lm->...km", pct, c, optimize=True)


def sht_forward(x, tables):
    x = np.asarray(x)
    assert x.shape[-2] == tables.nlat
    assert x.shape[-1] == tables.nlon
    X = rfft_lon(x.astype(np.float64), tables.mmax)
    return legendre_analysis(X, tables.weights)


def sht_inverse(c, tables):
    c = np.asarray(c)
    assert c.shape[-2] == tables.lmax
    assert c.shape[-1] == tables.mmax
    X = legendre_synthesis(c.astype(np.complex128), tables.pct)
    return irfft_lon(X, tables.nlon)
