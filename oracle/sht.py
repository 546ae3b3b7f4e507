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
import scipy.fft

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
        self._pfwd = None

    @property
    def weights(self):
        """Analysis table [m, l, k] (Legendre * quadrature weight)."""
        if self._weights is None:
            p = legpoly(self.mmax, self.lmax, self.theta, norm=self.norm, inverse=False, csphase=self.csphase, contiguous=False)
            p *= self.quad_w[None, None, :]
            self._weights = p
        return self._weights

    @property
    def p_analysis(self):
        """Legendre table of the forward transform without the quadrature weights, [m, l, k].

        For norm="ortho" it equals the synthesis table, which is then shared (the
        721-point tables are 3 GB each in float64).
        """
        if self.norm == "ortho":
            return self.pct
        if self._pfwd is None:
            self._pfwd = legpoly(self.mmax, self.lmax, self.theta, norm=self.norm, inverse=False, csphase=self.csphase, contiguous=False)
        return self._pfwd

    @property
    def pct(self):
        """Synthesis table [m, l, k]."""
        if self._pct is None:
            self._pct = legpoly(self.mmax, self.lmax, self.theta, norm=self.norm, inverse=True, csphase=self.csphase, contiguous=False)
        return self._pct


def rfft_lon(x, mmax):
    """Longitude stage of the forward transform: 2 pi/nlon * sum_n x e^{-i m phi_n}, m < mmax."""
    # scipy.fft is numpy's FFT routine with a thread pool (the full-resolution checks transform 384 x 721 rows)
    X = 2.0 * np.pi * scipy.fft.rfft(x, axis=-1, norm="forward", workers=-1)
    return X[..., :mmax]


def irfft_lon(X, nlon):
    """Longitude stage of the inverse: unnormalised C2R inverse DFT, zero-padded to nlon//2+1."""
    return scipy.fft.irfft(X, n=nlon, axis=-1, norm="forward", workers=-1)


def legendre_analysis(X, weights):
    """c[..., l, m] = sum_k X[..., k, m] weights[m, l, k] (per-order real contraction on Re and Im).

    Evaluated as one real matrix product per order m (the einsum '...km,mlk->...lm' of the
    reference, applied to Re and Im); degrees l < m have zero weights and are skipped.
    """
    mmax, lmax, nlat = weights.shape
    lead = X.shape[:-2]
    Xf = np.ascontiguousarray(X).reshape(-1, nlat, X.shape[-1])
    rows = Xf.shape[0]
    # order-major copies, so that every per-order product reads and writes contiguous memory
    # (real and imaginary planes apart: the strided .real / .imag views of a complex array would take numpy's own loop
    # instead of the BLAS routine)
    Xr = np.ascontiguousarray(Xf.real.transpose(2, 0, 1))  # (mmax, rows, nlat)
    Xi = np.ascontiguousarray(Xf.imag.transpose(2, 0, 1))
    ct = np.zeros((mmax, rows, lmax), dtype=np.complex128)
    for m in range(min(mmax, lmax)):
        w = np.ascontiguousarray(weights[m, m:, :].T)      # (nlat, lmax-m) real
        ct[m, :, m:] = (Xr[m] @ w) + 1j * (Xi[m] @ w)
    return np.ascontiguousarray(ct.transpose(1, 2, 0)).reshape(*lead, lmax, mmax)


def legendre_synthesis(c, pct):
    """X[..., k, m] = sum_l c[..., l, m] pct[m, l, k]."""
    mmax, lmax, nlat = pct.shape
    lead = c.shape[:-2]
    cf = np.ascontiguousarray(c).reshape(-1, lmax, mmax)
    rows = cf.shape[0]
    cr = np.ascontiguousarray(cf.real.transpose(2, 0, 1))  # (mmax, rows, lmax)
    ci = np.ascontiguousarray(cf.imag.transpose(2, 0, 1))
    Xt = np.zeros((mmax, rows, nlat), dtype=np.complex128)
    for m in range(min(mmax, lmax)):
        p = np.ascontiguousarray(pct[m, m:, :])            # (lmax-m, nlat)
        Xt[m] = (np.ascontiguousarray(cr[m, :, m:]) @ p) + 1j * (np.ascontiguousarray(ci[m, :, m:]) @ p)
    return np.ascontiguousarray(Xt.transpose(1, 2, 0)).reshape(*lead, nlat, mmax)


def sht_forward(x, tables):
    x = np.asarray(x)
    assert x.shape[-2] == tables.nlat
    assert x.shape[-1] == tables.nlon
    X = rfft_lon(np.asarray(x, dtype=np.float64), tables.mmax)
    # weights[m, l, k] = P[m, l, k] * w[k]: fold w into X instead of materialising a second table
    return legendre_analysis(X * tables.quad_w[:, None], tables.p_analysis)


def sht_inverse(c, tables):
    c = np.asarray(c)
    assert c.shape[-2] == tables.lmax
    assert c.shape[-1] == tables.mmax
    X = legendre_synthesis(np.asarray(c, dtype=np.complex128), tables.pct)
    return irfft_lon(X, tables.nlon)
