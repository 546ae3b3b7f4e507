"""Planar real FFT pair (oracle; numpy, float64 by default).  TEST INFRASTRUCTURE ONLY: the product never imports it.

Restates RealFFT2.forward and InverseRealFFT2.forward of makani/models/common/layers.py:219-287, the
planar counterparts of the spherical transform pair (selected by spectral_transform="fft",
makani/models/networks/sfnonet.py:542-556):

  forward : y = rfft2(x, s=(nlat, nlon), norm="ortho");  keep the first mmax longitude frequencies and, of the
            latitude frequencies, the first ceil(lmax/2) and the last floor(lmax/2), concatenated in that order
            (layers.py:242-248)
  inverse : take x[..., :mmax]; put rows [:ceil(lmax/2)] first, nlat - lmax zero rows, then the last
            floor(lmax/2) rows (layers.py:274-283); irfft2(s=(nlat, nlon), norm="ortho")

With lmax = 1 the reference's `-0:` slice would select every row; this restatement selects none, so only
lmax >= 2 restates the reference.

Pins: numpy.fft is the library statement of the same transform the reference calls through torch.fft;
tests/test_oracle_pins.py checks the pair against a brute-force double sum over the grid on a small case,
Parseval's identity for the untruncated transform, and the round trip of band-limited fields.
"""
import math

import numpy as np


class Fft2Modes:
    """Mode bookkeeping of one transform size (layers.py:225-240, 259-274)."""

    def __init__(self, nlat, nlon, lmax=None, mmax=None):
        self.nlat, self.nlon, self.grid = nlat, nlon, "planar"
        self.lmax = min(lmax or nlat, nlat)
        self.mmax = min(mmax or nlon // 2 + 1, nlon // 2 + 1)
        self.truncate = not (self.lmax == nlat and self.mmax == nlon // 2 + 1)
        self.lmax_high = math.ceil(self.lmax / 2)
        self.lmax_low = math.floor(self.lmax / 2)


def fft2_forward(x, t):
    """x [..., nlat, nlon] real -> [..., lmax, mmax] complex (layers.py:242-250)."""
    x = np.asarray(x)
    assert x.shape[-2:] == (t.nlat, t.nlon)
    y = np.fft.rfft2(x, s=(t.nlat, t.nlon), axes=(-2, -1), norm="ortho")
    if t.truncate:
        hi = y[..., : t.lmax_high, : t.mmax]
        lo = y[..., y.shape[-2] - t.lmax_low :, : t.mmax] if t.lmax_low > 0 else y[..., :0, : t.mmax]
        y = np.concatenate((hi, lo), axis=-2)
    return y


def fft2_inverse(c, t):
    """c [..., lmax, mmax] complex -> [..., nlat, nlon] real (layers.py:276-287)."""
    c = np.asarray(c)
    assert c.shape[-2] == t.lmax and c.shape[-1] >= t.mmax
    xt = c[..., : t.mmax]
    if t.truncate:
        hi = xt[..., : t.lmax_high, :]
        lo = xt[..., xt.shape[-2] - t.lmax_low :, :] if t.lmax_low > 0 else xt[..., :0, :]
        pad = np.zeros((*xt.shape[:-2], t.nlat - t.lmax, xt.shape[-1]), dtype=xt.dtype)
        xt = np.concatenate((hi, pad, lo), axis=-2)
    # irfft2 = inverse complex FFT along latitude, then complex-to-real along longitude; numpy zero-fills
    # the longitude frequencies from mmax to nlon/2 as torch.fft.irfft2 does
    return np.fft.irfft2(xt, s=(t.nlat, t.nlon), axes=(-2, -1), norm="ortho")
