"""Per-degree complex channel contraction and the SpectralConv op order (oracle).

dhconv restates makani/models/common/contractions.py:130-136
(einsum "bixy,iox->boxy" on complex tensors); spectral_conv restates the
orchestration of makani/models/common/spectral_convolution.py:124-148 for the
non-separable dhconv operator without bias.
"""
import numpy as np

from .sht import sht_forward, sht_inverse
from .fft2 import Fft2Modes, fft2_forward, fft2_inverse


def transform_forward(x, t):
    """The forward transform `t` describes: spherical tables or the planar pair's mode bookkeeping."""
    return fft2_forward(x, t) if isinstance(t, Fft2Modes) else sht_forward(x, t)


def transform_inverse(c, t):
    return fft2_inverse(c, t) if isinstance(t, Fft2Modes) else sht_inverse(c, t)


def dhconv(x, w):
    """y[b,o,l,m] = sum_i x[b,i,l,m] * w[i,o,l]."""
    x = np.asarray(x)
    w = np.asarray(w)
    assert x.shape[1] == w.shape[0] and x.shape[2] == w.shape[2]
    if x.shape[1] * w.shape[1] < 4096:
        return np.einsum("bixy,iox->boxy", x, w, optimize=True)
    # the same sum as one matrix product per (b, l): [O, I] @ [I, M]; einsum's own loop takes minutes at 384 channels
    # (contiguous operands: strided ones would take numpy's own loop instead of the BLAS routine)
    y = np.matmul(np.ascontiguousarray(w.transpose(2, 1, 0))[None], np.ascontiguousarray(x.transpose(0, 2, 1, 3)))      # [B, L, O, M]
    return np.ascontiguousarray(y.transpose(0, 2, 1, 3))


def diagonal(x, w):
    """y[b,o,l,m] = sum_i x[b,i,l,m] * w[i,o,l,m] (makani/models/common/contractions.py:121-127)."""
    x = np.asarray(x)
    w = np.asarray(w)
    assert x.shape[1] == w.shape[0] and x.shape[2:] == w.shape[2:]
    return np.einsum("bixy,ioxy->boxy", x, w, optimize=True)


def spectral_conv(x, w, fwd_tables, inv_tables, bias=None):
    """Returns (y, residual) as SpectralConv.forward does, all in float64.

    residual is the input itself unless the forward and inverse grids differ
    (spectral_convolution.py:62-64), in which case it is the inverse transform of the
    unfiltered coefficients (spectral_convolution.py:132-134).
    """
    scale_residual = (
        fwd_tables.nlat != inv_tables.nlat or fwd_tables.nlon != inv_tables.nlon or fwd_tables.grid != inv_tables.grid
    )
    residual = np.asarray(x, dtype=np.float64)
    contract = diagonal if np.asarray(w).ndim == 4 else dhconv
    c = transform_forward(x, fwd_tables)
    if scale_residual:
        residual = transform_inverse(c, inv_tables)
    y = contract(c, np.asarray(w, dtype=np.complex128))
    y = transform_inverse(y, inv_tables)
    if bias is not None:
        y = y + bias
    return y, residual
