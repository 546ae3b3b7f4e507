"""Orthonormal associated Legendre tables (oracle, float64).

Restates torch-harmonics' table builder used by RealSHT / InverseRealSHT
(constructed by Makani at makani/models/networks/sfnonet.py:536-539): the stable
three-term recursion in degree l on fully normalised functions
  Pbar_0^0 = 1/sqrt(4 pi)
  Pbar_l^l     = sqrt((2l+1)(1+c)(1-c)/(2l)) Pbar_{l-1}^{l-1}
  Pbar_l^{l-1} = sqrt(2l+1) c Pbar_{l-1}^{l-1}
  Pbar_l^m     = c sqrt((2l-1)(2l+1)/((l-m)(l+m))) Pbar_{l-1}^m
                 - sqrt((l+m-1)(l-m-1)(2l+1)/((l-m)(l+m)(2l-3))) Pbar_{l-2}^m
with c = cos(theta); Condon-Shortley phase flips odd m.
"""
import numpy as np


def legpoly(mmax, lmax, theta, norm="ortho", inverse=False, csphase=True):
    """Table vdm[m, l, k] = Pbar_l^m(cos theta_k), zero for l < m; float64."""
    theta = np.asarray(theta, dtype=np.float64)
    nmax = max(mmax, lmax)
    c = np.cos(theta)
    vdm = np.zeros((nmax, nmax, len(theta)), dtype=np.float64)
    norm_factor = 1.0 if norm == "ortho" else np.sqrt(4.0 * np.pi)
    norm_factor = 1.0 / norm_factor if inverse else norm_factor
    vdm[0, 0, :] = norm_factor / np.sqrt(4.0 * np.pi)
    for l in range(1, nmax):
        vdm[l - 1, l, :] = np.sqrt(2 * l + 1) * c * vdm[l - 1, l - 1, :]
        vdm[l, l, :] = np.sqrt((2 * l + 1) * (1 + c) * (1 - c) / 2 / l) * vdm[l - 1, l - 1, :]
    for l in range(2, nmax):
        m = np.arange(0, l - 1, dtype=np.float64)
        a = np.sqrt((2 * l - 1) / (l - m) * (2 * l + 1) / (l + m))
        b = np.sqrt((l + m - 1) / (l - m) * (2 * l + 1) / (2 * l - 3) * (l - m - 1) / (l + m))
        vdm[: l - 1, l, :] = c[None, :] * a[:, None] * vdm[: l - 1, l - 1, :] - b[:, None] * vdm[: l - 1, l - 2, :]
    if norm == "schmidt":
        fac = np.sqrt(2.0 * np.arange(nmax) + 1.0)
        vdm = vdm * fac[None, :, None] if inverse else vdm / fac[None, :, None]
    vdm = vdm[:mmax, :lmax].copy()
    if csphase:
        vdm[1::2] *= -1.0
    return vdm
