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


def legpoly(mmax, lmax, theta, norm="ortho", inverse=False, csphase=True, contiguous=True):
    """Table vdm[m, l, k] = Pbar_l^m(cos theta_k), zero for l < m; float64."""
    theta = np.asarray(theta, dtype=np.float64)
    nmax = max(mmax, lmax)
    c = np.cos(theta)
    # stored degree-major (v[l, m, k]) so that each recursion step touches contiguous memory;
    # the returned array is the [m, l, k] view of it
    v = np.zeros((nmax, nmax, len(theta)), dtype=np.float64)
    norm_factor = 1.0 if norm == "ortho" else np.sqrt(4.0 * np.pi)
    norm_factor = 1.0 / norm_factor if inverse else norm_factor
    v[0, 0, :] = norm_factor / np.sqrt(4.0 * np.pi)
    for l in range(1, nmax):
        v[l, l - 1, :] = np.sqrt(2 * l + 1) * c * v[l - 1, l - 1, :]
        v[l, l, :] = np.sqrt((2 * l + 1) * (1 + c) * (1 - c) / 2 / l) * v[l - 1, l - 1, :]
    for l in range(2, nmax):
        m = np.arange(0, l - 1, dtype=np.float64)
        a = np.sqrt((2 * l - 1) / (l - m) * (2 * l + 1) / (l + m))
        b = np.sqrt((l + m - 1) / (l - m) * (2 * l + 1) / (2 * l - 3) * (l - m - 1) / (l + m))
        # v[l] = c a v[l-1] - b v[l-2], evaluated in place (no full-size temporaries)
        cur = v[l, : l - 1, :]
        np.multiply(v[l - 1, : l - 1, :], c[None, :], out=cur)
        cur *= a[:, None]
        tmp = v[l - 2, : l - 1, :] * b[:, None]
        cur -= tmp
    if norm == "schmidt":
        fac = np.sqrt(2.0 * np.arange(nmax) + 1.0)
        v = v * fac[:, None, None] if inverse else v / fac[:, None, None]
    v = v[:lmax, :mmax]
    if csphase:
        v[:, 1::2] *= -1.0
    return np.ascontiguousarray(v.transpose(1, 0, 2)) if contiguous else v.transpose(1, 0, 2)
