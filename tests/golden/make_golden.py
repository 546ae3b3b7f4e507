"""Writes tests/golden/sht_32x64_known_answers.npz: known answers for the smallest benchmark configuration
(equiangular 32 x 64 grid, lmax = 32, mmax = 33, batch 2, 4 channels, N(0,1) inputs from a seed).

Nothing of the oracle or of the library is used here.  The expected values come from the definition of the
transform pair evaluated by brute force with library routines only:
  * spherical harmonics from scipy.special.sph_harm_y (orthonormal, Condon-Shortley phase),
  * Clenshaw-Curtis weights as the solution of the moment equations sum_k w_k P_j(x_k) = 2 delta_j0
    (numpy.polynomial.legendre), not from a closed form,
  * forward: c[l,m] = sum_{k,n} x[k,n] w_k (2 pi / nlon) conj(Y_l^m(theta_k, phi_n)),
  * inverse: x[k,n] = sum_l ( Re c[l,0] Y_l^0 + 2 sum_{0<m<nlon/2} Re(c[l,m] Y_l^m) + Re c[l,nlon/2] Pbar_l^{nlon/2} (-1)^n ),
    the real-signal (C2R) convention of the reference's inverse transform.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
from numpy.polynomial import legendre as npleg
from scipy.special import sph_harm_y

NLAT, NLON, LMAX, MMAX = 32, 64, 32, 33
BATCH, CHANS = 2, 4
SEED_X, SEED_C = 20240, 20241


def main():
    theta = np.arange(NLAT) * np.pi / (NLAT - 1)             # colatitudes, north pole first
    phi = 2.0 * np.pi * np.arange(NLON) / NLON
    x_nodes = np.cos(theta)
    V = npleg.legvander(x_nodes, NLAT - 1).T                  # V[j, k] = P_j(x_k)
    rhs = np.zeros(NLAT)
    rhs[0] = 2.0
    w = np.linalg.solve(V, rhs)
    assert abs(w.sum() - 2.0) < 1e-12 and np.all(w > 0)

    # Y[l, m, k, n]
    l = np.arange(LMAX)[:, None, None, None]
    m = np.arange(MMAX)[None, :, None, None]
    Y = sph_harm_y(l, m, theta[None, None, :, None], phi[None, None, None, :])
    Y = np.where(m <= l, Y, 0.0)

    rng = np.random.default_rng(SEED_X)
    x = rng.standard_normal((BATCH, CHANS, NLAT, NLON)).astype(np.float32)
    fwd = np.einsum("bckn,k,lmkn->bclm", x.astype(np.float64), w, np.conj(Y)) * (2.0 * np.pi / NLON)

    rng = np.random.default_rng(SEED_C)
    c = (rng.standard_normal((BATCH, CHANS, LMAX, MMAX)) + 1j * rng.standard_normal((BATCH, CHANS, LMAX, MMAX))).astype(np.complex64)
    c = c * (np.arange(MMAX)[None, :] <= np.arange(LMAX)[:, None])
    c64 = c.astype(np.complex128)
    factor = np.full(MMAX, 2.0)
    factor[0] = 1.0
    cc = c64.copy()
    cc[..., 0] = cc[..., 0].real                               # Im of the mean order is ignored
    inv = np.einsum("bclm,m,lmkn->bckn", cc[..., : NLON // 2], factor[: NLON // 2], Y[:, : NLON // 2]).real
    if MMAX > NLON // 2:                                       # Nyquist order: real part only, alternating sign
        pn = Y[:, NLON // 2, :, 0].real                        # Pbar_l^{N/2}(cos theta_k) (phi = 0)
        inv = inv + np.einsum("bcl,lk,n->bckn", c64[..., NLON // 2].real, pn, (-1.0) ** np.arange(NLON))

    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sht_32x64_known_answers.npz")
    np.savez_compressed(out, nlat=NLAT, nlon=NLON, lmax=LMAX, mmax=MMAX, weights=w, x=x, forward=fwd, coeffs=c, inverse=inv)
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
