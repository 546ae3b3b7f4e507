"""Writes tests/golden/fft2_24x32_known_answers.npz: known answers for the planar transform pair
(RealFFT2 / InverseRealFFT2, makani/models/common/layers.py:219-287) on a 24 x 32 grid with lmax = 13 kept latitude
frequencies (7 non-negative, 6 negative) and mmax = 12 longitude frequencies, batch 2, 3 channels.

Nothing of the oracle, of the library or of any FFT routine is used here: the expected values are the defining sums,
  forward: y[j, m] = (1 / sqrt(H W)) sum_{k,n} x[k,n] exp(-2 pi i (f_j k / H + m n / W)),   f_j = j (j < 7), H - 13 + j (j >= 7)
  inverse: z[k, m] = (1 / sqrt(H)) sum_j c[j, m] exp(+2 pi i f_j k / H)
           x[k, n] = (1 / sqrt(W)) ( Re z[k,0] + 2 sum_{0<m<W/2} Re(z[k,m] exp(2 pi i m n / W)) )      (mmax <= W/2: no Nyquist column)
evaluated with numpy.einsum in float64.

Run from the repository root:  python tests/golden/make_golden_fft2.py
"""
import os

import numpy as np

H, W, LMAX, MMAX = 24, 32, 13, 12
BATCH, CHANS = 2, 3
SEED_X, SEED_C = 30240, 30241


def main():
    lhigh = (LMAX + 1) // 2
    f = np.array([j if j < lhigh else H - LMAX + j for j in range(LMAX)])
    k, n, m = np.arange(H), np.arange(W), np.arange(MMAX)
    e_lat = np.exp(-2j * np.pi * np.outer(f, k) / H)           # [j, k]
    e_lon = np.exp(-2j * np.pi * np.outer(m, n) / W)           # [m, n]

    rng = np.random.default_rng(SEED_X)
    x = rng.standard_normal((BATCH, CHANS, H, W)).astype(np.float32)
    fwd = np.einsum("bckn,jk,mn->bcjm", x.astype(np.float64), e_lat, e_lon) / np.sqrt(H * W)

    rng = np.random.default_rng(SEED_C)
    c = (rng.standard_normal((BATCH, CHANS, LMAX, MMAX)) + 1j * rng.standard_normal((BATCH, CHANS, LMAX, MMAX))).astype(np.complex64)
    z = np.einsum("bcjm,jk->bckm", c.astype(np.complex128), np.conj(e_lat)) / np.sqrt(H)
    factor = np.full(MMAX, 2.0)
    factor[0] = 1.0
    zz = z.copy()
    zz[..., 0] = zz[..., 0].real                                 # the imaginary part of the mean column is dropped
    inv = np.einsum("bckm,m,mn->bckn", zz, factor, np.conj(e_lon)).real / np.sqrt(W)

    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fft2_24x32_known_answers.npz")
    np.savez_compressed(out, nlat=H, nlon=W, lmax=LMAX, mmax=MMAX, x=x, forward=fwd, coeffs=c, inverse=inv)
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
