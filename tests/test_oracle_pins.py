"""Pins the CPU oracle to facts it does not itself define (no GPU needed).

The reference tree holds no golden vectors for the transform values (its SHT tests are
shape checks, tests/test_models.py:45-69) and one numeric check at the quadrature
boundary (weights sum to 2, tests/test_metrics.py:37-45).  Everything else is pinned by
independent mathematics: scipy's spherical harmonics, closed forms, polynomial
exactness, brute-force DFTs and brute-force loops, chosen so that a dropped term, a wrong
sign, index or transposed operand fails at least one check.
"""
import numpy as np
import pytest
from scipy.special import sph_harm_y

from oracle.quadrature import legendre_gauss_weights, clenshaw_curtiss_weights, lobatto_weights, grid_nodes
from oracle.legendre import legpoly
from oracle.sht import ShtTables, sht_forward, sht_inverse, rfft_lon, irfft_lon
from oracle.dhconv import dhconv, spectral_conv


# ---- quadrature ------------------------------------------------------------------------------

@pytest.mark.parametrize("n", [2, 3, 20, 101, 721])
@pytest.mark.parametrize("rule", [legendre_gauss_weights, clenshaw_curtiss_weights, lobatto_weights])
def test_weights_integrate_one(rule, n):
    # the reference's own check (tests/test_metrics.py:37-45): sum of weights = 2 to rtol 1e-5; here to 1e-12
    x, w = rule(n)
    assert x.shape == (n,) and w.shape == (n,)
    assert np.all(np.diff(x) > 0)
    assert abs(w.sum() - 2.0) < 1e-12
    assert np.allclose(w, w[::-1], atol=1e-13) and np.allclose(x, -x[::-1], atol=1e-13)


@pytest.mark.parametrize("n", [5, 12, 33])
def test_polynomial_exactness(n):
    # Gauss: degree 2n-1, Lobatto: 2n-3, Clenshaw-Curtis: n-1; and NOT one even degree beyond (Gauss/Lobatto)
    def integral(p):
        return 0.0 if p % 2 else 2.0 / (p + 1)

    for rule, deg in ((legendre_gauss_weights, 2 * n - 1), (lobatto_weights, 2 * n - 3), (clenshaw_curtiss_weights, n - 1)):
        x, w = rule(n)
        for p in range(deg + 1):
            assert abs(np.sum(w * x**p) - integral(p)) < 1e-12, (rule.__name__, p)
    if n <= 12:          # one even degree further the rule is no longer exact (visible only for small n)
        x, w = legendre_gauss_weights(n)
        assert abs(np.sum(w * x ** (2 * n)) - integral(2 * n)) > 1e-9


def test_clenshaw_curtis_is_the_interpolatory_rule():
    # brute force: solve the Vandermonde moment equations on the nodes cos(k pi/(n-1))
    n = 9
    x, w = clenshaw_curtiss_weights(n)
    assert np.allclose(x, np.cos(np.linspace(np.pi, 0, n)))
    V = np.vander(x, n, increasing=True).T
    mom = np.array([0.0 if p % 2 else 2.0 / (p + 1) for p in range(n)])
    assert np.allclose(np.linalg.solve(V, mom), w, atol=1e-12)


def test_lobatto_nodes_are_roots_of_dP():
    n = 8
    x, w = lobatto_weights(n)
    assert x[0] == pytest.approx(-1) and x[-1] == pytest.approx(1)
    dP = np.polynomial.legendre.Legendre.basis(n - 1).deriv()
    assert np.allclose(dP(x[1:-1]), 0, atol=1e-10)


def test_grid_nodes_north_first():
    for grid in ("legendre-gauss", "equiangular", "lobatto"):
        theta, w = grid_nodes(16, grid)
        assert np.all(np.diff(theta) > 0) and theta[0] < np.pi / 2
    theta, _ = grid_nodes(17, "equiangular")
    assert np.allclose(theta, np.arange(17) * np.pi / 16)


# ---- Legendre table --------------------------------------------------------------------------

@pytest.mark.parametrize("grid,nlat", [("legendre-gauss", 24), ("equiangular", 33)])
def test_table_matches_scipy(grid, nlat):
    theta, _ = grid_nodes(nlat, grid)
    mmax, lmax = 19, 22
    tab = legpoly(mmax, lmax, theta)
    assert tab.shape == (mmax, lmax, nlat)
    for m in range(mmax):
        for l in range(lmax):
            ref = sph_harm_y(l, m, theta, 0.0).real if l >= m else np.zeros(nlat)
            assert np.allclose(tab[m, l], ref, atol=2e-14), (m, l)


def test_table_closed_forms_and_phase():
    theta = np.linspace(0.1, 3.0, 7)
    c, s = np.cos(theta), np.sin(theta)
    t = legpoly(3, 3, theta)
    assert np.allclose(t[0, 0], 1 / np.sqrt(4 * np.pi))
    assert np.allclose(t[0, 1], np.sqrt(3 / (4 * np.pi)) * c)
    assert np.allclose(t[1, 1], -np.sqrt(3 / (8 * np.pi)) * s)                # Condon-Shortley sign
    assert np.allclose(t[0, 2], np.sqrt(5 / (16 * np.pi)) * (3 * c * c - 1))
    assert np.allclose(t[1, 2], -np.sqrt(15 / (8 * np.pi)) * s * c)
    assert np.allclose(t[2, 2], np.sqrt(15 / (32 * np.pi)) * s * s)
    assert np.all(t[2, :2] == 0) and np.all(t[1, 0] == 0)
    t_nocs = legpoly(3, 3, theta, csphase=False)
    assert np.allclose(t_nocs[1], -t[1]) and np.allclose(t_nocs[0], t[0]) and np.allclose(t_nocs[2], t[2])


def test_table_norms():
    theta, _ = grid_nodes(12, "legendre-gauss")
    o = legpoly(6, 8, theta)
    assert np.allclose(legpoly(6, 8, theta, norm="four-pi"), o * np.sqrt(4 * np.pi))
    assert np.allclose(legpoly(6, 8, theta, norm="four-pi", inverse=True), o / np.sqrt(4 * np.pi))
    l = np.arange(8)
    assert np.allclose(legpoly(6, 8, theta, norm="schmidt"), o * np.sqrt(4 * np.pi) / np.sqrt(2 * l + 1)[None, :, None])
    assert np.allclose(legpoly(6, 8, theta, norm="schmidt", inverse=True), o / np.sqrt(4 * np.pi) * np.sqrt(2 * l + 1)[None, :, None])


def test_table_orthonormal_and_symmetric_at_scale():
    nlat = 240
    theta, w = grid_nodes(nlat, "legendre-gauss")
    tab = legpoly(8, 240, theta)
    for m in (0, 1, 7):
        G = (tab[m, m:] * w) @ tab[m, m:].T * 2 * np.pi
        assert np.allclose(G, np.eye(240 - m), atol=1e-11)
    l = np.arange(240)
    for m in (0, 3):
        sign = (-1.0) ** (l + m)
        assert np.allclose(tab[m][:, ::-1], tab[m] * sign[:, None], atol=1e-12)


def test_cropping_consistency():
    theta, _ = grid_nodes(20, "equiangular")
    big = legpoly(21, 20, theta)
    small = legpoly(7, 12, theta)
    assert np.array_equal(big[:7, :12], small)


# ---- longitude DFT -----------------------------------------------------------------------------

@pytest.mark.parametrize("nlon,mmax", [(8, 5), (9, 5), (12, 4), (30, 16)])
def test_rfft_is_scaled_dft(nlon, mmax):
    rng = np.random.default_rng(nlon)
    x = rng.standard_normal((3, nlon))
    n = np.arange(nlon)
    brute = np.stack([(2 * np.pi / nlon) * (x * np.exp(-2j * np.pi * m * n / nlon)).sum(-1) for m in range(mmax)], -1)
    assert np.allclose(rfft_lon(x, mmax), brute, atol=1e-13)


@pytest.mark.parametrize("nlon,mmax", [(8, 5), (9, 5), (12, 4), (30, 16)])
def test_irfft_is_c2r_sum(nlon, mmax):
    rng = np.random.default_rng(nlon + 1)
    X = rng.standard_normal((2, mmax)) + 1j * rng.standard_normal((2, mmax))     # Im(X_0), Im(Nyquist) set on purpose
    n = np.arange(nlon)
    brute = np.repeat(X[:, :1].real, nlon, axis=1)
    for m in range(1, mmax):
        if 2 * m == nlon:
            brute = brute + X[:, m : m + 1].real * (-1.0) ** n
        else:
            brute = brute + 2 * (X[:, m : m + 1] * np.exp(2j * np.pi * m * n / nlon)).real
    assert np.allclose(irfft_lon(X, nlon), brute, atol=1e-13)


# ---- transform pair ------------------------------------------------------------------------------

def test_constant_field():
    for grid, nlat in (("equiangular", 33), ("legendre-gauss", 32), ("lobatto", 33)):
        t = ShtTables(nlat, 64, grid=grid)
        c = sht_forward(np.ones((nlat, 64)), t)
        assert abs(c[0, 0] - np.sqrt(4 * np.pi)) < 1e-13
        c[0, 0] = 0
        assert np.abs(c).max() < 1e-13


def test_default_sizes():
    assert ShtTables(32, 64, grid="legendre-gauss").lmax == 32
    assert ShtTables(32, 64, grid="equiangular").lmax == 32
    assert ShtTables(32, 64, grid="lobatto").lmax == 31
    assert ShtTables(32, 64, grid="lobatto").mmax == 33


@pytest.mark.parametrize("grid,nlat,nlon,lmax", [("legendre-gauss", 24, 48, 24), ("equiangular", 33, 64, 16), ("lobatto", 25, 48, 23)])
def test_one_hot_harmonics(grid, nlat, nlon, lmax):
    """Analysis of a sampled real harmonic Re/Im(Y_l^m) gives a single coefficient."""
    t = ShtTables(nlat, nlon, lmax, lmax, grid)
    phi = 2 * np.pi * np.arange(nlon) / nlon
    for l, m in ((0, 0), (3, 0), (5, 2), (lmax - 1, lmax - 1), (lmax - 1, 1), (7, 7)):
        Y = sph_harm_y(l, m, t.theta[:, None], phi[None, :])
        for part, val in ((Y.real, 1.0), (Y.imag, -1j)):
            if m == 0 and val != 1.0:
                continue
            c = sht_forward(2 * part if m > 0 else part, t)
            expect = np.zeros_like(c)
            expect[l, m] = val
            assert np.allclose(c, expect, atol=1e-12), (l, m)


@pytest.mark.parametrize("grid,nlat,lmax", [("legendre-gauss", 32, 32), ("equiangular", 33, 16), ("lobatto", 33, 31)])
def test_roundtrip_bandlimited(grid, nlat, lmax):
    nlon = 64
    t = ShtTables(nlat, nlon, lmax, lmax + 1, grid)
    rng = np.random.default_rng(5)
    c = rng.standard_normal((2, lmax, lmax + 1)) + 1j * rng.standard_normal((2, lmax, lmax + 1))
    c[..., 0] = c[..., 0].real
    c *= np.tril(np.ones((lmax, lmax + 1)))
    x = sht_inverse(c, t)
    assert np.allclose(sht_forward(x, t), c, atol=1e-11)
    # Parseval on the sphere (orthonormal harmonics): integral of x^2 = sum_l (|c_l0|^2 + 2 sum_{m>0} |c_lm|^2)
    if grid == "legendre-gauss":
        t2 = ShtTables(2 * nlat, 2 * nlon, lmax, lmax + 1, grid)
        x2 = sht_inverse(c, t2)
        integral = (x2**2 * t2.quad_w[None, :, None]).sum(axis=(1, 2)) * (2 * np.pi / (2 * nlon))
        power = (np.abs(c[..., 0]) ** 2).sum(-1) + 2 * (np.abs(c[..., 1:]) ** 2).sum((-1, -2))
        assert np.allclose(integral, power, rtol=1e-11)


def test_inverse_ignores_imag_of_mean_and_nyquist():
    t = ShtTables(16, 32, 16, 17, "legendre-gauss")
    rng = np.random.default_rng(6)
    c = rng.standard_normal((16, 17)) + 1j * rng.standard_normal((16, 17))
    c2 = c.copy()
    c2[:, 0] = c[:, 0].real
    c2[:, 16] = c[:, 16].real
    assert np.allclose(sht_inverse(c, t), sht_inverse(c2, t), atol=1e-13)


def test_forward_brute_force_tiny():
    nlat, nlon, lmax, mmax = 5, 8, 4, 4
    t = ShtTables(nlat, nlon, lmax, mmax, "legendre-gauss")
    rng = np.random.default_rng(7)
    x = rng.standard_normal((nlat, nlon))
    phi = 2 * np.pi * np.arange(nlon) / nlon
    brute = np.zeros((lmax, mmax), dtype=complex)
    for l in range(lmax):
        for m in range(min(l, mmax - 1) + 1):
            Y = sph_harm_y(l, m, t.theta[:, None], phi[None, :])
            brute[l, m] = (x * np.conj(Y) * t.quad_w[:, None]).sum() * (2 * np.pi / nlon)
    assert np.allclose(sht_forward(x, t), brute, atol=1e-13)


# ---- dhconv and SpectralConv order -------------------------------------------------------------------

def test_dhconv_brute_force():
    rng = np.random.default_rng(8)
    B, I, O, L, M = 2, 3, 4, 5, 6
    x = rng.standard_normal((B, I, L, M)) + 1j * rng.standard_normal((B, I, L, M))
    w = rng.standard_normal((I, O, L)) + 1j * rng.standard_normal((I, O, L))
    y = np.zeros((B, O, L, M), dtype=complex)
    for b in range(B):
        for o in range(O):
            for l in range(L):
                for m in range(M):
                    for i in range(I):
                        y[b, o, l, m] += x[b, i, l, m] * w[i, o, l]
    assert np.allclose(dhconv(x, w), y, atol=1e-13)
    eye = np.zeros((I, I, L), dtype=complex)
    eye[np.arange(I), np.arange(I), :] = 1
    assert np.allclose(dhconv(x, eye), x)
    assert np.allclose(dhconv(x[:, :, :1], w[:, :, :1])[:, :, 0], np.einsum("bim,io->bom", x[:, :, 0], w[:, :, 0]))


def test_dhconv_many_channels_brute_force():
    """From 64 x 64 channels on the oracle evaluates the sum as matrix products; same brute-force loop pins that branch
    (distinct extents everywhere, so a transposed operand cannot pass)."""
    rng = np.random.default_rng(11)
    B, I, O, L, M = 2, 70, 64, 2, 3
    x = rng.standard_normal((B, I, L, M)) + 1j * rng.standard_normal((B, I, L, M))
    w = rng.standard_normal((I, O, L)) + 1j * rng.standard_normal((I, O, L))
    y = np.zeros((B, O, L, M), dtype=complex)
    for b in range(B):
        for o in range(O):
            for l in range(L):
                for m in range(M):
                    y[b, o, l, m] = sum(x[b, i, l, m] * w[i, o, l] for i in range(I))
    got = dhconv(x, w)
    assert got.shape == y.shape and np.allclose(got, y, atol=1e-12)


def test_diagonal_brute_force():
    from oracle.dhconv import diagonal

    rng = np.random.default_rng(10)
    B, I, O, L, M = 2, 3, 4, 5, 6
    x = rng.standard_normal((B, I, L, M)) + 1j * rng.standard_normal((B, I, L, M))
    w = rng.standard_normal((I, O, L, M)) + 1j * rng.standard_normal((I, O, L, M))
    y = np.zeros((B, O, L, M), dtype=complex)
    for b in range(B):
        for o in range(O):
            for l in range(L):
                for m in range(M):
                    for i in range(I):
                        y[b, o, l, m] += x[b, i, l, m] * w[i, o, l, m]
    assert np.allclose(diagonal(x, w), y, atol=1e-13)
    # a weight that does not depend on m is the dhconv operator
    wl = w[:, :, :, :1]
    assert np.allclose(diagonal(x, np.broadcast_to(wl, w.shape)), dhconv(x, wl[..., 0]), atol=1e-13)


def test_spectral_conv_residual_rule():
    rng = np.random.default_rng(9)
    same = ShtTables(12, 24, 12, 13, "legendre-gauss")
    up = ShtTables(25, 48, 12, 13, "equiangular")
    x = rng.standard_normal((1, 2, 12, 24))
    w = rng.standard_normal((2, 3, 12)) + 1j * rng.standard_normal((2, 3, 12))
    y, res = spectral_conv(x, w, same, same)
    assert np.array_equal(res, x) and y.shape == (1, 3, 12, 24)
    y, res = spectral_conv(x, w, same, up)
    assert res.shape == (1, 2, 25, 48) and y.shape == (1, 3, 25, 48)
    assert np.allclose(res, sht_inverse(sht_forward(x, same), up))
    assert np.allclose(y, sht_inverse(dhconv(sht_forward(x, same), w), up))


@pytest.mark.parametrize("grid,norm,nlat,nlon,lmax,mmax", [("equiangular", "ortho", 13, 24, 11, 9), ("legendre-gauss", "schmidt", 10, 19, 10, 10)])
def test_torch_restatement_matches_numpy_oracle_and_its_gradient_is_the_transpose(grid, norm, nlat, nlon, lmax, mmax):
    """oracle.torch_ref in float64 is the gradient oracle of the GPU backward tests.  Pinned two ways: its values
    equal the numpy oracle's, and its autograd gradient equals the explicit transpose of the real-linear map
    assembled column by column from the numpy oracle (a dropped factor 2 on the non-zero orders, or a kept
    imaginary part of the mean / Nyquist order, would show)."""
    import torch
    from oracle.torch_ref import TorchRefSHT
    from oracle.sht import ShtTables, sht_forward, sht_inverse

    t = ShtTables(nlat, nlon, lmax, mmax, grid, norm)
    ref = TorchRefSHT(nlat, nlon, lmax, mmax, grid, norm, dtype=torch.float64)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((nlat, nlon))
    c = rng.standard_normal((lmax, mmax)) + 1j * rng.standard_normal((lmax, mmax))
    np.testing.assert_allclose(ref.forward(torch.from_numpy(x)).numpy(), sht_forward(x, t), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(ref.inverse(torch.from_numpy(c)).numpy(), sht_inverse(c, t), rtol=1e-11, atol=1e-12)

    # forward: J[(l,m,re|im), (k,n)] from unit fields; gradient for cotangent g must be J^T [Re g; Im g]
    J = np.empty((lmax, mmax, 2, nlat * nlon))
    for j in range(nlat * nlon):
        e = np.zeros(nlat * nlon)
        e[j] = 1.0
        y = sht_forward(e.reshape(nlat, nlon), t)
        J[:, :, 0, j], J[:, :, 1, j] = y.real, y.imag
    g = rng.standard_normal((lmax, mmax)) + 1j * rng.standard_normal((lmax, mmax))
    xt = torch.from_numpy(x).requires_grad_(True)
    ref.forward(xt).backward(torch.from_numpy(g))
    want = np.einsum("lmj,lm->j", J[:, :, 0], g.real) + np.einsum("lmj,lm->j", J[:, :, 1], g.imag)
    np.testing.assert_allclose(xt.grad.numpy().ravel(), want, rtol=1e-10, atol=1e-12)

    # inverse: K[(k,n), (l,m,re|im)] from unit coefficients
    K = np.empty((nlat * nlon, lmax, mmax, 2))
    for l in range(lmax):
        for m in range(mmax):
            for p, v in enumerate((1.0, 1j)):
                e = np.zeros((lmax, mmax), dtype=np.complex128)
                e[l, m] = v
                K[:, l, m, p] = sht_inverse(e, t).ravel()
    gx = rng.standard_normal((nlat, nlon))
    ct = torch.from_numpy(c).requires_grad_(True)
    ref.inverse(ct).backward(torch.from_numpy(gx))
    want = np.einsum("jlmp,j->lmp", K, gx.ravel())
    np.testing.assert_allclose(torch.view_as_real(ct.grad).numpy(), want, rtol=1e-10, atol=1e-12)


def test_oracle_against_committed_known_answers():
    """tests/golden/sht_32x64_known_answers.npz (made by tests/golden/make_golden.py from scipy's spherical harmonics and
    moment-equation quadrature weights, without the oracle): smallest benchmark configuration, both directions."""
    import os
    from oracle.sht import ShtTables, sht_forward, sht_inverse

    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "sht_32x64_known_answers.npz"))
    t = ShtTables(int(g["nlat"]), int(g["nlon"]), int(g["lmax"]), int(g["mmax"]), "equiangular")
    np.testing.assert_allclose(t.quad_w, g["weights"], rtol=1e-11, atol=1e-14)
    fwd = sht_forward(g["x"].astype(np.float64), t)
    assert np.linalg.norm(fwd - g["forward"]) / np.linalg.norm(g["forward"]) < 1e-12
    inv = sht_inverse(g["coeffs"].astype(np.complex128), t)
    assert np.linalg.norm(inv - g["inverse"]) / np.linalg.norm(g["inverse"]) < 1e-12
