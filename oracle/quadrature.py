"""Quadrature rules on [-1, 1] used by the transform pair (oracle, float64).

Restates the rules torch-harmonics exposes as ``legendre_gauss_weights``,
``clenshaw_curtiss_weights`` and ``lobatto_weights``; Makani calls the first two at
makani/utils/grids.py:32,77,83 and the transforms use them for "legendre-gauss",
"equiangular" and "lobatto" grids.  All return (cos(theta) ascending from -1, weights).
"""
import numpy as np


def legendre_gauss_weights(n):
    """Gauss-Legendre nodes/weights of order n (unique rule; numpy's routine)."""
    x, w = np.polynomial.legendre.leggauss(n)
    return x.astype(np.float64), w.astype(np.float64)


def clenshaw_curtiss_weights(n):
    """Clenshaw-Curtis rule on x_k = cos(pi - k*pi/(n-1)), k = 0..n-1 (both poles).

    Closed form of the unique interpolatory rule on these nodes:
      w_k = c_k/N * (1 - sum_{j=1}^{floor(N/2)} b_j/(4j^2-1) cos(2 j theta_k)),
    N = n-1, b_j = 1 if 2j == N else 2, c_k = 1 at the end points else 2.
    """
    assert n > 1
    theta = np.linspace(np.pi, 0.0, n)
    x = np.cos(theta)
    if n == 2:
        return x, np.array([1.0, 1.0])
    N = n - 1
    j = np.arange(1, N // 2 + 1)
    b = np.where(2 * j == N, 1.0, 2.0)
    c = np.full(n, 2.0)
    c[0] = c[-1] = 1.0
    s = (b / (4.0 * j * j - 1.0))[None, :] * np.cos(2.0 * j[None, :] * theta[:, None])
    w = c / N * (1.0 - s.sum(axis=1))
    return x, w


def lobatto_weights(n, tol=1e-16, maxiter=100):
    """Gauss-Lobatto rule of order n (end points included)."""
    assert n > 1
    # Chebyshev-Gauss-Lobatto nodes as the initial guess, Newton on (1-x^2) P'_{n-1}
    x = -np.cos(np.pi * np.arange(n) / (n - 1))
    N = n - 1
    for _ in range(maxiter):
        P = np.zeros((n, n))
        P[:, 0] = 1.0
        P[:, 1] = x
        for k in range(2, n):
            P[:, k] = ((2 * k - 1) * x * P[:, k - 1] - (k - 1) * P[:, k - 2]) / k
        dx = (x * P[:, N] - P[:, N - 1]) / (n * P[:, N])
        x = x - dx
        if np.max(np.abs(dx)) < tol:
            break
    P = np.zeros((n, n))
    P[:, 0] = 1.0
    P[:, 1] = x
    for k in range(2, n):
        P[:, k] = ((2 * k - 1) * x * P[:, k - 1] - (k - 1) * P[:, k - 2]) / k
    w = 2.0 / (N * n * P[:, N] ** 2)
    return x, w


def grid_nodes(nlat, grid):
    """(theta ascending = north pole first, weights) for a named grid.

    Mirrors the grid switch of the transform constructors (legendre-gauss,
    lobatto, equiangular) and the flip of arccos(cost) to north-first ordering.
    """
    if grid == "legendre-gauss":
        cost, w = legendre_gauss_weights(nlat)
    elif grid == "lobatto":
        cost, w = lobatto_weights(nlat)
    elif grid == "equiangular":
        cost, w = clenshaw_curtiss_weights(nlat)
    else:
        raise ValueError("Unknown quadrature mode")
    theta = np.flip(np.arccos(np.clip(cost, -1.0, 1.0))).copy()
    # weights are symmetric under the flip; flip anyway so w[k] belongs to theta[k]
    return theta, np.flip(w).copy()


def default_lmax(nlat, grid):
    return nlat - 1 if grid == "lobatto" else nlat
