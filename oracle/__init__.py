"""CPU oracle for the SFNO spectral hot path (TEST INFRASTRUCTURE ONLY).

This package restates, in float64 numpy, the algorithm of the path that Makani's
SFNO spends its time in:

  * the real spherical harmonic transform pair that Makani constructs at
    makani/models/networks/sfnonet.py:524-539 and calls at
    makani/models/common/spectral_convolution.py:131,133,141.  The arithmetic of that
    pair lives in the third-party package torch-harmonics (pinned ">=0.6.5" in
    pyproject.toml:55, image tag v0.6.4 in docker/Dockerfile:78-81), which is not part
    of the reference tree; its published algorithm (quadrature rule, orthonormal
    associated Legendre recursion, rFFT + per-order contraction) is restated here.
  * the "dhconv" channel contraction, makani/models/common/contractions.py:130-136.
  * the SpectralConv orchestration, makani/models/common/spectral_convolution.py:124-148.

Nothing in the product (the HIP library and its Python host layer) may import this
package: it is the checker used by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py, never the thing measured or shipped.

Pinning status (what each function is checked against, see tests/test_oracle_*.py):
  quadrature.*            : sum of weights = 2 (the reference's own check,
                            tests/test_metrics.py:37-45), polynomial exactness,
                            numpy leggauss, brute-force interpolatory weights.
  legendre.legpoly        : scipy.special.sph_harm_y, closed forms l<=2,
                            discrete orthonormality, equatorial symmetry.
  sht.sht_forward/inverse : constant field, one-hot Y_l^m samples, band-limited
                            round trip, Parseval, brute-force O(N^2) DFT.
  dhconv.dhconv           : brute-force loops (both the einsum and the matrix-product branch), identity weights, L=1 matmul.
  sfno.SfnoOracle         : an independent evaluation from scipy's harmonics and explicit formulas (tests/test_oracle_sfno_pin.py).
  stepper.*               : hand-computed statistics and residual rule (tests/test_stepper.py).
  The reference holds no golden vectors for transform values (its tests check shapes
  only), so raw-coefficient sign/ordering conventions of torch-harmonics (latitude
  north->south, Condon-Shortley phase) are "parity unpinned" by reference fixtures;
  they are fixed here by the published definition and cancel in every
  inverse(per-degree op(forward(x))) composition the model uses.
"""
