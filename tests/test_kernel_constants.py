"""CPU pins of constants that live in the kernel sources: the GELU of the pointwise kernels is max(x, 0) - |x| 2^(Q(t) - 1) with a
polynomial Q(t) ~ log2 erfc(t / sqrt 2), t = min(|x|, T).  The coefficients are read from csrc/pointwise.hip and evaluated here in
float32 in the kernel's order; a mistyped coefficient, a wrong clamp or a lost factor 1/2 fails against scipy's erfc."""
import os
import re

import numpy as np
from scipy.special import erfc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def gelu_constants():
    src = open(os.path.join(ROOT, "modulus-makani_amd", "csrc", "pointwise.hip")).read()
    body = src[src.index("__device__ __forceinline__ float gelu(float x) {"):]
    body = body[:body.index("\n}\n")]
    clamp = float(re.search(r"fmed3f\(fabsf\(x\), 0\.f, ([0-9.eE+-]+)f\)", body).group(1))
    first = re.search(r"float q = fmaf\(t, ([0-9.eE+-]+)f, ([0-9.eE+-]+)f\);", body)
    coeffs = [float(first.group(1)), float(first.group(2))] + [float(m) for m in re.findall(r"q = fmaf\(t, q, ([0-9.eE+-]+)f\);", body)]
    assert "fmaf(-fabsf(x), __builtin_amdgcn_exp2f(q)" in body            # the factor 1/2 is in the constant term
    return clamp, coeffs


def kernel_gelu(x, clamp, coeffs):
    f = np.float32
    x = x.astype(f)
    t = np.minimum(np.abs(x), f(clamp)).astype(f)
    q = (t * f(coeffs[0]) + f(coeffs[1])).astype(f)
    for c in coeffs[2:]:
        q = (t * q + f(c)).astype(f)
    return (-np.abs(x) * np.exp2(q).astype(f) + np.maximum(x, f(0))).astype(f), q


def test_gelu_polynomial_follows_log2_erfc():
    clamp, coeffs = gelu_constants()
    assert 6.0 <= clamp <= 9.0 and 6 <= len(coeffs) <= 9
    t = np.linspace(0.0, clamp, 200001)
    _, q = kernel_gelu(t, clamp, coeffs)
    # Q(t) - 1 = log2(erfc(t / sqrt 2) / 2): relative error of the erfc factor below 1e-4 (a twentieth of the half ulp of bf16)
    rel = np.abs(np.exp2(q.astype(np.float64)) / (0.5 * erfc(t / np.sqrt(2.0))) - 1.0)
    assert rel.max() < 1e-4, rel.max()


def test_gelu_matches_the_erf_form_to_bf16_rounding():
    clamp, coeffs = gelu_constants()
    x = np.linspace(-12.0, 12.0, 400001)
    y, _ = kernel_gelu(x, clamp, coeffs)
    ref = 0.5 * x * erfc(-x / np.sqrt(2.0))
    # relative error far below bf16's half ulp wherever the value is representable at all; beyond the clamp the term no longer
    # decays and stays below 3e-10 |x| / clamp
    inside = x >= -clamp
    assert (np.abs(y[inside] - ref[inside]) <= 1.5e-4 * np.abs(ref[inside]) + 1e-12).all()
    assert (np.abs(y[~inside] - ref[~inside]) <= 3e-10 * np.abs(x[~inside]) / clamp).all()
    assert (y[x > 9.0] == x[x > 9.0].astype(np.float32)).all() and (y[x == 0.0] == 0.0).all()
