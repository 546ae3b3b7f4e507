"""CPU-side checks of the C ABI library: it loads, exports every declared symbol, and its
host-only table builders agree with the oracle (no GPU compute is called here)."""
import os
import re

import numpy as np
import pytest

from oracle.quadrature import grid_nodes
from oracle.legendre import legpoly

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "sfno_spectral.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sfno_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib_built):
    import ctypes

    lib = ctypes.CDLL(lib_built)
    names = declared_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), n
    import makani_amd._lib as L

    assert sorted(L.EXPORTS) == names
    assert L.lib.sfno_version() >= 1
    assert L.lib.sfno_strerror(-1).decode() == "invalid argument"


@pytest.mark.parametrize("grid", ["legendre-gauss", "lobatto", "equiangular"])
@pytest.mark.parametrize("nlat", [2, 3, 16, 33, 240, 721])
def test_quadrature_matches_oracle(lib_built, grid, nlat):
    import makani_amd as ma

    theta, w = ma.quadrature(grid, nlat)
    t0, w0 = grid_nodes(nlat, grid)
    assert np.allclose(theta, t0, atol=1e-13) and np.allclose(w, w0, atol=1e-13)
    assert abs(w.sum() - 2.0) < 1e-12


def test_quadrature_module_functions(lib_built):
    import makani_amd as ma

    for fn in (ma.legendre_gauss_weights, ma.clenshaw_curtiss_weights, ma.lobatto_weights):
        x, w = fn(20)
        assert np.all(np.diff(x) > 0) and abs(w.sum() - 2.0) < 1e-12       # tests/test_metrics.py:37-45
        x, w = fn(20, a=0.0, b=3.0)
        assert abs(w.sum() - 3.0) < 1e-12 and x.min() >= 0 and x.max() <= 3


@pytest.mark.parametrize("norm", ["ortho", "four-pi", "schmidt"])
@pytest.mark.parametrize("inverse", [False, True])
@pytest.mark.parametrize("csphase", [True, False])
def test_legendre_table_matches_oracle(lib_built, norm, inverse, csphase):
    import makani_amd as ma

    theta, _ = grid_nodes(40, "equiangular")
    for mmax, lmax in ((21, 20), (9, 33), (40, 40)):
        got = ma.legendre_table(mmax, lmax, theta, norm, inverse, csphase)
        ref = legpoly(mmax, lmax, theta, norm, inverse, csphase)
        assert np.allclose(got, ref, rtol=1e-11, atol=1e-14)


def test_legendre_table_large_orders(lib_built):
    import makani_amd as ma

    theta, _ = grid_nodes(721, "equiangular")
    got = ma.legendre_table(721, 721, theta[300:310], "ortho", False, True)
    ref = legpoly(721, 721, theta[300:310])
    assert np.isfinite(got).all()
    assert np.allclose(got, ref, rtol=1e-9, atol=1e-12)


def test_module_attributes_and_errors(lib_built):
    import torch
    import makani_amd as ma

    s = ma.RealSHT(32, 64, grid="legendre-gauss")
    assert (s.nlat, s.nlon, s.lmax, s.mmax, s.grid) == (32, 64, 32, 33, "legendre-gauss")
    assert ma.RealSHT(32, 64).lmax == 31                         # lobatto default
    assert ma.InverseRealSHT(32, 64, lmax=10, mmax=8, grid="equiangular").mmax == 8
    assert list(s.state_dict().keys()) == [] and list(s.buffers()) == []
    s.float()
    with pytest.raises(ValueError):
        ma.RealSHT(32, 64, grid="nope")
    with pytest.raises(RuntimeError):
        s(torch.zeros(1, 32, 64))                                # CPU tensors are refused: no fallback path
    w = s.weights
    assert tuple(w.shape) == (33, 32, 32) and w.dtype == torch.float32
    conv = ma.SpectralConv(s, ma.InverseRealSHT(32, 64, grid="legendre-gauss"), 4, 6, operator_type="dhconv", gain=2.0)
    assert tuple(conv.weight.shape) == (4, 6, 32) and conv.weight.dtype == torch.complex64
    assert not conv.scale_residual
    assert ma.SpectralConv(s, ma.InverseRealSHT(16, 32, lmax=32, mmax=33, grid="legendre-gauss"), 4, 6, operator_type="dhconv").scale_residual
    with pytest.raises(ValueError):
        ma.SpectralConv(s, ma.InverseRealSHT(32, 64, grid="legendre-gauss"), 4, 6, operator_type="bogus")


@pytest.mark.parametrize("nlat,lmax,mmax,grid", [(241, 241, 241, "legendre-gauss"), (361, 240, 241, "equiangular"), (32, 32, 33, "equiangular")])
@pytest.mark.parametrize("analysis", [True, False])
def test_stream_leaves_out_only_negligible_polar_chunks(lib_built, nlat, lmax, mmax, grid, analysis):
    """The device streams of the Legendre tables omit the leading K chunks of a 32-row block whose entries are all at most
    2^-64 of the largest entry of the order.  Checked against the oracle's float64 table: every omitted entry is that small, the
    first kept chunk holds a larger one (nothing more could have been dropped at this threshold), the index covers every row block,
    and at sizes where sin^m(theta) matters a noticeable share of the table is indeed left out."""
    import ctypes

    import makani_amd._lib as L

    theta, w = grid_nodes(nlat, grid)
    ref = legpoly(mmax, lmax, theta, "ortho", not analysis, True)          # [m][l][k]
    if analysis:
        ref = ref * w[None, None, :]
    K2 = (nlat + 1) // 2
    dp = ctypes.POINTER(ctypes.c_double)
    th = np.ascontiguousarray(theta, dtype=np.float64)
    lw = np.ascontiguousarray(w, dtype=np.float64)
    args = (mmax, lmax, nlat, th.ctypes.data_as(dp), lw.ctypes.data_as(dp) if analysis else None, 0, 0 if analysis else 1, 1, 1 if analysis else 0)
    n = L.lib.sfno_legendre_stream_skips(*args, None, 0)
    assert n > 0
    skips = np.zeros(n, dtype=np.int32)
    assert L.lib.sfno_legendre_stream_skips(*args, skips.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), n) == n
    pos, dense, kept = 0, 0, 0
    for m in range(mmax):
        a = np.abs(ref[m, :, :K2])
        thr = a.max() * 2.0 ** -64
        for p in (0, 1):
            rows_l = np.arange(m + p, lmax, 2)
            np0 = len(np.arange(m, lmax, 2))
            if analysis:
                blk = a[rows_l]                                            # rows = degrees, K = latitudes
                nc = (K2 + 15) // 16
            else:
                blk = np.zeros((K2, np0))                                  # rows = latitudes, K = degrees (padded to parity 0)
                blk[:, :len(rows_l)] = a[rows_l].T
                nc = (np0 + 15) // 16
                if m >= lmax:
                    blk = np.zeros((K2, 0))
            nrb = (blk.shape[0] + 31) // 32
            for rb in range(nrb):
                c0 = int(skips[pos])
                pos += 1
                assert 0 <= c0 <= nc
                sub = blk[32 * rb:32 * rb + 32]
                if c0 > 0:
                    assert sub[:, :16 * c0].max(initial=0.0) <= thr * (1 + 1e-9), (m, p, rb)
                if c0 < nc:
                    first = sub[:, 16 * c0:16 * c0 + 16].max(initial=0.0)
                    assert first > thr * (1 - 1e-9), (m, p, rb, c0)
                dense += nc
                kept += nc - c0
    assert pos == n
    if nlat >= 241:
        assert kept < 0.95 * dense
    print(f"{grid} {nlat} lmax {lmax} mmax {mmax} {'analysis' if analysis else 'synthesis'}: {kept} of {dense} blocks kept")


def test_pointwise_weight_grad_workspace_and_argument_checks(lib_built):
    """Host side of sfno_pointwise_weight_grad: the workspace query (a whole number of [O][K + bias] partial matrices, one
    per share of the pixel range: 8 to 256 shares, fewer for short inputs) and the argument checks that come before any launch."""
    import ctypes

    from makani_amd._lib import lib

    q = lib.sfno_pointwise_weight_grad_workspace_bytes
    for B, K, O, P, bias in [(1, 384, 768, 240 * 480, 1), (1, 768, 384, 240 * 480, 0), (2, 73, 384, 720, 1), (1, 1, 1, 8, 1), (4, 384, 73, 721 * 1440, 0),
                             (1, 4096, 4096, 64, 1)]:
        n = q(B, K, O, P, bias)
        per = 4 * O * (K + bias)
        assert n > 0 and n % per == 0, (B, K, O, P, bias, n)
        shares = n // per
        chunks = B * ((P + 31) // 32)
        assert 1 <= shares <= 256 and shares <= max(1, (chunks + 7) // 8)
        if chunks >= 8 * 256:
            assert shares >= 8
    # pixel counts the kernels do not take, and non-positive sizes: no workspace
    for args in [(1, 8, 8, 12, 0), (1, 8, 8, 4, 0), (0, 8, 8, 64, 0), (1, 0, 8, 64, 0), (1, 8, 0, 64, 0)]:
        assert q(*args) == 0
    # null pointers, bad pixel counts and misaligned operands are refused before anything is launched
    f = lib.sfno_pointwise_weight_grad
    buf = ctypes.create_string_buffer(4096 + 64)
    base = (ctypes.addressof(buf) + 63) & ~63
    ok = ctypes.c_void_p(base)
    assert f(None, ok, ok, None, 1, 8, 8, 64, ok, 4096, None) != 0
    assert f(ok, ok, ok, None, 1, 8, 8, 12, ok, 4096, None) != 0
    assert f(ctypes.c_void_p(base + 2), ok, ok, None, 1, 8, 8, 64, ok, 4096, None) != 0
    assert f(ok, ok, ok, None, 1, 8, 8, 64, ctypes.c_void_p(base + 4), 4096, None) != 0
