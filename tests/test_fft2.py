"""Planar transform pair RealFFT2 / InverseRealFFT2 (makani/models/common/layers.py:219-287).

CPU tests pin the oracle (oracle/fft2.py) against what the mathematics fixes: the truncated double sum
over the grid on a small case, the complex-to-real synthesis sum with a non-Hermitian input, Parseval,
and round trips of band-limited fields.  GPU tests compare the HIP path with the oracle (fp32, relative
L2 <= 1e-5 as for the spherical pair), its gradients with torch autograd through the reference's op
sequence in float64, and SpectralConv / the SFNO network built on the planar pair with the oracle model.
"""
import numpy as np
import pytest
import torch

from oracle.fft2 import Fft2Modes, fft2_forward, fft2_inverse
from oracle.dhconv import spectral_conv
from oracle.sfno import SfnoOracle
from oracle.torch_ref import TorchRefFFT2

TOL = 1e-5


def rel_l2(a, b):
    a, b = np.asarray(a), np.asarray(b)
    return float(np.linalg.norm((a - b).ravel()) / max(np.linalg.norm(b.ravel()), 1e-300))


def kept_frequencies(t):
    """Latitude frequency (as an index 0..nlat-1 of the full transform) of each of the lmax kept rows."""
    return [j if j < t.lmax_high else t.nlat - t.lmax + j for j in range(t.lmax)]


# ---- oracle pins (CPU) ----------------------------------------------------------------------------


@pytest.mark.parametrize("nlat,nlon,lmax,mmax", [(6, 8, None, None), (6, 8, 5, 4), (7, 9, 4, 3), (5, 6, 2, 4)])
def test_oracle_forward_is_the_truncated_double_sum(nlat, nlon, lmax, mmax):
    t = Fft2Modes(nlat, nlon, lmax, mmax)
    x = np.random.default_rng(0).standard_normal((nlat, nlon))
    k, n = np.arange(nlat)[:, None], np.arange(nlon)[None, :]
    want = np.empty((t.lmax, t.mmax), dtype=complex)
    for j, f in enumerate(kept_frequencies(t)):
        for m in range(t.mmax):
            want[j, m] = (x * np.exp(-2j * np.pi * (f * k / nlat + m * n / nlon))).sum() / np.sqrt(nlat * nlon)
    assert np.abs(fft2_forward(x, t) - want).max() < 1e-12


@pytest.mark.parametrize("nlat,nlon,lmax,mmax", [(6, 8, None, None), (6, 8, 5, 4), (7, 9, 4, 3), (6, 8, 4, 5)])
def test_oracle_inverse_is_the_complex_to_real_sum(nlat, nlon, lmax, mmax):
    """Inverse DFT along latitude over the kept frequencies, then the complex-to-real sum along longitude, which uses
    only the real part of the mean and Nyquist columns; the input is a general (non-Hermitian) complex array."""
    t = Fft2Modes(nlat, nlon, lmax, mmax)
    rng = np.random.default_rng(1)
    c = rng.standard_normal((t.lmax, t.mmax)) + 1j * rng.standard_normal((t.lmax, t.mmax))
    k = np.arange(nlat)
    z = np.zeros((nlat, t.mmax), dtype=complex)
    for j, f in enumerate(kept_frequencies(t)):
        z += c[j][None, :] * np.exp(2j * np.pi * f * k / nlat)[:, None] / np.sqrt(nlat)
    n = np.arange(nlon)
    want = np.zeros((nlat, nlon))
    for m in range(t.mmax):
        if m == 0:
            want += z[:, 0].real[:, None]
        elif nlon % 2 == 0 and m == nlon // 2:
            want += z[:, m].real[:, None] * (-1.0) ** n[None, :]
        else:
            want += 2.0 * (z[:, m][:, None] * np.exp(2j * np.pi * m * n / nlon)[None, :]).real
    want /= np.sqrt(nlon)
    assert np.abs(fft2_inverse(c, t) - want).max() < 1e-12


def test_oracle_parseval_and_roundtrip():
    rng = np.random.default_rng(2)
    t = Fft2Modes(10, 12)
    x = rng.standard_normal((3, 10, 12))
    y = fft2_forward(x, t)
    wm = np.full(t.mmax, 2.0)
    wm[0] = wm[-1] = 1.0
    assert abs((np.abs(y) ** 2 * wm).sum() - (x**2).sum()) < 1e-10 * (x**2).sum()
    assert np.abs(fft2_inverse(y, t) - x).max() < 1e-13
    # an odd number of kept latitude frequencies is closed under conjugation: fields synthesised from it survive the round trip
    t = Fft2Modes(10, 12, 5, 4)
    c = rng.standard_normal((5, 4)) + 1j * rng.standard_normal((5, 4))
    x0 = fft2_inverse(c, t)
    assert np.abs(fft2_inverse(fft2_forward(x0, t), t) - x0).max() < 1e-13


def test_oracle_default_and_clamped_modes():
    t = Fft2Modes(9, 16)
    assert (t.lmax, t.mmax, t.truncate) == (9, 9, False)
    t = Fft2Modes(9, 16, 20, 40)          # requests beyond the grid are clamped (layers.py:233-234)
    assert (t.lmax, t.mmax, t.truncate) == (9, 9, False)
    t = Fft2Modes(9, 16, 5, 9)
    assert (t.lmax_high, t.lmax_low, t.truncate) == (3, 2, True)


@pytest.mark.parametrize("nlat,nlon,lmax,mmax", [(8, 12, None, None), (9, 14, 6, 5)])
def test_torch_restatement_matches_numpy_oracle(nlat, nlon, lmax, mmax):
    t = Fft2Modes(nlat, nlon, lmax, mmax)
    ref = TorchRefFFT2(nlat, nlon, lmax, mmax)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, nlat, nlon))
    c = rng.standard_normal((2, t.lmax, t.mmax)) + 1j * rng.standard_normal((2, t.lmax, t.mmax))
    assert np.abs(ref.forward(torch.from_numpy(x)).numpy() - fft2_forward(x, t)).max() < 1e-12
    assert np.abs(ref.inverse(torch.from_numpy(c)).numpy() - fft2_inverse(c, t)).max() < 1e-12


def _golden():
    import os

    return np.load(os.path.join(os.path.dirname(__file__), "golden", "fft2_24x32_known_answers.npz"))


def test_oracle_against_committed_known_answers():
    """tests/golden/fft2_24x32_known_answers.npz holds the defining double sums (made by tests/golden/make_golden_fft2.py
    without any FFT routine): the oracle reproduces them."""
    g = _golden()
    t = Fft2Modes(int(g["nlat"]), int(g["nlon"]), int(g["lmax"]), int(g["mmax"]))
    assert np.abs(fft2_forward(g["x"].astype(np.float64), t) - g["forward"]).max() < 1e-12
    assert np.abs(fft2_inverse(g["coeffs"].astype(np.complex128), t) - g["inverse"]).max() < 1e-12


@pytest.mark.gpu
def test_hip_path_against_committed_known_answers(lib_built):
    import makani_amd as ma

    g = _golden()
    nlat, nlon, lmax, mmax = int(g["nlat"]), int(g["nlon"]), int(g["lmax"]), int(g["mmax"])
    y = ma.RealFFT2(nlat, nlon, lmax, mmax)(torch.from_numpy(g["x"]).cuda())
    z = ma.InverseRealFFT2(nlat, nlon, lmax, mmax)(torch.from_numpy(g["coeffs"]).cuda())
    torch.cuda.synchronize()
    assert rel_l2(y.cpu().numpy(), g["forward"]) < TOL
    assert rel_l2(z.cpu().numpy(), g["inverse"]) < TOL


def test_modules_mirror_the_reference_attributes():
    import makani_amd as ma

    f = ma.RealFFT2(721, 1440, lmax=240, mmax=241)
    i = ma.InverseRealFFT2(721, 1440)
    assert (f.nlat, f.nlon, f.lmax, f.mmax, f.truncate, f.lmax_high, f.lmax_low) == (721, 1440, 240, 241, True, 120, 120)
    assert (i.lmax, i.mmax, i.truncate) == (721, 721, False)
    assert len(list(f.parameters())) == 0 and len(f.state_dict()) == 0
    with pytest.raises(RuntimeError):
        f(torch.zeros(1, 721, 1440))       # no CPU fallback


# ---- HIP path (GPU) ---------------------------------------------------------------------------------

FFT2_CASES = [
    # nlat, nlon, lmax, mmax, lead
    (12, 16, None, None, (2, 3)),
    (12, 16, 7, 6, (5,)),
    (33, 64, 20, 20, (4,)),            # nlat = 3 * 11: a direct radix-11 pass
    (37, 50, 36, 26, (3,)),            # prime nlat, nlon outside the specialised longitude kernels
    (48, 96, 48, 49, (1, 7)),
    (91, 180, 30, 31, (9,)),
    (240, 480, 240, 241, (2, 5)),
    (16, 31, 5, 16, (3,)),             # odd nlon: no Nyquist column
    (64, 128, 40, 33, (11,)),          # latitude lengths with specialised passes: 64, 180, 240 (above), 720
    (180, 360, 101, 91, (2, 4)),
    (720, 1440, 240, 241, (3,)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("nlat,nlon,lmax,mmax,lead", FFT2_CASES)
def test_forward_and_inverse_match_oracle(lib_built, nlat, nlon, lmax, mmax, lead):
    import makani_amd as ma

    print(f"case fft2 {nlat}x{nlon} l{lmax} m{mmax} lead={lead}", flush=True)
    t = Fft2Modes(nlat, nlon, lmax, mmax)
    fwd, inv = ma.RealFFT2(nlat, nlon, lmax, mmax), ma.InverseRealFFT2(nlat, nlon, lmax, mmax)
    rng = np.random.default_rng(7)
    x = rng.standard_normal((*lead, nlat, nlon)).astype(np.float32)
    c = (rng.standard_normal((*lead, t.lmax, t.mmax)) + 1j * rng.standard_normal((*lead, t.lmax, t.mmax))).astype(np.complex64)
    y = fwd(torch.from_numpy(x).cuda())
    z = inv(torch.from_numpy(c).cuda())
    torch.cuda.synchronize()
    assert tuple(y.shape) == (*lead, t.lmax, t.mmax) and y.dtype == torch.complex64
    assert tuple(z.shape) == (*lead, nlat, nlon) and z.dtype == torch.float32
    assert rel_l2(y.cpu().numpy(), fft2_forward(x.astype(np.float64), t)) < TOL
    assert rel_l2(z.cpu().numpy(), fft2_inverse(c.astype(np.complex128), t)) < TOL


@pytest.mark.gpu
@pytest.mark.parametrize("nlat,nlon,lmax,mmax,lead", FFT2_CASES[:6] + FFT2_CASES[7:10])
def test_gradients_match_autograd_of_the_reference_ops(lib_built, nlat, nlon, lmax, mmax, lead):
    import makani_amd as ma

    print(f"case fft2-bwd {nlat}x{nlon} l{lmax} m{mmax} lead={lead}", flush=True)
    ref = TorchRefFFT2(nlat, nlon, lmax, mmax)
    fwd, inv = ma.RealFFT2(nlat, nlon, lmax, mmax), ma.InverseRealFFT2(nlat, nlon, lmax, mmax)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(*lead, nlat, nlon, generator=g)
    gy = torch.randn(*lead, ref.lmax, ref.mmax, 2, generator=g)
    c = torch.view_as_complex(torch.randn(*lead, ref.lmax, ref.mmax, 2, generator=g))
    gx = torch.randn(*lead, nlat, nlon, generator=g)
    gyc = torch.view_as_complex(gy)

    xr = x.double().requires_grad_(True)
    ref.forward(xr).backward(gyc.to(torch.complex128))
    xg = x.cuda().requires_grad_(True)
    fwd(xg).backward(gyc.cuda())
    cr = c.to(torch.complex128).requires_grad_(True)
    ref.inverse(cr).backward(gx.double())
    cg = c.cuda().requires_grad_(True)
    inv(cg).backward(gx.cuda())
    torch.cuda.synchronize()
    assert rel_l2(xg.grad.cpu().numpy(), xr.grad.numpy()) < TOL
    assert rel_l2(torch.view_as_real(cg.grad.cpu()).numpy(), torch.view_as_real(cr.grad).numpy()) < TOL


@pytest.mark.gpu
@pytest.mark.parametrize("operator_type", ["dhconv", "diagonal"])
@pytest.mark.parametrize("shapes", [((24, 48), (24, 48), 12, 12), ((33, 64), (16, 32), 16, 16)])
def test_spectral_conv_on_the_planar_pair(lib_built, operator_type, shapes):
    """SpectralConv(RealFFT2, InverseRealFFT2): forward against the oracle's op order, gradients against autograd of the
    reference ops; the second case has different input and output grids (the residual goes through the transforms)."""
    import makani_amd as ma

    (hi, wi), (ho, wo), lmax, mmax = shapes
    print(f"case fft2 spectral conv {operator_type} {shapes}", flush=True)
    torch.manual_seed(3)
    B, I, O = 2, 6, 4
    fwd, inv = ma.RealFFT2(hi, wi, lmax, mmax), ma.InverseRealFFT2(ho, wo, lmax, mmax)
    conv = ma.SpectralConv(fwd, inv, I, O, operator_type=operator_type).cuda()
    x = torch.randn(B, I, hi, wi)
    xg = x.cuda().requires_grad_(True)
    y, res = conv(xg)
    gy = torch.randn(B, O, ho, wo)
    y.backward(gy.cuda())
    torch.cuda.synchronize()
    w = conv.weight.detach().cpu().numpy().astype(np.complex128)
    want, want_res = spectral_conv(x.double().numpy(), w, Fft2Modes(hi, wi, lmax, mmax), Fft2Modes(ho, wo, lmax, mmax))
    assert rel_l2(y.detach().cpu().numpy(), want) < TOL
    assert rel_l2(res.detach().cpu().numpy(), want_res) < TOL

    rf, ri = TorchRefFFT2(hi, wi, lmax, mmax), TorchRefFFT2(ho, wo, lmax, mmax)
    xr = x.double().requires_grad_(True)
    wr = conv.weight.detach().cpu().to(torch.complex128).requires_grad_(True)
    eq = "bixy,iox->boxy" if operator_type == "dhconv" else "bixy,ioxy->boxy"
    ri.inverse(torch.einsum(eq, rf.forward(xr), wr)).backward(gy.double())
    assert rel_l2(xg.grad.cpu().numpy(), xr.grad.numpy()) < TOL
    assert rel_l2(torch.view_as_real(conv.weight.grad.cpu()).numpy(), torch.view_as_real(wr.grad).numpy()) < TOL


@pytest.mark.gpu
def test_network_with_the_planar_pair_matches_oracle(lib_built):
    """spectral_transform="fft" (sfnonet.py:542-556): fp32 forward against the float64 oracle model, and under bf16
    autocast with the fused pointwise tail."""
    from makani_amd.sfnonet import SphericalFourierNeuralOperatorNet

    cfg = dict(inp_shape=(48, 96), out_shape=(48, 96), inp_chans=3, out_chans=2, scale_factor=2, embed_dim=16, num_layers=3)
    print(f"case sfno fft {cfg}", flush=True)
    torch.manual_seed(4)
    net = SphericalFourierNeuralOperatorNet(spectral_transform="fft", **cfg).cuda().eval()
    x = torch.randn(2, 3, 48, 96, generator=torch.Generator().manual_seed(5))
    with torch.inference_mode():
        y = net(x.cuda())
        with torch.autocast("cuda", dtype=torch.bfloat16):
            yb = net(x.cuda())
    torch.cuda.synchronize()
    ref = SfnoOracle(cfg["inp_shape"], cfg["out_shape"], 2, 3, spectral_transform="fft").forward(net.state_dict(), x).numpy()
    assert rel_l2(y.cpu().double().numpy(), ref) < 1e-4
    assert rel_l2(yb.float().cpu().double().numpy(), ref) < 2e-2


@pytest.mark.gpu
def test_full_size_properties(lib_built):
    """720x1440, 73 channels: Parseval for the untruncated transform and the round trip, the properties that need no
    oracle run at this size; bf16 grid input is widened inside the longitude kernel to the same values."""
    import makani_amd as ma

    print("case fft2 720x1440x73", flush=True)
    fwd, inv = ma.RealFFT2(720, 1440), ma.InverseRealFFT2(720, 1440)
    x = torch.randn(1, 73, 720, 1440, device="cuda", generator=torch.Generator("cuda").manual_seed(1))
    y = fwd(x)
    wm = torch.full((721,), 2.0, device="cuda")
    wm[0] = wm[-1] = 1.0
    e_spec = float((y.abs().double() ** 2 * wm).sum())
    e_grid = float((x.double() ** 2).sum())
    assert abs(e_spec - e_grid) < 1e-5 * e_grid
    back = inv(y)
    assert float(torch.linalg.norm((back - x).double().ravel()) / torch.linalg.norm(x.double().ravel())) < TOL
    xb = x.to(torch.bfloat16)
    assert torch.equal(fwd.analysis(xb), fwd.analysis(xb.float()))


@pytest.mark.gpu
@pytest.mark.parametrize("nlat", [1024, 720, 512, 480, 360, 256, 240, 180, 128, 64])
def test_every_specialised_latitude_length(lib_built, nlat):
    """Each latitude length with compile-time passes, truncated and not, against the oracle."""
    import makani_amd as ma

    print(f"case specialised nlat={nlat}", flush=True)
    rng = np.random.default_rng(nlat)
    for lmax in (None, nlat // 3 + 1):
        t = Fft2Modes(nlat, 24, lmax, None)
        x = rng.standard_normal((7, nlat, 24)).astype(np.float32)
        c = (rng.standard_normal((7, t.lmax, t.mmax)) + 1j * rng.standard_normal((7, t.lmax, t.mmax))).astype(np.complex64)
        y = ma.RealFFT2(nlat, 24, lmax)(torch.from_numpy(x).cuda())
        z = ma.InverseRealFFT2(nlat, 24, lmax)(torch.from_numpy(c).cuda())
        torch.cuda.synchronize()
        assert rel_l2(y.cpu().numpy(), fft2_forward(x.astype(np.float64), t)) < TOL
        assert rel_l2(z.cpu().numpy(), fft2_inverse(c.astype(np.complex128), t)) < TOL


@pytest.mark.gpu
@pytest.mark.parametrize("nlat,lmax", [(721, None), (721, 240), (1300, 100)])
def test_long_latitude_lengths_without_specialised_passes(lib_built, nlat, lmax):
    """721 = 7 * 103 (the 0.25 degree grid with both poles) and 1300 = 4 * 25 * 13 run on the run-time radix passes
    with more than 64 KB of LDS per workgroup."""
    import makani_amd as ma

    print(f"case generic nlat={nlat} lmax={lmax}", flush=True)
    rng = np.random.default_rng(nlat)
    t = Fft2Modes(nlat, 16, lmax, None)
    x = rng.standard_normal((5, nlat, 16)).astype(np.float32)
    c = (rng.standard_normal((5, t.lmax, t.mmax)) + 1j * rng.standard_normal((5, t.lmax, t.mmax))).astype(np.complex64)
    y = ma.RealFFT2(nlat, 16, lmax)(torch.from_numpy(x).cuda())
    z = ma.InverseRealFFT2(nlat, 16, lmax)(torch.from_numpy(c).cuda())
    torch.cuda.synchronize()
    assert rel_l2(y.cpu().numpy(), fft2_forward(x.astype(np.float64), t)) < TOL
    assert rel_l2(z.cpu().numpy(), fft2_inverse(c.astype(np.complex128), t)) < TOL


@pytest.mark.gpu
def test_planar_plan_argument_checks(lib_built):
    """A planar plan keeps at most nlat latitude and nlon/2+1 longitude frequencies; the module clamps like the
    reference (layers.py:233-234), the C entry point rejects."""
    import ctypes

    import makani_amd as ma
    from makani_amd import _lib

    h = ctypes.c_void_p()
    planar, ortho = _lib.GRID["planar"], _lib.NORM["ortho"]
    assert _lib.lib.sfno_sht_plan_create(16, 32, 17, 17, planar, ortho, 1, _lib.DIR_FORWARD, _lib.COMPUTE_FP32, ctypes.byref(h)) == -1
    assert _lib.lib.sfno_sht_plan_create(16, 32, 16, 18, planar, ortho, 1, _lib.DIR_INVERSE, _lib.COMPUTE_FP32, ctypes.byref(h)) == -1
    assert not h.value
    f = ma.RealFFT2(16, 32, lmax=40, mmax=40)
    assert (f.lmax, f.mmax) == (16, 17)
    y = f(torch.ones(2, 16, 32, device="cuda"))
    torch.cuda.synchronize()
    # a constant field has a single non-zero coefficient, sqrt(nlat nlon) with the "ortho" normalisation
    want = torch.zeros(2, 16, 17, dtype=torch.complex64)
    want[:, 0, 0] = (16 * 32) ** 0.5
    assert torch.allclose(y.cpu(), want, atol=1e-5)
