"""GPU parity of the HIP transform pair against the float64 oracle.

Tolerance: relative L2 <= 1e-5 (fp32 arithmetic against a float64 oracle), the bound the
scope contract states for the fp32 path.
"""
import numpy as np
import pytest
import torch

from oracle.sht import ShtTables, sht_forward, sht_inverse

pytestmark = pytest.mark.gpu
TOL = 1e-5


def rel_l2(a, b):
    a = np.asarray(a)
    b = np.asarray(b)
    return np.linalg.norm((a - b).ravel()) / max(np.linalg.norm(b.ravel()), 1e-300)


CASES = [
    # nlat, nlon, lmax, mmax, grid, lead
    (32, 64, 32, 33, "equiangular", (2, 4)),      # BASELINE config 1
    (32, 64, None, None, "legendre-gauss", (3,)),
    (33, 64, None, None, "lobatto", (1, 5)),
    (16, 32, 16, 17, "legendre-gauss", (2, 6)),
    (33, 64, 16, 17, "equiangular", (2, 6)),
    (12, 30, 10, 9, "legendre-gauss", (7,)),      # nlon with factors 2*3*5, truncated orders
    (19, 45, 19, 23, "equiangular", (2, 3)),      # odd nlon
    (8, 14, 8, 8, "legendre-gauss", (4,)),        # radix 7 (generic butterfly)
    (91, 180, 60, 61, "equiangular", (5,)),       # several row blocks and K chunks
    (40, 96, 40, 49, "legendre-gauss", (2, 40)),  # 160 channel columns: more than one column tile
]


@pytest.mark.parametrize("nlat,nlon,lmax,mmax,grid,lead", CASES)
def test_forward_matches_oracle(lib_built, nlat, nlon, lmax, mmax, grid, lead):
    import makani_amd as ma

    print(f"case fwd {nlat}x{nlon} lmax={lmax} mmax={mmax} {grid} lead={lead}", flush=True)
    torch.manual_seed(0)
    x = torch.randn(*lead, nlat, nlon, dtype=torch.float32)
    sht = ma.RealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid=grid)
    got = sht(x.cuda())
    torch.cuda.synchronize()
    t = ShtTables(nlat, nlon, lmax, mmax, grid)
    ref = sht_forward(x.double().numpy(), t)
    assert got.shape == ref.shape and got.dtype == torch.complex64
    assert rel_l2(got.cpu().numpy(), ref) < TOL
    # structural zeros: no degree below the order
    g = got.cpu().numpy()
    for m in range(g.shape[-1]):
        assert np.all(g[..., : min(m, g.shape[-2]), m] == 0)


@pytest.mark.parametrize("nlat,nlon,lmax,mmax,grid,lead", CASES)
def test_inverse_matches_oracle(lib_built, nlat, nlon, lmax, mmax, grid, lead):
    import makani_amd as ma

    print(f"case inv {nlat}x{nlon} lmax={lmax} mmax={mmax} {grid} lead={lead}", flush=True)
    t = ShtTables(nlat, nlon, lmax, mmax, grid)
    torch.manual_seed(1)
    c = torch.randn(*lead, t.lmax, t.mmax, dtype=torch.complex64)
    # generic input: also fills l < m and Im(m=0), which the inverse must ignore / drop like the reference
    isht = ma.InverseRealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid=grid)
    got = isht(c.cuda())
    torch.cuda.synchronize()
    ref = sht_inverse(c.numpy().astype(np.complex128), t)
    assert got.shape == ref.shape and got.dtype == torch.float32
    assert rel_l2(got.cpu().numpy(), ref) < TOL


def test_roundtrip_bandlimited(lib_built):
    """inverse(forward(x)) = x for fields band-limited below the grid's exactness (Legendre-Gauss)."""
    import makani_amd as ma

    nlat, nlon = 48, 96
    t = ShtTables(nlat, nlon, 32, 33, "legendre-gauss")
    rng = np.random.default_rng(3)
    c = rng.standard_normal((5, 32, 33)) + 1j * rng.standard_normal((5, 32, 33))
    c[:, :, 0] = c[:, :, 0].real
    for m in range(33):
        c[:, :m, m] = 0
    c[:, :, 32] = 0
    x = sht_inverse(c, t)
    sht = ma.RealSHT(nlat, nlon, 32, 33, "legendre-gauss")
    isht = ma.InverseRealSHT(nlat, nlon, 32, 33, "legendre-gauss")
    xg = torch.from_numpy(x).float().cuda()
    cg = sht(xg)
    back = isht(cg)
    torch.cuda.synchronize()
    assert rel_l2(cg.cpu().numpy(), c) < TOL
    assert rel_l2(back.cpu().numpy(), x) < TOL


def test_constant_field(lib_built):
    import makani_amd as ma

    sht = ma.RealSHT(33, 64, grid="equiangular")
    c = sht(torch.ones(1, 33, 64, device="cuda")).cpu().numpy()
    assert abs(c[0, 0, 0] - np.sqrt(4 * np.pi)) < 1e-5
    c[0, 0, 0] = 0
    assert np.abs(c).max() < 1e-5


def test_shape_asserts(lib_built):
    import makani_amd as ma

    sht = ma.RealSHT(16, 32, grid="legendre-gauss")
    with pytest.raises(AssertionError):
        sht(torch.zeros(2, 16, 30, device="cuda"))
    isht = ma.InverseRealSHT(16, 32, grid="legendre-gauss")
    with pytest.raises(AssertionError):
        isht(torch.zeros(2, 16, 16, dtype=torch.complex64, device="cuda"))


def test_inverse_surplus_orders(lib_built):
    """mmax above nlon//2+1 (up-scaled coefficients synthesised on a coarser grid): surplus orders are dropped like irfft does."""
    import makani_amd as ma

    t = ShtTables(16, 32, 32, 33, "legendre-gauss")
    torch.manual_seed(5)
    c = torch.randn(3, 32, 33, dtype=torch.complex64)
    got = ma.InverseRealSHT(16, 32, lmax=32, mmax=33, grid="legendre-gauss")(c.cuda())
    ref = sht_inverse(c.numpy().astype(np.complex128), t)
    assert rel_l2(got.cpu().numpy(), ref) < TOL
    with pytest.raises(ValueError):
        ma.RealSHT(16, 32, lmax=32, mmax=33, grid="legendre-gauss")


@pytest.mark.parametrize("nlat,nlon,lmax,mmax,grid", [(32, 64, 20, 21, "equiangular"), (40, 480, 40, 41, "legendre-gauss"), (12, 30, 10, 9, "legendre-gauss")])
def test_bf16_grid_io_equals_cast_then_transform(lib_built, nlat, nlon, lmax, mmax, grid):
    """A bf16 field transformed directly equals the transform of its float32 widening, bit for bit; a bf16 output
    equals the float32 output rounded to nearest even (the reference's x.float() / x.to(dtype) around the transforms)."""
    import makani_amd as ma

    torch.manual_seed(7)
    sht = ma.RealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid=grid)
    isht = ma.InverseRealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid=grid)
    xb = torch.randn(3, 5, nlat, nlon).to(torch.bfloat16).cuda()
    s_direct = sht.analysis(xb)
    s_cast = sht.analysis(xb.float())
    # entries with l < m (and the channel padding) are never written: compare the defined part
    valid = (torch.arange(s_cast.shape[1])[None, :] >= torch.arange(s_cast.shape[0])[:, None]).cuda()
    assert torch.equal(s_direct[..., : 2 * 15][valid], s_cast[..., : 2 * 15][valid])
    y32 = isht.synthesis(s_cast, (3, 5))
    yb = isht.synthesis(s_cast, (3, 5), dtype=torch.bfloat16)
    assert yb.dtype == torch.bfloat16 and torch.equal(yb, y32.to(torch.bfloat16))


@pytest.mark.parametrize("nlat,nlon,lmax,mmax,grid,lead", [CASES[0], CASES[3], CASES[4], CASES[8], CASES[9], (241, 480, 241, 241, "legendre-gauss", (12,))])
def test_bf16_compute_variant(lib_built, nlat, nlon, lmax, mmax, grid, lead):
    """Legendre stage on bf16 MFMA (bf16 tables and activations, fp32 accumulation): relative L2 <= 1e-2 vs the float64 oracle."""
    import makani_amd as ma

    print(f"case bf16 compute {nlat}x{nlon} lmax={lmax} mmax={mmax} {grid} lead={lead}", flush=True)
    t = ShtTables(nlat, nlon, lmax, mmax, grid)
    torch.manual_seed(8)
    x = torch.randn(*lead, nlat, nlon)
    got = ma.RealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid=grid, compute="bf16")(x.cuda())
    ref = sht_forward(x.double().numpy(), t)
    e_fwd = rel_l2(got.cpu().numpy(), ref)
    c = torch.randn(*lead, t.lmax, t.mmax, dtype=torch.complex64)
    goti = ma.InverseRealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid=grid, compute="bf16")(c.cuda())
    refi = sht_inverse(c.numpy().astype(np.complex128), t)
    e_inv = rel_l2(goti.cpu().numpy(), refi)
    print(f"   rel-L2 forward {e_fwd:.2e} inverse {e_inv:.2e}", flush=True)
    assert e_fwd < 1e-2 and e_inv < 1e-2
    assert e_fwd > 1e-5 or e_inv > 1e-5          # it is the reduced-precision path that ran


@pytest.mark.parametrize("nlat,nlon,lmax,mmax,grid,lead", [CASES[0], CASES[8], CASES[9], (241, 480, 241, 241, "legendre-gauss", (12,))])
def test_fp32_on_bf16_pipe_is_as_accurate_as_fp32_mfma(lib_built, nlat, nlon, lmax, mmax, grid, lead):
    """The default fp32 mode cuts every operand of the Legendre stage exactly into three bf16 numbers and keeps the six
    largest partial products; "fp32_mfma" runs the same contraction on the fp32 matrix instruction.  Both meet the fp32
    bound against the float64 oracle, and the split path is not less accurate than the plain one (its dropped terms are
    below one fp32 rounding of a product)."""
    import makani_amd as ma

    print(f"case fp32 modes {nlat}x{nlon} lmax={lmax} mmax={mmax} {grid} lead={lead}", flush=True)
    t = ShtTables(nlat, nlon, lmax, mmax, grid)
    torch.manual_seed(9)
    # a wide spread of magnitudes and all 24 significant bits in use
    x = torch.randn(*lead, nlat, nlon) * torch.exp(3.0 * torch.randn(*lead, 1, 1))
    c = torch.randn(*lead, t.lmax, t.mmax, dtype=torch.complex64) * torch.exp(3.0 * torch.randn(*lead, 1, 1))
    ref = sht_forward(x.double().numpy(), t)
    refi = sht_inverse(c.numpy().astype(np.complex128), t)
    err = {}
    for mode in ("fp32", "fp32_mfma"):
        got = ma.RealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid=grid, compute=mode)(x.cuda())
        goti = ma.InverseRealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid=grid, compute=mode)(c.cuda())
        err[mode] = (rel_l2(got.cpu().numpy(), ref), rel_l2(goti.cpu().numpy(), refi))
        print(f"   {mode}: rel-L2 forward {err[mode][0]:.2e} inverse {err[mode][1]:.2e}", flush=True)
        assert err[mode][0] < TOL and err[mode][1] < TOL
    assert err["fp32"][0] <= 2.0 * err["fp32_mfma"][0] + 1e-7
    assert err["fp32"][1] <= 2.0 * err["fp32_mfma"][1] + 1e-7


def test_unknown_compute_mode_raises(lib_built):
    import makani_amd as ma

    with pytest.raises(ValueError):
        ma.RealSHT(8, 16, compute="fp16")


def test_known_answers_config0(lib_built):
    """configs[0] (equiangular 32 x 64, lmax 32, mmax 33, batch 2, 4 channels) against the committed known answers
    of tests/golden (scipy spherical harmonics, no oracle involved): rel-L2 <= 1e-5 both ways."""
    import os
    import makani_amd as ma

    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "sht_32x64_known_answers.npz"))
    nlat, nlon, lmax, mmax = int(g["nlat"]), int(g["nlon"]), int(g["lmax"]), int(g["mmax"])
    fwd = ma.RealSHT(nlat, nlon, lmax, mmax, grid="equiangular")
    inv = ma.InverseRealSHT(nlat, nlon, lmax, mmax, grid="equiangular")
    c = fwd(torch.from_numpy(g["x"]).cuda())
    x = inv(torch.from_numpy(g["coeffs"]).cuda())
    torch.cuda.synchronize()
    assert np.linalg.norm(c.cpu().numpy() - g["forward"]) / np.linalg.norm(g["forward"]) < 1e-5
    assert np.linalg.norm(x.cpu().numpy() - g["inverse"]) / np.linalg.norm(g["inverse"]) < 1e-5


@pytest.mark.parametrize("nlon", [1536, 1440, 1024, 720, 512, 480, 360, 256, 240, 180, 128, 64])
def test_every_specialised_longitude_length(lib_built, nlon):
    """Each transform length with compile-time passes, through the whole pair on a small latitude count: forward and
    inverse against the oracle, and bf16 grid input equal to its float32 widening."""
    import makani_amd as ma

    nlat, mmax, lead = 9, min(nlon // 2 + 1, 300), (2, 5)
    print(f"case specialised nlon={nlon}", flush=True)
    t = ShtTables(nlat, nlon, nlat, mmax, "legendre-gauss")
    torch.manual_seed(nlon)
    x = torch.randn(*lead, nlat, nlon)
    c = torch.randn(*lead, t.lmax, t.mmax, dtype=torch.complex64)
    sht = ma.RealSHT(nlat, nlon, lmax=nlat, mmax=mmax, grid="legendre-gauss")
    isht = ma.InverseRealSHT(nlat, nlon, lmax=nlat, mmax=mmax, grid="legendre-gauss")
    got_f, got_i = sht(x.cuda()), isht(c.cuda())
    torch.cuda.synchronize()
    assert rel_l2(got_f.cpu().numpy(), sht_forward(x.double().numpy(), t)) < TOL
    assert rel_l2(got_i.cpu().numpy(), sht_inverse(c.numpy().astype(np.complex128), t)) < TOL
    xb = x.to(torch.bfloat16).cuda()
    a, b = sht.analysis(xb), sht.analysis(xb.float())
    m, l = torch.arange(mmax)[:, None], torch.arange(nlat)[None, :]
    keep = (m <= l).cuda()
    assert torch.equal(a[..., : 2 * 10][keep], b[..., : 2 * 10][keep])


def test_empty_ragged_and_strided_inputs(lib_built):
    """Edge shapes at the module boundary: no leading dimensions, an empty batch, a non-contiguous view, half and double
    precision inputs (the reference up-casts half inputs itself; float64 is not this path's arithmetic)."""
    import makani_amd as ma

    nlat, nlon = 12, 24
    sht, isht = ma.RealSHT(nlat, nlon, grid="legendre-gauss"), ma.InverseRealSHT(nlat, nlon, grid="legendre-gauss")
    fft, ifft = ma.RealFFT2(nlat, nlon), ma.InverseRealFFT2(nlat, nlon)
    t = ShtTables(nlat, nlon, None, None, "legendre-gauss")
    torch.manual_seed(12)
    x = torch.randn(nlat, nlon)
    for f, inv in ((sht, isht), (fft, ifft)):
        y = f(x.cuda())                                         # a single field, no batch or channel axis
        assert tuple(y.shape) == (f.lmax, f.mmax)
        assert tuple(inv(y).shape) == (nlat, nlon)
        e = f(torch.empty(0, 3, nlat, nlon, device="cuda"))      # empty batch
        assert tuple(e.shape) == (0, 3, f.lmax, f.mmax)
        assert tuple(inv(e).shape) == (0, 3, nlat, nlon)
    assert rel_l2(sht(x.cuda()).cpu().numpy(), sht_forward(x.double().numpy(), t)) < TOL
    big = torch.randn(2, nlat, 3, nlon)
    view = big.permute(0, 2, 1, 3)                               # [2, 3, nlat, nlon], not contiguous
    got = sht(view.cuda())
    assert rel_l2(got.cpu().numpy(), sht_forward(view.double().numpy(), t)) < TOL
    half = torch.randn(2, nlat, nlon).half()
    assert rel_l2(sht(half.cuda()).cpu().numpy(), sht_forward(half.double().numpy(), t)) < TOL
    with pytest.raises(TypeError):
        sht(torch.randn(2, nlat, nlon, dtype=torch.float64).cuda())
    with pytest.raises(TypeError):
        isht(torch.randn(2, isht.lmax, isht.mmax).cuda())        # real input where coefficients are expected
