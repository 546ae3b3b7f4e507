"""Scale behaviour of the default arithmetic (operands scaled by powers of two and cut into two fp16 parts, three products on
the fp16 matrix pipe).  The scales are powers of two taken from the data, so multiplying a channel (a column of the Legendre
panel), a sample (the rows of the channel mix) or an output channel of the weight by 2^k must change nothing but the exponent of
the result: bit-identical mantissas, over the whole fp32 range and with very different magnitudes side by side in one launch.
A mistake in a scale (a bound taken over the wrong index, a rescale of partial sums that is off by one chunk, a saturated fp16
part) shows up here as a result that is not an exact power-of-two multiple."""
import pytest
import torch

pytestmark = pytest.mark.gpu

KS = [-90, -37, 0, 11, 64, 90]          # 2^-90 = 8.1e-28 ... 2^90 = 1.2e27 (results stay clear of denormals and of overflow)


def _pow2(ks):
    return torch.ldexp(torch.ones(len(ks)), torch.tensor(ks, dtype=torch.int32))


@pytest.mark.parametrize("nlat,nlon,lmax,mmax,grid", [(91, 180, 60, 61, "equiangular"), (40, 96, 40, 49, "legendre-gauss"), (721, 1440, 240, 241, "equiangular")])
def test_transforms_commute_with_power_of_two_channel_scales(lib_built, nlat, nlon, lmax, mmax, grid):
    import makani_amd as ma

    print(f"case scales sht {nlat}x{nlon} l{lmax} m{mmax} {grid}", flush=True)
    torch.manual_seed(5)
    # (rows 2p and 2p + 1 share one complex FFT along longitude -- real and imaginary part of one sequence --, so the rounding
    # error of a channel's coefficients is relative to the larger of the two: the two channels of a pair get the same scale)
    C = 2 * len(KS)
    ks = [k for k in KS for _ in range(2)]
    s = _pow2(ks).cuda()
    sht = ma.RealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid=grid)
    isht = ma.InverseRealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid=grid)
    x = torch.randn(C, nlat, nlon).cuda()
    base = sht(x)
    got = sht(x * s[:, None, None])
    torch.cuda.synchronize()
    assert torch.isfinite(torch.view_as_real(got)).all()
    assert torch.equal(torch.view_as_real(got), torch.view_as_real(base) * s[:, None, None, None])
    c = torch.randn(C, sht.lmax, sht.mmax, dtype=torch.complex64).cuda()
    base = isht(c)
    got = isht(c * s[:, None, None])
    torch.cuda.synchronize()
    assert torch.isfinite(got).all()
    assert torch.equal(got, base * s[:, None, None])


@pytest.mark.parametrize("B,I,O,L,M", [(len(KS), 20, 36, 33, 33), (len(KS), 384, 384, 24, 25)])
def test_dhconv_commutes_with_power_of_two_sample_and_output_scales(lib_built, B, I, O, L, M):
    import makani_amd as ma

    print(f"case scales dhconv B={B} I={I} O={O} L={L} M={M}", flush=True)
    torch.manual_seed(6)
    x = (torch.randn(B, I, L, M, dtype=torch.complex64) * torch.exp(torch.randn(B, I, 1, 1))).cuda()
    w = (torch.randn(I, O, L, dtype=torch.complex64) / I**0.5).cuda()
    base = ma._contract_dhconv(x, w)
    sb = _pow2(KS).cuda()                                     # one scale per sample: the rows (m, b) of the mix
    got = ma._contract_dhconv(x * sb[:, None, None, None], w)
    torch.cuda.synchronize()
    assert torch.isfinite(torch.view_as_real(got)).all()
    assert torch.equal(torch.view_as_real(got), torch.view_as_real(base) * sb[:, None, None, None, None])
    so = _pow2([KS[o % len(KS)] // 2 for o in range(O)]).cuda()        # one scale per output channel: the columns of the packed weight
    got = ma._contract_dhconv(x, w * so[None, :, None])
    torch.cuda.synchronize()
    assert torch.isfinite(torch.view_as_real(got)).all()
    assert torch.equal(torch.view_as_real(got), torch.view_as_real(base) * so[None, :, None, None, None])


def test_a_non_finite_channel_stays_in_its_channel(lib_built):
    """A NaN or an infinity in one channel of the transform's input comes out as NaN in that channel and leaves its neighbours
    in the same column tile bit-identical."""
    import makani_amd as ma

    print("case scales non-finite", flush=True)
    torch.manual_seed(7)
    nlat, nlon = 40, 96
    sht = ma.RealSHT(nlat, nlon, grid="legendre-gauss")
    x = torch.randn(8, nlat, nlon).cuda()
    base = sht(x)
    bad = x.clone()
    bad[2, 17, 5] = float("nan")
    bad[5, 3, 40] = float("inf")
    got = sht(bad)
    torch.cuda.synchronize()
    # (the partner in the FFT pair -- rows 3 and 4 -- is lost with it; the other pairs of the same column tile are untouched)
    for c in (0, 1, 6, 7):
        assert torch.equal(torch.view_as_real(got[c]), torch.view_as_real(base[c]))
    for c in (2, 5):
        g = torch.view_as_real(got[c])
        assert not torch.isfinite(g).all()
