"""GeometricH1Loss on the HIP transform (makani/utils/losses.py:268-360).

CPU part: the float64 restatement (oracle.losses) against what the mathematics fixes -- the closed form for a single
harmonic (pins the weights 1 / 2 of the orders and l(l+1) of the degrees) and Parseval on a Legendre-Gauss grid.
GPU part: the HIP path against that restatement (rel 1e-5, the fp32 bound of the path) and, for the gradient, against
torch autograd in float64 through the restated op sequence.
"""
import numpy as np
import pytest
import torch

from oracle.losses import GeometricH1Loss as OracleH1, degree_power
from oracle.sht import ShtTables, sht_forward, sht_inverse
from oracle.torch_ref import TorchRefSHT


@pytest.mark.parametrize("l,m", [(0, 0), (3, 0), (5, 2), (9, 9)])
def test_oracle_loss_single_harmonic(l, m):
    nlat, nlon, alpha, a = 16, 32, 0.3, 0.7 - 0.4j
    t = ShtTables(nlat, nlon, None, None, "legendre-gauss")
    c = np.zeros((1, 1, t.lmax, t.mmax), dtype=np.complex128)
    c[0, 0, l, m] = a.real if m == 0 else a
    f = sht_inverse(c, t)
    p = (abs(a.real) if m == 0 else abs(a)) ** 2 * (1.0 if m == 0 else 2.0)
    loss = OracleH1((nlat, nlon), absolute=True, alpha=alpha, grid="legendre-gauss")
    want = alpha * np.sqrt(p) + (1 - alpha) * np.sqrt(l * (l + 1) * p)
    assert abs(loss(f, np.zeros_like(f)) - want) < 1e-12 * max(1.0, want)
    sq = OracleH1((nlat, nlon), absolute=True, squared=True, alpha=alpha, grid="legendre-gauss")
    assert abs(sq(f, np.zeros_like(f)) - (alpha * p + (1 - alpha) * l * (l + 1) * p)) < 1e-12 * max(1.0, want * want)


def test_oracle_power_is_parseval():
    nlat, nlon = 12, 24
    t = ShtTables(nlat, nlon, None, None, "legendre-gauss")
    rng = np.random.default_rng(3)
    c = rng.standard_normal((2, 3, t.lmax, t.mmax)) + 1j * rng.standard_normal((2, 3, t.lmax, t.mmax))
    c[..., 0] = c[..., 0].real
    c[..., -1] = 0                                 # the Nyquist order of a real field is not free
    c *= np.tril(np.ones((t.lmax, t.mmax)))        # only m <= l exists
    f = sht_inverse(c, t)
    integral = (f ** 2 * t.quad_w[:, None]).sum(axis=(-2, -1)) * 2 * np.pi / nlon
    assert np.allclose(degree_power(sht_forward(f, t)).sum(axis=-1), integral, rtol=1e-12)


def _fields(seed, shape):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g), torch.randn(*shape, generator=g)


@pytest.mark.gpu
@pytest.mark.parametrize("nlat,nlon,lead", [(32, 64, (2, 4)), (33, 64, (3,)), (91, 180, (2, 5))])
def test_degree_power_matches_oracle(lib_built, nlat, nlon, lead):
    import makani_amd as ma
    from makani_amd.losses import degree_power as hip_power

    print(f"case degree power {nlat}x{nlon} lead={lead}", flush=True)
    x, _ = _fields(31, (*lead, nlat, nlon))
    sht = ma.RealSHT(nlat, nlon, grid="equiangular")
    got = hip_power(sht, x.cuda()).cpu().double().numpy()
    t = ShtTables(nlat, nlon, None, None, "equiangular")
    ref = degree_power(sht_forward(x.double().numpy(), t))
    assert got.shape == ref.shape
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("absolute,squared,size_average,reduction,mask", [
    (False, False, False, True, False),            # the reference's defaults
    (True, False, False, True, False),
    (True, True, True, True, False),
    (False, True, False, False, False),
    (False, False, True, True, True),
    (False, False, False, True, True),
])
def test_h1_loss_matches_oracle(lib_built, absolute, squared, size_average, reduction, mask):
    from makani_amd.losses import GeometricH1Loss

    nlat, nlon, B, C = 32, 64, 3, 4
    print(f"case h1 loss abs={absolute} sq={squared} avg={size_average} red={reduction} mask={mask}", flush=True)
    prd, tar = _fields(32, (B, C, nlat, nlon))
    kw = dict(absolute=absolute, squared=squared, size_average=size_average, reduction=reduction, alpha=0.4)
    m = torch.tensor([1.0, 0.0, 1.0]) if mask else None
    got = GeometricH1Loss((nlat, nlon), **kw).cuda()(prd.cuda(), tar.cuda(), m.cuda() if mask else None)
    ref = OracleH1((nlat, nlon), **kw)(prd.numpy(), tar.numpy(), m.numpy() if mask else None)
    assert np.allclose(got.detach().cpu().double().numpy(), ref, rtol=1e-5, atol=0)


@pytest.mark.gpu
@pytest.mark.parametrize("absolute,squared", [(False, False), (True, True)])
def test_h1_loss_gradient(lib_built, absolute, squared):
    """d loss / d prd against float64 autograd through the restated op sequence (rfft, einsum with the dense table,
    power, weights, norms)."""
    from makani_amd.losses import GeometricH1Loss

    nlat, nlon, B, C, alpha = 33, 64, 2, 3, 0.5
    print(f"case h1 loss gradient abs={absolute} sq={squared}", flush=True)
    prd, tar = _fields(33, (B, C, nlat, nlon))
    x = prd.cuda().requires_grad_(True)
    loss = GeometricH1Loss((nlat, nlon), absolute=absolute, squared=squared, alpha=alpha).cuda()
    loss(x, tar.cuda()).backward()

    ref_sht = TorchRefSHT(nlat, nlon, grid="equiangular", directions=("fwd",), dtype=torch.float64)
    h1 = torch.arange(ref_sht.lmax, dtype=torch.float64)
    h1 = h1 * (h1 + 1)

    def norms(f):
        c = torch.view_as_real(ref_sht.forward(f))
        p = c[..., 0] ** 2 + c[..., 1] ** 2
        n2 = p[..., :, 0] + 2 * p[..., :, 1:].sum(dim=-1)
        l2, hh = n2.reshape(B, -1).sum(-1), (n2 * h1).reshape(B, -1).sum(-1)
        return alpha * l2 + (1 - alpha) * hh if squared else alpha * l2.sqrt() + (1 - alpha) * hh.sqrt()

    xr = prd.double().requires_grad_(True)
    v = norms(xr - tar.double())
    (v if absolute else v / norms(tar.double())).sum().backward()
    g, gr = x.grad.cpu().double(), xr.grad
    assert float(torch.linalg.norm(g - gr) / torch.linalg.norm(gr)) < 1e-5
