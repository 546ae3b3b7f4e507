"""GPU parity of the dhconv contraction and of SpectralConv against the oracle (rel-L2 <= 1e-5, fp32)."""
import numpy as np
import pytest
import torch

from oracle.dhconv import dhconv, spectral_conv
from oracle.sht import ShtTables

pytestmark = pytest.mark.gpu
TOL = 1e-5


def rel_l2(a, b):
    return np.linalg.norm((np.asarray(a) - np.asarray(b)).ravel()) / max(np.linalg.norm(np.asarray(b).ravel()), 1e-300)


@pytest.mark.parametrize(
    "B,I,O,L,M",
    # even in_channels run on the bf16 matrix pipe with operands cut into three bf16 planes, odd ones on fp32 MFMA
    [(1, 3, 2, 4, 5), (2, 8, 8, 6, 7), (1, 20, 36, 33, 33), (3, 17, 5, 12, 9), (1, 64, 48, 40, 41), (4, 24, 24, 70, 71),
     (1, 384, 384, 24, 25), (2, 6, 70, 9, 9)],
)
def test_contract_dhconv_full(lib_built, B, I, O, L, M):
    import makani_amd as ma

    print(f"case dhconv B={B} I={I} O={O} L={L} M={M}", flush=True)
    torch.manual_seed(2)
    # magnitudes over several decades and all 24 significant bits in use
    x = torch.randn(B, I, L, M, dtype=torch.complex64) * torch.exp(2.0 * torch.randn(B, I, 1, 1))
    w = torch.randn(I, O, L, dtype=torch.complex64) / np.sqrt(I) * torch.exp(2.0 * torch.randn(1, O, 1))
    got = ma._contract_dhconv(x.cuda(), w.cuda())
    torch.cuda.synchronize()
    ref = dhconv(x.numpy().astype(np.complex128), w.numpy().astype(np.complex128))
    assert got.shape == ref.shape and got.is_contiguous()
    err = rel_l2(got.cpu().numpy(), ref)
    print(f"   rel-L2 {err:.2e}", flush=True)
    assert err < TOL
    # per output channel as well: a channel of small magnitude must not drown in the error of a large one
    for o in range(0, O, max(1, O // 7)):
        assert rel_l2(got.cpu().numpy()[:, o], ref[:, o]) < TOL


def test_contract_fun_interface(lib_built):
    import makani_amd as ma

    w = torch.randn(4, 4, 6, dtype=torch.complex64).cuda()
    f = ma.get_contract_fun(w, implementation="factorized", separable=False, complex=True, operator_type="dhconv")
    x = torch.randn(1, 4, 6, 7, dtype=torch.complex64).cuda()
    y = f(x, w, separable=False, operator_type="dhconv")
    ref = torch.einsum("bixy,iox->boxy", x.cpu(), w.cpu())
    assert rel_l2(y.cpu().numpy(), ref.numpy()) < TOL
    with pytest.raises(ValueError):
        f(x, w, operator_type="nonsense")


def test_weight_update_is_seen(lib_built):
    import makani_amd as ma

    w = torch.randn(4, 4, 6, dtype=torch.complex64).cuda()
    x = torch.randn(1, 4, 6, 7, dtype=torch.complex64).cuda()
    y0 = ma._contract_dhconv(x, w)
    w.mul_(2.0)
    y1 = ma._contract_dhconv(x, w)
    assert rel_l2(y1.cpu().numpy(), 2 * y0.cpu().numpy()) < 1e-6


@pytest.mark.parametrize(
    "fwd,inv,B,C,O",
    [
        ((33, 64, 16, 17, "equiangular"), (16, 32, 16, 17, "legendre-gauss"), 2, 6, 4),   # down-scaling block (residual re-synthesised)
        ((16, 32, 16, 17, "legendre-gauss"), (16, 32, 16, 17, "legendre-gauss"), 1, 8, 8),  # same-grid block
        ((16, 32, 16, 17, "legendre-gauss"), (33, 64, 16, 17, "equiangular"), 3, 5, 7),   # up-scaling block, odd channel counts
        ((48, 96, 48, 49, "legendre-gauss"), (48, 96, 48, 49, "legendre-gauss"), 1, 40, 40),
    ],
)
def test_spectral_conv_matches_oracle(lib_built, fwd, inv, B, C, O):
    import makani_amd as ma

    print(f"case spectral_conv fwd={fwd} inv={inv} B={B} C={C} O={O}", flush=True)
    torch.manual_seed(4)
    ft = ma.RealSHT(fwd[0], fwd[1], lmax=fwd[2], mmax=fwd[3], grid=fwd[4])
    it = ma.InverseRealSHT(inv[0], inv[1], lmax=inv[2], mmax=inv[3], grid=inv[4])
    conv = ma.SpectralConv(ft, it, C, O, operator_type="dhconv", gain=2.0).cuda()
    assert tuple(conv.weight.shape) == (C, O, inv[2]) and conv.weight.dtype == torch.complex64
    assert list(conv.state_dict().keys()) == ["weight"]
    x = torch.randn(B, C, fwd[0], fwd[1])
    with torch.no_grad():
        y, res = conv(x.cuda())
    torch.cuda.synchronize()
    y_ref, res_ref = spectral_conv(x.double().numpy(), conv.weight.detach().cpu().numpy().astype(np.complex128), ShtTables(*fwd), ShtTables(*inv))
    assert y.shape == y_ref.shape and res.shape == res_ref.shape
    assert rel_l2(y.cpu().numpy(), y_ref) < TOL
    assert rel_l2(res.cpu().numpy(), res_ref) < TOL


@pytest.mark.parametrize("B,I,O,L,M", [(1, 4, 2, 4, 5), (2, 8, 8, 6, 7), (1, 64, 48, 40, 41), (3, 18, 6, 12, 9), (1, 384, 384, 24, 25), (4, 24, 200, 70, 71)])
def test_contract_dhconv_bf16(lib_built, B, I, O, L, M):
    """bf16 MFMA variant (inputs rounded to bf16, fp32 accumulation): relative L2 <= 1e-2 against the float64 oracle."""
    import makani_amd as ma

    print(f"case dhconv bf16 B={B} I={I} O={O} L={L} M={M}", flush=True)
    torch.manual_seed(2)
    x = torch.randn(B, I, L, M, dtype=torch.complex64)
    w = torch.randn(I, O, L, dtype=torch.complex64) / np.sqrt(I)
    got = ma._contract_dhconv(x.cuda(), w.cuda(), compute="bf16")
    torch.cuda.synchronize()
    ref = dhconv(x.numpy().astype(np.complex128), w.numpy().astype(np.complex128))
    err = rel_l2(got.cpu().numpy(), ref)
    assert err < 1e-2
    # and it really is a reduced-precision path: exact bf16 rounding of the inputs reproduces it much more closely
    xb = torch.view_as_complex(torch.view_as_real(x).to(torch.bfloat16).float())
    wb = torch.view_as_complex(torch.view_as_real(w).to(torch.bfloat16).float())
    ref_b = dhconv(xb.numpy().astype(np.complex128), wb.numpy().astype(np.complex128))
    assert rel_l2(got.cpu().numpy(), ref_b) < 1e-5


@pytest.mark.parametrize("B,I,O,L,M", [(1, 3, 2, 4, 5), (2, 8, 8, 6, 7), (5, 17, 5, 12, 9), (1, 32, 48, 33, 34), (6, 4, 3, 7, 7)])
def test_contract_diagonal_and_its_gradients(lib_built, B, I, O, L, M):
    """operator_type "diagonal" (contractions.py:121-127): values against the oracle, gradients against float64 autograd
    of the same einsum (odd L*M exercises the unaligned path, B > 4 the batch loop)."""
    import makani_amd as ma
    from oracle.dhconv import diagonal

    print(f"case diagonal B={B} I={I} O={O} L={L} M={M}", flush=True)
    torch.manual_seed(3)
    x = torch.randn(B, I, L, M, dtype=torch.complex64)
    w = torch.randn(I, O, L, M, dtype=torch.complex64) / np.sqrt(I)
    g = torch.randn(B, O, L, M, dtype=torch.complex64)
    xg, wg = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    y = ma._contract_diagonal(xg, wg)
    y.backward(g.cuda())
    torch.cuda.synchronize()
    assert rel_l2(y.detach().cpu().numpy(), diagonal(x.numpy().astype(np.complex128), w.numpy().astype(np.complex128))) < TOL
    xr, wr = x.to(torch.complex128).requires_grad_(True), w.to(torch.complex128).requires_grad_(True)
    torch.einsum("bixy,ioxy->boxy", xr, wr).backward(g.to(torch.complex128))
    assert rel_l2(xg.grad.cpu().numpy(), xr.grad.numpy()) < TOL
    assert rel_l2(wg.grad.cpu().numpy(), wr.grad.numpy()) < TOL
    f = ma.get_contract_fun(wg, implementation="factorized", separable=False, complex=True, operator_type="diagonal")
    assert torch.equal(f(xg.detach(), wg.detach(), separable=False, operator_type="diagonal"), y.detach())


def test_spectral_conv_diagonal(lib_built):
    """SpectralConv with operator_type="diagonal" against the oracle (weight [I, O, L, M], lmax == mmax as the
    reference's initialisation requires)."""
    import makani_amd as ma

    torch.manual_seed(4)
    fwd = ma.RealSHT(16, 32, lmax=12, mmax=12, grid="legendre-gauss")
    inv = ma.InverseRealSHT(16, 32, lmax=12, mmax=12, grid="legendre-gauss")
    conv = ma.SpectralConv(fwd, inv, 5, 3, operator_type="diagonal").cuda()
    assert tuple(conv.weight.shape) == (5, 3, 12, 12)
    x = torch.randn(2, 5, 16, 32)
    y, res = conv(x.cuda())
    torch.cuda.synchronize()
    t = ShtTables(16, 32, 12, 12, "legendre-gauss")
    ref, _ = spectral_conv(x.double().numpy(), conv.weight.detach().cpu().numpy().astype(np.complex128), t, t)
    assert rel_l2(y.detach().cpu().numpy(), ref) < TOL
    assert torch.equal(res, x.cuda())


def test_packed_weight_cache_and_data_writes(lib_built):
    """The packed operand copy follows in-place updates through the parameter's version counter; a write through ``.data``
    leaves that counter alone and needs the explicit invalidation hook."""
    import makani_amd as ma
    from makani_amd import contractions

    torch.manual_seed(8)
    ft = ma.RealSHT(16, 32, lmax=16, mmax=17, grid="legendre-gauss")
    it = ma.InverseRealSHT(16, 32, lmax=16, mmax=17, grid="legendre-gauss")
    conv = ma.SpectralConv(ft, it, 4, 4, operator_type="dhconv").cuda()
    x = torch.randn(1, 4, 16, 32).cuda()
    with torch.no_grad():
        y0, _ = conv(x)
        conv.weight.data.mul_(3.0)             # invisible to the cache
        y_stale, _ = conv(x)
        conv.invalidate_packed()
        y1, _ = conv(x)
        conv.weight.data.mul_(2.0)
        contractions.clear_cache()             # the module-wide form
        y2, _ = conv(x)
    torch.cuda.synchronize()
    assert torch.equal(y_stale, y0)
    assert rel_l2(y1.cpu().numpy(), 3 * y0.cpu().numpy()) < 1e-6
    assert rel_l2(y2.cpu().numpy(), 6 * y0.cpu().numpy()) < 1e-6


@pytest.mark.parametrize("updown", [False, True])
def test_spectral_conv_empty_batch(lib_built, updown):
    """Batch size 0 returns empty tensors of the right shape, as the reference's einsum path does."""
    import makani_amd as ma

    ft = ma.RealSHT(33, 64, lmax=16, mmax=17, grid="equiangular") if updown else ma.RealSHT(16, 32, lmax=16, mmax=17, grid="legendre-gauss")
    it = ma.InverseRealSHT(16, 32, lmax=16, mmax=17, grid="legendre-gauss")
    conv = ma.SpectralConv(ft, it, 6, 4, operator_type="dhconv").cuda()
    x = torch.empty(0, 6, ft.nlat, ft.nlon, device="cuda")
    with torch.no_grad():
        y, res = conv(x)
    assert tuple(y.shape) == (0, 4, 16, 32)
    assert tuple(res.shape) == ((0, 6, 16, 32) if updown else (0, 6, 16, 32))
    xg = torch.empty(0, 6, ft.nlat, ft.nlon, device="cuda", requires_grad=True)
    y, _ = conv(xg)
    y.sum().backward()
    assert tuple(xg.grad.shape) == tuple(xg.shape) and tuple(conv.weight.grad.shape) == tuple(conv.weight.shape)
    assert float(conv.weight.grad.abs().max()) == 0.0


@pytest.mark.parametrize("operator_type", ["dhconv", "diagonal"])
def test_real_weight_contractions_and_their_gradients(lib_built, operator_type):
    """complex=False (contractions.py:157-166): activations as float32 [..., 2], real weights -- values and gradients against
    float64 autograd of the reference's einsum strings."""
    import makani_amd as ma

    print(f"case real-weight contraction {operator_type}", flush=True)
    torch.manual_seed(8)
    B, I, O, L, M = 2, 6, 4, 9, 7
    eq = "bixys,iox->boxys" if operator_type == "dhconv" else "bixys,ioxy->boxys"
    a = torch.randn(B, I, L, M, 2)
    w = torch.randn(*((I, O, L) if operator_type == "dhconv" else (I, O, L, M))) / np.sqrt(I)
    g = torch.randn(B, O, L, M, 2)
    ag, wg = a.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    f = ma.get_contract_fun(wg, implementation="factorized", separable=False, complex=False, operator_type=operator_type)
    y = f(ag, wg)
    assert y.dtype == torch.float32 and tuple(y.shape) == (B, O, L, M, 2) and y.is_contiguous()
    y.backward(g.cuda())
    torch.cuda.synchronize()
    ar, wr = a.double().requires_grad_(True), w.double().requires_grad_(True)
    yr = torch.einsum(eq, ar, wr)
    yr.backward(g.double())
    assert rel_l2(y.detach().cpu().numpy(), yr.detach().numpy()) < TOL
    assert rel_l2(ag.grad.cpu().numpy(), ar.grad.numpy()) < TOL
    assert wg.grad.dtype == torch.float32 and rel_l2(wg.grad.cpu().numpy(), wr.grad.numpy()) < TOL
    with pytest.raises(NotImplementedError):
        ma.get_contract_fun(wg, separable=True, complex=False, operator_type=operator_type)(ag, wg)
