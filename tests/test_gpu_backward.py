"""GPU parity of the backward (adjoint) kernels.

The reference has no hand-written backward: autograd differentiates its einsum + FFT op sequence.
The gradient oracle is therefore torch autograd (CPU, float64) through oracle.torch_ref, the
restatement of that op sequence; tolerance as for the forward pass (rel-L2 <= 1e-5 in fp32).
"""
import numpy as np
import pytest
import torch

from oracle.torch_ref import TorchRefSHT

pytestmark = pytest.mark.gpu
TOL = 1e-5


def rel_l2(a, b):
    a, b = a.detach().cpu(), b.detach().cpu()
    if a.is_complex():
        a, b = torch.view_as_real(a.resolve_conj()), torch.view_as_real(b.resolve_conj())
    a, b = a.double(), b.double()
    return float(torch.linalg.norm((a - b).ravel()) / max(float(torch.linalg.norm(b.ravel())), 1e-300))


SHT_CASES = [
    # nlat, nlon, lmax, mmax, grid, norm, lead
    (12, 24, None, None, "legendre-gauss", "ortho", (2, 3)),
    (33, 64, 33, 33, "equiangular", "ortho", (5,)),
    (17, 30, None, None, "lobatto", "four-pi", (1, 4)),
    (16, 31, 12, 10, "legendre-gauss", "schmidt", (3,)),     # odd nlon: no Nyquist bin, truncated orders
    (91, 180, 91, 91, "equiangular", "ortho", (7,)),
    (20, 38, 20, 20, "legendre-gauss", "ortho", (4,)),        # mmax = nlon/2 + 1: Nyquist bin kept
]


@pytest.mark.parametrize("nlat,nlon,lmax,mmax,grid,norm,lead", SHT_CASES)
def test_forward_sht_backward(lib_built, nlat, nlon, lmax, mmax, grid, norm, lead):
    import makani_amd as ma

    print(f"case sht-fwd-bwd {nlat}x{nlon} l{lmax} m{mmax} {grid} {norm} lead={lead}", flush=True)
    torch.manual_seed(5)
    mod = ma.RealSHT(nlat, nlon, lmax, mmax, grid=grid, norm=norm)
    ref = TorchRefSHT(nlat, nlon, lmax, mmax, grid, norm, directions=("fwd",), dtype=torch.float64)
    x = torch.randn(*lead, nlat, nlon)
    g = torch.randn(*lead, mod.lmax, mod.mmax, dtype=torch.complex64)
    xr = x.double().requires_grad_(True)
    ref.forward(xr).backward(g.to(torch.complex128))
    xg = x.cuda().requires_grad_(True)
    y = mod(xg)
    y.backward(g.cuda())
    torch.cuda.synchronize()
    assert xg.grad.shape == x.shape and xg.grad.dtype == torch.float32
    assert rel_l2(xg.grad, xr.grad) < TOL


@pytest.mark.parametrize("nlat,nlon,lmax,mmax,grid,norm,lead", SHT_CASES)
def test_inverse_sht_backward(lib_built, nlat, nlon, lmax, mmax, grid, norm, lead):
    import makani_amd as ma

    print(f"case sht-inv-bwd {nlat}x{nlon} l{lmax} m{mmax} {grid} {norm} lead={lead}", flush=True)
    torch.manual_seed(6)
    mod = ma.InverseRealSHT(nlat, nlon, lmax, mmax, grid=grid, norm=norm)
    ref = TorchRefSHT(nlat, nlon, lmax, mmax, grid, norm, directions=("inv",), dtype=torch.float64)
    c = torch.randn(*lead, mod.lmax, mod.mmax, dtype=torch.complex64)
    g = torch.randn(*lead, nlat, nlon)
    cr = c.to(torch.complex128).requires_grad_(True)
    ref.inverse(cr).backward(g.double())
    cg = c.cuda().requires_grad_(True)
    mod(cg).backward(g.cuda())
    torch.cuda.synchronize()
    # the dense reference table is zero for m > l, and so is its gradient there
    assert cg.grad.shape == c.shape and cg.grad.dtype == torch.complex64
    assert rel_l2(cg.grad, cr.grad) < TOL


def test_sht_adjoint_dot_product_full_size(lib_built):
    """<S x, y> = <x, S^T y> and the same for the inverse at 721 x 1440 (config 1 size, 2 channels)."""
    import makani_amd as ma

    print("case sht adjoint identity 721x1440", flush=True)
    torch.manual_seed(7)
    nlat, nlon = 721, 1440
    fwd = ma.RealSHT(nlat, nlon, grid="equiangular")
    inv = ma.InverseRealSHT(nlat, nlon, grid="equiangular")
    x = torch.randn(2, nlat, nlon, device="cuda", requires_grad=True)
    y = torch.randn(2, fwd.lmax, fwd.mmax, dtype=torch.complex64, device="cuda")
    out = fwd(x)
    out.backward(y)
    lhs = float((torch.view_as_real(out.detach()).double() * torch.view_as_real(y).double()).sum())
    rhs = float((x.detach().double() * x.grad.double()).sum())
    assert abs(lhs - rhs) < 1e-6 * float(torch.linalg.norm(out.detach()) * torch.linalg.norm(y))
    # the inverse reads only m <= l
    l = torch.arange(inv.lmax, device="cuda")[:, None]
    m = torch.arange(inv.mmax, device="cuda")[None, :]
    c = (torch.randn(2, inv.lmax, inv.mmax, dtype=torch.complex64, device="cuda") * (m <= l)).requires_grad_(True)
    g = torch.randn(2, nlat, nlon, device="cuda")
    z = inv(c)
    z.backward(g)
    lhs = float((z.detach().double() * g.double()).sum())
    rhs = float((torch.view_as_real(c.detach()).double() * torch.view_as_real(c.grad).double()).sum())
    assert abs(lhs - rhs) < 1e-6 * float(torch.linalg.norm(z.detach()) * torch.linalg.norm(g))
    assert float(torch.abs(c.grad * (m > l)).max()) == 0.0


@pytest.mark.parametrize(
    "B,I,O,L,M",
    [(1, 3, 2, 4, 5), (2, 8, 8, 6, 7), (1, 20, 36, 33, 33), (3, 17, 5, 12, 9), (1, 70, 130, 21, 22), (2, 64, 48, 40, 41)],
)
def test_contract_dhconv_backward(lib_built, B, I, O, L, M):
    import makani_amd as ma

    print(f"case dhconv-bwd B={B} I={I} O={O} L={L} M={M}", flush=True)
    torch.manual_seed(8)
    x = torch.randn(B, I, L, M, dtype=torch.complex64)
    w = torch.randn(I, O, L, dtype=torch.complex64) / np.sqrt(I)
    g = torch.randn(B, O, L, M, dtype=torch.complex64)
    xr = x.to(torch.complex128).requires_grad_(True)
    wr = w.to(torch.complex128).requires_grad_(True)
    torch.einsum("bixy,iox->boxy", xr, wr).backward(g.to(torch.complex128))
    xg = x.cuda().requires_grad_(True)
    wg = w.cuda().requires_grad_(True)
    ma._contract_dhconv(xg, wg).backward(g.cuda())
    torch.cuda.synchronize()
    assert rel_l2(xg.grad, xr.grad) < TOL
    assert rel_l2(wg.grad, wr.grad) < TOL


@pytest.mark.parametrize("scale", ["same", "down"])
def test_spectral_conv_backward(lib_built, scale):
    """Fused SpectralConv path (spectral layout end to end): gradients of input, weight and bias."""
    import makani_amd as ma

    print(f"case spectralconv-bwd {scale}", flush=True)
    torch.manual_seed(9)
    nlat, nlon = 24, 48
    nlat_o, nlon_o = (24, 48) if scale == "same" else (12, 24)
    lmax = mmax = 12
    B, C, O = 2, 6, 5
    fwd = ma.RealSHT(nlat, nlon, lmax, mmax, grid="equiangular")
    inv = ma.InverseRealSHT(nlat_o, nlon_o, lmax, mmax, grid="legendre-gauss")
    conv = ma.SpectralConv(fwd, inv, C, O, operator_type="dhconv", bias="constant").cuda()
    rf = TorchRefSHT(nlat, nlon, lmax, mmax, "equiangular", directions=("fwd",), dtype=torch.float64)
    ri = TorchRefSHT(nlat_o, nlon_o, lmax, mmax, "legendre-gauss", directions=("inv",), dtype=torch.float64)
    x = torch.randn(B, C, nlat, nlon)
    g = torch.randn(B, O, nlat_o, nlon_o)
    gres = torch.randn(B, C, nlat_o, nlon_o)

    xr = x.double().requires_grad_(True)
    wr = conv.weight.detach().cpu().to(torch.complex128).requires_grad_(True)
    br = conv.bias.detach().cpu().double().requires_grad_(True)
    spec = rf.forward(xr)
    res_r = ri.inverse(spec)                     # the reference recomputes the residual when the grids differ
    out_r = ri.inverse(torch.einsum("bixy,iox->boxy", spec, wr)) + br
    ((out_r * g.double()).sum() + (res_r * gres.double()).sum()).backward()

    xg = x.cuda().requires_grad_(True)
    out, res = conv(xg)
    ((out * g.cuda()).sum() + (res * gres.cuda()).sum()).backward()
    torch.cuda.synchronize()
    assert rel_l2(out, out_r) < TOL and rel_l2(res, res_r) < TOL
    assert rel_l2(xg.grad, xr.grad) < TOL
    assert rel_l2(conv.weight.grad, wr.grad) < TOL
    assert rel_l2(conv.bias.grad, br.grad) < TOL


def test_weight_grad_config2_size(lib_built):
    """Weight gradient at the config-2 block size (384 x 384 channels, 240 degrees) against a channel slice
    computed in float64, plus linearity in the output gradient."""
    import makani_amd as ma
    from makani_amd.contractions import dhconv_spectral
    from makani_amd._lib import lib

    print("case wgrad 384x384x240", flush=True)
    torch.manual_seed(10)
    I = O = 384
    L, M = 240, 241
    ld = int(lib.sfno_spectral_ld(I))
    spec = torch.randn(M, L, ld, device="cuda")
    w = (torch.randn(I, O, L, dtype=torch.complex64, device="cuda") / np.sqrt(I)).requires_grad_(True)
    g = torch.randn(M, L, ld, device="cuda")
    dhconv_spectral(spec, w, 1, M, triangular=True).backward(g)
    torch.cuda.synchronize()
    gw = w.grad.clone()
    # reference for input channels 5..8 and output channels 100..103
    xs = torch.view_as_complex(spec[:, :, : 2 * I].reshape(M, L, I, 2))[:, :, 5:9].cpu().to(torch.complex128)
    gs = torch.view_as_complex(g[:, :, : 2 * O].reshape(M, L, O, 2))[:, :, 100:104].cpu().to(torch.complex128)
    mask = (torch.arange(M)[:, None] <= torch.arange(L)[None, :]).to(torch.complex128)
    ref = torch.einsum("mli,mlo,ml->iol", xs.conj(), gs, mask)
    assert rel_l2(gw[5:9, 100:104], ref) < TOL
    w.grad = None
    dhconv_spectral(spec, w, 1, M, triangular=True).backward(2.0 * g)
    torch.cuda.synchronize()
    assert rel_l2(w.grad, 2.0 * gw) < 1e-6


def test_sfno_training_step_gradients(lib_built):
    """loss.backward() through the whole SFNO network (the reference's own model test checks that the input
    receives a gradient, tests/test_models.py:149-157).  The reference run keeps the same PyTorch modules but
    evaluates every spectral operator with the float64 torch restatement, differentiated by autograd."""
    import makani_amd.sht as sht
    from makani_amd.sfnonet import SphericalFourierNeuralOperatorNet
    from makani_amd.spectral_convolution import SpectralConv

    print("case sfno training step", flush=True)
    torch.manual_seed(11)
    net = SphericalFourierNeuralOperatorNet(inp_shape=(33, 64), out_shape=(33, 64), inp_chans=3, out_chans=3, scale_factor=2,
                                            embed_dim=16, num_layers=2).cuda().train()
    x = torch.randn(2, 3, 33, 64, generator=torch.Generator().manual_seed(12)).cuda()
    g = torch.randn(2, 3, 33, 64, generator=torch.Generator().manual_seed(13)).cuda()

    def step():
        net.zero_grad(set_to_none=True)
        xi = x.clone().requires_grad_(True)
        (net(xi) * g).sum().backward()
        torch.cuda.synchronize()
        grads = {n: p.grad.detach().clone() for n, p in net.named_parameters() if p.grad is not None}
        grads["input"] = xi.grad.detach().clone()
        return grads

    got = step()
    assert "input" in got and all(n in got for n, p in net.named_parameters() if p.requires_grad)

    refs = {}

    def ref_for(mod, direction):
        key = (id(mod), direction)
        if key not in refs:
            refs[key] = TorchRefSHT(mod.nlat, mod.nlon, mod.lmax, mod.mmax, mod.grid, mod.norm, directions=(direction,), dtype=torch.float64)
        return refs[key]

    def ref_forward(self, inp):
        return ref_for(self, "fwd").forward(inp.double().cpu()).to(torch.complex64).to(inp.device)

    def ref_inverse(self, c):
        return ref_for(self, "inv").inverse(c.to(torch.complex128).cpu()).float().to(c.device)

    convs = [m for m in net.modules() if isinstance(m, SpectralConv)]
    saved = (sht.RealSHT.forward, sht.InverseRealSHT.forward)
    try:
        sht.RealSHT.forward, sht.InverseRealSHT.forward = ref_forward, ref_inverse
        for c in convs:
            c._fused = False
            c._contract = lambda a, w, **kw: torch.einsum("bixy,iox->boxy", a, w)
        want = step()
    finally:
        sht.RealSHT.forward, sht.InverseRealSHT.forward = saved
    assert set(got) == set(want)
    # some gradients vanish identically (a bias in front of an instance norm) and hold rounding noise only:
    # errors are measured against the gradient's own norm, but not below 1 % of the largest gradient norm
    def norm(t):
        return float(torch.linalg.norm(torch.view_as_real(t) if t.is_complex() else t))

    gmax = max(norm(want[n]) for n in want)
    assert gmax > 0
    for n in got:
        assert norm(got[n] - want[n]) < 1e-4 * max(norm(want[n]), 1e-2 * gmax), n


@pytest.mark.parametrize("spectral", [False, True])
def test_inverse_with_surplus_orders_backward(lib_built, spectral):
    """An inverse transform may keep more orders than its longitude grid resolves (mmax > nlon // 2 + 1): the surplus is
    dropped like a complex-to-real FFT drops it, so its gradient is exactly zero and the rest equals the gradient of the
    reference op sequence (float64 autograd through the einsum + irfft, which crops the same way)."""
    import makani_amd as ma

    nlat, nlon, lmax, mmax = 12, 16, 12, 12
    print(f"case sht-inv-bwd surplus orders {nlat}x{nlon} l{lmax} m{mmax} spectral={spectral}", flush=True)
    torch.manual_seed(16)
    mod = ma.InverseRealSHT(nlat, nlon, lmax, mmax, grid="legendre-gauss")
    ref = TorchRefSHT(nlat, nlon, lmax, mmax, "legendre-gauss", "ortho", directions=("inv",), dtype=torch.float64)
    c = torch.randn(2, 3, lmax, mmax, dtype=torch.complex64)
    g = torch.randn(2, 3, nlat, nlon)
    cr = c.to(torch.complex128).requires_grad_(True)
    ref.inverse(cr).backward(g.double())
    cg = c.cuda().requires_grad_(True)
    if spectral:
        # the same transform on the order-major layout, as SpectralConv chains it
        from makani_amd.contractions import _to_spectral
        from makani_amd._lib import lib, check
        import ctypes

        spec = _to_spectral(c.cuda().contiguous(), 6, lmax, mmax, True).requires_grad_(True)
        mod.synthesis(spec, (2, 3)).backward(g.cuda())
        gs = spec.grad
        assert tuple(gs.shape) == mod.spectral_shape(6) and float(gs[nlon // 2 + 1:].abs().max()) == 0.0
        grad = torch.empty(2, 3, lmax, mmax, dtype=torch.complex64, device="cuda")
        check(lib.sfno_spectral_to_coeffs(ctypes.c_void_p(gs.contiguous().data_ptr()), ctypes.c_void_p(grad.data_ptr()), 6, lmax, mmax, 1,
                                          ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)), "to_coeffs")
    else:
        mod(cg).backward(g.cuda())
        grad = cg.grad
    torch.cuda.synchronize()
    assert grad.shape == c.shape
    assert float(grad[..., nlon // 2 + 1:].abs().max()) == 0.0 and float(cr.grad[..., nlon // 2 + 1:].abs().max()) == 0.0
    assert rel_l2(grad, cr.grad) < TOL
