"""GPU parity of the fused pointwise kernels (bf16 activations) against float64 PyTorch-CPU evaluation of
the same reference ops (nn.Conv2d(k=1) + bias, nn.GELU(), nn.InstanceNorm2d) on the same bf16-rounded
inputs.  The kernels accumulate in fp32 and round once, so the only difference is the final bf16
rounding: relative L2 <= 3e-3 (bf16 tolerance of the path: 1e-2)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu
TOL = 3e-3


def rel_l2(a, b):
    a, b = a.detach().cpu().double(), b.detach().cpu().double()
    return float(torch.linalg.norm((a - b).ravel()) / max(float(torch.linalg.norm(b.ravel())), 1e-300))


CONV_CASES = [
    # B, K, O, H, W, bias, act, addend, affine
    (2, 384, 768, 16, 24, True, "gelu", False, False),     # MLP fc1
    (1, 768, 384, 16, 24, True, None, False, False),       # MLP fc2
    (2, 384, 384, 13, 8, False, None, True, True),         # outer skip + norm1(y); strip shorter than a tile
    (1, 73, 384, 20, 36, True, "gelu", False, False),      # encoder fc1: K padded 73 -> 96
    (1, 384, 73, 20, 36, False, None, True, False),        # decoder fc2 + big skip (O < 96: four wavefronts along pixels)
    (3, 73, 73, 9, 8, False, None, False, False),
    (1, 100, 200, 11, 24, True, "gelu", True, True),       # nothing a multiple of the tile sizes
    (1, 8, 5, 721, 1440, True, None, False, False),        # full-resolution grid, tiny channels
    # several tiles per persistent workgroup (O > 96): the operand rings wrap and run on across tile boundaries
    (1, 100, 500, 160, 1000, True, "gelu", True, True),    # two row blocks, the second partly filled; ragged last strip
    (2, 73, 384, 125, 1000, False, None, False, False),    # four K chunks per tile, two samples
    (1, 384, 200, 90, 1000, True, None, True, False),      # twelve K chunks per tile
    (2, 128, 200, 123, 1000, True, "gelu", True, True),    # ragged last strip of every sample, several tiles per workgroup
]


@pytest.mark.parametrize("B,K,O,H,W,bias,act,addend,affine", CONV_CASES)
def test_conv1x1(lib_built, B, K, O, H, W, bias, act, addend, affine):
    from makani_amd import pointwise as pw

    print(f"case conv1x1 B={B} K={K} O={O} {H}x{W} bias={bias} act={act} addend={addend} affine={affine}", flush=True)
    g = torch.Generator().manual_seed(21)
    x = torch.randn(B, K, H, W, generator=g).bfloat16()
    w = (torch.randn(O, K, 1, 1, generator=g) / np.sqrt(K))
    bvec = torch.randn(O, generator=g) if bias else None
    r = torch.randn(B, O, H, W, generator=g).bfloat16() if addend else None
    sc = torch.randn(B, O, generator=g) if affine else None
    sh = torch.randn(B, O, generator=g) if affine else None

    ref = F.conv2d(x.double(), w.bfloat16().double(), bvec.double() if bias else None)
    if act == "gelu":
        ref = F.gelu(ref)
    if addend:
        ref = ref + (r.double() * sc.double()[:, :, None, None] + sh.double()[:, :, None, None] if affine else r.double())

    wg = w.cuda()
    got = pw.conv1x1(x.cuda(), wg, bvec.cuda() if bias else None, act, r.cuda() if addend else None,
                     sc.cuda() if affine else None, sh.cuda() if affine else None)
    torch.cuda.synchronize()
    assert got.dtype == torch.bfloat16 and got.shape == ref.shape
    assert rel_l2(got, ref) < TOL
    # the error of every element is bf16 rounding of the float64 value (plus fp32 accumulation noise)
    err = (got.cpu().double() - ref).abs()
    assert float((err - (ref.abs() * 2.0**-8 + 1e-3)).max()) <= 0.0


def test_weight_repack_on_update(lib_built):
    from makani_amd import pointwise as pw

    x = torch.randn(1, 16, 4, 8).bfloat16().cuda()
    w = torch.randn(8, 16, 1, 1).cuda()
    y0 = pw.conv1x1(x, w)
    w.mul_(2.0)
    y1 = pw.conv1x1(x, w)
    assert rel_l2(y1, 2.0 * y0.float()) < TOL


@pytest.mark.parametrize("B,C,H,W", [(2, 6, 16, 24), (1, 384, 24, 48), (1, 3, 721, 1440)])
def test_instance_norm_coeffs(lib_built, B, C, H, W):
    from makani_amd import pointwise as pw

    print(f"case instnorm B={B} C={C} {H}x{W}", flush=True)
    g = torch.Generator().manual_seed(22)
    # a mean several times the spread is the hard case for the variance; the scale/shift form itself loses
    # about eps_fp32 * |mean| / sigma of relative accuracy, so the spread is kept away from zero
    x = (torch.randn(B, C, H, W, generator=g) * (0.5 + torch.rand(B, C, 1, 1, generator=g)) + 5.0 * torch.randn(B, C, 1, 1, generator=g)).bfloat16()
    gamma, beta = torch.randn(C, generator=g), torch.randn(C, generator=g)
    ref = F.instance_norm(x.double(), weight=gamma.double(), bias=beta.double(), eps=1e-6)
    scale, shift = pw.instance_norm_coeffs(x.cuda(), gamma.cuda(), beta.cuda(), eps=1e-6)
    got = scale.cpu().double()[:, :, None, None] * x.double() + shift.cpu().double()[:, :, None, None]
    assert rel_l2(got, ref) < 1e-5
    y = pw.scale_shift_act(x.cuda(), scale, shift, None)
    torch.cuda.synchronize()
    assert rel_l2(y, ref) < TOL
    y = pw.scale_shift_act(x.cuda(), scale, shift, "gelu")
    assert rel_l2(y, F.gelu(ref)) < TOL


def test_gelu_matches_erf_form(lib_built):
    """The kernel's GELU against torch's exact (erf) GELU over [-12, 12]: equal after bf16 rounding up to one ulp
    (2^-8 relative) plus 1e-8 absolute, which only matters in the far negative tail where |gelu| < 1e-6."""
    from makani_amd import pointwise as pw

    x = torch.linspace(-12.0, 12.0, 8 * 4096).bfloat16().reshape(1, 1, 8, 4096).cuda()
    one = torch.ones(1, 1, device="cuda")
    y = pw.scale_shift_act(x, one, torch.zeros_like(one), "gelu").float().cpu()
    ref = F.gelu(x.cpu().double())
    err = (y.double() - ref).abs()
    assert float((err - ref.abs() * 2.0**-8).max()) <= 1e-8


def test_unsupported_inputs_raise(lib_built):
    from makani_amd import pointwise as pw

    w = torch.randn(4, 4, 1, 1).cuda()
    with pytest.raises(RuntimeError):
        pw.conv1x1(torch.randn(1, 4, 4, 8).cuda(), w)                 # float32 activations
    with pytest.raises(RuntimeError):
        pw.conv1x1(torch.randn(1, 4, 3, 5).bfloat16().cuda(), w)      # H*W not a multiple of 8
    with pytest.raises(RuntimeError):
        pw.conv1x1(torch.randn(1, 4, 4, 8).bfloat16(), w.cpu())       # CPU tensor


@pytest.mark.parametrize("nlat,nlon,lmax,mmax,lead,dtype", [
    (24, 64, 24, 33, (2, 5), torch.float32),          # Nyquist order kept; odd channel count (one padded slot in the last pair)
    (31, 480, 31, 40, (1, 9), torch.bfloat16),
    (40, 180, 30, 31, (3, 4), torch.bfloat16),
])
def test_instance_norm_coeffs_from_latitude_moments(lib_built, nlat, nlon, lmax, mmax, lead, dtype):
    """The inverse transform's by-product (per-latitude mean and mean squared deviation over longitude, by Parseval on the
    Fourier coefficients) gives the instance-norm statistics of the field it writes: (scale, shift) against float64
    statistics of the float32 field, and the field itself unchanged."""
    import makani_amd as ma
    from makani_amd import pointwise as pw

    print(f"case lat-moments {nlat}x{nlon} l{lmax} m{mmax} lead={lead} {dtype}", flush=True)
    torch.manual_seed(31)
    isht = ma.InverseRealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid="legendre-gauss")
    B, C = lead
    c = torch.randn(B, C, lmax, mmax, dtype=torch.complex64) * torch.exp(torch.randn(B, C, 1, 1))
    c[:, :, 0, 0] += 3.0 * torch.randn(B, C)                     # channel means well away from zero
    spec = torch.zeros(isht.spectral_shape(B * C), device="cuda")
    from makani_amd._lib import lib, check
    import ctypes
    check(lib.sfno_coeffs_to_spectral(ctypes.c_void_p(c.cuda().contiguous().data_ptr()), ctypes.c_void_p(spec.data_ptr()), B * C, lmax, mmax, 1,
                                      ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)), "to_spectral")
    torch.cuda.synchronize()
    with torch.no_grad():
        x32 = isht.synthesis(spec, (B, C))
        x, stats = isht.synthesis_with_lat_stats(spec, (B, C), dtype=dtype)
    assert stats is not None and tuple(stats.shape) == (B * C, nlat, 2)
    assert torch.equal(x, x32.to(dtype))
    gamma, beta = torch.randn(C).cuda(), torch.randn(C).cuda()
    sc, sh = pw.instance_norm_coeffs_lat(stats, B, gamma, beta, 1e-6)
    torch.cuda.synchronize()
    xd = x32.double().cpu()
    mean, var = xd.mean(dim=(2, 3)), xd.var(dim=(2, 3), unbiased=False)
    want_sc = gamma.cpu().double()[None, :] / torch.sqrt(var + 1e-6)
    want_sh = beta.cpu().double()[None, :] - mean * want_sc
    assert rel_l2(sc, want_sc) < 1e-5
    assert rel_l2(sh, want_sh) < 1e-5
    # per-latitude values themselves
    a = xd.mean(dim=3).reshape(B * C, nlat)
    d = ((xd - xd.mean(dim=3, keepdim=True)) ** 2).mean(dim=3).reshape(B * C, nlat)
    assert rel_l2(stats[..., 0], a) < 1e-5
    assert rel_l2(stats[..., 1], d) < 1e-5


def test_latitude_moments_absent_without_specialised_longitude_kernel(lib_built):
    """A longitude length served by the run-time radix kernels delivers no moments: the caller gets None and falls back to
    the statistics pass; the C entry point says unsupported."""
    import ctypes

    import makani_amd as ma
    from makani_amd._lib import lib

    isht = ma.InverseRealSHT(12, 50, lmax=12, mmax=13, grid="legendre-gauss")
    spec = torch.zeros(isht.spectral_shape(4), device="cuda")
    with torch.no_grad():
        x, stats = isht.synthesis_with_lat_stats(spec, (1, 4))
    assert stats is None and tuple(x.shape) == (1, 4, 12, 50)
    plan = isht.plan(spec.device)
    assert lib.sfno_sht_lat_stats_supported(plan.handle) == 0
    ws, nbytes = isht.workspace(plan, 4, spec.device)
    out = torch.empty(1, 4, 12, 50, device="cuda")
    st = torch.empty(4, 12, 2, device="cuda")
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.sfno_sht_synthesis_lat_stats(plan.handle, P(spec), P(out), 0, 4, P(ws), nbytes, P(st), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == -5


@pytest.mark.parametrize("nlat,nlon,lmax,mmax,C", [(721, 1440, 240, 241, 24), (64, 128, 40, 41, 10)])
def test_latitude_moments_against_statistics_of_the_rounded_field(lib_built, nlat, nlon, lmax, mmax, C):
    """norm0 on the fused path takes its statistics from the field before it is rounded to bfloat16 (the inverse transform's
    by-product), the reference's InstanceNorm2d from the rounded tensor it is given.  The means agree (rounding to nearest
    averages out); the variance of the rounded tensor is larger by the variance of the rounding error, ulp^2 / 12, which is
    1e-3 of the field's variance for a channel whose mean is ten standard deviations from zero, as in this test.  The
    normalised outputs of the two conventions therefore differ by a factor 1 +- 6e-4 around the mean: bounded here at 2e-3
    relative L2 and at 8e-3 (one bfloat16 ulp at one; measured 3.5e-3) in the largest element, in units of the normalised field."""
    import makani_amd as ma
    from makani_amd import pointwise as pw

    print(f"case lat-moments vs rounded statistics {nlat}x{nlon} C={C}", flush=True)
    torch.manual_seed(33)
    isht = ma.InverseRealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid="equiangular")
    sht = ma.RealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid="equiangular")
    field = torch.randn(1, C, nlat, nlon).cuda() + 2.0 * torch.randn(1, C, 1, 1).cuda()
    with torch.no_grad():
        spec = sht.analysis(field)
        x, stats = isht.synthesis_with_lat_stats(spec, (1, C), dtype=torch.bfloat16)
    gamma, beta = (1.0 + 0.2 * torch.randn(C)).cuda(), torch.randn(C).cuda()
    sc_l, sh_l = pw.instance_norm_coeffs_lat(stats, 1, gamma, beta, 1e-6)
    sc_r, sh_r = pw.instance_norm_coeffs(x, gamma, beta, 1e-6)
    torch.cuda.synchronize()
    xf = x.float()
    y_l = (sc_l[:, :, None, None] * xf + sh_l[:, :, None, None] - beta[None, :, None, None]) / gamma[None, :, None, None]
    y_r = (sc_r[:, :, None, None] * xf + sh_r[:, :, None, None] - beta[None, :, None, None]) / gamma[None, :, None, None]
    e2 = ((y_l - y_r).norm() / y_r.norm()).item()
    emax = (y_l - y_r).abs().max().item()
    mean_gap = ((sh_l - beta) / sc_l - (sh_r - beta) / sc_r).abs().div(xf.std(dim=(2, 3))).max().item()     # difference of the means, in standard deviations
    print(f"  normalised fields differ by {e2:.2e} (relative L2), {emax:.2e} at most; means by {mean_gap:.2e} standard deviations", flush=True)
    assert e2 < 2e-3 and emax < 8e-3 and mean_gap < 1e-3


def test_conv1x1_over_two_tensors(lib_built):
    """sfno_pointwise_conv_cat: the convolution over the channel-wise concatenation of two tensors equals the convolution of the
    concatenated tensor (same kernel, same order of the sum: bit for bit), with bias and GELU, K1 and K2 not multiples of the chunk,
    on both kernels (more and at most 96 output channels)."""
    from makani_amd import pointwise as pw

    g = torch.Generator().manual_seed(21)
    for (B, K1, K2, O, H, W) in ((1, 384, 384, 384, 24, 40), (2, 50, 77, 128, 16, 24), (1, 32, 416, 200, 8, 64), (2, 384, 73, 73, 16, 40), (1, 5, 3, 7, 8, 8),
                                 (1, 73, 100, 200, 125, 1000)):     # several tiles per persistent workgroup, odd K1
        x1 = torch.randn(B, K1, H, W, generator=g).bfloat16().cuda()
        x2 = torch.randn(B, K2, H, W, generator=g).bfloat16().cuda()
        w = (torch.randn(O, K1 + K2, generator=g) / (K1 + K2) ** 0.5).cuda()
        bias = torch.randn(O, generator=g).cuda()
        for act in (None, "gelu"):
            got = pw.conv1x1_cat(x1, x2, w, bias, act)
            want = pw.conv1x1(torch.cat([x1, x2], dim=1).contiguous(), w, bias, act)
            assert torch.equal(got, want), (B, K1, K2, O, act)
    with pytest.raises(RuntimeError):
        pw.conv1x1_cat(x1, x2, torch.randn(64, K1 + K2 + 1).cuda())      # weight of another width
