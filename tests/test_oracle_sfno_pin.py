"""Pins oracle.sfno.SfnoOracle (the network-level composition every GPU network test compares with) on the CPU.

An independent evaluation of the same network, assembled here from other primitives: spherical transforms as the defining
sums over scipy's sph_harm_y and the quadrature nodes and weights (no FFT, no Legendre table), the channel mix as explicit
loops over degrees, 1x1 convolutions as einsum, instance norm from the explicit mean and biased variance, GELU from erf.
It follows makani/models/networks/sfnonet.py:587-640 (network), 239-267 (block), makani/models/common/layers.py:86-216
and makani/models/common/spectral_convolution.py:124-148 independently of oracle/sfno.py, so a wrong eps, pad side of the
frequency position embedding, block-to-transform assignment, residual rule or op order in either fails the comparison."""
import numpy as np
import pytest
import torch
from scipy.special import erf, sph_harm_y

from oracle.quadrature import grid_nodes
from oracle.sfno import SfnoOracle


class BruteTransform:
    """x -> c[l, m] = sum_{k, n} w_k (2 pi / nlon) x[k, n] conj(Y_l^m(theta_k, phi_n)) and its synthesis
    x[k, n] = sum_l Re(c[l, 0]) Y_l^0 + 2 sum_{m >= 1} Re(c[l, m] Y_l^m): the imaginary part of the order-0 coefficients is dropped."""

    def __init__(self, nlat, nlon, lmax, mmax, grid):
        theta, w = grid_nodes(nlat, grid)
        phi = 2 * np.pi * np.arange(nlon) / nlon
        self.lmax, self.mmax = lmax, mmax
        self.Y = np.zeros((lmax, mmax, nlat, nlon), dtype=complex)
        for l in range(lmax):
            for m in range(min(l, mmax - 1) + 1):
                self.Y[l, m] = sph_harm_y(l, m, theta[:, None], phi[None, :])
        self.qw = w[:, None] * (2 * np.pi / nlon)

    def forward(self, x):
        return np.einsum("...kn,lmkn->...lm", x * self.qw, np.conj(self.Y))

    def inverse(self, c):
        x = np.einsum("...l,lkn->...kn", c[..., 0].real, self.Y[:, 0].real)
        return x + 2 * np.einsum("...lm,lmkn->...kn", c[..., 1:], self.Y[:, 1:]).real


def gelu(x):
    return 0.5 * x * (1.0 + erf(x / np.sqrt(2.0)))


def conv(x, sd, name):
    y = np.einsum("oi,bihw->bohw", sd[name + ".weight"][:, :, 0, 0], x)
    return y + sd[name + ".bias"][None, :, None, None] if name + ".bias" in sd else y


def inorm(x, sd, name, eps=1e-6):
    mean = x.mean(axis=(2, 3), keepdims=True)
    var = ((x - mean) ** 2).mean(axis=(2, 3), keepdims=True)
    return (x - mean) / np.sqrt(var + eps) * sd[name + ".weight"][None, :, None, None] + sd[name + ".bias"][None, :, None, None]


def independent_forward(sd, x, down, mid, up, num_layers, eps=1e-6):
    sd = {k: v.detach().cpu().numpy().astype(np.complex128 if v.is_complex() else np.float64) for k, v in sd.items()}
    residual = x
    y = conv(gelu(conv(x, sd, "encoder.fwd.0")), sd, "encoder.fwd.2")
    if "pos_embed.0" in sd:
        re, im = sd["pos_embed.0"], sd["pos_embed.1"]
        c = re.astype(complex)
        c[..., 1:] += 1j * im               # the imaginary parts belong to the orders m >= 1
        y = y + up.inverse(c)
    for i in range(num_layers):
        fwd = down if i == 0 else mid
        inv = up if i == num_layers - 1 else mid
        p = f"blocks.{i}."
        w = sd[p + "filter.filter.weight"]
        c = fwd.forward(y)
        res = inv.inverse(c) if fwd is not inv else y
        mixed = np.zeros((y.shape[0], w.shape[1]) + c.shape[2:], dtype=complex)
        for l in range(c.shape[2]):
            mixed[:, :, l, :] = np.einsum("bim,io->bom", c[:, :, l, :], w[:, :, l])
        z = gelu(inorm(inv.inverse(mixed), sd, p + "norm0", eps))
        z = conv(gelu(conv(z, sd, p + "mlp.fwd.0")), sd, p + "mlp.fwd.3")
        y = inorm(z, sd, p + "norm1", eps) + conv(res, sd, p + "outer_skip")
    y = conv(gelu(conv(y, sd, "decoder.fwd.0")), sd, "decoder.fwd.2")
    return y + conv(residual, sd, "residual_transform")


@pytest.mark.parametrize("pos_embed,num_layers", [("none", 3), ("frequency", 2)])
def test_sfno_oracle_matches_independent_evaluation(lib_built, pos_embed, num_layers):
    from makani_amd.sfnonet import SphericalFourierNeuralOperatorNet

    torch.manual_seed(17)
    inp, scale, embed = (13, 24), 2, 5
    net = SphericalFourierNeuralOperatorNet(inp_shape=inp, out_shape=inp, scale_factor=scale, inp_chans=3, out_chans=2, embed_dim=embed,
                                            num_layers=num_layers, pos_embed=pos_embed)
    g = torch.Generator().manual_seed(18)
    with torch.no_grad():
        for n, p in net.named_parameters():       # norms, biases and the embedding start at 1 / 0 / tiny values: make every one matter
            if "norm" in n or n.endswith(".bias"):
                p.add_(0.5 * torch.randn(p.shape, generator=g))
            if n == "pos_embed.0":
                p.copy_(torch.tril(torch.randn(p.shape, generator=g), diagonal=0))
            if n == "pos_embed.1":
                p.copy_(torch.tril(torch.randn(p.shape, generator=g), diagonal=-1))
    sd = net.state_dict()
    h, w = inp[0] // scale, inp[1] // scale
    lmax, mmax = h, w // 2 + 1                    # sfnonet.py:516-520 with hard_thresholding_fraction = 1
    assert (net.trans.lmax, net.trans.mmax, net.trans.nlat, net.trans.nlon) == (lmax, mmax, h, w)
    down = BruteTransform(inp[0], inp[1], lmax, mmax, "equiangular")
    mid = BruteTransform(h, w, lmax, mmax, "legendre-gauss")
    x = torch.randn(2, 3, *inp, generator=g)
    want = independent_forward(sd, x.double().numpy(), down, mid, down, num_layers)
    got = SfnoOracle(inp, inp, scale, num_layers).forward(sd, x).numpy()
    assert got.shape == want.shape == (2, 2, *inp)
    assert np.allclose(got, want, rtol=1e-9, atol=1e-10)
    # the comparison has teeth: the embedding, a swapped transform or a different eps changes the result visibly
    if pos_embed == "frequency":
        sd0 = {k: v for k, v in sd.items() if "pos_embed" not in k}
        assert np.abs(SfnoOracle(inp, inp, scale, num_layers).forward(sd0, x).numpy() - want).max() > 1e-3
    # PyTorch's default eps instead of the 1e-6 of sfnonet.py:379-386, or the internal transform on the wrong grid
    assert not np.allclose(independent_forward(sd, x.double().numpy(), down, mid, down, num_layers, eps=1e-5), want, rtol=1e-9, atol=1e-10)
    wrong = BruteTransform(h, w, lmax, mmax, "equiangular")
    assert np.abs(independent_forward(sd, x.double().numpy(), down, wrong, down, num_layers) - want).max() > 1e-3
