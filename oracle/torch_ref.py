"""PyTorch-CPU float32 restatement of the reference op sequence (oracle; CPU baseline).

This is what the reference executes on a CPU: dense float32 tables held as tensors,
``torch.fft.rfft`` -> two ``torch.einsum('...km,mlk->...lm')`` -> (dhconv einsum) ->
two ``torch.einsum('...lm,mlk->...km')`` -> ``torch.fft.irfft`` (torch-harmonics'
RealSHT / InverseRealSHT forward as called from
makani/models/common/spectral_convolution.py:131,141, and
makani/models/common/contractions.py:134).  It is timed by bench.py's cpu_baseline leg
and never used by the product.

With ``dtype=torch.float64`` the same op sequence is the gradient oracle of the tests: the
reference has no hand-written backward, autograd differentiates exactly these ops
(tests/test_models.py:149-157 of the reference checks the resulting input gradient).
"""
import numpy as np
import torch

from .sht import ShtTables


class TorchRefSHT:
    def __init__(self, nlat, nlon, lmax=None, mmax=None, grid="lobatto", norm="ortho", csphase=True, directions=("fwd", "inv"),
                 dtype=torch.float32):
        t = ShtTables(nlat, nlon, lmax, mmax, grid, norm, csphase)
        self.nlat, self.nlon, self.lmax, self.mmax = nlat, nlon, t.lmax, t.mmax
        self.weights = None
        self.pct = None
        if "inv" in directions:
            self.pct = torch.from_numpy(np.ascontiguousarray(t.pct)).to(dtype)
        if "fwd" in directions:
            if dtype == torch.float32:
                w = t.p_analysis.astype(np.float32)
                w *= t.quad_w[None, None, :].astype(np.float32)
            else:
                w = t.p_analysis * t.quad_w[None, None, :]
            self.weights = torch.from_numpy(np.ascontiguousarray(w)).to(dtype)

    def forward(self, x):
        x = 2.0 * torch.pi * torch.fft.rfft(x, dim=-1, norm="forward")
        x = torch.view_as_real(x)
        out_shape = list(x.size())
        out_shape[-3] = self.lmax
        out_shape[-2] = self.mmax
        xout = torch.zeros(out_shape, dtype=x.dtype)
        xout[..., 0] = torch.einsum("...km,mlk->...lm", x[..., : self.mmax, 0], self.weights)
        xout[..., 1] = torch.einsum("...km,mlk->...lm", x[..., : self.mmax, 1], self.weights)
        return torch.view_as_complex(xout)

    def inverse(self, c):
        c = torch.view_as_real(c)
        rl = torch.einsum("...lm,mlk->...km", c[..., 0], self.pct)
        im = torch.einsum("...lm,mlk->...km", c[..., 1], self.pct)
        x = torch.view_as_complex(torch.stack((rl, im), -1))
        return torch.fft.irfft(x, n=self.nlon, dim=-1, norm="forward")


class TorchRefFFT2:
    """The torch op sequence of RealFFT2.forward / InverseRealFFT2.forward (makani/models/common/layers.py:242-250,
    276-287); autograd through it is the gradient oracle of the planar pair."""

    def __init__(self, nlat, nlon, lmax=None, mmax=None):
        from .fft2 import Fft2Modes

        t = Fft2Modes(nlat, nlon, lmax, mmax)
        self.nlat, self.nlon, self.lmax, self.mmax, self.truncate = nlat, nlon, t.lmax, t.mmax, t.truncate
        self.lmax_high, self.lmax_low = t.lmax_high, t.lmax_low

    def forward(self, x):
        y = torch.fft.rfft2(x, s=(self.nlat, self.nlon), dim=(-2, -1), norm="ortho")
        if self.truncate:
            lo = y[..., y.shape[-2] - self.lmax_low :, : self.mmax]
            y = torch.cat((y[..., : self.lmax_high, : self.mmax], lo), dim=-2)
        return y

    def inverse(self, c):
        xt = c[..., : self.mmax]
        if self.truncate:
            xth = xt[..., : self.lmax_high, :]
            xtl = xt[..., xt.shape[-2] - self.lmax_low :, :]
            xthp = torch.nn.functional.pad(xth, (0, 0, 0, self.nlat - self.lmax))
            xt = torch.cat([xthp, xtl], dim=-2)
        return torch.fft.irfft2(xt, s=(self.nlat, self.nlon), dim=(-2, -1), norm="ortho")


def dhconv(x, w):
    return torch.einsum("bixy,iox->boxy", x, w)
