"""Spectral losses on the HIP transform: GeometricH1Loss (makani/utils/losses.py:268-360).

The reference transforms `prd - tar` (and `tar`) with RealSHT(*img_shape, grid="equiangular"), reduces the coefficients
to a per-degree power |c_l0|^2 + 2 sum_{m>0} |c_lm|^2 and weights the degrees with 1 (L2 part) and l(l+1) (H1 part).
Here the power comes from one kernel that reads the output of the Legendre analysis in place (no pass to the reference
coefficient layout, no intermediate tensors of the coefficients' size); its gradient feeds the adjoint transform.
"""
import ctypes

import torch
from torch import nn
from torch.autograd.function import once_differentiable

from ._lib import lib, check
from .sht import RealSHT


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class _DegreePowerFn(torch.autograd.Function):
    """spectral-layout coefficients [mmax, lmax, ld] -> power [rows, lmax]."""

    @staticmethod
    def forward(ctx, spec, rows, lmax, mmax):
        spec = spec.contiguous()
        power = torch.empty((rows, lmax), dtype=torch.float32, device=spec.device)
        check(lib.sfno_degree_power(_ptr(spec), _ptr(power), rows, lmax, mmax, _stream(spec.device)), "sfno_degree_power")
        ctx.save_for_backward(spec)
        ctx.cfg = (rows, lmax, mmax)
        return power

    @staticmethod
    @once_differentiable
    def backward(ctx, g):
        (spec,) = ctx.saved_tensors
        rows, lmax, mmax = ctx.cfg
        g = g.float().contiguous()
        gspec = torch.empty_like(spec)
        check(lib.sfno_degree_power_grad(_ptr(spec), _ptr(g), _ptr(gspec), rows, lmax, mmax, _stream(spec.device)), "sfno_degree_power_grad")
        return gspec, None, None, None


def degree_power(sht, x):
    """|c_l0|^2 + 2 sum_{m>0} |c_lm|^2 of sht(x) for every leading index: x [..., nlat, nlon] -> [..., lmax]."""
    lead = x.shape[:-2]
    rows = 1
    for n in lead:
        rows *= int(n)
    if rows == 0:
        return x.new_zeros((*lead, sht.lmax), dtype=torch.float32)
    spec = sht.analysis(x)
    return _DegreePowerFn.apply(spec, rows, sht.lmax, sht.mmax).reshape(*lead, sht.lmax)


class GeometricH1Loss(nn.Module):
    """Weighted H1 loss on the sphere; `alpha` balances the L2 and H1 seminorms (makani/utils/losses.py:268-360)."""

    def __init__(self, img_shape, p=2.0, size_average=False, reduction=True, absolute=False, squared=False, alpha=0.5):
        super().__init__()
        self.reduction = reduction
        self.size_average = size_average
        self.absolute = absolute
        self.squared = squared
        self.alpha = alpha
        self.sht = RealSHT(*img_shape, grid="equiangular").float()
        h1_weights = torch.arange(self.sht.lmax).float()
        self.register_buffer("h1_weights", h1_weights * (h1_weights + 1))

    def _norms(self, x):
        num_examples = x.size()[0]
        norm2 = degree_power(self.sht, x)
        l2_norm2 = norm2.reshape(num_examples, -1).sum(dim=-1)
        h1_norm2 = (norm2 * self.h1_weights).reshape(num_examples, -1).sum(dim=-1)
        if not self.squared:
            return self.alpha * torch.sqrt(l2_norm2) + (1 - self.alpha) * torch.sqrt(h1_norm2)
        return self.alpha * l2_norm2 + (1 - self.alpha) * h1_norm2

    def abs(self, prd, tar):
        all_norms = self._norms(prd - tar)
        if self.reduction:
            return torch.mean(all_norms) if self.size_average else torch.sum(all_norms)
        return all_norms

    def rel(self, prd, tar, mask=None):
        retval = self._norms(prd - tar) / self._norms(tar)
        if mask is not None:
            retval = retval * mask
        if self.reduction:
            if self.size_average:
                retval = torch.mean(retval) if mask is None else torch.sum(retval) / torch.sum(mask)
            else:
                retval = torch.sum(retval)
        return retval

    def forward(self, prd, tar, mask=None):
        if self.absolute:
            return self.abs(prd, tar)
        return self.rel(prd, tar, mask)
