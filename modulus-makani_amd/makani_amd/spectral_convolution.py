"""SpectralConv with the interface of makani/models/common/spectral_convolution.py:43-148,
running the forward transform, the dhconv channel mix and the inverse transform on the
HIP kernels without leaving the order-major spectral layout in between.
"""
import math

import torch
import torch.nn as nn

from .contractions import get_contract_fun, dhconv_spectral, clear_cache
from .sht import RealSHT, InverseRealSHT


class SpectralConv(nn.Module):
    """Spectral convolution on the sphere: SHT -> per-degree complex channel mix -> inverse SHT."""

    # per-mode extent of the weight behind [in_channels, out_channels]: the contract of spectral_convolution.py:89-96
    _MODE_DIMS = {"diagonal": ("modes_lat_local", "modes_lon_local"), "dhconv": ("modes_lat_local",)}

    def __init__(self, forward_transform, inverse_transform, in_channels, out_channels, operator_type="diagonal", separable=False, bias=False, gain=1.0,
                 compute="fp32"):
        """Attribute names, the shape of ``weight`` and its initial distribution are those of the reference module
        (spectral_convolution.py:50-122), so that its checkpoints load and its callers find what they read.

        compute: arithmetic of the channel mix -- "fp32" (default, the reference's precision), "fp32_bf16x3" or "bf16"
        (bf16 matrix inputs, fp32 accumulation)."""
        super().__init__()
        if operator_type not in self._MODE_DIMS:
            raise ValueError(f"unsupported operator type {operator_type!r}, expected one of {sorted(self._MODE_DIMS)}")
        if separable:
            raise NotImplementedError("the HIP path implements the non-separable operators")
        fwd, inv = forward_transform, inverse_transform
        self.forward_transform, self.inverse_transform = fwd, inv
        self.in_channels, self.out_channels = in_channels, out_channels
        self.operator_type, self.separable, self.compute = operator_type, separable, compute

        # the filter lives on the modes of the inverse transform; one process holds all of them
        self.modes_lat = self.modes_lat_local = inv.lmax
        self.modes_lon = self.modes_lon_local = inv.mmax
        self.nlat_local, self.nlon_local = inv.nlat, inv.nlon
        # input and output grids differ: the residual then has to pass through the transforms as well (forward)
        same_grid = (fwd.nlat, fwd.nlon) == (inv.nlat, inv.nlon) and getattr(fwd, "grid", None) == getattr(inv, "grid", None)
        self.scale_residual = not same_grid

        # weight ~ sqrt(gain / in_channels) * CN(0, 1) per mode, the degree-0 row larger by sqrt(2)
        shape = (in_channels, out_channels) + tuple(getattr(self, d) for d in self._MODE_DIMS[operator_type])
        std = torch.full((self.modes_lat_local,), math.sqrt(gain / in_channels), dtype=torch.complex64)
        std[0] *= math.sqrt(2.0)
        # (broadcast along the last axis of the weight: the degree axis for dhconv)
        self.weight = nn.Parameter(std * torch.randn(*shape, dtype=torch.complex64))
        self._contract = get_contract_fun(self.weight, implementation="factorized", separable=separable, complex=True, operator_type=operator_type)

        bias_shape = {"constant": (1, out_channels, 1, 1), "position": (1, out_channels, self.nlat_local, self.nlon_local)}.get(bias)
        if bias_shape is not None:
            self.bias = nn.Parameter(torch.zeros(bias_shape))

        # forward transform -> dhconv -> inverse transform without leaving the order-major spectral layout
        self._fused = (
            operator_type == "dhconv"
            and isinstance(fwd, RealSHT)
            and isinstance(inv, InverseRealSHT)
            and (fwd.lmax, fwd.mmax, fwd._planar) == (inv.lmax, inv.mmax, inv._planar)
        )
        # coefficients of a spherical transform vanish for l < m; the planar pair fills the whole rectangle
        self._triangular = not getattr(fwd, "_planar", False)

    def invalidate_packed(self):
        """Drops the packed MFMA operand copies of ``weight``; call after writing the parameter through ``.data``."""
        clear_cache(self.weight)

    def forward(self, x, lat_stats=False):
        """Returns (x, residual) as the reference does.  With lat_stats=True (inference on the fused path only) a third value
        follows: per-latitude moments of x from InverseRealSHT.synthesis_with_lat_stats, or None where they are not available."""
        dtype = x.dtype
        residual = x
        B, C, H, W = x.shape
        stats = None

        if self._fused:
            # The transforms and the contraction work in float32 regardless of autocast.  A bf16 input is
            # widened while the FFT kernel loads it and the output is rounded while it is stored: the
            # same values as the reference's x.float() ... x.to(dtype) without the two full-tensor passes.
            fuse_cast = dtype == torch.bfloat16 and not hasattr(self, "bias")
            spec = self.forward_transform.analysis(x if dtype == torch.bfloat16 else x.float())
            if self.scale_residual:
                residual = self.inverse_transform.synthesis(spec, (B, C), dtype=dtype if dtype == torch.bfloat16 else torch.float32).to(dtype)
            spec = dhconv_spectral(spec, self.weight, B, self.modes_lon, triangular=self._triangular, compute=self.compute)
            if lat_stats and fuse_cast and not torch.is_grad_enabled():
                x, stats = self.inverse_transform.synthesis_with_lat_stats(spec, (B, self.out_channels), dtype=dtype)
            else:
                x = self.inverse_transform.synthesis(spec, (B, self.out_channels), dtype=dtype if fuse_cast else torch.float32)
        else:
            x = x.float()
            with torch.autocast(device_type="cuda", enabled=False):
                x = self.forward_transform(x).contiguous()
                if self.scale_residual:
                    residual = self.inverse_transform(x)
                    residual = residual.to(dtype)
            xp = self._contract(x, self.weight, separable=self.separable, operator_type=self.operator_type)
            x = xp.contiguous()
            with torch.autocast(device_type="cuda", enabled=False):
                x = self.inverse_transform(x)

        if hasattr(self, "bias"):
            x = x + self.bias
        x = x.to(dtype=dtype)
        return (x, residual, stats) if lat_stats else (x, residual)
