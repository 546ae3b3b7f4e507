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

    def __init__(self, forward_transform, inverse_transform, in_channels, out_channels, operator_type="diagonal", separable=False, bias=False, gain=1.0,
                 compute="fp32"):
        super().__init__()
        # compute = "bf16" runs the channel mix on bf16 MFMA (fp32 accumulate); the reference and the default stay fp32
        self.compute = compute
        self.forward_transform = forward_transform
        self.inverse_transform = inverse_transform
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.modes_lat = self.inverse_transform.lmax
        self.modes_lon = self.inverse_transform.mmax
        self.scale_residual = (self.forward_transform.nlat != self.inverse_transform.nlat) or (self.forward_transform.nlon != self.inverse_transform.nlon)
        if hasattr(self.forward_transform, "grid"):
            self.scale_residual = self.scale_residual or (self.forward_transform.grid != self.inverse_transform.grid)
        self.operator_type = operator_type
        self.separable = separable
        assert self.inverse_transform.lmax == self.modes_lat
        assert self.inverse_transform.mmax == self.modes_lon

        weight_shape = [in_channels]
        if not self.separable:
            weight_shape += [out_channels]
        self.modes_lat_local = self.modes_lat
        self.modes_lon_local = self.modes_lon
        self.nlat_local = self.inverse_transform.nlat
        self.nlon_local = self.inverse_transform.nlon
        if self.operator_type == "diagonal":
            weight_shape += [self.modes_lat_local, self.modes_lon_local]
        elif self.operator_type == "dhconv":
            weight_shape += [self.modes_lat_local]
        else:
            raise ValueError(f"Unsupported operator type f{self.operator_type}")
        if self.separable:
            raise NotImplementedError("the HIP path implements the non-separable operators")

        # same initialisation as the reference (spectral_convolution.py:97-102)
        scale = math.sqrt(gain / in_channels) * torch.ones(self.modes_lat_local, dtype=torch.complex64)
        scale[0] *= math.sqrt(2.0)
        init = scale * torch.randn(*weight_shape, dtype=torch.complex64)
        self.weight = nn.Parameter(init)

        self._contract = get_contract_fun(self.weight, implementation="factorized", separable=separable, complex=True, operator_type=operator_type)

        if bias == "constant":
            self.bias = nn.Parameter(torch.zeros(1, self.out_channels, 1, 1))
        elif bias == "position":
            self.bias = nn.Parameter(torch.zeros(1, self.out_channels, self.nlat_local, self.nlon_local))

        self._fused = (
            operator_type == "dhconv"
            and isinstance(forward_transform, RealSHT)
            and isinstance(inverse_transform, InverseRealSHT)
            and forward_transform.lmax == inverse_transform.lmax
            and forward_transform.mmax == inverse_transform.mmax
            and forward_transform._planar == inverse_transform._planar
        )
        # coefficients of a spherical transform vanish for l < m; the planar pair fills the whole rectangle
        self._triangular = not getattr(forward_transform, "_planar", False)

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
