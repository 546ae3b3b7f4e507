"""RealSHT / InverseRealSHT with the torch-harmonics module interface, running on the
hand-written HIP kernels of libsfno_spectral (gfx950).

Drop-in for the objects Makani builds at makani/models/networks/sfnonet.py:524-539
(``sht_handle(nlat, nlon, lmax=, mmax=, grid=).float()``) and calls at
makani/models/common/spectral_convolution.py:131,133,141 and sfnonet.py:596,598,616:
same constructor arguments, same ``nlat/nlon/lmax/mmax/grid/norm/csphase`` attributes,
``forward`` maps real ``[..., nlat, nlon]`` to complex ``[..., lmax, mmax]`` and back.
The Legendre tables live inside a device plan (packed, triangular), not in module
buffers, so the modules add nothing to a state_dict -- like the non-persistent buffers
of the reference modules.
"""
import ctypes

import numpy as np
import torch
import torch.nn as nn
from torch.autograd.function import once_differentiable

from . import _lib
from ._lib import lib, check


def quadrature(grid, nlat):
    """(theta ascending, weights) of a latitude grid, float64 numpy, from the library's host code."""
    theta = np.empty(nlat, dtype=np.float64)
    w = np.empty(nlat, dtype=np.float64)
    dp = ctypes.POINTER(ctypes.c_double)
    check(lib.sfno_quadrature(_lib.GRID[grid], nlat, theta.ctypes.data_as(dp), w.ctypes.data_as(dp)), "sfno_quadrature")
    return theta, w


def legendre_gauss_weights(n, a=-1.0, b=1.0):
    """(cos(theta) ascending, weights) as torch_harmonics.quadrature.legendre_gauss_weights returns them."""
    theta, w = quadrature("legendre-gauss", n)
    x = np.cos(theta)[::-1].copy()
    return (b - a) * 0.5 * x + (b + a) * 0.5, w[::-1].copy() * (b - a) * 0.5


def clenshaw_curtiss_weights(n, a=-1.0, b=1.0):
    theta, w = quadrature("equiangular", n)
    x = np.cos(theta)[::-1].copy()
    return (b - a) * 0.5 * x + (b + a) * 0.5, w[::-1].copy() * (b - a) * 0.5


def lobatto_weights(n, a=-1.0, b=1.0):
    theta, w = quadrature("lobatto", n)
    x = np.cos(theta)[::-1].copy()
    return (b - a) * 0.5 * x + (b + a) * 0.5, w[::-1].copy() * (b - a) * 0.5


def legendre_table(mmax, lmax, theta, norm="ortho", inverse=False, csphase=True):
    """Dense float64 table [mmax, lmax, nlat] from the library's host recursion."""
    theta = np.ascontiguousarray(theta, dtype=np.float64)
    out = np.empty((mmax, lmax, len(theta)), dtype=np.float64)
    dp = ctypes.POINTER(ctypes.c_double)
    check(
        lib.sfno_legendre_table(mmax, lmax, len(theta), theta.ctypes.data_as(dp), _lib.NORM[norm], int(inverse), int(csphase), out.ctypes.data_as(dp)),
        "sfno_legendre_table",
    )
    return out


class _Plan:
    """Owns one sfno_sht_plan on one device."""

    def __init__(self, mod, device, directions):
        self.handle = ctypes.c_void_p()
        with torch.cuda.device(device):
            check(
                lib.sfno_sht_plan_create(
                    mod.nlat, mod.nlon, mod.lmax, mod.mmax, _lib.GRID[mod.grid], _lib.NORM[mod.norm], int(mod.csphase), directions,
                    {"fp32": _lib.COMPUTE_FP32, "bf16": _lib.COMPUTE_BF16, "fp32_mfma": _lib.COMPUTE_FP32_MFMA, "fp32_bf16x3": _lib.COMPUTE_FP32_BF16X3}[mod.compute], ctypes.byref(self.handle),
                ),
                "sfno_sht_plan_create",
            )

    def __del__(self):
        if getattr(self, "handle", None):
            lib.sfno_sht_plan_destroy(self.handle)
            self.handle = None


def _stream_ptr(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


class _SHTBase(nn.Module):
    _directions = 0
    _adjoint_direction = 0
    _planar = False    # True in the planar FFT pair of layers.py, which shares the plan, layouts and entry points

    def __init__(self, nlat, nlon, lmax=None, mmax=None, grid="lobatto", norm="ortho", csphase=True, compute="fp32"):
        super().__init__()
        # compute = "fp32" (default, the reference's arithmetic): fp32 operands and accumulation, the Legendre stage on the
        #   fp16 matrix pipe with every operand scaled by a power of two and cut into two fp16 numbers (three products);
        # "fp32_bf16x3": every operand cut exactly into three bf16 numbers (six products, no scales);
        # "fp32_mfma": the fp32 matrix instruction on fp32 tables;
        # "bf16": bf16 tables and inputs, fp32 accumulation.
        if compute not in ("fp32", "bf16", "fp32_mfma", "fp32_bf16x3"):
            raise ValueError(f"unknown compute mode {compute!r}, expected 'fp32', 'fp32_mfma', 'fp32_bf16x3' or 'bf16'")
        self.compute = compute
        self.nlat = nlat
        self.nlon = nlon
        self.grid = grid
        self.norm = norm
        self.csphase = csphase
        if grid == "legendre-gauss" or grid == "equiangular":
            self.lmax = lmax or self.nlat
        elif grid == "lobatto":
            self.lmax = lmax or self.nlat - 1
        elif grid == "planar" and self._planar:
            self.lmax = lmax or self.nlat
        else:
            raise ValueError("Unknown quadrature mode")
        if norm not in _lib.NORM:
            raise ValueError("Unknown normalization mode")
        self.mmax = mmax or self.nlon // 2 + 1
        if (self._directions & _lib.DIR_FORWARD) and self.mmax > self.nlon // 2 + 1:
            raise ValueError("mmax must not exceed nlon // 2 + 1 for the forward transform")
        self._plans = {}

    def extra_repr(self):
        return f"nlat={self.nlat}, nlon={self.nlon},\n lmax={self.lmax}, mmax={self.mmax},\n grid={self.grid}, csphase={self.csphase}"

    def plan(self, device, adjoint=False):
        """Device plan of the transform, or (built on the first backward pass) of its adjoint."""
        device = torch.device(device)
        if device.type != "cuda":
            raise RuntimeError("the SFNO spectral kernels run on a HIP device only; move the input to the GPU")
        index = device.index if device.index is not None else torch.cuda.current_device()
        key = (index, adjoint)
        p = self._plans.get(key)
        if p is None:
            p = _Plan(self, torch.device("cuda", index), self._adjoint_direction if adjoint else self._directions)
            self._plans[key] = p
        return p

    def _adjoint_module(self):
        """The module whose adjoint plan serves this module's backward pass: the module itself, except for an inverse
        transform that keeps more orders than the longitude grid resolves (mmax > nlon // 2 + 1).  Such an inverse drops
        the surplus orders like a complex-to-real FFT does, so their cotangents are exactly zero and the adjoint is that of
        the same transform truncated to nlon // 2 + 1 orders."""
        if self.mmax <= self.nlon // 2 + 1 or self._directions != _lib.DIR_INVERSE:
            return self
        if getattr(self, "_truncated", None) is None:
            object.__setattr__(self, "_truncated", type(self)(self.nlat, self.nlon, self.lmax, self.nlon // 2 + 1, self.grid, self.norm, self.csphase,
                                                              self.compute))
        return self._truncated

    def workspace(self, plan, rows, device):
        nbytes = lib.sfno_sht_workspace_bytes(plan.handle, rows)
        return torch.empty(nbytes, dtype=torch.uint8, device=device), nbytes

    def spectral_shape(self, rows):
        return (self.mmax, self.lmax, int(lib.sfno_spectral_ld(rows)))

    def __getstate__(self):
        state = dict(self.__dict__)
        state["_plans"] = {}
        state.pop("_truncated", None)
        return state

    def __deepcopy__(self, memo):
        return type(self)(self.nlat, self.nlon, self.lmax, self.mmax, self.grid, self.norm, self.csphase, self.compute)


def _as_fp32_rows(x, tail):
    if x.is_complex() != (tail == "coeffs"):
        raise TypeError("expected a real field" if tail == "grid" else "expected complex coefficients")
    if tail == "grid":
        if x.dtype in (torch.float16, torch.bfloat16):
            x = x.float()
        if x.dtype != torch.float32:
            raise TypeError(f"the HIP transform computes in float32; got {x.dtype}")
    else:
        if x.dtype != torch.complex64:
            raise TypeError(f"the HIP transform computes in complex64; got {x.dtype}")
    return x.contiguous()


def _rows(lead):
    return int(np.prod(lead)) if len(lead) else 1


class _ForwardFn(torch.autograd.Function):
    """RealSHT.forward on the reference layout; backward = sfno_sht_forward_adjoint."""

    @staticmethod
    def forward(ctx, x, mod):
        ctx.mod = mod
        return mod._forward(x)

    @staticmethod
    @once_differentiable
    def backward(ctx, g):
        mod = ctx.mod
        g = g.contiguous()
        lead = g.shape[:-2]
        gx = torch.empty((*lead, mod.nlat, mod.nlon), dtype=torch.float32, device=g.device)
        if gx.numel():
            plan = mod.plan(g.device, adjoint=True)
            ws, nbytes = mod.workspace(plan, _rows(lead), g.device)
            check(lib.sfno_sht_forward_adjoint(plan.handle, _ptr(g), _ptr(gx), _rows(lead), _ptr(ws), nbytes, _stream_ptr(g.device)),
                  "sfno_sht_forward_adjoint")
        return gx, None


class _AnalysisFn(torch.autograd.Function):
    """Grid field -> spectral layout; backward = sfno_sht_analysis_adjoint in the dtype of the field."""

    @staticmethod
    def forward(ctx, x, mod, dt):
        ctx.mod, ctx.dt, ctx.shape = mod, dt, x.shape
        return mod._analysis(x, dt)

    @staticmethod
    @once_differentiable
    def backward(ctx, g):
        mod = ctx.mod
        g = g.contiguous()
        rows = _rows(ctx.shape[:-2])
        gx = torch.empty(ctx.shape, dtype=torch.bfloat16 if ctx.dt == _lib.DTYPE_BF16 else torch.float32, device=g.device)
        if rows == 0:
            return gx, None, None
        plan = mod.plan(g.device, adjoint=True)
        ws, nbytes = mod.workspace(plan, rows, g.device)
        check(lib.sfno_sht_analysis_adjoint(plan.handle, _ptr(g), _ptr(gx), ctx.dt, rows, _ptr(ws), nbytes, _stream_ptr(g.device)),
              "sfno_sht_analysis_adjoint")
        return gx, None, None


class _InverseFn(torch.autograd.Function):
    """InverseRealSHT.forward on the reference layout; backward = sfno_sht_inverse_adjoint."""

    @staticmethod
    def forward(ctx, c, mod):
        ctx.mod = mod
        return mod._inverse(c)

    @staticmethod
    @once_differentiable
    def backward(ctx, g):
        full, mod = ctx.mod, ctx.mod._adjoint_module()
        g = g.float().contiguous()
        lead = g.shape[:-2]
        gc = torch.empty((*lead, mod.lmax, mod.mmax), dtype=torch.complex64, device=g.device)
        if gc.numel():
            plan = mod.plan(g.device, adjoint=True)
            ws, nbytes = mod.workspace(plan, _rows(lead), g.device)
            check(lib.sfno_sht_inverse_adjoint(plan.handle, _ptr(g), _ptr(gc), _rows(lead), _ptr(ws), nbytes, _stream_ptr(g.device)),
                  "sfno_sht_inverse_adjoint")
        if mod is not full:      # orders the longitude grid does not resolve receive no gradient
            gc = torch.nn.functional.pad(gc, (0, full.mmax - mod.mmax))
        return gc, None


class _SynthesisFn(torch.autograd.Function):
    """Spectral layout -> grid field; backward = sfno_sht_synthesis_adjoint."""

    @staticmethod
    def forward(ctx, spec, mod, lead, fused):
        ctx.mod, ctx.lead = mod, tuple(lead)
        return mod._synthesis(spec, lead, fused)

    @staticmethod
    @once_differentiable
    def backward(ctx, g):
        full, mod = ctx.mod, ctx.mod._adjoint_module()
        rows = _rows(ctx.lead)
        if rows == 0:
            return torch.zeros(full.spectral_shape(0), dtype=torch.float32, device=g.device), None, None, None
        plan = mod.plan(g.device, adjoint=True)
        if g.dtype == torch.bfloat16 and lib.sfno_sht_io_dtype_supported(plan.handle, _lib.DTYPE_BF16):
            g, dt = g.contiguous(), _lib.DTYPE_BF16
        else:
            g, dt = g.float().contiguous(), _lib.DTYPE_F32
        gspec = torch.empty(mod.spectral_shape(rows), dtype=torch.float32, device=g.device)
        ws, nbytes = mod.workspace(plan, rows, g.device)
        check(lib.sfno_sht_synthesis_adjoint(plan.handle, _ptr(g), dt, _ptr(gspec), rows, _ptr(ws), nbytes, _stream_ptr(g.device)),
              "sfno_sht_synthesis_adjoint")
        if mod is not full:      # orders the longitude grid does not resolve receive no gradient (the order axis comes first)
            gspec = torch.cat((gspec, gspec.new_zeros((full.mmax - mod.mmax,) + tuple(gspec.shape[1:]))), dim=0)
        return gspec, None, None, None


class RealSHT(_SHTBase):
    """Forward real spherical harmonic transform (analysis)."""

    _directions = _lib.DIR_FORWARD
    _adjoint_direction = _lib.DIR_FORWARD_ADJOINT

    @property
    def weights(self):
        """Dense analysis table [mmax, lmax, nlat] (float32), as the reference module's buffer of that name."""
        theta, w = quadrature(self.grid, self.nlat)
        return torch.from_numpy(legendre_table(self.mmax, self.lmax, theta, self.norm, False, self.csphase) * w).float()

    def forward(self, x):
        assert x.shape[-2] == self.nlat
        assert x.shape[-1] == self.nlon
        return _ForwardFn.apply(_as_fp32_rows(x, "grid"), self)

    def _forward(self, x):
        lead = x.shape[:-2]
        rows = _rows(lead)
        out = torch.empty((*lead, self.lmax, self.mmax), dtype=torch.complex64, device=x.device)
        if rows == 0:
            return out
        plan = self.plan(x.device)
        ws, nbytes = self.workspace(plan, rows, x.device)
        check(lib.sfno_sht_forward(plan.handle, _ptr(x), _ptr(out), rows, _ptr(ws), nbytes, _stream_ptr(x.device)), "sfno_sht_forward")
        return out

    def analysis(self, x):
        """x [..., nlat, nlon] (float32, or bfloat16 widened inside the FFT kernel) -> spectral-layout float32 [mmax, lmax, ld]."""
        assert x.shape[-2] == self.nlat
        assert x.shape[-1] == self.nlon
        plan = self.plan(x.device)
        if x.dtype == torch.bfloat16 and lib.sfno_sht_io_dtype_supported(plan.handle, _lib.DTYPE_BF16):
            return _AnalysisFn.apply(x.contiguous(), self, _lib.DTYPE_BF16)
        return _AnalysisFn.apply(_as_fp32_rows(x, "grid"), self, _lib.DTYPE_F32)

    def _analysis(self, x, dt):
        plan = self.plan(x.device)
        rows = _rows(x.shape[:-2])
        spec = torch.empty(self.spectral_shape(rows), dtype=torch.float32, device=x.device)
        if rows == 0:
            return spec
        ws, nbytes = self.workspace(plan, rows, x.device)
        check(lib.sfno_sht_analysis(plan.handle, _ptr(x), dt, _ptr(spec), rows, _ptr(ws), nbytes, _stream_ptr(x.device)), "sfno_sht_analysis")
        return spec


class InverseRealSHT(_SHTBase):
    """Inverse real spherical harmonic transform (synthesis)."""

    _directions = _lib.DIR_INVERSE
    _adjoint_direction = _lib.DIR_INVERSE_ADJOINT

    @property
    def pct(self):
        """Dense synthesis table [mmax, lmax, nlat] (float32), as the reference module's buffer of that name."""
        theta, _ = quadrature(self.grid, self.nlat)
        return torch.from_numpy(legendre_table(self.mmax, self.lmax, theta, self.norm, True, self.csphase)).float()

    def forward(self, x):
        assert x.shape[-2] == self.lmax
        assert x.shape[-1] == self.mmax
        return _InverseFn.apply(_as_fp32_rows(x, "coeffs"), self)

    def _inverse(self, x):
        lead = x.shape[:-2]
        rows = _rows(lead)
        out = torch.empty((*lead, self.nlat, self.nlon), dtype=torch.float32, device=x.device)
        if rows == 0:
            return out
        plan = self.plan(x.device)
        ws, nbytes = self.workspace(plan, rows, x.device)
        check(lib.sfno_sht_inverse(plan.handle, _ptr(x), _ptr(out), rows, _ptr(ws), nbytes, _stream_ptr(x.device)), "sfno_sht_inverse")
        return out

    def synthesis(self, spec, lead, dtype=torch.float32):
        """spectral-layout float32 [mmax, lmax, ld] -> x [*lead, nlat, nlon]; dtype bfloat16 rounds inside the FFT kernel."""
        rows = _rows(lead)
        assert tuple(spec.shape) == self.spectral_shape(rows) and spec.dtype == torch.float32
        plan = self.plan(spec.device)
        fused = bool(dtype == torch.bfloat16 and lib.sfno_sht_io_dtype_supported(plan.handle, _lib.DTYPE_BF16))
        out = _SynthesisFn.apply(spec.contiguous(), self, tuple(lead), fused)
        return out if out.dtype == dtype else out.to(dtype)

    def synthesis_with_lat_stats(self, spec, lead, dtype=torch.float32):
        """synthesis() without autograd that also returns float32 [rows, nlat, 2]: per channel row and latitude the mean
        over longitude of the field and of its squared deviation from that mean (a by-product of the longitude kernel,
        enough for the instance norm that follows); (field, None) where the longitude length has no specialised kernel."""
        rows = _rows(lead)
        assert tuple(spec.shape) == self.spectral_shape(rows) and spec.dtype == torch.float32
        plan = self.plan(spec.device)
        if not lib.sfno_sht_lat_stats_supported(plan.handle):
            return self.synthesis(spec, lead, dtype), None
        fused = dtype == torch.bfloat16
        out = torch.empty((*lead, self.nlat, self.nlon), dtype=torch.bfloat16 if fused else torch.float32, device=spec.device)
        stats = torch.empty((rows, self.nlat, 2), dtype=torch.float32, device=spec.device)
        if rows == 0:
            return (out if out.dtype == dtype else out.to(dtype)), stats
        ws, nbytes = self.workspace(plan, rows, spec.device)
        check(lib.sfno_sht_synthesis_lat_stats(plan.handle, _ptr(spec.contiguous()), _ptr(out), _lib.DTYPE_BF16 if fused else _lib.DTYPE_F32, rows,
                                               _ptr(ws), nbytes, _ptr(stats), _stream_ptr(spec.device)), "sfno_sht_synthesis_lat_stats")
        return (out if out.dtype == dtype else out.to(dtype)), stats

    def _synthesis(self, spec, lead, fused):
        rows = _rows(lead)
        plan = self.plan(spec.device)
        out = torch.empty((*lead, self.nlat, self.nlon), dtype=torch.bfloat16 if fused else torch.float32, device=spec.device)
        if rows == 0:
            return out
        ws, nbytes = self.workspace(plan, rows, spec.device)
        check(lib.sfno_sht_synthesis(plan.handle, _ptr(spec), _ptr(out), _lib.DTYPE_BF16 if fused else _lib.DTYPE_F32, rows, _ptr(ws), nbytes,
                                     _stream_ptr(spec.device)), "sfno_sht_synthesis")
        return out
