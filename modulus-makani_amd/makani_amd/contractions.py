"""dhconv contraction on the HIP kernels, with the call signatures of
makani/models/common/contractions.py:130-136 (``_contract_dhconv``) and of the callable
returned by makani/models/common/factorizations.py:212-232 (``get_contract_fun``).
"""
import ctypes
import weakref
from functools import partial

import torch
from torch.autograd.function import once_differentiable

from . import _lib
from ._lib import lib, check


class PackedWeights:
    """Device handle holding a SpectralConv weight packed as per-degree MFMA operand stream."""

    def __init__(self, in_channels, out_channels, lmax, device, compute="fp32"):
        self.handle = ctypes.c_void_p()
        self.shape = (in_channels, out_channels, lmax)
        self.device = torch.device(device)
        self.compute = compute
        self.stamp = None
        with torch.cuda.device(self.device):
            check(lib.sfno_dhconv_weights_create(in_channels, out_channels, lmax, COMPUTE[compute], ctypes.byref(self.handle)), "sfno_dhconv_weights_create")

    def refresh(self, weight, adjoint=False):
        """Re-pack if the parameter changed (in-place updates bump ``_version``).

        adjoint: this handle has shape (O, I, L) and is filled with the conjugate transpose of ``weight`` [I, O, L]."""
        stamp = (weight.data_ptr(), -1 if weight.is_inference() else weight._version)
        if stamp != self.stamp:
            w = weight.detach()
            if w.dtype != torch.complex64:
                raise TypeError(f"dhconv weight must be complex64, got {w.dtype}")
            w = w.contiguous()
            s = ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)
            if adjoint:
                check(lib.sfno_dhconv_weights_update_adjoint(self.handle, ctypes.c_void_p(w.data_ptr()), s), "sfno_dhconv_weights_update_adjoint")
            else:
                check(lib.sfno_dhconv_weights_update(self.handle, ctypes.c_void_p(w.data_ptr()), s), "sfno_dhconv_weights_update")
            self.stamp = stamp
        return self

    def __del__(self):
        if getattr(self, "handle", None):
            lib.sfno_dhconv_weights_destroy(self.handle)
            self.handle = None


# arithmetic of the contraction: fp32 MFMA, or bf16 MFMA inputs with fp32 accumulation
COMPUTE = {"fp32": _lib.COMPUTE_FP32, "bf16": _lib.COMPUTE_BF16, "fp32_bf16x3": _lib.COMPUTE_FP32_BF16X3}

# (id(tensor), compute) -> (weak reference to the tensor, PackedWeights); tensors compare element-wise,
# so they cannot key a WeakKeyDictionary directly
_cache = {}


def packed_for(weight, compute="fp32", adjoint=False):
    """Packed handle for a weight tensor (or, for the backward pass, for its conjugate transpose), cached per
    tensor object and refreshed when it changes."""
    if weight.device.type != "cuda":
        raise RuntimeError("the dhconv kernel runs on a HIP device only")
    if compute not in COMPUTE:
        raise ValueError(f"unknown compute mode {compute!r}, expected 'fp32', 'fp32_bf16x3' or 'bf16'")
    key = (id(weight), compute, adjoint)
    shape = (weight.shape[1], weight.shape[0], weight.shape[2]) if adjoint else tuple(weight.shape)
    hit = _cache.get(key)
    p = hit[1] if hit is not None and hit[0]() is weight else None
    if p is None or p.device != weight.device or p.shape != shape:
        p = PackedWeights(shape[0], shape[1], shape[2], weight.device, compute)
        _cache[key] = (weakref.ref(weight, lambda _, k=key: _cache.pop(k, None)), p)
    return p.refresh(weight, adjoint)


def clear_cache(weight=None):
    """Forgets the packed copies of `weight` (of every weight if None), so that the next call packs the parameter again.

    The cache notices in-place updates through the tensor's version counter (optimizer steps, ``copy_`` under
    ``no_grad``).  Writes through ``param.data`` (``p.data.add_()``, EMA swaps, some fused optimizers) do not move that
    counter: call this, or ``SpectralConv.invalidate_packed()``, after such a write."""
    if weight is None:
        _cache.clear()
        return
    for key in [k for k in _cache if k[0] == id(weight)]:
        _cache.pop(key, None)


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _weight_grad(spec_in, gspec_out, shape, batch, mmax, triangular):
    """gw[i,o,l] = sum_{b,m} conj(x[b,i,l,m]) g[b,o,l,m] from spectral-layout buffers."""
    I, O, L = shape
    if batch == 0:
        return torch.zeros((I, O, L), dtype=torch.complex64, device=spec_in.device)
    gw = torch.empty((I, O, L), dtype=torch.complex64, device=spec_in.device)
    check(
        lib.sfno_dhconv_weight_grad(I, O, L, ctypes.c_void_p(spec_in.data_ptr()), ctypes.c_void_p(gspec_out.data_ptr()),
                                    ctypes.c_void_p(gw.data_ptr()), batch, mmax, int(triangular), _stream(spec_in.device)),
        "sfno_dhconv_weight_grad",
    )
    return gw


class _DhconvSpectralFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, spec_in, weight, batch, mmax, triangular, compute):
        ctx.save_for_backward(spec_in, weight)
        ctx.cfg = (batch, mmax, triangular, compute)
        return _dhconv_spectral(spec_in, weight, batch, mmax, triangular, compute, False)

    @staticmethod
    @once_differentiable
    def backward(ctx, g):
        spec_in, weight = ctx.saved_tensors
        batch, mmax, triangular, compute = ctx.cfg
        g = g.contiguous()
        gin = gw = None
        if ctx.needs_input_grad[0]:
            gin = _dhconv_spectral(g, weight, batch, mmax, triangular, compute, True)
        if ctx.needs_input_grad[1]:
            gw = _weight_grad(spec_in, g, tuple(weight.shape), batch, mmax, triangular)
        return gin, gw, None, None, None, None


def dhconv_spectral(spec_in, weight, batch, mmax, triangular=True, compute="fp32"):
    """Spectral-layout contraction: [mmax, L, ld(batch*I)] -> [mmax, L, ld(batch*O)]."""
    return _DhconvSpectralFn.apply(spec_in.contiguous(), weight, batch, mmax, triangular, compute)


def _dhconv_spectral(spec_in, weight, batch, mmax, triangular, compute, adjoint):
    pw = packed_for(weight, compute, adjoint)
    I, O, L = pw.shape
    ld_out = int(lib.sfno_spectral_ld(batch * O))
    out = torch.empty((mmax, L, ld_out), dtype=torch.float32, device=spec_in.device)
    if ld_out != 2 * batch * O:
        out.zero_()
    if batch == 0:
        return out
    s = ctypes.c_void_p(torch.cuda.current_stream(spec_in.device).cuda_stream)
    check(
        lib.sfno_dhconv_spectral(pw.handle, ctypes.c_void_p(spec_in.data_ptr()), ctypes.c_void_p(out.data_ptr()), batch, mmax, int(triangular), s),
        "sfno_dhconv_spectral",
    )
    return out


def _contract_dhconv(ac: torch.Tensor, bc: torch.Tensor, triangular: bool = False, compute: str = "fp32") -> torch.Tensor:
    """einsum("bixy,iox->boxy") on complex64 tensors (contractions.py:130-136)."""
    if ac.dim() != 4 or bc.dim() != 3 or ac.shape[1] != bc.shape[0] or ac.shape[2] != bc.shape[2]:
        raise RuntimeError(f"dhconv: shapes {tuple(ac.shape)} and {tuple(bc.shape)} do not match 'bixy,iox->boxy'")
    if ac.dtype != torch.complex64:
        raise TypeError(f"dhconv input must be complex64, got {ac.dtype}")
    return _DhconvFn.apply(ac.contiguous(), bc, triangular, compute)


def _to_spectral(c, rows, L, M, triangular):
    spec = torch.empty((M, L, int(lib.sfno_spectral_ld(rows))), dtype=torch.float32, device=c.device)
    check(lib.sfno_coeffs_to_spectral(ctypes.c_void_p(c.data_ptr()), ctypes.c_void_p(spec.data_ptr()), rows, L, M, int(triangular),
                                      _stream(c.device)), "sfno_coeffs_to_spectral")
    return spec


class _DhconvFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, ac, bc, triangular, compute):
        ctx.save_for_backward(ac, bc)
        ctx.cfg = (triangular, compute)
        return _dhconv(ac, bc, triangular, compute, False)

    @staticmethod
    @once_differentiable
    def backward(ctx, g):
        ac, bc = ctx.saved_tensors
        triangular, compute = ctx.cfg
        g = g.contiguous()
        B, I, L, M = ac.shape
        O = bc.shape[1]
        gac = gbc = None
        if ctx.needs_input_grad[0]:
            gac = _dhconv(g, bc, triangular, compute, True)
        if ctx.needs_input_grad[1]:
            if g.numel() == 0:
                gbc = torch.zeros_like(bc)
            else:
                gbc = _weight_grad(_to_spectral(ac, B * I, L, M, triangular), _to_spectral(g, B * O, L, M, triangular), (I, O, L), B, M, triangular)
        return gac, gbc, None, None


def _dhconv(ac, bc, triangular, compute, adjoint):
    B, _, L, M = ac.shape
    pw = packed_for(bc, compute, adjoint)
    O = pw.shape[1]
    out = torch.empty((B, O, L, M), dtype=torch.complex64, device=ac.device)
    if out.numel() == 0:
        return out
    nbytes = lib.sfno_dhconv_workspace_bytes(pw.handle, B, M)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=ac.device)
    s = ctypes.c_void_p(torch.cuda.current_stream(ac.device).cuda_stream)
    check(
        lib.sfno_dhconv(pw.handle, ctypes.c_void_p(ac.data_ptr()), ctypes.c_void_p(out.data_ptr()), B, M, int(triangular),
                        ctypes.c_void_p(ws.data_ptr()), nbytes, s),
        "sfno_dhconv",
    )
    return out


class _DiagonalFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, ac, bc):
        ctx.save_for_backward(ac, bc)
        return _diagonal(ac, bc, False)

    @staticmethod
    @once_differentiable
    def backward(ctx, g):
        ac, bc = ctx.saved_tensors
        g = g.contiguous()
        B, I, L, M = ac.shape
        O = bc.shape[1]
        gac = gbc = None
        if ctx.needs_input_grad[0]:
            gac = _diagonal(g, bc, True)
        if ctx.needs_input_grad[1]:
            gbc = torch.zeros_like(bc)
            if g.numel():
                check(lib.sfno_diagonal_weight_grad(ctypes.c_void_p(ac.data_ptr()), ctypes.c_void_p(g.data_ptr()), ctypes.c_void_p(gbc.data_ptr()),
                                                    B, I, O, L * M, _stream(ac.device)), "sfno_diagonal_weight_grad")
        return gac, gbc


def _diagonal(ac, bc, adjoint):
    B, _, L, M = ac.shape
    I, O = bc.shape[0], bc.shape[1]
    out = torch.empty((B, I if adjoint else O, L, M), dtype=torch.complex64, device=ac.device)
    if out.numel():
        check(lib.sfno_diagonal_contract(ctypes.c_void_p(ac.data_ptr()), ctypes.c_void_p(bc.data_ptr()), ctypes.c_void_p(out.data_ptr()),
                                         B, I, O, L * M, int(adjoint), _stream(ac.device)), "sfno_diagonal_contract")
    return out


def _contract_diagonal(ac: torch.Tensor, bc: torch.Tensor) -> torch.Tensor:
    """einsum("bixy,ioxy->boxy") on complex64 tensors (contractions.py:121-127)."""
    if ac.dim() != 4 or bc.dim() != 4 or ac.shape[1] != bc.shape[0] or ac.shape[2:] != bc.shape[2:]:
        raise RuntimeError(f"diagonal: shapes {tuple(ac.shape)} and {tuple(bc.shape)} do not match 'bixy,ioxy->boxy'")
    if ac.dtype != torch.complex64 or bc.dtype != torch.complex64:
        raise TypeError(f"diagonal contraction computes in complex64, got {ac.dtype} and {bc.dtype}")
    if ac.device.type != "cuda":
        raise RuntimeError("the diagonal contraction kernel runs on a HIP device only")
    return _DiagonalFn.apply(ac.contiguous(), bc.contiguous())


def _as_complex_weight(b):
    """A real weight as the complex one with zero imaginary part (differentiable: the gradient is the real part of the complex one's)."""
    return torch.complex(b, torch.zeros_like(b))


def _contract_diagonal_real(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """einsum("bixys,ioxy->boxys"): complex activations as float32 [..., 2], real weight (contractions.py:157-160)."""
    if a.dim() != 5 or a.shape[-1] != 2 or b.is_complex():
        raise RuntimeError(f"diagonal (real weight): shapes {tuple(a.shape)} and {tuple(b.shape)} do not match 'bixys,ioxy->boxys'")
    return torch.view_as_real(_contract_diagonal(torch.view_as_complex(a.contiguous()), _as_complex_weight(b))).contiguous()


def _contract_dhconv_real(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """einsum("bixys,iox->boxys"): complex activations as float32 [..., 2], real weight (contractions.py:163-166)."""
    if a.dim() != 5 or a.shape[-1] != 2 or b.is_complex():
        raise RuntimeError(f"dhconv (real weight): shapes {tuple(a.shape)} and {tuple(b.shape)} do not match 'bixys,iox->boxys'")
    return torch.view_as_real(_contract_dhconv(torch.view_as_complex(a.contiguous()), _as_complex_weight(b))).contiguous()


def _contract_dense(x, weight, separable=False, operator_type="diagonal", complex=True):
    """Mirror of _contract_dense_pytorch (factorizations.py:167-200).

    The separable variants are not provided: the reference's einsums for them ("bixy,ixy->boxy", "bixy,ix->boxy",
    contractions.py:139-154) name an output index that no input carries, so they cannot be evaluated there either."""
    if operator_type not in ("diagonal", "dhconv"):
        raise ValueError(f"unknown operator type {operator_type!r}, expected 'diagonal' or 'dhconv'")
    if separable:
        raise NotImplementedError("the separable operators are not provided (see above)")
    if operator_type == "diagonal":
        return _contract_diagonal(x, weight) if complex else _contract_diagonal_real(x, weight)
    return _contract_dhconv(x, weight) if complex else _contract_dhconv_real(x, weight)


def get_contract_fun(weight, implementation="reconstructed", separable=False, operator_type="diagonal", complex=True):
    """Same selection interface as factorizations.py:212-247, dense tensor weights only."""
    if implementation not in ("reconstructed", "factorized"):
        raise ValueError(f'Got {implementation=}, expected "reconstructed" or "factorized"')
    if not torch.is_tensor(weight):
        raise ValueError(f"Got unexpected weight type of class {weight.__class__.__name__}")
    return partial(_contract_dense, separable=separable, complex=complex, operator_type=operator_type)
