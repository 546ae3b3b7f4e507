"""dhconv contraction on the HIP kernels, with the call signatures of
makani/models/common/contractions.py:130-136 (``_contract_dhconv``) and of the callable
returned by makani/models/common/factorizations.py:212-232 (``get_contract_fun``).
"""
import ctypes
import weakref
from functools import partial

import torch

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

    def refresh(self, weight):
        """Re-pack if the parameter changed (in-place updates bump ``_version``)."""
        stamp = (weight.data_ptr(), weight._version)
        if stamp != self.stamp:
            w = weight.detach()
            if w.dtype != torch.complex64:
                raise TypeError(f"dhconv weight must be complex64, got {w.dtype}")
            w = w.contiguous()
            s = ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)
            check(lib.sfno_dhconv_weights_update(self.handle, ctypes.c_void_p(w.data_ptr()), s), "sfno_dhconv_weights_update")
            self.stamp = stamp
        return self

    def __del__(self):
        if getattr(self, "handle", None):
            lib.sfno_dhconv_weights_destroy(self.handle)
            self.handle = None


# arithmetic of the contraction: fp32 MFMA, or bf16 MFMA inputs with fp32 accumulation
COMPUTE = {"fp32": _lib.COMPUTE_FP32, "bf16": _lib.COMPUTE_BF16}

# (id(tensor), compute) -> (weak reference to the tensor, PackedWeights); tensors compare element-wise,
# so they cannot key a WeakKeyDictionary directly
_cache = {}


def packed_for(weight, compute="fp32"):
    """Packed handle for a weight tensor, cached per tensor object and refreshed when it changes."""
    if weight.device.type != "cuda":
        raise RuntimeError("the dhconv kernel runs on a HIP device only")
    if compute not in COMPUTE:
        raise ValueError(f"unknown compute mode {compute!r}, expected 'fp32' or 'bf16'")
    key = (id(weight), compute)
    hit = _cache.get(key)
    p = hit[1] if hit is not None and hit[0]() is weight else None
    if p is None or p.device != weight.device or p.shape != tuple(weight.shape):
        p = PackedWeights(weight.shape[0], weight.shape[1], weight.shape[2], weight.device, compute)
        _cache[key] = (weakref.ref(weight, lambda _, k=key: _cache.pop(k, None)), p)
    return p.refresh(weight)


def dhconv_spectral(spec_in, weight, batch, mmax, triangular=True, compute="fp32"):
    """Spectral-layout contraction: [mmax, L, ld(batch*I)] -> [mmax, L, ld(batch*O)]."""
    pw = packed_for(weight, compute)
    I, O, L = pw.shape
    ld_out = int(lib.sfno_spectral_ld(batch * O))
    out = torch.empty((mmax, L, ld_out), dtype=torch.float32, device=spec_in.device)
    if ld_out != 2 * batch * O:
        out.zero_()
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
    if (ac.requires_grad or bc.requires_grad) and torch.is_grad_enabled():
        raise NotImplementedError("backward through the HIP dhconv kernel is not implemented")
    ac = ac.contiguous()
    B, I, L, M = ac.shape
    O = bc.shape[1]
    pw = packed_for(bc, compute)
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


def _contract_dense(x, weight, separable=False, operator_type="diagonal", complex=True):
    """Mirror of _contract_dense_pytorch (factorizations.py:167-200) for the operator this library implements."""
    if operator_type == "diagonal":
        raise NotImplementedError("only operator_type='dhconv' runs on the HIP path")
    if operator_type != "dhconv":
        raise ValueError(f"Unkonw operator type {operator_type}")
    if separable or not complex:
        raise NotImplementedError("only the non-separable complex dhconv runs on the HIP path")
    return _contract_dhconv(x, weight)


def get_contract_fun(weight, implementation="reconstructed", separable=False, operator_type="diagonal", complex=True):
    """Same selection interface as factorizations.py:212-247, dense tensor weights only."""
    if implementation not in ("reconstructed", "factorized"):
        raise ValueError(f'Got {implementation=}, expected "reconstructed" or "factorized"')
    if not torch.is_tensor(weight):
        raise ValueError(f"Got unexpected weight type of class {weight.__class__.__name__}")
    return partial(_contract_dense, separable=separable, complex=complex, operator_type=operator_type)
