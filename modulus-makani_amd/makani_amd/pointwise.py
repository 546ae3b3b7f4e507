"""Pointwise tail of the SFNO block on the HIP kernels, for bfloat16 NCHW activations.

1x1 convolutions with fused bias / exact GELU / "+ scale * addend + shift" epilogue, and
instance norm split into its statistics (a per-(b, c) scale and shift) and their application.
These replace the nn.Conv2d(kernel_size=1) / nn.InstanceNorm2d / nn.GELU sequences of
makani/models/networks/sfnonet.py:246-262 and makani/models/common/layers.py:86-216 on the
inference path under bf16 autocast.  The plain convolution (with its bias) also has a backward on the HIP
kernels -- conv1x1_trainable, the forward of PointwiseConv2d when a gradient is asked for --, so that training under
bf16 autocast keeps its 1x1 convolutions here; the fused epilogues have none.
"""
import ctypes
import weakref

import torch

from . import _lib
from ._lib import lib, check

ACT = {None: _lib.ACT_NONE, "none": _lib.ACT_NONE, "gelu": _lib.ACT_GELU}

# id(parameter) -> (weakref, stamp, packed bf16 [O, Kpad])
_wcache = {}


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def packed_weight(weight):
    """MFMA operand stream of a 1x1 convolution weight ([O, K, 1, 1] or [O, K]); cached per parameter and
    rebuilt when the parameter changes."""
    key = id(weight)
    # (tensors made under inference_mode carry no version counter: they are packed once per tensor object)
    stamp = (weight.data_ptr(), -1 if weight.is_inference() else weight._version, weight.device)
    hit = _wcache.get(key)
    if hit is not None and hit[0]() is weight and hit[1] == stamp:
        return hit[2]
    w = weight.detach().reshape(weight.shape[0], -1).float().contiguous()
    O, K = w.shape
    p = torch.empty(lib.sfno_pointwise_weight_elems(O, K), dtype=torch.bfloat16, device=w.device)
    check(lib.sfno_pointwise_pack_weight(_ptr(w), _ptr(p), O, K, _stream(w.device)), "sfno_pointwise_pack_weight")
    _wcache[key] = (weakref.ref(weight, lambda _, k=key: _wcache.pop(k, None)), stamp, p)
    return p


def clear_cache(weight=None):
    """Forgets the packed copy of `weight` (of every weight if None); needed only after writes through ``param.data``, which
    the version stamp of the cache does not see."""
    if weight is None:
        _wcache.clear()
    else:
        _wcache.pop(id(weight), None)


def supported(x):
    """Whether the fused kernels take this activation tensor."""
    return x.is_cuda and x.dim() == 4 and x.dtype == torch.bfloat16 and (x.shape[2] * x.shape[3]) % 8 == 0 and x.shape[2] * x.shape[3] >= 8


def conv1x1(x, weight, bias=None, act=None, addend=None, add_scale=None, add_shift=None):
    """act(conv1x1(x, weight) + bias) + add_scale * addend + add_shift  ->  bf16 [B, O, H, W]."""
    if not supported(x):
        raise RuntimeError("the fused pointwise kernels take contiguous bfloat16 NCHW HIP tensors with H*W a multiple of 8")
    x = x.contiguous()
    B, K, H, W = x.shape
    pw = packed_weight(weight)
    O = weight.shape[0]
    if weight.shape[1] != K:
        raise RuntimeError(f"conv1x1: input has {K} channels, weight expects {weight.shape[1]}")
    y = torch.empty((B, O, H, W), dtype=torch.bfloat16, device=x.device)
    if bias is not None:
        bias = bias.detach().float().contiguous()
    if addend is not None:
        if addend.shape != y.shape or addend.dtype != torch.bfloat16:
            raise RuntimeError("conv1x1: addend must be a bfloat16 tensor of the output's shape")
        addend = addend.contiguous()
        if add_scale is not None:
            add_scale = add_scale.float().contiguous()
            add_shift = add_shift.float().contiguous()
            assert add_scale.numel() == B * O and add_shift.numel() == B * O
    check(
        lib.sfno_pointwise_conv(_ptr(x), _ptr(pw), _ptr(bias), _ptr(y), B, K, O, H * W, ACT[act], _ptr(addend), _ptr(add_scale),
                                _ptr(add_shift), _stream(x.device)),
        "sfno_pointwise_conv",
    )
    return y


def conv1x1_cat(x1, x2, weight, bias=None, act=None, out=None):
    """act(conv1x1(cat([x1, x2], dim=1), weight) + bias) without building the concatenation  ->  bf16 [B, O, H, W];
    weight [O, K1 + K2] (or [O, K1 + K2, 1, 1]); out: a contiguous bf16 tensor of the result's shape to write into."""
    if not (supported(x1) and supported(x2)) or x1.shape[0] != x2.shape[0] or x1.shape[2:] != x2.shape[2:]:
        raise RuntimeError("conv1x1_cat takes two contiguous bfloat16 NCHW HIP tensors of one batch and grid size, H*W a multiple of 8")
    x1, x2 = x1.contiguous(), x2.contiguous()
    B, K1, H, W = x1.shape
    K2 = x2.shape[1]
    O = weight.shape[0]
    if weight.reshape(O, -1).shape[1] != K1 + K2:
        raise RuntimeError(f"conv1x1_cat: inputs have {K1} + {K2} channels, weight expects {weight.reshape(O, -1).shape[1]}")
    pw = packed_weight(weight)
    if out is None:
        y = torch.empty((B, O, H, W), dtype=torch.bfloat16, device=x1.device)
    else:
        if tuple(out.shape) != (B, O, H, W) or out.dtype != torch.bfloat16 or not out.is_contiguous() or out.device != x1.device:
            raise RuntimeError("conv1x1_cat: out must be a contiguous bfloat16 tensor of the result's shape")
        y = out
    if bias is not None:
        bias = bias.detach().float().contiguous()
    check(lib.sfno_pointwise_conv_cat(_ptr(x1), K1, _ptr(x2), K2, _ptr(pw), _ptr(bias), _ptr(y), B, O, H * W, ACT[act], _stream(x1.device)),
          "sfno_pointwise_conv_cat")
    return y


def instance_norm_coeffs(x, gamma=None, beta=None, eps=1e-5):
    """(scale, shift) float32 [B, C] such that instance_norm(x) = scale * x + shift."""
    if not supported(x):
        raise RuntimeError("the fused pointwise kernels take contiguous bfloat16 NCHW HIP tensors with H*W a multiple of 8")
    x = x.contiguous()
    B, C, H, W = x.shape
    rows, P = B * C, H * W
    scale = torch.empty((B, C), dtype=torch.float32, device=x.device)
    shift = torch.empty_like(scale)
    nbytes = lib.sfno_instance_norm_workspace_bytes(rows, P)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    g = gamma.detach().float().contiguous() if gamma is not None else None
    b = beta.detach().float().contiguous() if beta is not None else None
    check(
        lib.sfno_instance_norm_coeffs(_ptr(x), _ptr(g), _ptr(b), _ptr(scale), _ptr(shift), rows, C, P, float(eps), _ptr(ws), nbytes, _stream(x.device)),
        "sfno_instance_norm_coeffs",
    )
    return scale, shift


def instance_norm_coeffs_lat(lat_stats, batch, gamma=None, beta=None, eps=1e-5):
    """(scale, shift) float32 [B, C] from the per-latitude moments [B*C, nlat, 2] that InverseRealSHT.synthesis_with_lat_stats returns."""
    rows, nlat, _ = lat_stats.shape
    C = rows // batch
    scale = torch.empty((batch, C), dtype=torch.float32, device=lat_stats.device)
    shift = torch.empty_like(scale)
    g = gamma.detach().float().contiguous() if gamma is not None else None
    b = beta.detach().float().contiguous() if beta is not None else None
    check(lib.sfno_instance_norm_coeffs_lat(_ptr(lat_stats), _ptr(g), _ptr(b), _ptr(scale), _ptr(shift), rows, C, nlat, float(eps),
                                            _stream(lat_stats.device)), "sfno_instance_norm_coeffs_lat")
    return scale, shift


def scale_shift_act(x, scale, shift, act=None):
    """act(scale[b, c] * x + shift[b, c]) -> bf16, same shape."""
    if not supported(x):
        raise RuntimeError("the fused pointwise kernels take contiguous bfloat16 NCHW HIP tensors with H*W a multiple of 8")
    x = x.contiguous()
    B, C, H, W = x.shape
    y = torch.empty_like(x)
    check(lib.sfno_scale_shift_act(_ptr(x), _ptr(scale), _ptr(shift), _ptr(y), B * C, H * W, ACT[act], _stream(x.device)), "sfno_scale_shift_act")
    return y


def conv1x1_weight_grad(gy, x, with_bias):
    """(gweight float32 [O, K], gbias float32 [O] or None) of y = conv1x1(x, weight) + bias for the output gradient gy:
    gweight[o, k] = sum_{b,p} gy[b, o, p] x[b, k, p], gbias[o] = sum_{b,p} gy[b, o, p]; bf16 operands, fp32 sums in a fixed order."""
    if not (supported(x) and supported(gy)) or gy.shape[0] != x.shape[0] or gy.shape[2:] != x.shape[2:]:
        raise RuntimeError("conv1x1_weight_grad takes two contiguous bfloat16 NCHW HIP tensors of one batch and grid size, H*W a multiple of 8")
    x, gy = x.contiguous(), gy.contiguous()
    B, K, H, W = x.shape
    O = gy.shape[1]
    gw = torch.empty((O, K), dtype=torch.float32, device=x.device)
    gb = torch.empty((O,), dtype=torch.float32, device=x.device) if with_bias else None
    nbytes = lib.sfno_pointwise_weight_grad_workspace_bytes(B, K, O, H * W, 1 if with_bias else 0)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    check(lib.sfno_pointwise_weight_grad(_ptr(gy), _ptr(x), _ptr(gw), _ptr(gb), B, K, O, H * W, _ptr(ws), nbytes, _stream(x.device)),
          "sfno_pointwise_weight_grad")
    return gw, gb


class _Conv1x1(torch.autograd.Function):
    """y = conv1x1(x, weight) + bias on the HIP kernels, with the three gradients autograd derives for nn.Conv2d(kernel_size=1)
    (makani/models/common/layers.py:95-116,160-216): the input gradient is the same convolution with the transposed weight."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        xb = x.detach().to(torch.bfloat16).contiguous()
        ctx.save_for_backward(xb, weight)
        ctx.has_bias = bias is not None
        ctx.x_dtype = x.dtype
        ctx.b_dtype = bias.dtype if bias is not None else None
        # (the parameter itself goes in: its packed copy is cached per parameter object and version)
        return conv1x1(xb, weight, bias)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, gy):
        xb, weight = ctx.saved_tensors
        gy = gy.to(torch.bfloat16).contiguous()
        gx = gw = gb = None
        if ctx.needs_input_grad[0]:
            wt = weight.detach().reshape(weight.shape[0], -1).t().contiguous()       # [K, O]: packed afresh, it is no parameter
            gx = conv1x1(gy, wt).to(ctx.x_dtype)
        if ctx.needs_input_grad[1] or (ctx.has_bias and ctx.needs_input_grad[2]):
            gw, gb = conv1x1_weight_grad(gy, xb, ctx.has_bias)
            gw = gw.reshape(weight.shape).to(weight.dtype)
            if gb is not None:
                gb = gb.to(ctx.b_dtype)
        return gx, gw, gb


def trainable_active(x):
    """Whether PointwiseConv2d routes this call through the HIP kernels: a gradient is being recorded and the activations are
    bf16 (or will be under bf16 autocast) HIP tensors the kernels take."""
    if not torch.is_grad_enabled() or not x.is_cuda or x.dim() != 4:
        return False
    bf16 = x.dtype == torch.bfloat16 or (torch.is_autocast_enabled() and torch.get_autocast_dtype("cuda") == torch.bfloat16)
    return bf16 and (x.shape[2] * x.shape[3]) % 8 == 0 and x.shape[2] * x.shape[3] >= 8


def conv1x1_trainable(x, weight, bias=None):
    """conv1x1(x, weight) + bias -> bf16, differentiable with respect to x, weight and bias (HIP kernels in both directions)."""
    return _Conv1x1.apply(x, weight, bias)


class PointwiseConv2d(torch.nn.Conv2d):
    """nn.Conv2d(kernel_size=1) whose training forward and backward under bf16 run on the HIP kernels; every other call (fp32,
    CPU, no gradient) is nn.Conv2d.  Same parameters and state-dict keys."""

    def __init__(self, in_channels, out_channels, bias=True):
        super().__init__(in_channels, out_channels, 1, bias=bias)

    def forward(self, x):
        if trainable_active(x) and (x.requires_grad or self.weight.requires_grad):
            return conv1x1_trainable(x, self.weight, self.bias)
        return super().forward(x)
