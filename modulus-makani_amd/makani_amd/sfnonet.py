"""Spherical Fourier Neural Operator network on the HIP spectral path.

Caller-side mirror of makani/models/networks/sfnonet.py for the single-GPU, linear-filter
configuration that Makani's recipes use (config/sfnonet.yaml:24-40,149-174): same
constructor keywords, same layer order and parameter names (``encoder.fwd.N``,
``blocks.i.{norm0,norm1,filter.filter,mlp.fwd.N,outer_skip}``, ``decoder.fwd.N``,
``residual_transform``), so a Makani state_dict loads with ``strict=True``.  The spectral
filter runs on makani_amd.SpectralConv (HIP kernels).  The pointwise parts are plain PyTorch
modules, as in the reference; for inference under bf16 autocast (no gradient recorded) the
same modules are evaluated by the fused HIP kernels of makani_amd.pointwise instead.
"""
import math
from functools import partial

import torch
import torch.nn as nn

from . import pointwise as pw
from .sht import RealSHT, InverseRealSHT
from .layers import RealFFT2, InverseRealFFT2
from .spectral_convolution import SpectralConv
from .contractions import dhconv_spectral

_ACTIVATIONS = {"relu": nn.ReLU, "gelu": nn.GELU, "silu": nn.SiLU}


def _is_gelu(m):
    return isinstance(m, nn.GELU) and getattr(m, "approximate", "none") == "none"


def _is_conv1x1(m):
    return isinstance(m, nn.Conv2d) and m.kernel_size == (1, 1) and m.stride == (1, 1) and m.padding == (0, 0) and m.groups == 1


def _norm_fusable(m):
    return isinstance(m, nn.Identity) or (isinstance(m, nn.InstanceNorm2d) and not m.track_running_stats)


def _norm_coeffs(m, x):
    """(scale, shift) of a fusable normalisation layer, or (None, None) for the identity."""
    if isinstance(m, nn.Identity):
        return None, None
    return pw.instance_norm_coeffs(x, m.weight if m.affine else None, m.bias if m.affine else None, m.eps)


def _fused_chain(mods):
    """Splits a Sequential of 1x1 convolutions, GELUs and identities into (conv, act) steps; None if it holds anything else."""
    steps = []
    for m in mods:
        if isinstance(m, nn.Identity):
            continue
        if _is_conv1x1(m):
            steps.append([m, None])
        elif _is_gelu(m) and steps and steps[-1][1] is None:
            steps[-1][1] = "gelu"
        else:
            return None
    return steps or None


def _run_chain(steps, x, addend=None, add_scale=None, add_shift=None):
    for i, (conv, act) in enumerate(steps):
        last = i == len(steps) - 1
        x = pw.conv1x1(x, conv.weight, conv.bias, act, addend if last else None, add_scale if last else None, add_shift if last else None)
    return x


def _stamp(*tensors):
    """Identity of the current values of some parameters, for the caches of tensors derived from them: storage address and
    version counter (inference tensors have none: they cannot be updated in place)."""
    return tuple((t.data_ptr(), -1 if t.is_inference() else t._version) for t in tensors)


def fused_pointwise_active(x):
    """The fused kernels serve inference on bf16 activations: bf16 input or bf16 autocast, and no autograd graph (the callers
    also require ``eval()`` mode: a module in training mode always runs the PyTorch modules)."""
    if torch.is_grad_enabled() or not x.is_cuda or x.dim() != 4:
        return False
    bf16 = x.dtype == torch.bfloat16 or (torch.is_autocast_enabled() and torch.get_autocast_dtype("cuda") == torch.bfloat16)
    return bf16 and (x.shape[2] * x.shape[3]) % 8 == 0


def _pointwise(cin, cout, bias, std):
    conv = pw.PointwiseConv2d(cin, cout, bias=bias)
    nn.init.normal_(conv.weight, mean=0.0, std=std)
    if bias:
        nn.init.constant_(conv.bias, 0.0)
    return conv


class EncoderDecoder(nn.Module):
    """Stack of 1x1 convolutions: (conv + bias, activation) x num_layers, then a bias-free conv (layers.py:86-133)."""

    def __init__(self, num_layers, input_dim, output_dim, hidden_dim, act_layer, gain=1.0, input_format="nchw"):
        super().__init__()
        if input_format != "nchw":
            raise NotImplementedError(f"Error, input format {input_format} not supported.")
        mods, cur = [], input_dim
        for _ in range(num_layers):
            mods += [_pointwise(cur, hidden_dim, True, math.sqrt(2.0 / cur)), act_layer()]
            cur = hidden_dim
        mods.append(_pointwise(cur, output_dim, False, math.sqrt(gain / cur)))
        self.fwd = nn.Sequential(*mods)

    def forward(self, x):
        return self.fwd(x)


class MLP(nn.Module):
    """conv1x1 -> activation -> dropout -> conv1x1 -> dropout (layers.py:136-216); parameters at fwd.0 and fwd.3."""

    def __init__(self, in_features, hidden_features=None, out_features=None, act_layer=nn.GELU, output_bias=True, drop_rate=0.0,
                 drop_type="iid", gain=1.0, **kwargs):
        super().__init__()
        out_features = out_features or in_features
        hidden_features = hidden_features or in_features
        fc1 = _pointwise(in_features, hidden_features, True, math.sqrt(2.0 / in_features))
        fc2 = _pointwise(hidden_features, out_features, output_bias, math.sqrt(gain / hidden_features))
        if drop_rate > 0.0:
            drop = nn.Dropout(drop_rate) if drop_type == "iid" else nn.Dropout2d(drop_rate)
        else:
            drop = nn.Identity()
        self.fwd = nn.Sequential(fc1, act_layer(), drop, fc2, drop)

    def forward(self, x):
        return self.fwd(x)


class SpectralFilterLayer(nn.Module):
    """Holder of the spectral operator under the name ``filter`` (sfnonet.py:51-116); linear, unfactorized filters only."""

    def __init__(self, forward_transform, inverse_transform, embed_dim, filter_type="linear", operator_type="diagonal", hidden_size_factor=1,
                 factorization=None, rank=1.0, separable=False, complex_activation="real", spectral_layers=1, bias=False, drop_rate=0.0, gain=1.0):
        super().__init__()
        if filter_type != "linear" or factorization is not None:
            raise NotImplementedError("the HIP path implements filter_type='linear' without factorization")
        self.filter = SpectralConv(forward_transform, inverse_transform, embed_dim, embed_dim, operator_type=operator_type, separable=separable,
                                   bias=bias, gain=gain)

    def forward(self, x, lat_stats=False):
        return self.filter(x, lat_stats=lat_stats) if lat_stats else self.filter(x)


class FourierNeuralOperatorBlock(nn.Module):
    """filter -> norm0 -> (+ inner skip) -> act -> MLP -> norm1 -> (+ outer skip) (sfnonet.py:119-267)."""

    def __init__(self, forward_transform, inverse_transform, embed_dim, filter_type="linear", operator_type="diagonal", mlp_ratio=2.0,
                 mlp_drop_rate=0.0, path_drop_rate=0.0, act_layer=nn.GELU, norm_layer=(nn.Identity, nn.Identity), rank=1.0, factorization=None,
                 separable=False, inner_skip="linear", outer_skip=None, use_mlp=False, complex_activation="real", spectral_layers=1, bias=False,
                 final_activation=False, fused_pointwise=True, **kwargs):
        super().__init__()
        # fused_pointwise (not a Makani option): evaluate the tail of the block with the fused HIP kernels when no gradient
        # is recorded and the activations are bfloat16; False keeps the PyTorch modules in every situation
        self.fused_pointwise = fused_pointwise
        if path_drop_rate > 0.0:
            raise NotImplementedError("stochastic depth is a training feature outside this path")
        self.input_shape_loc = (forward_transform.nlat, forward_transform.nlon)
        self.output_shape_loc = (inverse_transform.nlat, inverse_transform.nlon)
        self.norm0 = norm_layer[0]()

        gain_factor = 1.0 if act_layer == nn.Identity else 2.0
        if inner_skip == "linear":
            gain_factor /= 2.0
            self.inner_skip = _pointwise(embed_dim, embed_dim, False, math.sqrt(gain_factor / embed_dim))
        elif inner_skip == "identity":
            self.inner_skip = nn.Identity()
            gain_factor /= 2.0
        elif inner_skip != "none":
            raise ValueError(f"Unknown skip connection type {inner_skip}")

        self.filter = SpectralFilterLayer(forward_transform, inverse_transform, embed_dim, filter_type, operator_type, hidden_size_factor=mlp_ratio,
                                          factorization=factorization, rank=rank, separable=separable, complex_activation=complex_activation,
                                          spectral_layers=spectral_layers, bias=bias, drop_rate=path_drop_rate, gain=gain_factor)
        self.act_layer0 = act_layer()
        self.norm1 = norm_layer[1]()

        gain_factor = 2.0 if (final_activation and act_layer != nn.Identity) else 1.0
        if outer_skip == "linear":
            gain_factor /= 2.0
            self.outer_skip = _pointwise(embed_dim, embed_dim, False, math.sqrt(gain_factor / embed_dim))
        elif outer_skip == "identity":
            self.outer_skip = nn.Identity()
            gain_factor /= 2.0
        elif outer_skip not in ("none", None):
            raise ValueError(f"Unknown skip connection type {outer_skip}")

        if use_mlp:
            self.mlp = MLP(in_features=embed_dim, hidden_features=int(embed_dim * mlp_ratio), act_layer=act_layer, drop_rate=mlp_drop_rate,
                           drop_type="features", gain=gain_factor)
        if final_activation:
            self.act_layer1 = act_layer()

    def _fusable(self):
        if not (hasattr(self, "mlp") and _fused_chain(self.mlp.fwd) and _is_gelu(self.act_layer0)):
            return False
        if hasattr(self, "inner_skip") or hasattr(self, "act_layer1") or not _norm_fusable(self.norm0) or not _norm_fusable(self.norm1):
            return False
        return hasattr(self, "outer_skip") and _is_conv1x1(self.outer_skip) and self.outer_skip.bias is None

    def _forward_fused(self, x, residual, lat_stats=None, skip_weight=None, defer_skip=False):
        """norm0 -> GELU -> MLP -> norm1 -> + outer_skip(residual) in five kernels: row statistics (or, for norm0, the
        per-latitude moments the inverse transform delivered with x), scale/shift + GELU, two 1x1 convolutions with bias
        (+ GELU) epilogues, row statistics, and the skip convolution whose epilogue adds the normalised MLP output."""
        if lat_stats is not None and isinstance(self.norm0, nn.InstanceNorm2d):
            m = self.norm0
            sc, sh = pw.instance_norm_coeffs_lat(lat_stats, x.shape[0], m.weight if m.affine else None, m.bias if m.affine else None, m.eps)
        else:
            sc, sh = _norm_coeffs(self.norm0, x)
        if sc is None:
            sc = torch.ones(x.shape[:2], dtype=torch.float32, device=x.device)
            sh = torch.zeros_like(sc)
        x = pw.scale_shift_act(x, sc, sh, "gelu")
        x = _run_chain(_fused_chain(self.mlp.fwd), x)
        sc, sh = _norm_coeffs(self.norm1, x)
        if defer_skip:
            # the caller merges "norm1(x) + outer_skip(residual)" into the linear layer that follows (the network's _decoder_merge)
            return x, residual, sc, sh
        # skip_weight: the skip convolution composed with a linear map the caller pulled out of `residual` (see the network's
        # _encoder_fold)
        return pw.conv1x1(residual, self.outer_skip.weight if skip_weight is None else skip_weight, None, None, x, sc, sh)

    def forward(self, x, defer_skip=False):
        # on the fused inference path the inverse transform hands over the moments norm0 needs together with its output
        want_stats = getattr(self, "fused_pointwise", True) and not self.training and fused_pointwise_active(x) and x.dtype == torch.bfloat16 and self._fusable()
        if want_stats:
            x, residual, lat_stats = self.filter(x, lat_stats=True)
        else:
            (x, residual), lat_stats = self.filter(x), None
        if getattr(self, "fused_pointwise", True) and not self.training and fused_pointwise_active(x) and x.dtype == torch.bfloat16 and residual.dtype == torch.bfloat16 \
                and residual.shape[2:] == x.shape[2:] and self._fusable():
            return self._forward_fused(x.contiguous(), residual.contiguous(), lat_stats, defer_skip=defer_skip)
        # (defer_skip is honoured on the fused path only; here the block's output comes back whole)
        x = self.norm0(x)
        if hasattr(self, "inner_skip"):
            x = x + self.inner_skip(residual)
        x = self.act_layer0(x)
        if hasattr(self, "mlp"):
            x = self.mlp(x)
        x = self.norm1(x)
        if hasattr(self, "outer_skip"):
            x = x + self.outer_skip(residual)
        if hasattr(self, "act_layer1"):
            x = self.act_layer1(x)
        return x


class SphericalFourierNeuralOperatorNet(nn.Module):
    """SFNO (sfnonet.py:270-640): encoder -> num_layers blocks -> decoder, plus the big skip connection."""

    def __init__(self, spectral_transform="sht", model_grid_type="equiangular", sht_grid_type="legendre-gauss", filter_type="linear",
                 operator_type="dhconv", inp_shape=(721, 1440), out_shape=(721, 1440), scale_factor=8, inp_chans=2, out_chans=2, embed_dim=32,
                 num_layers=4, repeat_layers=1, use_mlp=True, mlp_ratio=2.0, encoder_ratio=1, decoder_ratio=1, activation_function="gelu",
                 encoder_layers=1, pos_embed="none", pos_drop_rate=0.0, path_drop_rate=0.0, mlp_drop_rate=0.0,
                 normalization_layer="instance_norm", max_modes=None, hard_thresholding_fraction=1.0, big_skip=True, rank=1.0,
                 factorization=None, separable=False, complex_activation="real", spectral_layers=3, bias=False, checkpointing=0,
                 spectral_compute="fp32", fused_pointwise=True, fold_encoder=True, merge_decoder=True, **kwargs):
        super().__init__()
        # fold_encoder (not a Makani option): on the fused inference path the encoder's last (linear) convolution is applied in
        # spectral space, inside the first block's weights, instead of at full resolution; see _encoder_fold
        self.fold_encoder = fold_encoder
        self._fold_cache = None
        # merge_decoder (not a Makani option): on the same path the last block's skip convolution and norm1 are merged into the
        # decoder's first convolution; see _decoder_merge_ok
        self.merge_decoder = merge_decoder
        self._merge_cache = None
        self._tail_cache = None
        # fused_pointwise (not a Makani option): under torch.no_grad() / inference_mode() with bf16 autocast the 1x1 convolutions,
        # instance norms and GELUs run on the fused HIP kernels (weights rounded to bf16 once, fp32 accumulation, one rounding per
        # layer, norm0 statistics from the unrounded field).  A forward that records gradients always runs the PyTorch modules, so
        # a validation pass under no_grad does not follow the training forward's arithmetic to the bit: pass False (or set the
        # attribute on the network and on every block) where train and validation numbers must come from the same path.
        self.fused_pointwise = fused_pointwise
        # spectral_compute = "bf16" (not a Makani option) runs the Legendre and dhconv contractions on bf16 MFMA
        self.spectral_compute = spectral_compute
        if spectral_transform not in ("sht", "fft"):
            raise ValueError("Unknown spectral transform")
        self.spectral_transform = spectral_transform
        self.inp_shape, self.out_shape = tuple(inp_shape), tuple(out_shape)
        self.inp_chans, self.out_chans, self.embed_dim = inp_chans, out_chans, embed_dim
        self.repeat_layers, self.big_skip = repeat_layers, big_skip
        self.h = int(self.inp_shape[0] // scale_factor)
        self.w = int(self.inp_shape[1] // scale_factor)
        self._init_spectral_transforms(model_grid_type, sht_grid_type, hard_thresholding_fraction, max_modes)

        if activation_function not in _ACTIVATIONS:
            raise ValueError(f"Unknown activation function {activation_function}")
        act = _ACTIVATIONS[activation_function]

        self.encoder = EncoderDecoder(encoder_layers, inp_chans, embed_dim, int(encoder_ratio * embed_dim), act)
        self.pos_drop = nn.Dropout(p=pos_drop_rate) if pos_drop_rate > 0.0 else nn.Identity()

        if normalization_layer == "layer_norm":
            raise NotImplementedError("layer_norm over channels of an nchw tensor is Makani's own distributed module; use instance_norm or none")
        elif normalization_layer == "instance_norm":
            norm = partial(nn.InstanceNorm2d, num_features=embed_dim, eps=1e-6, affine=True, track_running_stats=False)
        elif normalization_layer == "none":
            norm = nn.Identity
        else:
            raise NotImplementedError(f"Error, normalization {normalization_layer} not implemented.")

        self.blocks = nn.ModuleList()
        for i in range(num_layers):
            fwd = self.trans_down if i == 0 else self.trans
            inv = self.itrans_up if i == num_layers - 1 else self.itrans
            self.blocks.append(
                FourierNeuralOperatorBlock(fwd, inv, embed_dim, filter_type=filter_type, operator_type=operator_type, mlp_ratio=mlp_ratio,
                                           mlp_drop_rate=mlp_drop_rate, path_drop_rate=0.0 if path_drop_rate == 0.0 else path_drop_rate * i / max(num_layers - 1, 1),
                                           act_layer=act, norm_layer=(norm, norm), inner_skip="none", outer_skip="linear", use_mlp=use_mlp, rank=rank,
                                           factorization=factorization, separable=separable, complex_activation=complex_activation,
                                           spectral_layers=spectral_layers, bias=bias, fused_pointwise=fused_pointwise))
            self.blocks[-1].filter.filter.compute = spectral_compute

        self.decoder = EncoderDecoder(encoder_layers, embed_dim, out_chans, int(decoder_ratio * embed_dim), act, gain=0.5 if big_skip else 1.0)
        if big_skip:
            self.residual_transform = _pointwise(inp_chans, out_chans, False, math.sqrt(0.5 / inp_chans))

        if pos_embed == "direct":
            self.pos_embed = nn.Parameter(torch.zeros(1, embed_dim, self.inp_shape[0], self.inp_shape[1]))
            self.pos_embed.type = "direct"
            with torch.no_grad():
                nn.init.trunc_normal_(self.pos_embed, std=0.02)
        elif pos_embed == "frequency":
            lmax, mmax = self.itrans_up.lmax, self.itrans_up.mmax
            rcoeffs = nn.Parameter(torch.tril(torch.randn(1, embed_dim, lmax, mmax), diagonal=0))
            ccoeffs = nn.Parameter(torch.tril(torch.randn(1, embed_dim, lmax, mmax - 1), diagonal=-1))
            with torch.no_grad():
                nn.init.trunc_normal_(rcoeffs, std=0.02)
                nn.init.trunc_normal_(ccoeffs, std=0.02)
            self.pos_embed = nn.ParameterList([rcoeffs, ccoeffs])
            self.pos_embed.type = "frequency"
        elif pos_embed not in ("none", "None", None):
            raise ValueError("Unknown position embedding type")

    def _init_spectral_transforms(self, model_grid_type, sht_grid_type, hard_thresholding_fraction, max_modes):
        # mode counts and the four transform objects exactly as sfnonet.py:503-571 derives them
        if max_modes is not None:
            modes_lat, modes_lon = max_modes
        else:
            modes_lat = int(self.h * hard_thresholding_fraction)
            modes_lon = int((self.w // 2 + 1) * hard_thresholding_fraction)
        c = self.spectral_compute
        if self.spectral_transform == "fft":
            # planar pair (sfnonet.py:542-556); the grid type arguments do not apply
            self.trans_down = RealFFT2(*self.inp_shape, lmax=modes_lat, mmax=modes_lon).float()
            self.itrans_up = InverseRealFFT2(*self.out_shape, lmax=modes_lat, mmax=modes_lon).float()
            self.trans = RealFFT2(self.h, self.w, lmax=modes_lat, mmax=modes_lon).float()
            self.itrans = InverseRealFFT2(self.h, self.w, lmax=modes_lat, mmax=modes_lon).float()
            self.inp_shape_loc = (self.trans_down.nlat, self.trans_down.nlon)
            self.out_shape_loc = (self.itrans_up.nlat, self.itrans_up.nlon)
            self.h_loc, self.w_loc = self.itrans.nlat, self.itrans.nlon
            return
        self.trans_down = RealSHT(*self.inp_shape, lmax=modes_lat, mmax=modes_lon, grid=model_grid_type, compute=c).float()
        self.itrans_up = InverseRealSHT(*self.out_shape, lmax=modes_lat, mmax=modes_lon, grid=model_grid_type, compute=c).float()
        self.trans = RealSHT(self.h, self.w, lmax=modes_lat, mmax=modes_lon, grid=sht_grid_type, compute=c).float()
        self.itrans = InverseRealSHT(self.h, self.w, lmax=modes_lat, mmax=modes_lon, grid=sht_grid_type, compute=c).float()
        self.inp_shape_loc = (self.trans_down.nlat, self.trans_down.nlon)
        self.out_shape_loc = (self.itrans_up.nlat, self.itrans_up.nlon)
        self.h_loc, self.w_loc = self.itrans.nlat, self.itrans.nlon

    def _forward_features(self, x):
        for _ in range(self.repeat_layers):
            for blk in self.blocks:
                x = blk(x)
        return x

    # The encoder ends in a bias-free 1x1 convolution W2 (layers.py:129-131) and the first block starts with a transform to a
    # different grid, so the encoder's output x = W2 h is used by nothing but that transform (the block takes its residual from
    # the coefficients, spectral_convolution.py:132-134).  Channel mixing commutes with the transforms: SHT(W2 h) = W2 SHT(h).  On
    # the fused inference path the convolution at full resolution is therefore not run at all: the transform takes h, W2 goes
    # into the block's spectral weight (w'[j, o, l] = sum_i W2[i, j] w[i, o, l], computed once per weight update) and into the
    # skip convolution of the residual (W_skip W2).  W2 enters with its bf16-rounded values, as autocast would use it; what
    # differs from the layer-by-layer evaluation is one bf16 rounding of the 384-channel field that is no longer made.
    def _encoder_fold(self):
        """(encoder steps without the last convolution, folded spectral weight, folded skip weight), or None where the
        shortcut does not apply."""
        if not getattr(self, "fold_encoder", True) or self.repeat_layers != 1 or len(self.blocks) == 0:
            return None
        enc = _fused_chain(self.encoder.fwd)
        blk = self.blocks[0]
        conv = blk.filter.filter
        if enc is None or len(enc) < 2 or enc[-1][1] is not None or enc[-1][0].bias is not None:
            return None
        # the fold moves the first block's transforms, channel mix and skip convolution from the encoder's output channels to
        # its hidden channels: worth it only if those are not more
        if enc[-1][0].in_channels > enc[-1][0].out_channels:
            return None
        if not (isinstance(blk, FourierNeuralOperatorBlock) and blk._fusable() and getattr(blk, "fused_pointwise", True)):
            return None
        if not (conv._fused and conv.scale_residual and not hasattr(conv, "bias") and conv.in_channels == enc[-1][0].out_channels):
            return None
        w2, w0, ws = enc[-1][0].weight, conv.weight, blk.outer_skip.weight
        stamp = _stamp(w2, w0, ws)
        cached = getattr(self, "_fold_cache", None)
        if cached is None or cached[0] != stamp:
            # (ordinary tensors, also when called under inference_mode: the packed-operand caches read version counters)
            with torch.inference_mode(False), torch.no_grad():
                w2b = w2.detach().reshape(w2.shape[0], w2.shape[1]).to(torch.bfloat16).float()        # [i, j]
                wf = torch.einsum("ij,iol->jol", w2b.to(torch.complex64), w0.detach()).contiguous()
                wsb = ws.detach().reshape(ws.shape[0], ws.shape[1]).to(torch.bfloat16).float()
                wsk = (wsb @ w2b).reshape(ws.shape[0], w2.shape[1], 1, 1).contiguous()
            cached = (stamp, wf, wsk)
            self._fold_cache = cached
        return enc[:-1], cached[1], cached[2]

    def clear_fold_cache(self):
        """Forgets the folded weights (they follow in-place updates of their three parameters through the version counters;
        call this after writing one of them through ``.data``)."""
        self._fold_cache = None
        self._merge_cache = None
        self._tail_cache = None

    def _block0_folded(self, h, wf, wsk):
        blk = self.blocks[0]
        conv = blk.filter.filter
        B = h.shape[0]
        spec = conv.forward_transform.analysis(h)
        residual = conv.inverse_transform.synthesis(spec, (B, h.shape[1]), dtype=torch.bfloat16)
        spec = dhconv_spectral(spec, wf, B, conv.modes_lon, triangular=conv._triangular, compute=conv.compute)
        x, stats = conv.inverse_transform.synthesis_with_lat_stats(spec, (B, conv.out_channels), dtype=torch.bfloat16)
        return blk._forward_fused(x.contiguous(), residual.contiguous(), stats, skip_weight=wsk)

    # The last block ends in  x = scale * m + shift + W_skip r  (norm1 of the MLP output m as a per-(sample, channel) affine, plus
    # the skip convolution of the residual r) and nothing but the decoder's first convolution W_d, b_d reads x.  Both steps are
    # linear, so they are one convolution over the two tensors m and r, with the weight [W_d diag(scale) | W_d W_skip] and the
    # bias W_d shift + b_d of each sample: the sum is never written and the skip convolution's 384 x 384 products per pixel at
    # full resolution are not computed.  W_d and W_skip enter with their bf16-rounded values, as autocast would use them.
    def _decoder_merge_ok(self):
        if not getattr(self, "merge_decoder", True) or self.repeat_layers != 1 or len(self.blocks) < 2:
            return False
        dec = _fused_chain(self.decoder.fwd)
        blk = self.blocks[-1]
        if dec is None or not (isinstance(blk, FourierNeuralOperatorBlock) and blk._fusable() and getattr(blk, "fused_pointwise", True)):
            return False
        wd = dec[0][0].weight
        return wd.shape[0] > 96 and wd.shape[1] == blk.outer_skip.weight.shape[0]

    def _tail_cat_ok(self):
        dec = _fused_chain(self.decoder.fwd)
        return bool(self.big_skip and getattr(self, "merge_decoder", True) and dec and dec[-1][1] is None)

    def _tail_weight(self, conv):
        """[W_last | W_res] of the decoder's last convolution and residual_transform, cached until one of them changes."""
        wl, wr = conv.weight, self.residual_transform.weight
        stamp = _stamp(wl, wr)
        cached = getattr(self, "_tail_cache", None)
        if cached is None or cached[0] != stamp:
            with torch.inference_mode(False), torch.no_grad():
                w = torch.cat([wl.detach().reshape(wl.shape[0], -1).float(), wr.detach().reshape(wr.shape[0], -1).float()], dim=1).contiguous()
            cached = (stamp, w)
            self._tail_cache = cached
        return cached[1]

    def _decoder_merged(self, x):
        """Last block and the decoder's first step for the output x of the block before it; returns the result and the decoder
        steps still to run."""
        blk, dec = self.blocks[-1], _fused_chain(self.decoder.fwd)
        conv_d = dec[0][0]
        out = blk(x, defer_skip=True)
        if not isinstance(out, tuple):           # the block could not take its fused path after all: layer by layer from here
            return out, dec
        m, r, sc, sh = out
        B, C = m.shape[:2]
        with torch.inference_mode(False), torch.no_grad():
            cached = getattr(self, "_merge_cache", None)
            stamp = _stamp(conv_d.weight, blk.outer_skip.weight)
            if cached is None or cached[0] != stamp:
                wd = conv_d.weight.detach().reshape(conv_d.weight.shape[0], -1).to(torch.bfloat16).float()
                ws = blk.outer_skip.weight.detach().reshape(C, -1).to(torch.bfloat16).float()
                cached = (stamp, wd, (wd @ ws).contiguous())
                self._merge_cache = cached
            wd, wds = cached[1], cached[2]
            if sc is None:
                sc = torch.ones((B, C), dtype=torch.float32, device=m.device)
                sh = torch.zeros_like(sc)
            sc, sh = sc.clone(), sh.clone()          # ordinary tensors for the arithmetic below
            # all samples at once: [W_d diag(scale_b) | W_d W_skip] and W_d shift_b (+ bias); only the left half depends on b
            wcat = torch.cat([wd[None] * sc[:, None, :], wds[None].expand(B, -1, -1)], dim=2).contiguous()
            bias = sh @ wd.t()
            if conv_d.bias is not None:
                bias = bias + conv_d.bias.detach().float()
        y = torch.empty((B, wd.shape[0], m.shape[2], m.shape[3]), dtype=torch.bfloat16, device=m.device)
        for b in range(B):
            pw.conv1x1_cat(m[b:b + 1], r[b:b + 1], wcat[b], bias[b], dec[0][1], out=y[b:b + 1])
        return y, dec[1:]

    def _forward_fused(self, x):
        """Encoder, blocks and decoder with every 1x1 convolution on the fused bf16 kernels (inference under bf16 autocast)."""
        enc, dec = _fused_chain(self.encoder.fwd), _fused_chain(self.decoder.fwd)
        xb = x.to(torch.bfloat16).contiguous()
        cat_tail = False
        if self.big_skip:
            if self.out_shape != self.inp_shape:
                residual = self.itrans_up(self.trans_down(x.to(torch.float32)).contiguous()).to(torch.bfloat16).contiguous()
            else:
                residual = xb
            # the decoder's last convolution and residual_transform feed one sum (sfnonet.py:636-638): one convolution over
            # the two tensors with the weight [W_last | W_res]; where that does not apply the residual is convolved here
            cat_tail = self._tail_cat_ok()
            if not cat_tail:
                residual = pw.conv1x1(residual, self.residual_transform.weight)
        fold = self._encoder_fold()
        merge = self._decoder_merge_ok()
        if fold is not None:
            x = self._block0_folded(_run_chain(fold[0], xb), fold[1], fold[2])
            rest = self.blocks[1:]
        elif merge:
            x = _run_chain(enc, xb)
            rest = self.blocks
        else:
            x = _run_chain(enc, xb)
            x = self._forward_features(x)
            rest = []
        for blk in (rest[:-1] if merge else rest):
            x = blk(x)
        if merge:
            x, dec = self._decoder_merged(x.to(torch.bfloat16).contiguous())
        x = x.to(torch.bfloat16).contiguous()
        if self.big_skip and cat_tail:
            if not dec:                           # the merged convolution was the decoder's last step: the residual is still to be added
                return x + pw.conv1x1(residual, self.residual_transform.weight)
            x = _run_chain(dec[:-1], x)
            conv = dec[-1][0]
            return pw.conv1x1_cat(x, residual, self._tail_weight(conv), conv.bias, None)
        if not dec:
            return x + residual if self.big_skip else x
        return _run_chain(dec, x, residual if self.big_skip else None)

    def _fusable(self, x):
        if not (getattr(self, "fused_pointwise", True) and not self.training and fused_pointwise_active(x)) or hasattr(self, "pos_embed"):
            return False
        if not isinstance(self.pos_drop, nn.Identity) or (self.out_shape[0] * self.out_shape[1]) % 8 != 0:
            return False
        if self.big_skip and not (_is_conv1x1(self.residual_transform) and self.residual_transform.bias is None):
            return False
        return _fused_chain(self.encoder.fwd) is not None and _fused_chain(self.decoder.fwd) is not None

    def forward(self, x):
        if self._fusable(x):
            return self._forward_fused(x)
        if self.big_skip:
            if self.out_shape != self.inp_shape:
                xtype = x.dtype
                residual = self.itrans_up(self.trans_down(x.to(torch.float32)).contiguous()).to(dtype=xtype)
            else:
                residual = x
        x = self.encoder(x)
        if hasattr(self, "pos_embed"):
            if self.pos_embed.type == "frequency":
                pe = torch.stack([self.pos_embed[0], nn.functional.pad(self.pos_embed[1], (1, 0), "constant", 0)], dim=-1)
                pe = self.itrans_up(torch.view_as_complex(pe.float().contiguous()))
            else:
                pe = self.pos_embed
            x = x + pe
        x = self.pos_drop(x)
        x = self._forward_features(x)
        x = self.decoder(x)
        if self.big_skip:
            x = x + self.residual_transform(residual)
        return x
