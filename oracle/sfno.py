"""Float64 CPU restatement of the SFNO forward pass (oracle).

Functional form of makani/models/networks/sfnonet.py:587-640 (network forward),
119-267 (block), makani/models/common/layers.py:86-133,136-216 (1x1-conv stacks) and
makani/models/common/spectral_convolution.py:124-148 for the linear/dhconv/instance-norm
recipe of config/sfnonet.yaml:24-40, driven by a state_dict with Makani's key names.
The spectral parts run on the numpy oracle, the pointwise parts on torch float64.
"""
import numpy as np
import torch
import torch.nn.functional as F

from .sht import ShtTables
from .fft2 import Fft2Modes
from .dhconv import spectral_conv, transform_forward, transform_inverse


class SfnoOracle:
    def __init__(self, inp_shape, out_shape, scale_factor, num_layers, model_grid_type="equiangular", sht_grid_type="legendre-gauss",
                 activation="gelu", normalization="instance_norm", big_skip=True, use_mlp=True, hard_thresholding_fraction=1.0,
                 spectral_transform="sht"):
        h, w = inp_shape[0] // scale_factor, inp_shape[1] // scale_factor
        ml, mm = int(h * hard_thresholding_fraction), int((w // 2 + 1) * hard_thresholding_fraction)
        if spectral_transform == "fft":      # sfnonet.py:542-556
            self.down = Fft2Modes(inp_shape[0], inp_shape[1], ml, mm)
            self.up = Fft2Modes(out_shape[0], out_shape[1], ml, mm)
            self.mid = Fft2Modes(h, w, ml, mm)
        else:
            self.down = ShtTables(inp_shape[0], inp_shape[1], ml, mm, model_grid_type)
            self.up = ShtTables(out_shape[0], out_shape[1], ml, mm, model_grid_type)
            self.mid = ShtTables(h, w, ml, mm, sht_grid_type)
        self.inp_shape, self.out_shape = tuple(inp_shape), tuple(out_shape)
        self.num_layers, self.big_skip, self.use_mlp = num_layers, big_skip, use_mlp
        self.act = {"gelu": F.gelu, "relu": F.relu, "silu": F.silu}[activation]
        self.normalization = normalization

    @staticmethod
    def _conv(x, sd, name):
        w = sd[name + ".weight"].double().to(x.device)
        b = sd.get(name + ".bias")
        if x.is_cuda:
            # a 1x1 convolution is a matrix product over channels; float64 convolutions have no device library behind them
            y = torch.einsum("oi,bihw->bohw", w[:, :, 0, 0], x)
            return y if b is None else y + b.double().to(x.device)[None, :, None, None]
        return F.conv2d(x, w, None if b is None else b.double())

    def _norm(self, x, sd, name):
        if self.normalization == "none":
            return x
        return F.instance_norm(x, weight=sd[name + ".weight"].double().to(x.device), bias=sd[name + ".bias"].double().to(x.device), eps=1e-6)

    def forward(self, sd, x, pointwise_device="cpu", taps=None):
        """pointwise_device: where the float64 torch ops between the spectral operators run ("cpu", or a HIP device for the
        full-size model, whose 1x1 convolutions are 4.5 TFLOP per sample); the spectral operators always run on the numpy
        oracle.  taps: optional dict that receives the input of every SpectralConv (key = block index) as a CPU tensor."""
        sd = {k: v.detach().cpu() for k, v in sd.items()}
        dev = torch.device(pointwise_device)
        x = x.detach().cpu().double()
        if self.big_skip:
            if self.out_shape != self.inp_shape:
                residual = torch.from_numpy(transform_inverse(transform_forward(x.numpy(), self.down), self.up))
            else:
                residual = x
        residual = residual.to(dev) if self.big_skip else None
        y = self._conv(self.act(self._conv(x.to(dev), sd, "encoder.fwd.0")), sd, "encoder.fwd.2")
        # position embedding (sfnonet.py:612-622): a learnt field, or learnt coefficients synthesised on the input grid
        if "pos_embed" in sd:
            y = y + sd["pos_embed"].double().to(dev)
        elif "pos_embed.0" in sd:
            re, im = sd["pos_embed.0"].double().numpy(), sd["pos_embed.1"].double().numpy()
            c = re + 1j * np.pad(im, ((0, 0), (0, 0), (0, 0), (1, 0)))
            y = y + torch.from_numpy(transform_inverse(c, self.up)).to(dev)
        for i in range(self.num_layers):
            fwd = self.down if i == 0 else self.mid
            inv = self.up if i == self.num_layers - 1 else self.mid
            p = f"blocks.{i}."
            w = sd[p + "filter.filter.weight"].numpy().astype(np.complex128)
            if taps is not None:
                taps[i] = y.cpu()
            z, res = spectral_conv(y.cpu().numpy(), w, fwd, inv)
            z, res = torch.from_numpy(z).to(dev), torch.from_numpy(np.asarray(res)).to(dev)
            if p + "filter.filter.bias" in sd:           # spectral_convolution.py:143-144
                z = z + sd[p + "filter.filter.bias"].double().to(dev)
            z = self.act(self._norm(z, sd, p + "norm0"))
            if self.use_mlp:
                z = self._conv(self.act(self._conv(z, sd, p + "mlp.fwd.0")), sd, p + "mlp.fwd.3")
            z = self._norm(z, sd, p + "norm1")
            y = z + self._conv(res, sd, p + "outer_skip")
        y = self._conv(self.act(self._conv(y, sd, "decoder.fwd.0")), sd, "decoder.fwd.2")
        if self.big_skip:
            y = y + self._conv(residual, sd, "residual_transform")
        return y.cpu()
