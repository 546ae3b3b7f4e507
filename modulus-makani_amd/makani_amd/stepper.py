"""Makani's model wrappers around the HIP network: input/output normalisation over the history, static features,
residual learning and the autoregressive feed-back, with the interfaces of makani/models/stepper.py:21-129
(SingleStepWrapper, MultiStepWrapper), makani/models/preprocessor.py:29-420 (Preprocessor2D) and the model
construction of makani/models/model_registry.py:119-166 (get_model).  Single GPU: the spatial reductions of the
reference (preprocessor.py:300-322) are plain sums here.

`params` is any object with Makani's attribute names (a types.SimpleNamespace, a YParams object, ...); entries that
Makani's trainer always sets and a stand-alone user may leave out fall back to the defaults of config/sfnonet.yaml.
"""
import importlib.util
import os
from functools import partial

import numpy as np
import torch
import torch.nn as nn


def _get(params, name, default=None):
    return getattr(params, name, default)


class Preprocessor2D(nn.Module):
    """History normalisation, static features, unpredicted (forcing) channels and the residual rule."""

    def __init__(self, params):
        super().__init__()
        self.n_history = int(_get(params, "n_history", 0))
        self.history_normalization_mode = _get(params, "history_normalization_mode", "none")
        nh = self.n_history + 1
        if self.history_normalization_mode == "exponential":
            decay = float(params.history_normalization_decay)
            # oldest step first: weight exp(-decay * age), normalised to one
            w = torch.exp(-decay * torch.arange(self.n_history, -1, -1, dtype=torch.float32))
            w = (w / w.sum()).reshape(1, nh, 1, 1, 1)
        elif self.history_normalization_mode == "mean":
            w = torch.full((1, nh, 1, 1, 1), 1.0 / nh, dtype=torch.float32)
        elif self.history_normalization_mode in ("none", "timediff"):
            w = torch.ones(nh, dtype=torch.float32)
        else:
            raise ValueError(f"unknown history_normalization_mode {self.history_normalization_mode!r}")
        self.register_buffer("history_normalization_weights", w, persistent=False)
        self.history_mean = self.history_std = None
        self.history_eps = 1e-6

        self.learn_residual = _get(params, "target", "default") == "residual"
        self.residual_scale = None
        if self.learn_residual and _get(params, "normalize_residual", False):
            self.register_buffer("residual_scale", torch.from_numpy(np.load(params.time_diff_stds_path)).to(torch.float32), persistent=False)

        self.img_shape = [params.img_shape_x, params.img_shape_y]
        # forcing channels that the model reads but does not predict, kept between calls (train and eval apart)
        self.unpredicted_inp_train = self.unpredicted_tar_train = None
        self.unpredicted_inp_eval = self.unpredicted_tar_eval = None

        feats = []
        if _get(params, "add_grid", False):
            if hasattr(params, "lat") and hasattr(params, "lon"):
                if _get(params, "data_grid_type", "equiangular") != _get(params, "model_grid_type", "equiangular"):
                    raise NotImplementedError("grid conversion between data and model grids is Makani's GridConverter; not part of this path")
                tx = torch.deg2rad(torch.as_tensor(params.lat, dtype=torch.float32))
                ty = torch.deg2rad(torch.as_tensor(params.lon, dtype=torch.float32))
            else:
                tx = torch.linspace(0, 1, params.img_shape_x + 1, dtype=torch.float32)[:-1]
                ty = torch.linspace(0, 1, params.img_shape_y + 1, dtype=torch.float32)[:-1]
            gx, gy = torch.meshgrid(tx, ty, indexing="ij")
            grid = torch.stack([gx, gy])[None]
            if _get(params, "gridtype", "sinusoidal") == "sinusoidal":
                nfreq = int(_get(params, "grid_num_frequencies", 1))
                grid = torch.cat([torch.sin(grid)] + [torch.sin(f * grid) for f in range(2, nfreq + 1)], dim=1)
            feats.append(grid)
        if _get(params, "add_orography", False):
            oro = torch.as_tensor(np.load(params.orography_path), dtype=torch.float32)[None, None]
            feats.append((oro - oro.mean()) / (oro.std() + 1.0e-6))
        if _get(params, "add_landmask", False):
            lsm = torch.as_tensor(np.load(params.landmask_path), dtype=torch.long)
            feats.append(torch.nn.functional.one_hot(lsm).permute(2, 0, 1).to(torch.float32)[None])
        self.do_add_static_features = bool(feats)
        if feats:
            self.register_buffer("static_features", torch.cat(feats, dim=1), persistent=False)

    # -- history bookkeeping: [B, T*C, H, W] <-> [B, T, C, H, W]
    def flatten_history(self, x):
        return x.reshape(x.shape[0], x.shape[1] * x.shape[2], *x.shape[3:]) if x.dim() == 5 else x

    def expand_history(self, x, nhist):
        return x.reshape(x.shape[0], nhist, x.shape[1] // nhist, *x.shape[2:]) if x.dim() == 4 else x

    def add_residual(self, x, dx):
        if not self.learn_residual:
            return dx
        if self.residual_scale is not None:
            dx = dx * self.residual_scale
        x = self.expand_history(x, self.n_history + 1)
        x[:, -1] = x[:, -1] + dx               # in place, as the reference does
        return self.flatten_history(x)

    def add_static_features(self, x):
        if self.do_add_static_features:
            x = torch.cat([x, self.static_features.expand(x.shape[0], -1, -1, -1).to(x.dtype)], dim=1)
        return x

    def remove_static_features(self, x):
        return x[:, : x.shape[1] - self.static_features.shape[1]] if self.do_add_static_features else x

    def _unpredicted(self, which):
        return getattr(self, f"unpredicted_{which}_{'train' if self.training else 'eval'}")

    def cache_unpredicted_features(self, x, y, xz=None, yz=None):
        for which, val in (("inp", xz), ("tar", yz)):
            name = f"unpredicted_{which}_{'train' if self.training else 'eval'}"
            cur = getattr(self, name)
            if cur is not None and val is not None:
                cur.copy_(val)
            else:
                setattr(self, name, val)
        return x, y

    def append_channels(self, x, xc):
        flat = x.dim() == 4
        out = torch.cat([self.expand_history(x, self.n_history + 1), self.expand_history(xc, self.n_history + 1)], dim=2)
        return self.flatten_history(out) if flat else out

    def append_unpredicted_features(self, inp):
        z = self._unpredicted("inp")
        return inp if z is None else self.append_channels(inp, z)

    def remove_unpredicted_features(self, inp):
        z = self._unpredicted("inp")
        if z is None:
            return inp
        x = self.expand_history(inp, self.n_history + 1)
        return self.flatten_history(x[:, :, : x.shape[2] - z.shape[2]])

    def append_history(self, x1, x2, step):
        """Next input of the rollout: drop the oldest step, append the prediction; the forcing of the target step moves in."""
        zin, ztar = self._unpredicted("inp"), self._unpredicted("tar")
        if ztar is not None and step < ztar.shape[1]:
            nxt = ztar[:, step : step + 1]
            zin.copy_(nxt if self.n_history == 0 else torch.cat([zin[:, 1:], nxt], dim=1))
        if self.n_history == 0:
            return x2
        x1 = self.expand_history(x1, self.n_history + 1)
        return self.flatten_history(torch.cat([x1[:, 1:], self.expand_history(x2, 1)], dim=1))

    # -- normalisation over space and (weighted) over the history
    def history_compute_stats(self, x):
        if self.history_normalization_mode == "none":
            self.history_mean = torch.zeros((1, 1, 1, 1), dtype=torch.float32, device=x.device)
            self.history_std = torch.ones((1, 1, 1, 1), dtype=torch.float32, device=x.device)
            return
        if self.history_normalization_mode == "timediff":
            raise NotImplementedError("timediff statistics are computed but never applied by the reference (preprocessor.py:325-326)")
        xr = self.expand_history(x, self.n_history + 1)
        npix = float(self.img_shape[0] * self.img_shape[1])
        w = self.history_normalization_weights
        mean = torch.sum(xr * w, dim=(1, 3, 4), keepdim=True) / npix
        var = torch.sum(torch.square(xr - mean) * w, dim=(1, 3, 4), keepdim=True) / npix
        self.history_mean, self.history_std = mean.squeeze(1), torch.sqrt(var).squeeze(1)

    def history_normalize(self, x, target=False):
        if self.history_normalization_mode in ("none", "timediff"):
            return x
        shape = x.shape
        x = self.flatten_history(x)
        if target:      # predicted channels only
            xn = (x - self.history_mean[:, : x.shape[1]]) / self.history_std[:, : x.shape[1]]
        else:
            rep = (1, self.n_history + 1, 1, 1)
            xn = (x - self.history_mean.repeat(rep)) / self.history_std.repeat(rep)
        return xn.reshape(shape)

    def history_denormalize(self, xn, target=False):
        if self.history_normalization_mode in ("none", "timediff"):
            return xn
        assert self.history_mean is not None and self.history_std is not None
        shape = xn.shape
        xn = self.flatten_history(xn)
        if target:
            x = xn * self.history_std[:, : xn.shape[1]] + self.history_mean[:, : xn.shape[1]]
        else:
            rep = (1, self.n_history + 1, 1, 1)
            x = xn * self.history_std.repeat(rep) + self.history_mean.repeat(rep)
        return x.reshape(shape)


class SingleStepWrapper(nn.Module):
    """forcing channels -> normalise -> static features -> model -> denormalise -> residual (stepper.py:21-47)."""

    def __init__(self, params, model_handle):
        super().__init__()
        self.preprocessor = Preprocessor2D(params)
        self.model = model_handle()

    def _step(self, inp):
        pre = self.preprocessor
        x = pre.append_unpredicted_features(inp)
        pre.history_compute_stats(x)
        x = pre.add_static_features(pre.history_normalize(x, target=False))
        y = pre.history_denormalize(self.model(x), target=True)
        return pre.add_residual(inp, y)

    def forward(self, inp):
        return self._step(inp)


class MultiStepWrapper(SingleStepWrapper):
    """Training: n_future + 1 fed-back steps, predictions concatenated along the channels; evaluation: one step
    (stepper.py:50-129)."""

    def __init__(self, params, model_handle):
        super().__init__(params, model_handle)
        self.residual_mode = _get(params, "target", "default") == "target"
        self.n_future = int(params.n_future)

    def forward(self, inp):
        if not self.training:
            return self._step(inp)
        preds, cur = [], inp
        for step in range(self.n_future + 1):
            pred = self._step(cur)          # denormalised with this step's statistics, before the next step replaces them
            preds.append(pred)
            if step < self.n_future:
                cur = self.preprocessor.append_history(cur, pred, step)
        return torch.cat(preds, dim=1)


class FourierNeuralOperatorNet(nn.Module):
    """The planar FNO: the SFNO network with spectral_transform="fft" (sfnonet.py:657-659).  Defined as a factory class so
    that `nettype: FNO` resolves to a torch module like in Makani."""

    def __new__(cls, *args, **kwargs):
        from .sfnonet import SphericalFourierNeuralOperatorNet

        kwargs.pop("spectral_transform", None)
        return SphericalFourierNeuralOperatorNet(*args, spectral_transform="fft", **kwargs)


def _registry():
    from .sfnonet import SphericalFourierNeuralOperatorNet

    reg = {"SFNO": SphericalFourierNeuralOperatorNet, "FNO": FourierNeuralOperatorNet}
    try:        # models other packages publish under Makani's entry-point group
        from importlib.metadata import entry_points

        for ep in entry_points(group="makani.models"):
            reg.setdefault(ep.name, ep)
    except Exception:
        pass
    return reg


def get_model(params, **kwargs):
    """Constructs the wrapped model the way Makani's registry does: the network named by params.nettype ("SFNO", "FNO", an
    entry point of the group makani.models, or "path/to/file.py:ClassName") receives inp_shape, out_shape, inp_chans,
    out_chans and every entry of params as keyword arguments, and is wrapped for single- or multi-step use."""
    inp_shape = (params.img_crop_shape_x, params.img_crop_shape_y)
    out_shape = (params.out_shape_x, params.out_shape_y) if hasattr(params, "out_shape_x") and hasattr(params, "out_shape_y") else inp_shape
    reg = _registry()
    name = params.nettype
    handle = reg.get(name)
    if handle is None:
        if ":" not in name or len(name.split(":")) != 2:
            raise KeyError(f"No model is registered under the name {name}")
        path, cls = name.split(":")
        if not os.path.exists(path):
            raise ValueError(f"Expected string of format 'path/to/model_file.py:ModuleName' but {path} does not exist.")
        spec = importlib.util.spec_from_file_location(cls, path)
        module = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(module)
        handle = getattr(module, cls)
    elif hasattr(handle, "load"):
        handle = handle.load()
    opts = params.to_dict() if hasattr(params, "to_dict") else dict(vars(params))
    for k in ("inp_shape", "out_shape", "inp_chans", "out_chans"):
        opts.pop(k, None)
    handle = partial(handle, inp_shape=inp_shape, out_shape=out_shape, inp_chans=params.N_in_channels, out_chans=params.N_out_channels, **opts, **kwargs)
    return MultiStepWrapper(params, handle) if int(_get(params, "n_future", 0)) > 0 else SingleStepWrapper(params, handle)
