"""Makani's wrapper layer (makani_amd.stepper) against the float64 restatement oracle/stepper.py, and the restatement
against hand-computed numbers.  CPU tests use a small stand-in network (the wrappers are device-agnostic torch code);
the GPU test wraps the HIP SFNO."""
import types

import numpy as np
import pytest
import torch
import torch.nn as nn

from oracle import stepper as ost


def params(**kw):
    base = dict(nettype="SFNO", img_crop_shape_x=8, img_crop_shape_y=16, img_shape_x=8, img_shape_y=16, N_in_channels=3, N_out_channels=3,
                n_future=0, n_history=0, history_normalization_mode="none", target="default", add_grid=False, add_orography=False,
                add_landmask=False)
    base.update(kw)
    return types.SimpleNamespace(**base)


class Mix(nn.Module):
    """stand-in network: a fixed 1x1 convolution followed by tanh"""

    def __init__(self, cin, cout, seed=0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.w = nn.Parameter(torch.randn(cout, cin, generator=g, dtype=torch.float64) / cin ** 0.5)

    def forward(self, x):
        return torch.tanh(torch.einsum("oi,bihw->bohw", self.w.to(x.dtype), x))

    def numpy(self):
        w = self.w.detach().numpy()
        return lambda x: np.tanh(np.einsum("oi,bihw->bohw", w, x))


def test_oracle_history_statistics_by_hand():
    # two history steps of one channel on a 1 x 2 grid, decay ln 2: weights (1/3, 2/3) for (older, newer)
    x = np.array([[[[1.0, 3.0]], [[5.0, 9.0]]]])                 # [B=1, T*C=2, 1, 2]
    w = ost.history_weights("exponential", 1, np.log(2.0))
    assert np.allclose(w, [1 / 3, 2 / 3])
    mean, std = ost.history_stats(x, 1, w)
    # weighted sum over steps of the SUM over the grid, divided by the number of grid points
    m = (1 / 3 * (1 + 3) + 2 / 3 * (5 + 9)) / 2
    v = (1 / 3 * ((1 - m) ** 2 + (3 - m) ** 2) + 2 / 3 * ((5 - m) ** 2 + (9 - m) ** 2)) / 2
    assert np.allclose(mean, m) and np.allclose(std, np.sqrt(v))
    # identity model, residual learning: the prediction is added to the newest step only
    out = ost.single_step(lambda z: z[:, -1:], x, n_history=1, mode="exponential", decay=np.log(2.0), learn_residual=True)
    assert np.allclose(out[:, 0], x[:, 0]) and np.allclose(out[:, 1], 2 * x[:, 1])


@pytest.mark.parametrize("mode,n_history,residual,grid", [("none", 0, False, False), ("exponential", 2, False, True), ("exponential", 1, True, False),
                                                           ("mean", 1, False, True)])
def test_single_step_wrapper_matches_restatement(mode, n_history, residual, grid):
    from makani_amd.stepper import SingleStepWrapper

    C, T = 3, n_history + 1
    p = params(n_history=n_history, history_normalization_mode=mode, history_normalization_decay=0.7, target="residual" if residual else "default",
               normalize_residual=False, add_grid=grid, gridtype="sinusoidal", grid_num_frequencies=2)
    nstatic = 4 if grid else 0
    net = Mix(T * C + nstatic, C, seed=3)
    wrap = SingleStepWrapper(p, lambda: net).double().eval()
    x = torch.randn(2, T * C, 8, 16, generator=torch.Generator().manual_seed(1), dtype=torch.float64) * 3 + 1
    static = wrap.preprocessor.static_features.double().numpy() if grid else None
    if grid:
        assert static.shape == (1, 4, 8, 16)
        tx = np.linspace(0, 1, 9)[:-1]
        assert np.allclose(static[0, 0, :, 3], np.sin(tx)) and np.allclose(static[0, 2, :, 3], np.sin(2 * tx))
    want = ost.single_step(net.numpy(), x.numpy().copy(), n_history=n_history, mode=mode, decay=0.7, static=static, learn_residual=residual)
    with torch.no_grad():
        got = wrap(x.clone()).numpy()
    # (the history weights and the static features are float32 buffers, as in the reference: agreement to float32 rounding)
    assert got.shape == want.shape == ((2, T * C, 8, 16) if residual else (2, C, 8, 16))
    assert np.allclose(got, want, rtol=1e-6, atol=1e-6)


def test_multi_step_wrapper_training_and_eval():
    from makani_amd.stepper import MultiStepWrapper

    C, n_history, n_future = 2, 1, 2
    p = params(N_in_channels=C, N_out_channels=C, n_history=n_history, n_future=n_future, history_normalization_mode="exponential",
               history_normalization_decay=0.3)
    net = Mix(2 * C, C, seed=5)
    wrap = MultiStepWrapper(p, lambda: net).double()
    x = torch.randn(2, 2 * C, 8, 16, generator=torch.Generator().manual_seed(2), dtype=torch.float64)
    wrap.train()
    with torch.no_grad():
        got = wrap(x.clone()).numpy()
    want = ost.multi_step_train(net.numpy(), x.numpy(), n_future, n_history=n_history, mode="exponential", decay=0.3)
    assert got.shape == (2, (n_future + 1) * C, 8, 16) and np.allclose(got, want, rtol=1e-6, atol=1e-6)
    wrap.eval()
    with torch.no_grad():
        one = wrap(x.clone()).numpy()
    assert np.allclose(one, want[:, :C], rtol=1e-6, atol=1e-6)


def test_forcing_channels_follow_the_rollout():
    """Unpredicted channels (e.g. the zenith angle) are appended to every history step of the input, and the target's forcing
    of step s becomes the input forcing of step s + 1 (preprocessor.py:209-226)."""
    from makani_amd.stepper import MultiStepWrapper

    C, n_future = 2, 1
    p = params(N_in_channels=C + 1, N_out_channels=C, n_future=n_future)
    seen = []

    class Spy(nn.Module):
        def forward(self, x):
            seen.append(x.clone())
            return x[:, :C] * 0.5

    wrap = MultiStepWrapper(p, Spy).train()
    x = torch.randn(1, C, 8, 16)
    xz = torch.full((1, 1, 1, 8, 16), 7.0)
    yz = torch.stack([torch.full((1, 1, 8, 16), 8.0), torch.full((1, 1, 8, 16), 9.0)], dim=1)
    wrap.preprocessor.cache_unpredicted_features(x, None, xz, yz)
    out = wrap(x)
    assert out.shape == (1, 2 * C, 8, 16) and len(seen) == 2
    assert torch.all(seen[0][:, C] == 7.0) and torch.all(seen[1][:, C] == 8.0)
    assert torch.allclose(seen[1][:, :C], 0.5 * x)


def test_get_model_and_registry(lib_built):
    import makani_amd as ma

    p = params(img_crop_shape_x=32, img_crop_shape_y=64, img_shape_x=32, img_shape_y=64, scale_factor=4, embed_dim=8, num_layers=2)
    m = ma.get_model(p)
    assert isinstance(m, ma.SingleStepWrapper) and isinstance(m.model, ma.SphericalFourierNeuralOperatorNet)
    assert all(k.startswith("model.") for k in m.state_dict())          # Makani checkpoints carry this prefix
    assert m.model.inp_chans == 3 and m.model.embed_dim == 8 and m.model.spectral_transform == "sht"
    p.nettype, p.n_future = "FNO", 1
    m = ma.get_model(p)
    assert isinstance(m, ma.MultiStepWrapper) and m.model.spectral_transform == "fft"
    # Makani's "path/to/file.py:ClassName" route executes the file on its own: the package ships an entry file for it
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p.nettype = os.path.join(root, "modulus-makani_amd", "makani_models.py") + ":SphericalFourierNeuralOperatorNet"
    assert type(ma.get_model(p).model).__name__ == "SphericalFourierNeuralOperatorNet"
    p.nettype = "NoSuchNet"
    with pytest.raises(KeyError):
        ma.get_model(p)
    # the packaging file publishes the same two names under Makani's entry-point group
    import tomli
    eps = tomli.load(open(os.path.join(root, "modulus-makani_amd", "pyproject.toml"), "rb"))["project"]["entry-points"]["makani.models"]
    assert eps == {"SFNO": "makani_amd.sfnonet:SphericalFourierNeuralOperatorNet", "FNO": "makani_amd.stepper:FourierNeuralOperatorNet"}


@pytest.mark.gpu
def test_wrapped_hip_sfno_matches_oracle(lib_built):
    """The HIP SFNO inside the single-step wrapper: with normalisation "none" it equals the bare network bit for bit; with
    exponential history normalisation, a sinusoidal grid and residual learning it equals the float64 restatement of the
    wrapper around the float64 oracle model (fp32 network tolerance 1e-4)."""
    import makani_amd as ma
    from oracle.sfno import SfnoOracle

    base = dict(img_crop_shape_x=33, img_crop_shape_y=64, img_shape_x=33, img_shape_y=64, N_in_channels=3, N_out_channels=3, scale_factor=2, embed_dim=16,
                num_layers=2)
    torch.manual_seed(4)
    plain = ma.get_model(params(**base)).cuda().eval()
    x = torch.randn(2, 3, 33, 64, generator=torch.Generator().manual_seed(5))
    with torch.inference_mode():
        assert torch.equal(plain(x.cuda()), plain.model(x.cuda()))
    # two history steps, two static channels: the network reads 2 * 3 + 2 channels and predicts 3
    p = params(**{**base, "N_in_channels": 8}, n_history=1, history_normalization_mode="exponential", history_normalization_decay=0.5, target="residual",
               normalize_residual=False, add_grid=True, gridtype="sinusoidal", grid_num_frequencies=1)
    torch.manual_seed(4)
    wrap = ma.get_model(p).cuda().eval()
    xh = torch.randn(2, 6, 33, 64, generator=torch.Generator().manual_seed(6)) * 2 + 0.5
    with torch.inference_mode():
        got = wrap(xh.cuda().clone())
    torch.cuda.synchronize()
    oracle = SfnoOracle((33, 64), (33, 64), 2, 2)
    sd = {k[len("model."):]: v for k, v in wrap.state_dict().items()}
    model = lambda z: oracle.forward(sd, torch.from_numpy(z)).numpy()
    want = ost.single_step(model, xh.double().numpy(), n_history=1, mode="exponential", decay=0.5,
                           static=wrap.preprocessor.static_features.double().cpu().numpy(), learn_residual=True)
    err = np.linalg.norm(got.double().cpu().numpy() - want) / np.linalg.norm(want)
    print(f"wrapped SFNO vs oracle: {err:.2e}", flush=True)
    assert got.shape == (2, 6, 33, 64) and err < 1e-4
