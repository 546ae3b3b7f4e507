"""SFNO network on the HIP spectral path against the float64 oracle model (same state_dict).

fp32: relative L2 <= 1e-4 on the network output (the 1e-5 bound of the spectral kernels,
relaxed for the fp32 PyTorch convolutions / instance norms around them over several layers).
bf16 autocast: relative L2 <= 1e-2 (the spectral path itself stays fp32, as in the reference:
makani/models/common/spectral_convolution.py:124-148).
"""
import numpy as np
import pytest
import torch

from oracle.sfno import SfnoOracle

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    return np.linalg.norm((np.asarray(a) - np.asarray(b)).ravel()) / max(np.linalg.norm(np.asarray(b).ravel()), 1e-300)


def build(**kw):
    from makani_amd.sfnonet import SphericalFourierNeuralOperatorNet

    torch.manual_seed(4)
    return SphericalFourierNeuralOperatorNet(**kw)


CASES = [
    # the reference's own smoke configuration (tests/test_models.py:26-69): 32x64, 4 in / 2 out, batch 4, defaults
    dict(inp_shape=(32, 64), out_shape=(32, 64), inp_chans=4, out_chans=2, batch=4),
    # recipe-like: scale factor 3, instance norm, MLP, 3 layers, odd latitude count like 721
    dict(inp_shape=(91, 180), out_shape=(91, 180), inp_chans=5, out_chans=5, scale_factor=3, embed_dim=48, num_layers=3, batch=1),
    # output grid differs from the input grid: the big skip goes through the transforms
    dict(inp_shape=(33, 64), out_shape=(17, 32), inp_chans=3, out_chans=3, scale_factor=2, embed_dim=16, num_layers=2, batch=2),
]


@pytest.mark.parametrize("case", CASES)
def test_forward_matches_oracle_fp32(lib_built, case):
    case = dict(case)
    batch = case.pop("batch")
    print(f"case sfno fp32 {case}", flush=True)
    net = build(**case).cuda().eval()
    x = torch.randn(batch, case["inp_chans"], *case["inp_shape"], generator=torch.Generator().manual_seed(5))
    with torch.inference_mode():
        y = net(x.cuda())
    torch.cuda.synchronize()
    assert tuple(y.shape) == (batch, case["out_chans"], *case["out_shape"])
    oracle = SfnoOracle(case["inp_shape"], case["out_shape"], case.get("scale_factor", 8), case.get("num_layers", 4))
    ref = oracle.forward(net.state_dict(), x)
    assert rel_l2(y.cpu().double().numpy(), ref.numpy()) < 1e-4


@pytest.mark.parametrize("extra", [dict(pos_embed="direct"), dict(pos_embed="frequency"), dict(bias="position"), dict(bias="constant")])
def test_position_embedding_and_filter_bias(lib_built, extra):
    """Learnt position embedding ("direct": a field on the input grid; "frequency": coefficients synthesised with the
    up-sampling inverse transform, sfnonet.py:479-495, 612-622) and the SpectralConv bias (spectral_convolution.py:117-122,
    143-144) against the oracle model, with the parameters set to random values (their defaults are zeros or tiny)."""
    case = dict(inp_shape=(33, 64), out_shape=(33, 64), inp_chans=3, out_chans=2, scale_factor=2, embed_dim=16, num_layers=2)
    print(f"case sfno {extra}", flush=True)
    net = build(**case, **extra).cuda().eval()
    g = torch.Generator().manual_seed(6)
    with torch.no_grad():
        for name, prm in net.named_parameters():
            if "pos_embed" in name or name.endswith("filter.filter.bias"):
                v = torch.randn(prm.shape, generator=g)
                if name == "pos_embed.0":
                    v = torch.tril(v, diagonal=0)
                if name == "pos_embed.1":
                    v = torch.tril(v, diagonal=-1)
                prm.copy_(v)
    x = torch.randn(2, 3, 33, 64, generator=g)
    with torch.inference_mode():
        y = net(x.cuda())
    oracle = SfnoOracle(case["inp_shape"], case["out_shape"], 2, 2)
    ref = oracle.forward(net.state_dict(), x)
    assert rel_l2(y.cpu().double().numpy(), ref.numpy()) < 1e-4
    # the extra parameters matter: without them the output differs (a bias that is constant over the grid does not:
    # the instance norm that follows the filter removes it)
    if extra != dict(bias="constant"):
        sd0 = {k: v for k, v in net.state_dict().items() if "pos_embed" not in k and not k.endswith("filter.filter.bias")}
        assert rel_l2(oracle.forward(sd0, x).numpy(), ref.numpy()) > 1e-2


def test_forward_bf16_autocast(lib_built):
    """Under bf16 autocast only the pointwise layers run in bf16; the spectral path stays fp32.

    The run on the HIP kernels is compared with the same PyTorch modules (same bf16 pointwise
    arithmetic on the GPU) whose spectral operator is evaluated by the float64 oracle, so the
    difference isolates the spectral path; tolerance 1e-2.  Against the all-float64 oracle model
    the bf16 rounding of the pointwise layers dominates (checked loosely, 5e-2).
    """
    import makani_amd.spectral_convolution as sc
    from oracle.dhconv import spectral_conv
    from oracle.sht import ShtTables

    case = dict(inp_shape=(91, 180), out_shape=(91, 180), inp_chans=5, out_chans=5, scale_factor=3, embed_dim=48, num_layers=3)
    print(f"case sfno bf16 {case}", flush=True)
    net = build(**case).cuda().eval()
    x = torch.randn(2, 5, 91, 180, generator=torch.Generator().manual_seed(5))
    with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
        y = net(x.cuda())
    torch.cuda.synchronize()
    assert y.dtype == torch.bfloat16

    def tables(t):
        return ShtTables(t.nlat, t.nlon, t.lmax, t.mmax, t.grid)

    def oracle_forward(self, inp, lat_stats=False):
        out, res = spectral_conv(inp.float().cpu().double().numpy(), self.weight.detach().cpu().numpy().astype(np.complex128),
                                 tables(self.forward_transform), tables(self.inverse_transform))
        out = torch.from_numpy(out).to(inp.device, inp.dtype)
        res = torch.from_numpy(np.asarray(res)).to(inp.device, inp.dtype) if self.scale_residual else inp
        return (out, res, None) if lat_stats else (out, res)      # no moments: the block computes the row statistics itself

    hip_forward = sc.SpectralConv.forward
    try:
        sc.SpectralConv.forward = oracle_forward
        with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
            y_ref = net(x.cuda())
    finally:
        sc.SpectralConv.forward = hip_forward
    assert rel_l2(y.float().cpu().numpy(), y_ref.float().cpu().numpy()) < 1e-2
    ref64 = SfnoOracle((91, 180), (91, 180), 3, 3).forward(net.state_dict(), x)
    assert rel_l2(y.float().cpu().double().numpy(), ref64.numpy()) < 5e-2


def test_rollout_feeds_output_back(lib_built):
    """Autoregressive use (makani/utils/inferencer.py:144-177 with n_history = 0): x_{t+1} = model(x_t)."""
    case = dict(inp_shape=(32, 64), out_shape=(32, 64), inp_chans=3, out_chans=3, scale_factor=4, embed_dim=16, num_layers=2)
    net = build(**case).cuda().eval()
    x = torch.randn(1, 3, 32, 64, generator=torch.Generator().manual_seed(6))
    oracle = SfnoOracle((32, 64), (32, 64), 4, 2)
    with torch.inference_mode():
        g, r = x.cuda(), x
        for _ in range(3):
            g = net(g)
            r = oracle.forward(net.state_dict(), r).float()
    assert rel_l2(g.cpu().double().numpy(), r.double().numpy()) < 1e-4


def test_fused_pointwise_tail_matches_module_path(lib_built):
    """Under bf16 autocast without autograd the 1x1 convolutions, instance norms and GELUs run on the fused HIP
    kernels.  Same network, fused against the PyTorch module path (the reference's execution).  Both round every
    layer's output to bf16, at different places, so they are compared through the float64 oracle model: the fused
    run (fp32 accumulation, one rounding per layer) must be no further from it than the module path is, and the
    two runs must agree within the sum of those distances."""
    case = dict(inp_shape=(91, 180), out_shape=(91, 180), inp_chans=5, out_chans=5, scale_factor=3, embed_dim=48, num_layers=3)
    print(f"case sfno fused pointwise {case}", flush=True)
    net = build(**case).cuda().eval()
    # non-trivial affine parameters and biases, which the initialisation leaves at one and zero
    g = torch.Generator().manual_seed(9)
    with torch.no_grad():
        for n, p in net.named_parameters():
            if "norm" in n or n.endswith(".bias"):
                p.add_(0.3 * torch.randn(p.shape, generator=g).to(p.device))
    x = torch.randn(2, 5, 91, 180, generator=torch.Generator().manual_seed(5))

    def run(fused):
        net.fused_pointwise = fused
        for b in net.blocks:
            b.fused_pointwise = fused
        with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
            return net(x.cuda())

    y_fused, y_mod = run(True), run(False)
    torch.cuda.synchronize()
    assert y_fused.dtype == torch.bfloat16 and y_fused.shape == y_mod.shape
    ref64 = SfnoOracle((91, 180), (91, 180), 3, 3).forward(net.state_dict(), x).numpy()
    e_fused = rel_l2(y_fused.float().cpu().double().numpy(), ref64)
    e_mod = rel_l2(y_mod.float().cpu().double().numpy(), ref64)
    print(f"fused {e_fused:.3e}  module path {e_mod:.3e}", flush=True)
    assert e_fused < 2e-2 and e_fused < 1.2 * e_mod
    assert rel_l2(y_fused.float().cpu().numpy(), y_mod.float().cpu().numpy()) < e_fused + e_mod
    # with autograd recording, the module path runs (the fused kernels have no backward)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y_grad = net(x.cuda().requires_grad_(True))
    assert y_grad.requires_grad


def test_fused_pointwise_switch(lib_built):
    """fused_pointwise=False at construction keeps the PyTorch modules under no_grad + bf16 autocast too: the result equals
    the one of a network built with the default and switched off attribute by attribute, and differs from the fused one."""
    case = dict(inp_shape=(33, 64), out_shape=(33, 64), inp_chans=3, out_chans=3, scale_factor=2, embed_dim=16, num_layers=2)
    torch.manual_seed(4)
    from makani_amd.sfnonet import SphericalFourierNeuralOperatorNet

    net_off = SphericalFourierNeuralOperatorNet(**case, fused_pointwise=False).cuda().eval()
    net_on = SphericalFourierNeuralOperatorNet(**case).cuda().eval()
    net_on.load_state_dict(net_off.state_dict())
    assert not net_off.fused_pointwise and all(not b.fused_pointwise for b in net_off.blocks)
    x = torch.randn(2, 3, 33, 64, generator=torch.Generator().manual_seed(5)).cuda()
    with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
        y_off, y_on = net_off(x), net_on(x)
        net_on.fused_pointwise = False
        for b in net_on.blocks:
            b.fused_pointwise = False
        y_on_off = net_on(x)
    torch.cuda.synchronize()
    assert torch.equal(y_off, y_on_off)
    assert not torch.equal(y_off, y_on)
    assert rel_l2(y_on.float().cpu().numpy(), y_off.float().cpu().numpy()) < 3e-2


def test_encoder_fold_matches_layer_by_layer(lib_built):
    """fold_encoder: the encoder's last (linear, bias-free) 1x1 convolution is applied in spectral space, inside block 0's
    weights and skip convolution, instead of at full resolution (channel mixing commutes with the transforms).  Same network,
    folded against layer by layer, both through the float64 oracle model: the folded run must not be further from it, the
    two must agree within the sum of their distances, the shortcut must really be taken where it applies (grids differ
    between encoder and block 0) and not where block 0 runs more than once."""
    case = dict(inp_shape=(92, 180), out_shape=(92, 180), inp_chans=5, out_chans=5, scale_factor=3, embed_dim=48, num_layers=3)
    print(f"case sfno encoder fold {case}", flush=True)
    net = build(**case).cuda().eval()
    g = torch.Generator().manual_seed(11)
    with torch.no_grad():
        for n, p in net.named_parameters():
            if "norm" in n or n.endswith(".bias"):
                p.add_(0.3 * torch.randn(p.shape, generator=g).to(p.device))
    x = torch.randn(2, 5, 92, 180, generator=torch.Generator().manual_seed(7))

    def run(fold):
        net.fold_encoder = fold
        net.clear_fold_cache()
        with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
            y = net(x.cuda())
        return y, net._fold_cache is not None

    (y_fold, taken), (y_layers, taken_off) = run(True), run(False)
    assert taken and not taken_off
    ref64 = SfnoOracle((92, 180), (92, 180), 3, 3).forward(net.state_dict(), x).numpy()
    e_fold = rel_l2(y_fold.float().cpu().double().numpy(), ref64)
    e_layers = rel_l2(y_layers.float().cpu().double().numpy(), ref64)
    d = rel_l2(y_fold.float().cpu().numpy(), y_layers.float().cpu().numpy())
    print(f"folded {e_fold:.3e}  layer by layer {e_layers:.3e}  between them {d:.3e}", flush=True)
    assert e_fold < 2e-2 and e_fold < 1.1 * e_layers and d < e_fold + e_layers
    # a weight update is followed: the fold is recomputed when one of its three parameters changes
    with torch.no_grad():
        net.encoder.fwd[2].weight.mul_(1.5)
    y2, _ = run(True)
    net.fold_encoder = False
    with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
        y2_layers = net(x.cuda())
    net.fold_encoder = True
    assert rel_l2(y2.float().cpu().numpy(), y2_layers.float().cpu().numpy()) < 2e-2
    assert rel_l2(y2.float().cpu().numpy(), y_fold.float().cpu().numpy()) > 5e-2
    # not applicable with repeated layers: block 0 then also receives a later block's output
    for kw in (dict(repeat_layers=2),):
        other = build(**{**case, **kw}).cuda().eval()
        with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
            y = other(x.cuda())
        assert other._fold_cache is None and torch.isfinite(y.float()).all()


def test_fused_path_needs_eval_mode(lib_built):
    """In training mode the network runs the PyTorch modules even under no_grad and bf16 autocast (a validation pass inside a
    training loop then follows the training forward's arithmetic); eval() switches the fused kernels on."""
    case = dict(inp_shape=(48, 96), out_shape=(48, 96), inp_chans=4, out_chans=3, scale_factor=2, embed_dim=32, num_layers=2)
    net = build(**case).cuda()
    x = torch.randn(1, 4, 48, 96, generator=torch.Generator().manual_seed(13)).cuda()
    net.train()
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        y_train = net(x)
    assert net._fold_cache is None                      # the fused forward (which folds the encoder) was not taken
    net.eval()
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        y_eval = net(x)
    assert net._fold_cache is not None
    assert rel_l2(y_eval.float().cpu().numpy(), y_train.float().cpu().numpy()) < 3e-2


def test_network_built_under_inference_mode(lib_built):
    """A network whose parameters are inference tensors (built and moved to the device under torch.inference_mode()) takes the
    fused path with the encoder fold and the merged decoder: the caches of derived weights must not ask such tensors for a
    version counter.  Same output as the same state dict in ordinary tensors."""
    case = dict(inp_shape=(92, 180), out_shape=(92, 180), inp_chans=5, out_chans=5, scale_factor=3, embed_dim=128, num_layers=3)
    print(f"case sfno inference-mode parameters {case}", flush=True)
    with torch.inference_mode():
        net_inf = build(**case).cuda().eval()
    assert all(p.is_inference() for p in net_inf.parameters())
    net = build(**case).cuda().eval()
    net.load_state_dict({k: v.clone() for k, v in net_inf.state_dict().items()})
    x = torch.randn(2, 5, 92, 180, generator=torch.Generator().manual_seed(9)).cuda()
    with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
        y_inf = net_inf(x)
        y = net(x)
    assert net_inf._fold_cache is not None and net_inf._merge_cache is not None and net_inf._tail_cache is not None
    assert torch.equal(y_inf, y)


def test_encoder_fold_not_taken_when_it_widens(lib_built):
    """encoder_ratio = 2: the encoder's hidden layer is wider than the embedding, so folding its last convolution into block 0
    would run the transforms on twice the channels; the network then evaluates layer by layer (and agrees with the oracle)."""
    case = dict(inp_shape=(48, 96), out_shape=(48, 96), inp_chans=4, out_chans=3, scale_factor=2, embed_dim=32, num_layers=2, encoder_ratio=2)
    print(f"case sfno wide encoder {case}", flush=True)
    net = build(**case).cuda().eval()
    x = torch.randn(1, 4, 48, 96, generator=torch.Generator().manual_seed(10))
    with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
        y = net(x.cuda())
    assert net._fold_cache is None
    # (the same network with encoder_ratio = 1 does take the fold: the size is one the fused path accepts)
    narrow = build(**{**case, "encoder_ratio": 1}).cuda().eval()
    with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
        narrow(x.cuda())
    assert narrow._fold_cache is not None
    # the bf16 forward is held against the fp32 forward of the same network (itself pinned against the oracle above)
    with torch.inference_mode():
        y32 = net(x.cuda())
    assert rel_l2(y.float().cpu().numpy(), y32.float().cpu().numpy()) < 2e-2


def test_decoder_merge_matches_layer_by_layer(lib_built):
    """merge_decoder: the last block's "norm1(mlp) + outer_skip(residual)" and the decoder's first convolution are one convolution
    over the two tensors (both steps are linear), with per-sample weights [W_d diag(scale) | W_d W_skip] and bias W_d shift + b_d.
    Same network, merged against layer by layer, through the float64 oracle model; batch 2, so that the per-sample weights differ."""
    case = dict(inp_shape=(92, 180), out_shape=(92, 180), inp_chans=5, out_chans=5, scale_factor=3, embed_dim=128, num_layers=3)
    print(f"case sfno decoder merge {case}", flush=True)
    net = build(**case).cuda().eval()
    g = torch.Generator().manual_seed(12)
    with torch.no_grad():
        for n, p in net.named_parameters():
            if "norm" in n or n.endswith(".bias"):
                p.add_(0.3 * torch.randn(p.shape, generator=g).to(p.device))
    x = torch.randn(2, 5, 92, 180, generator=torch.Generator().manual_seed(8))
    x[1] *= 3.0

    def run(merge):
        net.merge_decoder = merge
        net._merge_cache = None
        with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
            y = net(x.cuda())
        return y, net._merge_cache is not None

    (y_m, taken), (y_l, taken_off) = run(True), run(False)
    assert taken and not taken_off
    ref64 = SfnoOracle((92, 180), (92, 180), 3, 3).forward(net.state_dict(), x).numpy()
    e_m = rel_l2(y_m.float().cpu().double().numpy(), ref64)
    e_l = rel_l2(y_l.float().cpu().double().numpy(), ref64)
    d = rel_l2(y_m.float().cpu().numpy(), y_l.float().cpu().numpy())
    print(f"merged {e_m:.3e}  layer by layer {e_l:.3e}  between them {d:.3e}", flush=True)
    assert e_m < 2e-2 and e_m < 1.1 * e_l and d < e_m + e_l
    # narrow decoders (at most 96 channels) keep the layer-by-layer evaluation
    small = build(**{**case, "embed_dim": 48}).cuda().eval()
    with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
        y = small(x.cuda())
    assert small._merge_cache is None and torch.isfinite(y.float()).all()
