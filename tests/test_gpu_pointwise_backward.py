"""Gradients of the 1x1 convolution on the HIP kernels (bf16 activations) against float64 autograd of the reference op
(nn.Conv2d(kernel_size=1) + bias, makani/models/common/layers.py:95-116,160-216) on the same bf16-rounded operands.

weight / bias gradient: bf16 operands are exact inputs, products exact in fp32, fp32 sums -> relative L2 <= 1e-5, per row of
   the weight gradient too (a row whose pixels were dropped or counted twice fails by far more);
input gradient: the forward kernel on the transposed weight, one bf16 rounding at the store -> relative L2 <= 3e-3."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    a, b = a.detach().cpu().double(), b.detach().cpu().double()
    return float(torch.linalg.norm((a - b).ravel()) / max(float(torch.linalg.norm(b.ravel())), 1e-300))


WGRAD_CASES = [
    # B, K, O, H, W, bias
    (1, 20, 36, 13, 8, True),          # one tile, one share, rows and columns far inside the tile
    (2, 73, 384, 20, 36, True),        # encoder: three row tiles, bias column inside the first column tile
    (1, 384, 73, 45, 80, False),       # decoder: two column tiles, the second half empty
    (3, 256, 128, 9, 8, True),         # K = tile width: the bias column opens a second column tile of its own
    (2, 300, 260, 11, 24, True),       # nothing a multiple of the tile sizes; pixels per sample not a multiple of the 32-pixel chunk
    (1, 1, 1, 1, 8, True),             # smallest shape
    (1, 384, 768, 120, 240, True),     # MLP fc1 at a quarter of the model's grid: many shares
    (2, 768, 384, 60, 124, False),     # MLP fc2, two samples, 232.5 chunks per sample
]


@pytest.mark.parametrize("B,K,O,H,W,bias", WGRAD_CASES)
def test_weight_and_bias_gradient(lib_built, B, K, O, H, W, bias):
    from makani_amd import pointwise as pw

    assert (H * W) % 8 == 0              # the kernels take H*W a multiple of 8
    print(f"case pointwise wgrad B={B} K={K} O={O} {H}x{W} bias={bias}", flush=True)
    g = torch.Generator().manual_seed(31)
    x = torch.randn(B, K, H, W, generator=g).bfloat16()
    gy = (torch.randn(B, O, H, W, generator=g) * torch.exp(torch.randn(B, O, 1, 1, generator=g))).bfloat16()
    want_w = torch.einsum("bop,bkp->ok", gy.double().reshape(B, O, -1), x.double().reshape(B, K, -1))
    want_b = gy.double().sum(dim=(0, 2, 3))

    gw, gb = pw.conv1x1_weight_grad(gy.cuda(), x.cuda(), bias)
    torch.cuda.synchronize()
    assert gw.shape == (O, K) and gw.dtype == torch.float32
    assert torch.isfinite(gw).all()
    assert rel_l2(gw, want_w) < 1e-5
    rows = torch.linalg.norm(gw.cpu().double() - want_w, dim=1) / torch.linalg.norm(want_w, dim=1).clamp_min(1e-300)
    assert float(rows.max()) < 1e-4, (int(rows.argmax()), float(rows.max()))
    if bias:
        assert gb.shape == (O,) and rel_l2(gb, want_b) < 1e-5
    else:
        assert gb is None
    # the sums run in a fixed order: a second call gives the same bits
    gw2, gb2 = pw.conv1x1_weight_grad(gy.cuda(), x.cuda(), bias)
    torch.cuda.synchronize()
    assert torch.equal(gw, gw2) and (gb is None or torch.equal(gb, gb2))


def test_weight_gradient_counts_every_pixel_once(lib_built):
    """x = 1 and gy = 1 in bf16: every entry of the weight gradient is the number of pixels, exactly, for pixel counts around the
    chunk (32) and share boundaries and for several samples."""
    from makani_amd import pointwise as pw

    for B, P in [(1, 8), (1, 40), (2, 264), (3, 1000), (1, 32 * 4097 + 8)]:
        print(f"case pointwise wgrad count B={B} P={P}", flush=True)
        x = torch.ones(B, 5, 1, P, dtype=torch.bfloat16, device="cuda")
        gy = torch.ones(B, 3, 1, P, dtype=torch.bfloat16, device="cuda")
        gw, gb = pw.conv1x1_weight_grad(gy, x, True)
        torch.cuda.synchronize()
        assert torch.equal(gw.cpu(), torch.full((3, 5), float(B * P))) and torch.equal(gb.cpu(), torch.full((3,), float(B * P)))


AUTOGRAD_CASES = [
    # B, K, O, H, W, bias, x requires grad
    (2, 73, 384, 20, 36, True, False),      # first layer of the encoder: the input needs no gradient
    (1, 384, 768, 16, 24, True, True),
    (2, 768, 384, 13, 8, False, True),
    (1, 100, 200, 11, 24, True, True),
]


@pytest.mark.parametrize("B,K,O,H,W,bias,xgrad", AUTOGRAD_CASES)
def test_trainable_convolution_against_float64_autograd(lib_built, B, K, O, H, W, bias, xgrad):
    from makani_amd import pointwise as pw

    print(f"case pointwise autograd B={B} K={K} O={O} {H}x{W} bias={bias} xgrad={xgrad}", flush=True)
    g = torch.Generator().manual_seed(41)
    x = torch.randn(B, K, H, W, generator=g).bfloat16()
    w = torch.randn(O, K, 1, 1, generator=g) / np.sqrt(K)
    bvec = torch.randn(O, generator=g) if bias else None
    gy = torch.randn(B, O, H, W, generator=g).bfloat16()

    # float64 reference on the operands as the kernels see them (bf16 activations, bf16-rounded weight)
    xr = x.double().requires_grad_(xgrad)
    wr = w.bfloat16().double().requires_grad_(True)
    br = bvec.double().requires_grad_(True) if bias else None
    F.conv2d(xr, wr, br).backward(gy.double())

    conv = pw.PointwiseConv2d(K, O, bias=bias).cuda()
    with torch.no_grad():
        conv.weight.copy_(w)
        if bias:
            conv.bias.copy_(bvec)
    xg = x.cuda().requires_grad_(xgrad)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = conv(xg)
    assert y.dtype == torch.bfloat16 and y.grad_fn is not None and type(y.grad_fn).__name__.startswith("_Conv1x1")
    y.backward(gy.cuda())
    torch.cuda.synchronize()
    assert rel_l2(y, F.conv2d(x.double(), w.bfloat16().double(), bvec.double() if bias else None)) < 3e-3
    assert conv.weight.grad.dtype == torch.float32 and conv.weight.grad.shape == w.shape
    assert rel_l2(conv.weight.grad, wr.grad) < 1e-5
    if bias:
        assert rel_l2(conv.bias.grad, br.grad) < 1e-5
    if xgrad:
        assert xg.grad.dtype == torch.bfloat16 and rel_l2(xg.grad, xr.grad) < 3e-3
    else:
        assert xg.grad is None


def test_pointwise_conv2d_is_nn_conv2d_elsewhere(lib_built):
    """Without a gradient, in fp32 or on the CPU the module is nn.Conv2d: same values, same state-dict keys."""
    from makani_amd import pointwise as pw

    print("case pointwise module fallback", flush=True)
    torch.manual_seed(5)
    conv = pw.PointwiseConv2d(12, 7, bias=True)
    ref = torch.nn.Conv2d(12, 7, 1, bias=True)
    assert list(conv.state_dict().keys()) == list(ref.state_dict().keys())
    ref.load_state_dict(conv.state_dict())
    x = torch.randn(2, 12, 4, 8)
    assert torch.equal(conv(x), ref(x))                                   # CPU
    conv, ref, x = conv.cuda(), ref.cuda(), x.cuda()
    y = conv(x.requires_grad_(True))                                      # fp32 with a gradient: the library's convolution
    assert y.dtype == torch.float32 and not type(y.grad_fn).__name__.startswith("_Conv1x1")
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        assert torch.equal(conv(x), ref(x))                               # bf16 without a gradient


def test_training_step_through_the_network_matches_the_module_path(lib_built):
    """One forward + backward of a small SFNO under bf16 autocast in training mode: the 1x1 convolutions run on the HIP kernels
    in both directions (their nodes are in the graph) and every parameter gradient agrees with the same network evaluated with
    nn.Conv2d's own kernels to bf16 accuracy."""
    import makani_amd as ma
    from makani_amd import pointwise as pw

    print("case pointwise training step", flush=True)
    torch.manual_seed(11)
    kw = dict(inp_shape=(33, 64), out_shape=(33, 64), inp_chans=5, out_chans=3, scale_factor=2, embed_dim=32, num_layers=2)
    net = ma.SphericalFourierNeuralOperatorNet(**kw).cuda().train()
    x = torch.randn(2, 5, 33, 64, device="cuda")
    tgt = torch.randn(2, 3, 33, 64, device="cuda")

    def grads(use_hip):
        net.zero_grad(set_to_none=True)
        saved = pw.trainable_active
        if not use_hip:
            pw.trainable_active = lambda t: False
        try:
            with torch.autocast("cuda", dtype=torch.bfloat16):
                y = net(x)
            names = set()
            stack = [y.grad_fn]
            seen = set()
            while stack:
                f = stack.pop()
                if f is None or f in seen:
                    continue
                seen.add(f)
                names.add(type(f).__name__)
                stack.extend(n for n, _ in f.next_functions)
            loss = ((y.float() - tgt) ** 2).mean()
            loss.backward()
        finally:
            pw.trainable_active = saved
        torch.cuda.synchronize()
        real = lambda t: torch.view_as_real(t) if t.is_complex() else t
        return float(loss.detach()), {n: real(p.grad.detach()).clone() for n, p in net.named_parameters() if p.grad is not None}, names

    l_hip, g_hip, names_hip = grads(True)
    l_ref, g_ref, names_ref = grads(False)
    assert any(n.startswith("_Conv1x1") for n in names_hip) and not any(n.startswith("_Conv1x1") for n in names_ref)
    assert abs(l_hip - l_ref) <= 2e-2 * abs(l_ref)
    assert set(g_hip) == set(g_ref) and len(g_hip) > 10
    # (a bias in front of an instance norm has a zero gradient up to rounding noise: parameters whose gradient is far below the
    # largest one are judged together with the others, not one by one)
    norms = {n: float(torch.linalg.norm(g_ref[n].double())) for n in g_ref}
    top = max(norms.values())
    worst = max((rel_l2(g_hip[n], g_ref[n]), n) for n in g_ref if norms[n] > 1e-2 * top)
    assert worst[0] < 5e-2, worst
    err = sum(float(torch.linalg.norm((g_hip[n] - g_ref[n]).double())) ** 2 for n in g_ref) ** 0.5
    assert err < 3e-2 * sum(v * v for v in norms.values()) ** 0.5
