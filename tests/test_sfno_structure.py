"""CPU checks of the SFNO network mirror: parameter names, shapes and transform wiring."""
import torch


def test_state_dict_keys_and_wiring(lib_built):
    from makani_amd.sfnonet import SphericalFourierNeuralOperatorNet

    net = SphericalFourierNeuralOperatorNet(inp_shape=(721, 1440), out_shape=(721, 1440), scale_factor=3, inp_chans=73, out_chans=73,
                                            embed_dim=8, num_layers=3)
    # internal grid 240x480, 240 degrees, 241 orders (makani/models/networks/sfnonet.py:325-326,519-520)
    assert (net.h, net.w) == (240, 480)
    for t in (net.trans_down, net.itrans_up, net.trans, net.itrans):
        assert (t.lmax, t.mmax) == (240, 241)
    assert (net.trans_down.nlat, net.trans_down.nlon, net.trans_down.grid) == (721, 1440, "equiangular")
    assert (net.itrans.nlat, net.itrans.nlon, net.itrans.grid) == (240, 480, "legendre-gauss")
    assert net.blocks[0].filter.filter.forward_transform is net.trans_down and net.blocks[0].filter.filter.inverse_transform is net.itrans
    assert net.blocks[1].filter.filter.forward_transform is net.trans and net.blocks[2].filter.filter.inverse_transform is net.itrans_up
    assert net.blocks[0].filter.filter.scale_residual and not net.blocks[1].filter.filter.scale_residual and net.blocks[2].filter.filter.scale_residual
    keys = set(net.state_dict().keys())
    expect = {"encoder.fwd.0.weight", "encoder.fwd.0.bias", "encoder.fwd.2.weight", "decoder.fwd.0.weight", "decoder.fwd.0.bias",
              "decoder.fwd.2.weight", "residual_transform.weight"}
    for i in range(3):
        p = f"blocks.{i}."
        expect |= {p + "norm0.weight", p + "norm0.bias", p + "norm1.weight", p + "norm1.bias", p + "filter.filter.weight",
                   p + "mlp.fwd.0.weight", p + "mlp.fwd.0.bias", p + "mlp.fwd.3.weight", p + "mlp.fwd.3.bias", p + "outer_skip.weight"}
    assert keys == expect
    w = net.state_dict()["blocks.1.filter.filter.weight"]
    assert tuple(w.shape) == (8, 8, 240) and w.dtype == torch.complex64
    assert tuple(net.state_dict()["blocks.0.mlp.fwd.0.weight"].shape) == (16, 8, 1, 1)


def test_pointwise_convolutions_are_conv2d_modules_on_the_cpu(lib_built):
    """The network's 1x1 convolutions are PointwiseConv2d modules: nn.Conv2d in everything a checkpoint or a CPU run sees
    (class hierarchy, parameter names and shapes, values), the HIP route being taken only for bf16 HIP tensors with a gradient."""
    import copy

    from makani_amd import pointwise as pw
    from makani_amd.sfnonet import SphericalFourierNeuralOperatorNet

    torch.manual_seed(0)
    net = SphericalFourierNeuralOperatorNet(inp_shape=(16, 32), out_shape=(16, 32), scale_factor=2, inp_chans=3, out_chans=2, embed_dim=8,
                                            num_layers=2)
    convs = [m for m in net.modules() if isinstance(m, torch.nn.Conv2d)]
    assert convs and all(isinstance(m, pw.PointwiseConv2d) and m.kernel_size == (1, 1) for m in convs)
    conv = convs[0]
    ref = torch.nn.Conv2d(conv.in_channels, conv.out_channels, 1, bias=conv.bias is not None)
    ref.load_state_dict(conv.state_dict())                      # same keys and shapes
    x = torch.randn(2, conv.in_channels, 4, 8, requires_grad=True)
    assert not pw.trainable_active(x)                           # CPU tensor: the module path
    y = conv(x)
    assert torch.equal(y, ref(x)) and not type(y.grad_fn).__name__.startswith("_Conv1x1")
    with torch.autocast("cpu", dtype=torch.bfloat16):
        assert not pw.trainable_active(x)
    twin = copy.deepcopy(conv)
    assert isinstance(twin, pw.PointwiseConv2d) and torch.equal(twin.weight, conv.weight)
