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
