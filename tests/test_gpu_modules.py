"""GPU known-answer tests of the self-deforming layers
(ops/dconv-native/test/test_modules.py:8-73) plus replacement utilities."""
import pytest
import torch
import torch.nn as nn

import d2conv3d_amd as d2c
from d2conv3d_amd import modules as M
from d2conv3d_amd.util import add_deformable_conv

pytestmark = pytest.mark.gpu


def test_no_deform_dconv(dev):
    data = torch.randn(2, 3, 7, 7, 7, device=dev)
    conv = nn.Conv3d(3, 4, 3).to(dev)
    dconv = d2c.DConv3d(3, 4, 3).to(dev)
    dconv.deform_conv.weight.data = conv.weight.data
    dconv.deform_conv.bias.data = conv.bias.data
    assert torch.allclose(conv(data), dconv(data), atol=1e-6)


def test_no_deform_mdconv(dev):
    data = torch.randn(2, 3, 7, 7, 7, device=dev)
    conv = nn.Conv3d(3, 4, 3).to(dev)
    mdconv = d2c.MDConv3d(3, 4, 3).to(dev)
    mdconv.deform_conv.weight.data = conv.weight.data
    mdconv.deform_conv.bias.data = conv.bias.data
    assert torch.allclose(conv(data * 0.5), mdconv(data), atol=1e-6)   # sigmoid(0) = 0.5


def test_size_conditioning(dev):
    data = torch.randn(2, 3, 7, 7, 7, device=dev)
    conv = nn.Conv3d(3, 4, 3, padding=(1, 2, 2), dilation=(1, 2, 2)).to(dev)
    dconv = d2c.SizeConditionedDConv3d(3, 4, 3, padding=1).to(dev)
    dconv.deform_params.weight.data[0] = 0
    dconv.deform_params.bias.data[0] = 1          # ELU(1) + 1 = 2
    dconv.deform_conv.weight.data = conv.weight.data
    dconv.deform_conv.bias.data = conv.bias.data
    assert torch.allclose(conv(data), dconv(data), atol=1e-6)


def test_backward_runs(dev):
    data = torch.randn(2, 3, 7, 7, 7, device=dev)
    dconv = d2c.DConv3d(3, 4, 3, padding=1, bias=False).to(dev)
    dconv(data).mean().backward()
    assert dconv.deform_params.weight.grad is not None and dconv.deform_conv.weight.grad is not None


@pytest.mark.parametrize("cls", [M.XYZSizeConditionedMDConv3d, M.XXZSizeConditionedMDConv3d,
                                 M.XYSizeConditionedDConv3d, M.SpatialMDConv3d, M.TemporalDConv3d])
def test_variants_forward_backward(cls, dev):
    torch.manual_seed(0)
    layer = cls(4, 6, 3, padding=1).to(dev)
    nn.init.normal_(layer.deform_params.weight, std=0.05)
    x = torch.randn(2, 4, 5, 6, 7, device=dev, requires_grad=True)
    y = layer(x)
    assert y.shape == (2, 6, 5, 6, 7)
    y.square().mean().backward()
    assert torch.isfinite(x.grad).all() and layer.deform_params.weight.grad.abs().sum() > 0


def test_add_deformable_conv_replaces_and_keeps_weights(dev):
    net = nn.Sequential(nn.Conv3d(4, 8, 3, padding=1), nn.ReLU(), nn.Conv3d(8, 8, 1), nn.Conv3d(8, 4, 3, padding=1))
    ref = [m.weight.detach().clone() for m in net if isinstance(m, nn.Conv3d)]
    net2, n = add_deformable_conv(net, version="XYZSizeConditionedDCNv2")
    assert n == 2 and isinstance(net2[0], M.XYZSizeConditionedMDConv3d) and isinstance(net2[2], nn.Conv3d)
    assert torch.equal(net2[0].deform_conv.weight, ref[0]) and torch.equal(net2[3].deform_conv.weight, ref[2])
    net2 = net2.to(dev)
    x = torch.randn(1, 4, 4, 6, 6, device=dev)
    # zero-initialised deformation: modulation 0.5 everywhere, dilation ELU(0)+1 = 1
    y = net2(x)
    assert y.shape == (1, 4, 4, 6, 6) and torch.isfinite(y).all()
