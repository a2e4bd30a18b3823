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


# ---- the deformation producer of the size-conditioned layers as library kernels ------------------------
from d2conv3d_amd.grid import offsets_from_size_map, size_map_offsets  # noqa: E402


@pytest.mark.parametrize("mode,channels", [("xyz", 3), ("xxz", 2), ("xy", 2), ("x", 1)])
@pytest.mark.parametrize("activation", ["linear", "elu", "relu", "relu_plus_one"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_size_map_offsets_match_the_torch_formulation(mode, channels, activation, dtype, dev):
    # network/layers.py:171-181 + utils/grid.py:72-98 in torch against d2c_size_map_offsets_forward / _backward;
    # kernel (3, 5, 2) has an even extent (fractional kernel grid) and a non-unit dilation
    g = torch.Generator().manual_seed(17)
    raw = (torch.randn(2, channels, 3, 5, 6, generator=g) * 1.5).to(dev, dtype)
    kernel, dilation = (3, 5, 2), (1, 2, 1)
    a = raw.clone().requires_grad_(True)
    b = raw.clone().requires_grad_(True)
    ref = offsets_from_size_map(M._apply_size_activation(activation, a), mode, kernel, dilation)
    out = size_map_offsets(b, mode, kernel, dilation, activation)
    assert out.shape == ref.shape and out.dtype == ref.dtype
    if dtype == torch.float32:
        assert torch.allclose(out, ref, rtol=1e-6, atol=1e-6)
    else:
        assert torch.allclose(out.float(), ref.float(), rtol=1e-2, atol=1e-2)
    go = torch.randn(ref.shape, generator=g).to(dev, dtype)
    ref.backward(go)
    out.backward(go)
    if dtype == torch.float32:
        assert torch.allclose(b.grad, a.grad, rtol=1e-5, atol=1e-5)
    else:
        # torch rounds every partial sum to bfloat16, the kernel accumulates in float32
        scale = a.grad.float().abs().max().item()
        assert torch.allclose(b.grad.float(), a.grad.float(), rtol=5e-2, atol=5e-2 * scale)


@pytest.mark.parametrize("cls", ["XYZSizeConditionedMDConv3d", "XXZSizeConditionedDConv3d", "SizeConditionedMDConv3d"])
def test_size_conditioned_layers_same_with_and_without_the_fused_producer(cls, dev):
    torch.manual_seed(3)
    layer = getattr(M, cls)(4, 6, 3, padding=1).to(dev)
    with torch.no_grad():
        layer.deform_params.weight.normal_(0, 0.3)
        layer.deform_params.bias.normal_(0, 0.3)
    x = torch.randn(2, 4, 5, 6, 7, device=dev)
    outs, grads = [], []
    # True: the size map goes into the operator (deform_conv3d_sized); "expand": offsets tensor made by the library's
    # expansion kernel; False: the reference's torch formulation
    for fused in (True, "expand", False):
        layer.fused_deformation = fused
        layer.zero_grad()
        xi = x.clone().requires_grad_(True)
        out = layer(xi)
        out.square().sum().backward()
        outs.append(out.detach())
        grads.append([xi.grad.clone(), layer.deform_params.weight.grad.clone()])
    for i in (0, 1):
        assert torch.allclose(outs[i], outs[2], rtol=1e-5, atol=1e-5)
        for a, b in zip(grads[i], grads[2]):
            assert torch.allclose(a, b, rtol=1e-4, atol=1e-4 * max(1.0, b.abs().max().item()))


def test_size_map_offsets_reject_bad_arguments(dev):
    with pytest.raises(RuntimeError):
        size_map_offsets(torch.zeros(1, 3, 2, 2, 2), "xyz")                       # CPU tensor
    with pytest.raises(RuntimeError):
        size_map_offsets(torch.zeros(1, 2, 2, 2, 2, device=dev), "xyz")           # wrong channel count
    with pytest.raises(RuntimeError):
        size_map_offsets(torch.zeros(1, 3, 2, 2, 2, device=dev, dtype=torch.float64), "xyz")


def test_tap_statistics_match_the_oracle(dev):
    """Out-of-volume telemetry: the counts are those of the oracle's corner sets on the same offsets."""
    from d2conv3d_amd.util import tap_statistics
    from oracle import cpu
    g = torch.Generator().manual_seed(11)
    xshape, ks, stride, padding, dilation, G = (2, 8, 5, 9, 7), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 2
    off = torch.randn(2, G * 81, 5, 9, 7, generator=g) * 2.0
    _, ef = cpu.conv3d_corners(xshape, off, (8, 8) + ks, stride, padding, dilation, G)
    ef = ef.to(torch.int32)
    st = tap_statistics(xshape, off.to(dev), ks, stride, padding, dilation, G)
    n = ef.numel()
    assert st["taps"] == n
    assert st["dead"] == int((ef == 0).sum()) / n
    assert st["partial"] == int(((ef != 0) & (ef != 255)).sum()) / n
    assert st["corners_read"] == sum(int(((ef >> c) & 1).sum()) for c in range(8)) / (8.0 * n)
    assert 0.05 < st["dead"] < 0.6 and st["partial"] > 0.05     # the case does leave the volume


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("cls", ["MDConv3d", "DConv3d", "XYZSizeConditionedMDConv3d"])
def test_branch_convolution_on_the_operator(cls, dtype, dev):
    """The deformation branch's nn.Conv3d evaluated by the operator at zero offsets (modules._branch_conv: the default
    for bfloat16, "all" for float32 too) against the stock call, both held to a float64 run of the same layer (direct
    kernels): in bfloat16 the operator's branch is no further from it than the stock one (both carry the 5 - 10 % that
    bfloat16 offsets leave in the gradients that pass through them); in float32 the output agrees to 1e-4 and the
    gradients through the offsets to 1e-2 (sampling points that change their voxel, see _branch_conv)."""
    from d2conv3d_amd import modules as M
    torch.manual_seed(31)
    layer = getattr(M, cls)(128, 64, 3, padding=1).to(dev)
    with torch.no_grad():
        layer.deform_params.weight.normal_(0, 0.02)
        layer.deform_params.bias.normal_(0, 0.3)
    l64 = getattr(M, cls)(128, 64, 3, padding=1).to(dev).double()
    layer = layer.to(dtype)
    with torch.no_grad():
        for p64, p in zip(l64.parameters(), layer.parameters()):
            p64.copy_(p.double())
    x = torch.randn(1, 128, 5, 12, 13, device=dev).to(dtype)
    gout = torch.randn(1, 64, 5, 12, 13, device=dev).to(dtype)

    def step(lay, cast):
        lay.zero_grad()
        xi = cast(x).clone().requires_grad_(True)
        out = lay(xi)
        out.backward(cast(gout))
        return [out.detach().double(), xi.grad.double()] + [p.grad.double().clone() for p in lay.parameters()]

    exact = step(l64, lambda t: t.double())
    res = {}
    for on in ("all", False):
        layer.branch_on_operator = on
        res[on] = step(layer, lambda t: t)
    err = lambda a, e: ((a - e).norm() / e.norm().clamp_min(1e-30)).item()
    for i, e in enumerate(exact):
        on_op, stock = err(res["all"][i], e), err(res[False][i], e)
        if dtype == torch.bfloat16:
            assert on_op < max(1.5 * stock, 2e-2), (cls, i, on_op, stock)
        else:
            assert on_op < (1e-4 if i == 0 else 1e-2), (cls, i, on_op, stock)
    # the default: on for bfloat16 only
    layer.branch_on_operator = True
    out = step(layer, lambda t: t)[0]
    same, other = ("all", False) if dtype == torch.bfloat16 else (False, "all")
    assert err(out, res[same][0]) < 0.2 * err(out, res[other][0]), (err(out, res[same][0]), err(out, res[other][0]))
