"""The normalisation behind the convolution (network/modules/refinement.py:38-43: Sequential(ConvType, Activation,
GroupNorm)): per-channel sums added up by the forward kernels (d2c_conv3d_forward_stats), GroupNorm from them
(d2c_group_norm_forward / _backward), and the fused block of util.fuse_conv_act_norm.

Expected values: torch.nn.functional.group_norm and its autograd in float64 on the CPU (the routine the reference
calls), sums of the returned output in float64, and the unfused nn.Sequential with the same parameters.
float32: 1e-4 relative / 1e-5 absolute (scaled by the tensor's magnitude for gradients); bfloat16: 2e-2 of the scale."""
import copy

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import d2conv3d_amd as d2c
from d2conv3d_amd import _ops, modules as M, util
from _util import assert_close, rel_l2

pytestmark = pytest.mark.gpu


def _check(actual, expected, dtype, what):
    expected = expected.float()
    if dtype == torch.float32:
        assert_close(actual, expected, 1e-4, 1e-5 * max(1.0, expected.abs().max().item()), what)
    else:
        assert rel_l2(actual, expected) < 2e-2, (what, rel_l2(actual, expected))
        assert_close(actual, expected, 2e-2, 2e-2 * max(expected.abs().max().item(), 1e-6), what)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape,groups,affine", [
    ((2, 32, 4, 6, 8), 4, True),        # rows of 192 values: 16-byte accesses
    ((3, 24, 3, 5, 7), 24, True),       # one channel per group, rows of 105 values: element accesses
    ((1, 640, 2, 3, 5), 1, False),      # one group of 640 channels (LayerNorm-like), no affine parameters
    ((2, 16, 37), 2, True),             # any number of spatial dimensions
])
def test_group_norm_from_statistics_matches_torch(shape, groups, affine, dtype, dev):
    g = torch.Generator().manual_seed(31)
    x = (torch.randn(shape, generator=g) * 1.7 + 0.4).to(dtype)
    C = shape[1]
    w = (torch.rand(C, generator=g) + 0.5).to(dtype) if affine else None
    b = torch.randn(C, generator=g).to(dtype) if affine else None
    gy = torch.randn(shape, generator=g).to(dtype)
    xd = x.to(dev).requires_grad_(True)
    wd = w.to(dev).requires_grad_(True) if affine else None
    bd = b.to(dev).requires_grad_(True) if affine else None
    stats = _ops.channel_stats(xd.detach())
    x64 = x.double()
    e_stats = torch.stack([x64.flatten(2).sum(-1), (x64 * x64).flatten(2).sum(-1)], dim=-1)
    assert_close(stats, e_stats, 1e-5, 1e-5 * e_stats.abs().max().item(), "channel sums")
    y = _ops.group_norm_from_stats(xd, stats, wd, bd, groups, 1e-5)
    y.backward(gy.to(dev))
    xr = x64.clone().requires_grad_(True)
    wr = w.double().clone().requires_grad_(True) if affine else None
    br = b.double().clone().requires_grad_(True) if affine else None
    ey = F.group_norm(xr, groups, wr, br, 1e-5)
    ey.backward(gy.double())
    _check(y, ey.detach(), dtype, "group norm forward")
    _check(xd.grad, xr.grad, dtype, "grad_x")
    if affine:
        _check(wd.grad, wr.grad, dtype, "grad_gamma")
        _check(bd.grad, br.grad, dtype, "grad_beta")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_group_norm_of_values_far_from_zero(dtype, dev):
    """Activations whose mean is 30 standard deviations from zero: the variance is the small difference of
    sum_sq / m and mean^2.  The per-channel sums are float32 (their rounding, amplified by mean^2 / var = 900,
    bounds the result: 1e-3 relative is asked for here, where zero-mean data meets 1e-4); they are combined and
    the difference is taken in double, so nothing more is lost.  Expected: F.group_norm in float64."""
    g = torch.Generator().manual_seed(37)
    shape, groups = (2, 32, 4, 6, 8), 4
    x = (torch.randn(shape, generator=g) + 30.0).to(dtype)
    gy = torch.randn(shape, generator=g).to(dtype)
    xd = x.to(dev).requires_grad_(True)
    stats = _ops.channel_stats(xd.detach())
    y = _ops.group_norm_from_stats(xd, stats, None, None, groups, 1e-5)
    y.backward(gy.to(dev))
    xr = x.double().clone().requires_grad_(True)
    ey = F.group_norm(xr, groups, None, None, 1e-5)
    ey.backward(gy.double())
    if dtype == torch.float32:
        assert_close(y, ey.detach(), 1e-3, 1e-3, "group norm forward, mean 30")
        assert_close(xd.grad, xr.grad, 1e-3, 1e-3 * xr.grad.abs().max().item(), "grad_x, mean 30")
    else:
        assert rel_l2(y, ey.detach()) < 2e-2 and rel_l2(xd.grad, xr.grad) < 2e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", ["dma_o320", "dma_o200_ragged", "regs_c64_many_tiles", "small_c64", "depthwise", "generic"])
@pytest.mark.parametrize("relu", [None, 1.5])
def test_convolution_returns_the_sums_of_its_output(case, relu, dtype, dev):
    # (N, Cin, Cout, dims, groups): the matrix-core kernel that adds the sums up where it stores (wide weight groups
    # on at least 128 position tiles of 64: whole work items and items whose steps are shared out; N = 2 makes
    # tiles that straddle the two samples), the register-gather kernel on enough position tiles that no steps are
    # shared out (it adds into the result itself; blocks of 32 positions that straddle the samples add lane by
    # lane), and the families that run the separate sums kernel behind the convolution
    N, Cin, Cout, dims, groups = {"dma_o320": (2, 64, 320, (5, 29, 30), 1), "dma_o200_ragged": (2, 64, 200, (7, 25, 24), 1),
                                  "regs_c64_many_tiles": (2, 64, 64, (8, 31, 33), 1),
                                  "small_c64": (2, 64, 64, (4, 6, 7), 1), "depthwise": (2, 64, 64, (4, 6, 7), 64),
                                  "generic": (2, 6, 10, (3, 5, 6), 1)}[case]
    if case == "generic" and dtype == torch.bfloat16:
        pytest.skip("float32 covers the direct kernels")
    g = torch.Generator().manual_seed(77)
    x = torch.randn(N, Cin, *dims, generator=g).to(dtype)
    w = ((torch.rand(Cout, Cin // groups, 3, 3, 3, generator=g) * 2 - 1) / (Cin // groups * 27) ** 0.5).to(dtype)
    b = (torch.rand(Cout, generator=g) - 0.5).to(dtype)
    off = torch.randn(N, 81, *dims, generator=g) * 1.5
    m = torch.sigmoid(torch.randn(N, 27, *dims, generator=g))
    x, w, b, off, m = (t.to(dev) for t in (x, w, b, off, m))
    out, stats = d2c.deform_conv3d(x, off, m, w, b, 1, 1, 1, groups, 1, output_relu=relu, output_stats=True)
    ref = d2c.deform_conv3d(x, off, m, w, b, 1, 1, 1, groups, 1, output_relu=relu)
    _check(out, ref, dtype, "output with and without the sums")
    o64 = out.double()
    e = torch.stack([o64.flatten(2).sum(-1), (o64 * o64).flatten(2).sum(-1)], dim=-1)
    assert stats.shape == (N, Cout, 2) and stats.dtype == torch.float32
    assert_close(stats, e, 1e-4, 1e-5 * e.abs().max().item(), "sums of the stored output")


class _ScaledReLU(nn.Module):      # network/layers.py:414-419; recognised by its class name
    def forward(self, x):
        return 1.71285855 * F.relu(x)


_ScaledReLU.__name__ = "ScaledReLU"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cls,act,cin,cout,dims", [
    ("MDConv3d", nn.ReLU, 64, 192, (5, 29, 30)),                         # sums added up by the forward kernel
    ("XYZSizeConditionedMDConv3d", _ScaledReLU, 64, 160, (5, 29, 30)),   # ... with the offsets formed in the sampler
    ("DConv3d", nn.ReLU, 8, 16, (3, 6, 7)),                              # direct kernels + separate sums kernel
])
def test_fused_conv_act_norm_block_matches_the_sequence(cls, act, cin, cout, dims, dtype, dev):
    torch.manual_seed(5)
    seq = nn.Sequential(getattr(M, cls)(cin, cout, 3, padding=1), act(), nn.GroupNorm(8, cout))
    with torch.no_grad():
        seq[0].deform_params.weight.normal_(0, 0.05)
        seq[0].deform_params.bias.normal_(0, 0.3)
        seq[2].weight.uniform_(0.5, 1.5)
        seq[2].bias.normal_(0, 0.5)
    plain = nn.ModuleDict({"block": seq}).to(dev, dtype)
    fused = copy.deepcopy(plain)
    assert util.fuse_conv_act_norm(fused) == 1 and isinstance(fused["block"], util.ConvActGroupNorm)
    assert list(fused.state_dict()) == list(plain.state_dict())
    x = torch.randn(2, cin, *dims, device=dev).to(dtype)
    gy = torch.randn(2, cout, *dims, device=dev).to(dtype)
    res = []
    for net in (plain, fused):
        xi = x.clone().requires_grad_(True)
        y = net["block"](xi)
        y.backward(gy)
        res.append([y.detach(), xi.grad] + [p.grad for p in net.parameters()])
    names = ["output", "grad_input"] + [n for n, _ in plain.named_parameters()]
    for n, a, e in zip(names, res[1], res[0]):
        if dtype == torch.float32:
            assert_close(a, e, 1e-3, 1e-4 * max(1.0, e.abs().max().item()), n)
        else:
            assert rel_l2(a, e) < 3e-2, (n, rel_l2(a, e))
    # and the block's output against torch's group_norm in float64 on the convolution's own output
    conv, norm = plain["block"][0], plain["block"][2]
    with torch.no_grad():
        h = plain["block"][1](conv(x)).double().cpu()
        ey = F.group_norm(h, 8, norm.weight.double().cpu(), norm.bias.double().cpu(), norm.eps)
    _check(res[1][0], ey, dtype, "fused block vs torch group_norm")
