"""Offsets held at zero along some axes inside the operator (descriptor field offset_axes): what the Spatial and
Temporal layers of the reference do by overwriting channels of a cloned offsets tensor
(ops/dconv-native/src/dconv_native/modules.py:87-120).  Expected values: the CPU oracle on the offsets tensor with
those channels zeroed; their gradient channels must come back exactly zero."""
import pytest
import torch

import d2conv3d_amd as d2c
from d2conv3d_amd import modules as M
from oracle import cpu
from _util import assert_close, rel_l2

pytestmark = pytest.mark.gpu


def _case(N, Cin, Cout, dims, G, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, Cin, *dims, generator=g)
    w = (torch.rand(Cout, Cin, 3, 3, 3, generator=g) * 2 - 1) / (Cin * 27) ** 0.5
    b = (torch.rand(Cout, generator=g) * 2 - 1) / (Cin * 27) ** 0.5
    off = torch.randn(N, G * 81, *dims, generator=g) * 1.5
    m = torch.sigmoid(torch.randn(N, G * 27, *dims, generator=g))
    gout = torch.randn(N, Cout, *dims, generator=g)
    if dtype == torch.bfloat16:
        x, w, b, gout = x.bfloat16(), w.bfloat16(), b.bfloat16(), gout.bfloat16()
    return x, off, m, w, b, gout


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("axes", [6, 1, 2, 5])      # spatial (y, x), temporal (z), y only, (z, x)
@pytest.mark.parametrize("shape", [(2, 64, 64, (4, 6, 7), 1), (1, 128, 320, (7, 35, 34), 2)])
def test_fixed_offset_axes_against_oracle(shape, axes, dtype, dev):
    N, Cin, Cout, dims, G = shape
    x, off, m, w, b, gout = _case(N, Cin, Cout, dims, G, 61 + axes, dtype)
    masked = off.clone()
    for a in range(3):
        if not (axes >> a) & 1:
            masked[:, a::3] = 0
    f = lambda t: t.float()
    e_out = cpu.conv3d_forward(f(x), masked, m, f(w), f(b), 1, 1, 1, 1, G)
    e = list(cpu.conv3d_backward(f(gout), f(x), masked, m, f(w), True, 1, 1, 1, 1, G))
    for a in range(3):
        if not (axes >> a) & 1:
            e[1][:, a::3] = 0           # the overwritten channels get no gradient
    ts = [t.to(dev).requires_grad_(True) for t in (x, off, m, w, b)]      # the unmasked tensor goes in
    out = d2c.deform_conv3d(*ts, 1, 1, 1, 1, G, offset_axes=axes)
    out.backward(gout.to(dev))
    for a in range(3):
        if not (axes >> a) & 1:
            assert bool((ts[1].grad[:, a::3] == 0).all()), f"gradient channels of fixed axis {a} must be zero"
    for n, a, ee in [("out", out, e_out)] + list(zip(("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias"),
                                                     [t.grad for t in ts], e)):
        if dtype == torch.float32:
            assert_close(a, ee, 1e-4, 1e-5 * max(1.0, ee.abs().max().item()), n)
        else:
            assert rel_l2(a, ee) < 2e-2, (n, rel_l2(a, ee))
            assert_close(a, ee, 2e-2, 2e-2 * ee.abs().max().item(), n)


def test_fixed_offset_axes_need_the_matrix_core_kernels(dev):
    x, off, m, w, b, _ = _case(1, 6, 4, (3, 4, 5), 1, 3, torch.float32)
    with pytest.raises(RuntimeError, match="matrix-core"):
        d2c.deform_conv3d(*(t.to(dev) for t in (x, off, m, w, b)), 1, 1, 1, 1, 1, offset_axes=6)
    with pytest.raises(RuntimeError, match="offset_axes"):
        d2c.deform_conv3d(*(t.to(dev) for t in (x, off, m, w, b)), 1, 1, 1, 1, 1, offset_axes=9)


def test_fixed_offset_axes_refused_where_the_backward_would_leave_the_matrix_core_kernels(dev):
    """An offset group that spans several weight groups (groups=2, offset_groups=1): the backward pass of such a
    shape runs on the direct kernels, which know nothing of offset_axes, so the operator refuses the field as a
    whole instead of sampling with unzeroed offsets in one direction."""
    from d2conv3d_amd import _ops
    g = torch.Generator().manual_seed(5)
    x = torch.randn(1, 128, 3, 5, 6, generator=g).to(dev)
    w = (torch.randn(128, 64, 3, 3, 3, generator=g) * 0.02).to(dev)
    off = torch.randn(1, 81, 3, 5, 6, generator=g).to(dev)
    m = torch.rand(1, 27, 3, 5, 6, generator=g).to(dev)
    assert _ops.conv3d_algo(x, off, m, w, (1, 1, 1), (1, 1, 1), (1, 1, 1), 2, 1) == "mfma"
    assert _ops.conv3d_algo(x, off, m, w, (1, 1, 1), (1, 1, 1), (1, 1, 1), 2, 1, offset_axes=6) == "invalid"
    with pytest.raises(RuntimeError, match="offset_axes"):
        d2c.deform_conv3d(x, off, m, w, None, 1, 1, 1, 2, 1, offset_axes=6)


@pytest.mark.parametrize("cls", ["SpatialMDConv3d", "TemporalMDConv3d"])
def test_grouped_spatial_and_temporal_layers_against_oracle(cls, dev):
    """groups=2 with one offset group: the layers must fall back to zeroing a copy of the offsets, and every
    gradient must match the oracle run on the zeroed offsets (the fixed axes' offset channels get none)."""
    torch.manual_seed(11)
    C, dims = 128, (3, 5, 6)
    layer = getattr(M, cls)(C, C, 3, padding=1, groups=2).to(dev)
    layer.checkpoint_deformation = False
    with torch.no_grad():
        layer.deform_params.weight.normal_(0, 0.02)
        layer.deform_params.bias.normal_(0, 0.5)
    x = torch.randn(1, C, *dims, device=dev)
    gout = torch.randn(1, C, *dims, device=dev)
    axes = layer._offset_axes
    with torch.no_grad():
        deformation = layer.deform_params(x)
        offsets = deformation[:, :81].clone()
        alpha = torch.sigmoid(deformation[:, 81:])
        for a in range(3):
            if not (axes >> a) & 1:
                offsets[:, a::3] = 0
    dc = layer.deform_conv
    f = lambda t: t.detach().float().cpu()
    e_out = cpu.conv3d_forward(f(x), f(offsets), f(alpha), f(dc.weight), f(dc.bias), 1, 1, 1, 2, 1)
    e = cpu.conv3d_backward(f(gout), f(x), f(offsets), f(alpha), f(dc.weight), True, 1, 1, 1, 2, 1)
    # through the layer: the deformation is a function of x too, so compare the operator's own gradients by
    # cutting the graph at the deformation
    xi = x.clone().requires_grad_(True)
    captured = {}
    hook = layer.deform_params.register_forward_hook(lambda mod, inp, out: captured.setdefault("d", out))
    y = layer(xi)
    hook.remove()
    assert_close(y, e_out, 1e-4, 1e-5, cls + " out")
    gd, gw_, gb_ = torch.autograd.grad(y, [captured["d"], dc.weight, dc.bias], gout)
    goff, gmask = gd[:, :81], gd[:, 81:]
    for a in range(3):
        if not (axes >> a) & 1:
            assert bool((goff[:, a::3] == 0).all())
            e[1][:, a::3] = 0
    sg = f(alpha) * (1 - f(alpha))
    for n, a_, e_ in (("grad_offset", goff, e[1]), ("grad_mask", gmask, e[2] * sg), ("grad_weight", gw_, e[3]),
                      ("grad_bias", gb_, e[4])):
        assert_close(a_, e_, 1e-4, 1e-5 * max(1.0, e_.abs().max().item()), f"{cls} {n}")


@pytest.mark.parametrize("cls", ["SpatialMDConv3d", "TemporalMDConv3d", "SpatialDConv3d", "TemporalDConv3d"])
@pytest.mark.parametrize("channels", [64, 6])      # matrix-core kernels (axes fixed in the kernel) / direct kernels (copy)
def test_spatial_and_temporal_layers_with_and_without_the_kernel_path(cls, channels, dev):
    torch.manual_seed(9)
    layer = getattr(M, cls)(channels, channels, 3, padding=1).to(dev)
    with torch.no_grad():
        layer.deform_params.weight.normal_(0, 0.05)
        layer.deform_params.bias.normal_(0, 0.4)
    x = torch.randn(2, channels, 4, 6, 7, device=dev)
    res = []
    for in_kernel in (True, False):
        layer.fixed_axes_in_kernel = in_kernel
        layer.zero_grad()
        xi = x.clone().requires_grad_(True)
        y = layer(xi)
        y.square().sum().backward()
        res.append([y.detach(), xi.grad] + [p.grad.clone() for p in layer.parameters()])
    for a, e in zip(*res):
        assert_close(a, e, 1e-4, 1e-5 * max(1.0, e.abs().max().item()), cls)
    # the fixed axes really are fixed: a reference run with explicitly zeroed offsets
    with torch.no_grad():
        deformation = layer.deform_params(x)
        n_off = 81
        offsets = deformation[:, :n_off].clone()
        alpha = torch.sigmoid(deformation[:, n_off:]) if "MD" in cls else None
        if cls.startswith("Spatial"):
            offsets[:, 0::3] = 0
        else:
            offsets[:, 1::3] = 0
            offsets[:, 2::3] = 0
        ref = layer.deform_conv(x, offsets, alpha)
    assert_close(res[0][0], ref, 1e-4, 1e-5, cls + " vs explicit zeroing")
