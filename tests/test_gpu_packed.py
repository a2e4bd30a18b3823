"""The operator on the un-split output of the deformation branch (description fields deform_channels and
mask_activation): what MDConv3d's `torch.split` + modulation activation do in front of the operator in the reference
(network/layers.py:107-120, ops/dconv-native/src/dconv_native/modules.py:71-84), done by the sampler itself.

Expected values: the CPU oracle on the split tensors, with torch's own activation and its autograd for the modulation
part; and the layers with the fusion switched off."""
import pytest
import torch

import d2conv3d_amd as d2c
from d2conv3d_amd import _ops, modules as M
from oracle import cpu
from _util import assert_close, rel_l2

pytestmark = pytest.mark.gpu

ACT = {"sigmoid": torch.sigmoid, "relu": torch.relu, "tanh": torch.tanh, "linear": lambda t: t}


def _check(a, e, dtype, what):
    if dtype == torch.float32:
        assert_close(a, e, 1e-4, 1e-5 * max(1.0, e.abs().max().item()), what)
    else:
        assert rel_l2(a, e) < 2e-2, (what, rel_l2(a, e))
        assert_close(a, e, 2e-2, 2e-2 * max(e.abs().max().item(), 1e-6), what)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("act", ["sigmoid", "relu", "tanh", "linear"])
@pytest.mark.parametrize("shape", [(2, 64, 64, (3, 6, 7), 1), (1, 128, 192, (7, 35, 34), 2)])
def test_deformation_tensor_read_in_place_against_oracle(shape, act, dtype, dev):
    N, Cin, Cout, dims, G = shape
    g = torch.Generator().manual_seed(41)
    GK = G * 27
    x = torch.randn(N, Cin, *dims, generator=g).to(dtype)
    w = ((torch.rand(Cout, Cin, 3, 3, 3, generator=g) * 2 - 1) / (Cin * 27) ** 0.5).to(dtype)
    b = ((torch.rand(Cout, generator=g) * 2 - 1) / (Cin * 27) ** 0.5).to(dtype)
    deformation = torch.cat([torch.randn(N, 3 * GK, *dims, generator=g) * 1.5,
                             torch.randn(N, GK, *dims, generator=g) * 1.2], dim=1).to(dtype)
    gout = torch.randn(N, Cout, *dims, generator=g).to(dtype)
    ts = [t.to(dev).requires_grad_(True) for t in (x, deformation, w, b)]
    assert _ops.deform_conv3d_packed_supported(ts[0], ts[1], ts[2], 3 * GK, act, None, "linear", (1, 1, 1), (1, 1, 1),
                                               (1, 1, 1), 1, G)
    out = _ops.deform_conv3d_packed(ts[0], ts[1], ts[2], ts[3], 3 * GK, act, (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, G)
    out.backward(gout.to(dev))
    # expected: the reference's sequence on the same values (the activation in the tensors' own type, like torch)
    raw = deformation[:, 3 * GK:].clone().requires_grad_(True)
    alpha = ACT[act](raw)
    off = deformation[:, :3 * GK].float()
    f = lambda t: t.detach().float()
    e_out = cpu.conv3d_forward(f(x), off, f(alpha), f(w), f(b), 1, 1, 1, 1, G)
    e = cpu.conv3d_backward(f(gout), f(x), off, f(alpha), f(w), True, 1, 1, 1, 1, G)
    alpha.backward(e[2].to(dtype))
    e_gdef = torch.cat([e[1], raw.grad.float()], dim=1)
    _check(out, e_out, dtype, "out")
    _check(ts[0].grad, e[0], dtype, "grad_input")
    _check(ts[1].grad[:, :3 * GK], e_gdef[:, :3 * GK], dtype, "grad of the offsets part")
    _check(ts[1].grad[:, 3 * GK:], e_gdef[:, 3 * GK:], dtype, "grad of the raw modulation part")
    _check(ts[2].grad, e[3], dtype, "grad_weight")
    _check(ts[3].grad, e[4], dtype, "grad_bias")


@pytest.mark.parametrize("wanted", ["x+deformation", "weights", "deformation"])
def test_packed_backward_with_some_gradients_only(wanted, dev):
    """grad_input from the lists without the offset / mask gradient kernel (the list pass then reads the mask through
    the activation), grad_weight by sampling again, and the deformation gradient alone."""
    g = torch.Generator().manual_seed(43)
    N, C, dims, GK = 1, 64, (4, 9, 10), 27
    x = torch.randn(N, C, *dims, generator=g)
    w = (torch.rand(C, C, 3, 3, 3, generator=g) * 2 - 1) / (C * 27) ** 0.5
    deformation = torch.cat([torch.randn(N, 81, *dims, generator=g) * 1.5, torch.randn(N, 27, *dims, generator=g)], dim=1)
    gout = torch.randn(N, C, *dims, generator=g)
    need = {"x+deformation": (1, 1, 0), "weights": (0, 0, 1), "deformation": (0, 1, 0)}[wanted]
    ts = [t.to(dev).requires_grad_(bool(r)) for t, r in zip((x, deformation, w), need)]
    _ops.deform_conv3d_packed(ts[0], ts[1], ts[2], None, 81, "sigmoid", (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, 1).backward(gout.to(dev))
    raw = deformation[:, 81:].clone().requires_grad_(True)
    alpha = torch.sigmoid(raw)
    e = cpu.conv3d_backward(gout, x, deformation[:, :81], alpha.detach(), w, False, 1, 1, 1, 1, 1)
    alpha.backward(e[2])
    exp = (e[0], torch.cat([e[1], raw.grad], dim=1), e[3])
    for t, r, ee, n in zip(ts, need, exp, ("grad_input", "grad_deformation", "grad_weight")):
        if r:
            assert_close(t.grad, ee, 1e-4, 1e-5 * max(1.0, ee.abs().max().item()), n)
        else:
            assert t.grad is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cls,kw", [
    ("MDConv3d", {}), ("MDConv3d", {"activation": "tanh"}), ("MDConv3d", {"offset_groups": 2}),
    ("SpatialMDConv3d", {}), ("TemporalMDConv3d", {}),
    ("XYZSizeConditionedMDConv3d", {}), ("XYSizeConditionedMDConv3d", {"size_activation": "relu_plus_one"}),
    ("SizeConditionedMDConv3d", {}),
])
def test_layers_with_and_without_the_fused_deformation(cls, kw, dtype, dev):
    torch.manual_seed(17)
    C = 64
    layer = getattr(M, cls)(C, C, 3, padding=1, **kw).to(dev)
    with torch.no_grad():
        layer.deform_params.weight.normal_(0, 0.03)
        layer.deform_params.bias.normal_(0, 0.5)
    layer = layer.to(dtype)
    x = torch.randn(2, C, 4, 7, 9, device=dev).to(dtype)
    gout = torch.randn(2, C, 4, 7, 9, device=dev).to(dtype)
    res = []
    for fused in (True, False):
        layer.fused_deformation = fused
        if hasattr(layer, "fixed_axes_in_kernel"):
            layer.fixed_axes_in_kernel = fused
        layer.zero_grad()
        xi = x.clone().requires_grad_(True)
        y = layer(xi)
        y.backward(gout)
        res.append([y.detach(), xi.grad] + [p.grad.clone() for p in layer.parameters()])
    names = ["output", "grad_input"] + [n for n, _ in layer.named_parameters()]
    for n, a, e in zip(names, *res):
        if dtype == torch.float32:
            assert_close(a, e, 1e-3, 1e-4 * max(1.0, e.abs().max().item()), f"{cls} {n}")
        else:
            assert rel_l2(a, e) < 3e-2, (cls, n, rel_l2(a, e))


def test_the_fused_path_makes_no_copies_of_the_deformation(dev):
    """What the fusion is for: between the deformation branch's convolution and the operator no kernel runs -- no
    split copies, no sigmoid, and in the backward pass no sigmoid_backward and no concatenation of gradients."""
    from torch.profiler import ProfilerActivity, profile
    torch.manual_seed(3)
    layer = M.MDConv3d(64, 64, 3, padding=1).to(dev)
    x = torch.randn(1, 64, 4, 9, 10, device=dev, requires_grad=True)
    gout = torch.randn(1, 64, 4, 9, 10, device=dev)
    calls = {}
    for fused in (True, False):
        layer.fused_deformation = fused
        layer(x).backward(gout)             # warm-up (workspace, library load)
        with profile(activities=[ProfilerActivity.CPU]) as prof:
            layer(x).backward(gout)
        calls[fused] = {e.key: e.count for e in prof.key_averages()}
    gone = ("aten::sigmoid", "aten::sigmoid_backward", "aten::split", "aten::split_with_sizes", "aten::cat")
    assert "aten::sigmoid" in calls[False] and "aten::sigmoid_backward" in calls[False]
    assert not any(k in calls[True] for k in gone), sorted(calls[True])


def test_shapes_outside_the_matrix_core_kernels_fall_back(dev):
    torch.manual_seed(5)
    layer = M.MDConv3d(6, 4, 3, padding=1).to(dev)          # direct kernels: split + activation as in the reference
    with torch.no_grad():
        layer.deform_params.weight.normal_(0, 0.05)
    x = torch.randn(1, 6, 3, 5, 6, device=dev)
    res = []
    for fused in (True, False):
        layer.fused_deformation = fused
        res.append(layer(x))
    assert_close(res[0], res[1], 1e-6, 1e-6, "fallback")
    d = layer.deform_params(x)
    assert not _ops.deform_conv3d_packed_supported(x, d, layer.deform_conv.weight, 81, "sigmoid", None, "linear",
                                                   (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, 1)
    with pytest.raises(RuntimeError, match="matrix-core"):
        _ops.deform_conv3d_packed(x, d, layer.deform_conv.weight, None, 81, "sigmoid", (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, 1)
