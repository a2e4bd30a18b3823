"""The deformable convolution fed by the size map itself (d2c_conv3d_sized_forward / _backward,
deform_conv3d_sized): against the CPU oracle -- offsets from the numpy closed form of oracle/sizemap.py (pinned in
tests/test_size_map_pins.py), convolution and gradients from the C oracle, grad_size by the transpose of the
expansion times the derivative of the size activation -- and against the two-step path (expansion kernel, then
deform_conv3d) on the same tensors.  Shapes cover the matrix-core kernels, which form the offsets inside the
sampler, and the families that expand the map inside the workspace (direct kernels, channel-separated kernels).

float32: 1e-4 relative / 1e-5 absolute (absolute part scaled by the tensor's magnitude for the gradients);
bfloat16: 2e-2 of the tensor's scale."""
import numpy as np
import pytest
import torch

import d2conv3d_amd as d2c
from d2conv3d_amd import _ops
from d2conv3d_amd.grid import size_map_offsets
from oracle import cpu, sizemap
from _util import assert_close, rel_l2

pytestmark = pytest.mark.gpu

# name: (N, Cin, Cout, dims, kernel, stride, pad, dil, groups, mask, bias, family)
SHAPES = {
    "mfma_c64": (2, 64, 64, (4, 6, 7), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, True, True, "mfma"),
    "mfma_c128_o96_nomask": (1, 128, 96, (3, 6, 9), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, False, True, "mfma"),
    "mfma_stride_dil_k352": (2, 64, 40, (5, 9, 8), (3, 5, 2), (1, 2, 1), (1, 2, 1), (1, 2, 1), 1, True, False, "mfma"),
    "mfma_groups2": (1, 128, 64, (3, 5, 6), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 2, True, True, "mfma"),
    "mfma_dma_big": (1, 64, 320, (7, 35, 34), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, True, True, "mfma"),
    "generic_c6": (2, 6, 4, (3, 5, 6), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, True, True, "generic"),
    "depthwise_c64": (2, 64, 64, (4, 6, 7), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 64, True, True, "depthwise"),
}
MODES = {"xyz": 3, "xxz": 2, "xy": 2, "x": 1}


def make(name, mode, dtype, aux16=False, seed=0):
    N, Cin, Cout, dims, k, s, p, d, groups, mask, bias, _ = SHAPES[name]
    od = tuple((n + 2 * pp - (dd * (kk - 1) + 1)) // ss + 1 for n, kk, ss, pp, dd in zip(dims, k, s, p, d))
    K = k[0] * k[1] * k[2]
    g = torch.Generator().manual_seed(5000 + seed)
    x = torch.randn(N, Cin, *dims, generator=g)
    fan_in = Cin // groups * K
    w = (torch.rand(Cout, Cin // groups, *k, generator=g) * 2 - 1) / fan_in ** 0.5
    b = (torch.rand(Cout, generator=g) * 2 - 1) / fan_in ** 0.5 if bias else None
    raw = torch.randn(N, MODES[mode], *od, generator=g) * 1.2 + 0.5      # raw size prediction, both signs
    m = torch.sigmoid(torch.randn(N, K, *od, generator=g)) if mask else None
    gout = torch.randn(N, Cout, *od, generator=g)
    if dtype == torch.bfloat16:
        x, w, gout = x.bfloat16(), w.bfloat16(), gout.bfloat16()
        b = b.bfloat16() if b is not None else None
        if aux16:
            raw, m = raw.bfloat16(), (m.bfloat16() if m is not None else None)
    return (x, raw, m, w, b), gout, (k, s, p, d, groups)


def f32(t):
    return t.float() if t is not None else None


def oracle(x, raw, m, w, b, gout, mode, act, k, s, p, d, groups, aux16=False):
    """Expected forward value and gradients (input, raw size map, mask, weight, bias) in float32 / float64."""
    r64 = raw.double().numpy()
    if aux16:
        # a bfloat16 size map: the offsets the sampler uses are those the torch formulation makes in bfloat16
        # (every intermediate rounded); many then sit exactly on voxels, where the derivative is one-sided, so the
        # oracle has to see these very offsets
        from d2conv3d_amd.grid import offsets_from_size_map
        from d2conv3d_amd.modules import _apply_size_activation
        off = offsets_from_size_map(_apply_size_activation(act, raw.bfloat16()), mode, k, d).float()
    else:
        off = torch.from_numpy(sizemap.offsets(sizemap.activate(r64, act), mode, k, d)).float()
    out = cpu.conv3d_forward(f32(x), off, f32(m), f32(w), f32(b), s, p, d, groups, 1)
    gx, goff, gm, gw, gb = cpu.conv3d_backward(f32(gout), f32(x), off, f32(m), f32(w), b is not None, s, p, d, groups, 1)
    graw = sizemap.offsets_backward(goff.double().numpy(), mode, k, d) * sizemap.activate_grad(r64, act)
    return out, [gx, torch.from_numpy(graw).float(), gm, gw, gb]


def check(actual, expected, dtype, what):
    if dtype == torch.float32:
        assert_close(actual, expected, 1e-4, 1e-5 * max(1.0, expected.abs().max().item()), what)
    else:
        assert rel_l2(actual, expected) < 2e-2, (what, rel_l2(actual, expected))
        assert_close(actual, expected, 2e-2, 2e-2 * expected.abs().max().item(), what)


CASES = [("mfma_c64", "xyz", "elu"), ("mfma_c64", "x", "linear"), ("mfma_c128_o96_nomask", "xy", "relu_plus_one"),
         ("mfma_stride_dil_k352", "xxz", "elu"), ("mfma_groups2", "xyz", "relu"), ("mfma_dma_big", "xyz", "elu"),
         ("generic_c6", "xxz", "elu"), ("depthwise_c64", "xyz", "linear")]


@pytest.mark.parametrize("dtype,aux16", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
@pytest.mark.parametrize("name,mode,act", CASES)
def test_sized_operator_against_oracle_and_two_step_path(name, mode, act, dtype, aux16, dev):
    if SHAPES[name][-1] == "generic" and dtype == torch.bfloat16 and aux16:
        pytest.skip("one bfloat16 case of the direct kernels is enough")
    (x, raw, m, w, b), gout, (k, s, p, d, groups) = make(name, mode, dtype, aux16)
    # the oracle sees what the kernels see: bfloat16-rounded values up-cast
    e_out, e_grads = oracle(f32(x), f32(raw), m, w, b, gout, mode, act, k, s, p, d, groups, aux16)
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, raw, m, w, b)]
    out = d2c.deform_conv3d_sized(ts[0], ts[1], ts[2], ts[3], ts[4], mode, act, s, p, d, groups)
    out.backward(gout.to(dev))
    # the same through the expansion kernel and the ordinary operator
    t2 = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, raw, m, w, b)]
    off = size_map_offsets(t2[1], mode, k, d, act)
    assert _ops.conv3d_algo(t2[0], off, t2[2], t2[3], s, p, d, groups, 1) == SHAPES[name][-1]
    out2 = d2c.deform_conv3d(t2[0], off, t2[2], t2[3], t2[4], s, p, d, groups, 1)
    out2.backward(gout.to(dev))
    # forward: same offsets bit for bit, same kernels (sums may be ordered differently where steps are shared out)
    if dtype == torch.float32:
        assert_close(out, out2, 1e-5, 1e-6, "sized vs two-step forward")
    else:
        assert_close(out, out2, 1e-2, 1e-2 * e_out.abs().max().item(), "sized vs two-step forward")
    names = ("grad_input", "grad_size", "grad_mask", "grad_weight", "grad_bias")
    check(out, e_out, dtype, "forward")
    for n, t, t_, e in zip(names, ts, t2, e_grads):
        if t is None:
            continue
        if n == "grad_size" and dtype == torch.bfloat16 and aux16:
            # a bfloat16 size map: the two-step path rounds 3K offset gradients to bfloat16 before they add up, the
            # oracle and the fused path do not; hold the fused path to the oracle, the two-step path loosely
            check(t.grad, e, dtype, n)
            assert rel_l2(t_.grad, e) < 6e-2
            continue
        check(t.grad, e, dtype, n)
        check(t_.grad, e, dtype, n + " (two-step)")


def test_sized_operator_argument_checks(dev):
    (x, raw, m, w, b), _, (k, s, p, d, groups) = make("mfma_c64", "xyz", torch.float32)
    x, raw, m, w, b = (t.to(dev) for t in (x, raw, m, w, b))
    with pytest.raises(RuntimeError):
        d2c.deform_conv3d_sized(x, raw[:, :2], m, w, b, "xyz", "elu", s, p, d)          # wrong channel count
    with pytest.raises(RuntimeError):
        d2c.deform_conv3d_sized(x, raw[..., :-1].contiguous(), m, w, b, "xyz", "elu", s, p, d)   # wrong output size
    with pytest.raises(RuntimeError):
        d2c.deform_conv3d_sized(x, raw.cpu(), m, w, b, "xyz", "elu", s, p, d)            # CPU size map
    with pytest.raises(KeyError):
        d2c.deform_conv3d_sized(x, raw, m, w, b, "zyx", "elu", s, p, d)


def test_sized_operator_fused_relu(dev):
    (x, raw, m, w, b), gout, (k, s, p, d, groups) = make("mfma_c64", "xyz", torch.float32, seed=3)
    ts = [t.to(dev).requires_grad_(True) for t in (x, raw, m, w, b)]
    t2 = [t.to(dev).requires_grad_(True) for t in (x, raw, m, w, b)]
    out = d2c.deform_conv3d_sized(*ts, "xyz", "elu", s, p, d, groups, output_relu=1.5)
    ref = 1.5 * torch.relu(d2c.deform_conv3d_sized(*t2, "xyz", "elu", s, p, d, groups))
    out.backward(gout.to(dev))
    ref.backward(gout.to(dev))
    assert_close(out, ref, 1e-5, 1e-6, "fused relu forward")
    for a, e in zip(ts, t2):
        assert_close(a.grad, e.grad, 1e-4, 1e-5 * max(1.0, e.grad.abs().max().item()), "fused relu gradient")
