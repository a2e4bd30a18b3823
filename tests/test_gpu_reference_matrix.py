"""GPU parity, small shapes: the reference's own test matrix
(ops/dconv-native/test/test_deform_conv.py:232-505) run through the Python
surface -> C ABI -> HIP kernels, checked against the CPU oracle and, as in the
reference, with float64 gradcheck and the stock-convolution known answers.

Tolerances: float64 1e-9; float32 1e-4 relative / 1e-5 absolute (forward and
gradients; atomics reorder sums); bfloat16 2e-2 relative to the tensor's scale.
"""
import pytest
import torch
import torch.nn.functional as F
from torch.autograd import gradcheck

import d2conv3d_amd as d2c
from d2conv3d_amd import _ops
from oracle import cpu
from _util import assert_close, generate_data, rel_l2, to_dev

pytestmark = pytest.mark.gpu

CASES_3D = {
    "default": dict(),
    "stride": dict(stride=3),
    "offset_groups": dict(channels_in=6, channels_out=4, n_offset_groups=2),
    "weight_groups": dict(channels_in=12, channels_out=6, n_weight_groups=3),
    "groups": dict(channels_in=24, channels_out=12, n_weight_groups=6, n_offset_groups=2),
    "channel_sep": dict(channels_in=6, channels_out=6, n_weight_groups=6, n_offset_groups=3),
    "aniso_fwd": dict(channels_in=2, channels_out=3, dimensions=(5, 7, 7), stride=(1, 2, 1),
                      padding=(0, 1, 2), dilation=(1, 1, 2)),
    "large_batch": dict(batch_size=21, channels_in=2, channels_out=2, dimensions=(3, 5, 5), kernel_size=(1, 3, 3)),
    "aniso_bwd": dict(channels_in=3, channels_out=5, dimensions=(2, 3, 5), kernel_size=(3, 5, 3),
                      stride=(1, 2, 1), padding=(1, 3, 5), dilation=(1, 1, 2)),
    "no_bias": dict(bias=False),
    "far_offsets": dict(offset_scale=3.0, padding=1),
}
CASES_1D = {
    "default": dict(dimensions=12),
    "stride": dict(dimensions=13, stride=3),
    "offset_groups": dict(dimensions=12, channels_in=6, channels_out=4, n_offset_groups=2),
    "weight_groups": dict(dimensions=12, channels_in=12, channels_out=6, n_weight_groups=3),
    "groups": dict(dimensions=12, channels_in=24, channels_out=12, n_weight_groups=6, n_offset_groups=2),
    "aniso": dict(dimensions=15, stride=2, padding=3, dilation=2, kernel_size=5),
    "no_bias": dict(dimensions=12, bias=False),
    "far_offsets": dict(dimensions=12, offset_scale=4.0, padding=1),
}
TOL = {torch.float64: (1e-9, 1e-9), torch.float32: (1e-4, 1e-5)}


def _geo(kw):
    return (kw.get("stride", 1), kw.get("padding", 0), kw.get("dilation", 1),
            kw.get("n_weight_groups", 1), kw.get("n_offset_groups", 1))


def _run(nd, fn, oracle_fwd, oracle_bwd, kw, dtype, dev, with_mask=True, seed=0):
    x, off, a, w, b = generate_data(nd, dtype=dtype, seed=seed, **kw)
    if not with_mask:
        a = None
    s, p, d, g, og = _geo(kw)
    exp = oracle_fwd(x, off, a, w, b, s, p, d, g, og)
    gout = torch.randn(exp.shape, generator=torch.Generator().manual_seed(seed + 1), dtype=torch.float64).to(dtype)
    egrads = oracle_bwd(gout, x, off, a, w, b is not None, s, p, d, g, og)
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, a, w, b)]
    out = fn(*ts, s, p, d, g, og)
    rtol, atol = TOL[dtype]
    assert_close(out, exp, rtol, atol, "forward")
    out.backward(gout.to(dev))
    for name, t, e in zip(("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias"), ts, egrads):
        if t is None:
            continue
        # gradients are sums of many terms: the absolute floor scales with the tensor
        assert_close(t.grad, e, rtol, atol * max(1.0, e.abs().max().item()), name)


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("case", list(CASES_3D))
def test_conv3d_forward_backward_vs_oracle(case, dtype, dev):
    _run(3, d2c.deform_conv3d, cpu.conv3d_forward, cpu.conv3d_backward, CASES_3D[case], dtype, dev)


def test_conv3d_no_alpha(dev):
    # test_deform_conv.py:481-484
    _run(3, d2c.deform_conv3d, cpu.conv3d_forward, cpu.conv3d_backward, {}, torch.float64, dev, with_mask=False)
    _run(3, d2c.deform_conv3d, cpu.conv3d_forward, cpu.conv3d_backward, dict(padding=1), torch.float32, dev,
         with_mask=False)


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("case", list(CASES_1D))
def test_conv1d_forward_backward_vs_oracle(case, dtype, dev):
    _run(1, d2c.deform_conv1d, cpu.conv1d_forward, cpu.conv1d_backward, CASES_1D[case], dtype, dev)


def test_conv1d_no_alpha_no_bias(dev):
    _run(1, d2c.deform_conv1d, cpu.conv1d_forward, cpu.conv1d_backward, dict(dimensions=12, bias=False),
         torch.float64, dev, with_mask=False)


def test_conv3d_no_deformation(dev):
    # test_deform_conv.py:347-371
    x, off, a, w, b = to_dev(dev, *generate_data(3, kernel_size=3))
    out = d2c.deform_conv3d(x, torch.zeros_like(off), torch.ones_like(a), w, b)
    assert torch.allclose(out, F.conv3d(x, w, b), atol=1e-7)


def test_conv1d_no_deformation(dev):
    # test_deform_conv.py:236-255
    x, off, a, w, b = to_dev(dev, *generate_data(1, dimensions=256, kernel_size=3, channels_in=24,
                                                 channels_out=6, n_weight_groups=3))
    out = d2c.deform_conv1d(x, torch.zeros_like(off), torch.ones_like(a), w, b, n_weight_groups=3)
    assert torch.allclose(out, F.conv1d(x, w, b, groups=3), atol=1e-7)


def test_conv3d_known_offset(dev):
    # test_deform_conv.py:486-505
    x, off, a, w, b = to_dev(dev, *generate_data(3))
    shifted = F.pad(x[:, :, 1:, 1:, 1:], (0, 1, 0, 1, 0, 1))
    out = d2c.deform_conv3d(x, torch.ones_like(off), torch.ones_like(a), w, b)
    assert torch.allclose(out, F.conv3d(shifted, w, b), atol=1e-7)


def test_half_inputs_give_float32(dev):
    # test_deform_conv.py:471-474
    x, off, a, w, b = to_dev(dev, *generate_data(3, bias=False, dtype=torch.half))
    out = d2c.deform_conv3d(x.float(), off, a, w, b)
    assert out.dtype == torch.float
    exp = cpu.conv3d_forward(x.float().cpu(), off.float().cpu(), a.float().cpu(), w.float().cpu(), None)
    assert_close(out, exp, 1e-4, 1e-5, "half->float forward")


@pytest.mark.parametrize("case", ["default", "groups", "aniso_bwd", "no_bias"])
def test_conv3d_gradcheck_float64(case, dev):
    # test_deform_conv.py:216-229
    kw = CASES_3D[case]
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in generate_data(3, seed=5, **kw)]
    s, p, d, g, og = _geo(kw)
    assert gradcheck(lambda *a: d2c.deform_conv3d(*a, s, p, d, g, og), tuple(ts), nondet_tol=1e-6)


@pytest.mark.parametrize("case", ["default", "groups", "aniso"])
def test_conv1d_gradcheck_float64(case, dev):
    kw = CASES_1D[case]
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in generate_data(1, seed=6, **kw)]
    s, p, d, g, og = _geo(kw)
    assert gradcheck(lambda *a: d2c.deform_conv1d(*a, s, p, d, g, og), tuple(ts), nondet_tol=1e-6)


def test_conv1d_integer_position_rule(dev):
    # dconv1d_gpu.cu:332-351 (see the oracle's own test of the same rule)
    L = 6
    x = torch.randn(1, 1, L, dtype=torch.float64)
    w = torch.ones(1, 1, 1, dtype=torch.float64)
    off = torch.zeros(1, 1, L, dtype=torch.float64)
    a = torch.full((1, 1, L), 0.5, dtype=torch.float64)
    gout = torch.ones(1, 1, L, dtype=torch.float64)
    for quirks in (True, False):
        e = cpu.conv1d_backward(gout, x, off, a, w, False, quirks=quirks)
        ts = [t.to(dev).requires_grad_(True) for t in (x, off, a, w)]
        out = _ops.deform_conv1d(ts[0], ts[1], ts[2], ts[3], None, 1, 0, 1, 1, 1, reference_quirks=quirks)
        out.backward(gout.to(dev))
        assert_close(ts[1].grad, e[1], 1e-12, 1e-12, f"grad_offset quirks={quirks}")
        assert_close(ts[2].grad, e[2], 1e-12, 1e-12, f"grad_mask quirks={quirks}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_corner_index_bit_exact(dtype, dev):
    g = torch.Generator().manual_seed(3)
    xshape, ks = (2, 4, 6, 9, 11), (3, 3, 3)
    stride, padding, dilation, G = (1, 2, 1), (1, 1, 2), (1, 1, 2), 2
    od = tuple((d + 2 * p - (a * 2 + 1)) // s + 1 for d, s, p, a in zip(xshape[2:], stride, padding, dilation))
    off = (torch.randn(2, G * 81, *od, generator=g, dtype=torch.float64) * 2.5).to(dtype)
    off.view(-1)[::7] = torch.round(off.view(-1)[::7])
    off.view(-1)[5::97] = 1e9
    off.view(-1)[11::101] = -1e9
    off.view(-1)[13::103] = float("inf")
    eb, ef = cpu.conv3d_corners(xshape, off, (4, 4) + ks, stride, padding, dilation, G)
    base, flags = _ops.conv3d_corner_index(xshape, off.to(dev), ks, stride, padding, dilation, G)
    assert torch.equal(flags.cpu(), ef)
    assert torch.equal(base.cpu(), eb)


@pytest.mark.parametrize("case", ["default", "groups", "far_offsets"])
def test_conv3d_bfloat16_generic(case, dev):
    kw = CASES_3D[case]
    x, off, a, w, b = generate_data(3, dtype=torch.float32, seed=9, **kw)
    xb, wb, bb = x.bfloat16(), w.bfloat16(), (b.bfloat16() if b is not None else None)
    s, p, d, g, og = _geo(kw)
    exp = cpu.conv3d_forward(xb.float(), off, a, wb.float(), bb.float() if bb is not None else None, s, p, d, g, og)
    gout = torch.randn(exp.shape, generator=torch.Generator().manual_seed(2)).bfloat16()
    eg = cpu.conv3d_backward(gout.float(), xb.float(), off, a, wb.float(), b is not None, s, p, d, g, og)
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (xb, off, a, wb, bb)]
    out = d2c.deform_conv3d(*ts, s, p, d, g, og)
    assert out.dtype == torch.bfloat16
    assert rel_l2(out, exp) < 2e-2
    out.backward(gout.to(dev))
    for name, t, e in zip(("gx", "goff", "gmask", "gw", "gb"), ts, eg):
        if t is not None:
            assert t.grad.dtype == t.dtype
            assert rel_l2(t.grad, e) < 2e-2, name
