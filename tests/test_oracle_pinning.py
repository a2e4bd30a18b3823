"""Pins the CPU oracle (oracle/) before anything is compared with it.

Nothing here retypes the oracle's formulas.  The checks are the reference
test-suite's own known answers (ops/dconv-native/test/test_deform_conv.py,
test_modules.py), library routines (torch's stock convolutions and autograd),
central finite differences in float64, hand-computed special cases, and an
independent loop-by-loop restatement of the reference's expected_fn
(oracle/brute.py).
"""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import brute, cpu
from d2conv3d_amd.grid import offsets_from_size_map
from _util import generate_data

F64 = dict(rtol=1e-10, atol=1e-10)


def close(a, b, rtol=1e-10, atol=1e-10):
    return torch.allclose(a.double(), b.double(), rtol=rtol, atol=atol)


# ---------------------------------------------------------------- forward, 3-D
def test_no_deformation_is_stock_conv3d():
    # test_deform_conv.py:347-371
    x, off, a, w, b = generate_data(3, kernel_size=3)
    out = cpu.conv3d_forward(x, torch.zeros_like(off), torch.ones_like(a), w, b)
    assert torch.allclose(out, F.conv3d(x, w, b), atol=1e-7)


@pytest.mark.parametrize("stride,padding,dilation,groups", [
    (1, 1, 1, 1), (2, 1, 1, 1), ((1, 2, 1), (0, 1, 2), (1, 1, 2), 1), (1, 1, 1, 3), (1, (1, 2, 2), (1, 2, 2), 1),
])
def test_no_deformation_with_geometry(stride, padding, dilation, groups):
    x, off, a, w, b = generate_data(3, channels_in=6, channels_out=3, dimensions=(5, 7, 7), stride=stride,
                                    padding=padding, dilation=dilation, n_weight_groups=groups)
    out = cpu.conv3d_forward(x, torch.zeros_like(off), None, w, b, stride, padding, dilation, groups, 1)
    assert close(out, F.conv3d(x, w, b, stride, padding, dilation, groups), 1e-9, 1e-9)


def test_known_offset_plus_one():
    # test_deform_conv.py:486-505: offsets == +1 sample the input shifted by (1,1,1), zero filled
    x, off, a, w, b = generate_data(3)
    shifted = F.pad(x[:, :, 1:, 1:, 1:], (0, 1, 0, 1, 0, 1))
    out = cpu.conv3d_forward(x, torch.ones_like(off), torch.ones_like(a), w, b)
    assert torch.allclose(out, F.conv3d(shifted, w, b), atol=1e-7)


@pytest.mark.parametrize("shift", [(-1, 0, 2), (2, -2, 1), (0, 3, -3), (-6, 0, 0)])
def test_integer_offsets_are_shifted_convs(shift):
    x, off, a, w, b = generate_data(3, dimensions=(5, 6, 7), padding=1)
    off = torch.zeros_like(off)
    for ax in range(3):
        off[:, ax::3] = shift[ax]
    # out(p) samples x(p - 1 + tap + shift) with zeros outside the volume: an unpadded stock
    # convolution over the zero-extended input, cut out at [shift - 1, shift + size + 1)
    big = F.pad(x, (8, 8, 8, 8, 8, 8))
    sl = [slice(None), slice(None)] + [slice(8 + s - 1, 8 + s + n + 1) for s, n in zip(shift, x.shape[2:])]
    shifted = big[tuple(sl)]
    out = cpu.conv3d_forward(x, off, None, w, b, padding=1)
    assert close(out, F.conv3d(shifted, w, b), 1e-9, 1e-9)


BRUTE_CASES = [
    dict(),                                                         # defaults of generate_data
    dict(stride=3),                                                 # test_stride
    dict(channels_in=6, channels_out=4, n_offset_groups=2),         # test_offset_groups
    dict(channels_in=12, channels_out=6, n_weight_groups=3, dimensions=4),        # test_weight_groups
    dict(channels_in=12, channels_out=6, n_weight_groups=6, n_offset_groups=2, dimensions=4),  # test_groups
    dict(channels_in=6, channels_out=6, n_weight_groups=6, n_offset_groups=3),    # test_channel_sep_groups
    dict(channels_in=2, channels_out=3, dimensions=(5, 7, 7), stride=(1, 2, 1), padding=(0, 1, 2),
         dilation=(1, 1, 2)),                                       # test_forward
    dict(batch_size=3, channels_in=2, channels_out=2, dimensions=(3, 5, 5), kernel_size=(1, 3, 3)),
    dict(channels_in=3, channels_out=5, dimensions=(2, 3, 5), kernel_size=(3, 5, 3), stride=(1, 2, 1),
         padding=(1, 3, 5), dilation=(1, 1, 2)),                    # test_backward geometry
    dict(bias=False),
    dict(offset_scale=3.0, padding=1),                              # many taps outside the volume
]


@pytest.mark.parametrize("case", range(len(BRUTE_CASES)))
def test_forward_3d_against_loop_restatement(case):
    kw = dict(BRUTE_CASES[case])
    x, off, a, w, b = generate_data(3, seed=10 + case, **kw)
    geo = {k: kw.get(k, d) for k, d in (("stride", 1), ("padding", 0), ("dilation", 1))}
    out = cpu.conv3d_forward(x, off, a, w, b, geo["stride"], geo["padding"], geo["dilation"],
                             kw.get("n_weight_groups", 1), kw.get("n_offset_groups", 1))
    exp = brute.deform_conv_forward(x, off, a, w, b, geo["stride"], geo["padding"], geo["dilation"])
    assert close(out, exp), (out - exp).abs().max()


def test_forward_3d_without_mask_is_unit_mask():
    x, off, a, w, b = generate_data(3, seed=3)
    assert close(cpu.conv3d_forward(x, off, None, w, b), cpu.conv3d_forward(x, off, torch.ones_like(a), w, b))


def test_constant_integer_dilation_map_is_dilated_conv():
    # test_modules.py:48-67 generalised: size 2 on (y, x) == Conv3d(padding=(1,2,2), dilation=(1,2,2))
    x, _, _, w, b = generate_data(3, channels_in=3, channels_out=4, dimensions=7, padding=1)
    for size, pad, dil in [((1.0, 2.0, 2.0), (1, 2, 2), (1, 2, 2)), ((2.0, 1.0, 3.0), (2, 1, 3), (2, 1, 3))]:
        sm = torch.tensor(size, dtype=torch.float64).view(1, 3, 1, 1, 1).expand(2, 3, 7, 7, 7)
        off = offsets_from_size_map(sm, "xyz", (3, 3, 3), (1, 1, 1))
        out = cpu.conv3d_forward(x, off, None, w, b, padding=1)
        assert close(out, F.conv3d(x, w, b, padding=pad, dilation=dil), 1e-9, 1e-9)


def test_f32_oracle_agrees_with_f64_oracle():
    x, off, a, w, b = generate_data(3, channels_in=4, channels_out=4, padding=1, seed=5)
    o64 = cpu.conv3d_forward(x, off, a, w, b, padding=1)
    o32 = cpu.conv3d_forward(*(t.float() for t in (x, off, a, w, b)), padding=1)
    # same float32-rounded inputs in float64
    o64r = cpu.conv3d_forward(*(t.float().double() for t in (x, off, a, w, b)), padding=1)
    assert torch.allclose(o32.double(), o64r, rtol=1e-4, atol=1e-4)
    assert torch.allclose(o64, o64r, rtol=1e-3, atol=1e-3)


# --------------------------------------------------------------- backward, 3-D
def _fd_check(fwd, inputs, gout, analytic, h=1e-6, tol=2e-6, max_coords=400, seed=0):
    """Central differences of L = sum(out * gout) against the analytic gradients."""
    rng = np.random.default_rng(seed)
    for t, g in zip(inputs, analytic):
        if t is None:
            continue
        flat = t.view(-1)
        idxs = np.arange(flat.numel())
        if len(idxs) > max_coords:
            idxs = rng.choice(idxs, max_coords, replace=False)
        for i in idxs:
            old = flat[i].item()
            flat[i] = old + h
            lp = (fwd(*inputs) * gout).sum().item()
            flat[i] = old - h
            lm = (fwd(*inputs) * gout).sum().item()
            flat[i] = old
            num = (lp - lm) / (2 * h)
            ana = g.view(-1)[i].item()
            assert abs(num - ana) <= tol * (1 + abs(num)), (i, num, ana)


BWD_CASES = [
    dict(),
    dict(stride=3),
    dict(channels_in=6, channels_out=4, n_offset_groups=2, dimensions=4),
    dict(channels_in=12, channels_out=6, n_weight_groups=3, dimensions=4),
    dict(channels_in=12, channels_out=6, n_weight_groups=6, n_offset_groups=2, dimensions=4),
    dict(channels_in=6, channels_out=6, n_weight_groups=6, n_offset_groups=3, dimensions=4),
    dict(channels_in=3, channels_out=5, dimensions=(2, 3, 5), kernel_size=(3, 5, 3), stride=(1, 2, 1),
         padding=(1, 3, 5), dilation=(1, 1, 2)),
    dict(bias=False, dimensions=4),
]


@pytest.mark.parametrize("case", range(len(BWD_CASES)))
@pytest.mark.parametrize("with_mask", [True, False])
def test_backward_3d_against_finite_differences(case, with_mask):
    # the float64 gradcheck of test_deform_conv.py:216-229, done by hand on the oracle
    kw = dict(BWD_CASES[case])
    x, off, a, w, b = generate_data(3, seed=40 + case, **kw)
    if not with_mask:
        a = None
    s, p, d = kw.get("stride", 1), kw.get("padding", 0), kw.get("dilation", 1)
    g, og = kw.get("n_weight_groups", 1), kw.get("n_offset_groups", 1)

    def fwd(x_, off_, a_, w_, b_):
        return cpu.conv3d_forward(x_, off_, a_, w_, b_, s, p, d, g, og)
    out = fwd(x, off, a, w, b)
    gout = torch.randn(out.shape, generator=torch.Generator().manual_seed(7), dtype=torch.float64)
    grads = cpu.conv3d_backward(gout, x, off, a, w, b is not None, s, p, d, g, og)
    _fd_check(fwd, [x, off, a, w, b], gout, grads, max_coords=150)


def test_backward_3d_no_deformation_is_conv_autograd():
    x, off, a, w, b = generate_data(3, channels_in=4, channels_out=6, n_weight_groups=2, padding=1)
    xr, wr, br = (t.clone().requires_grad_(True) for t in (x, w, b))
    out = F.conv3d(xr, wr, br, padding=1, groups=2)
    gout = torch.randn_like(out)
    out.backward(gout)
    gx, goff, gm, gw, gb = cpu.conv3d_backward(gout, x, torch.zeros_like(off), torch.ones_like(a), w, True,
                                               1, 1, 1, 2, 1)
    assert close(gx, xr.grad, 1e-9, 1e-9) and close(gw, wr.grad, 1e-9, 1e-9) and close(gb, br.grad, 1e-9, 1e-9)
    assert close(gb, gout.sum((0, 2, 3, 4)))


def test_derivative_is_right_sided_at_integer_positions():
    # 1 channel, 1x1x1 kernel, weight 1: out(p) = trilinear(x, p + off).  At off == 0 the derivative
    # w.r.t. the z-offset is the forward difference x[z+1] - x[z] (floor-based corners); the last
    # slice sees zero beyond the volume.
    x = torch.randn(1, 1, 4, 3, 3, dtype=torch.float64)
    w = torch.ones(1, 1, 1, 1, 1, dtype=torch.float64)
    off = torch.zeros(1, 3, 4, 3, 3, dtype=torch.float64)
    gout = torch.ones(1, 1, 4, 3, 3, dtype=torch.float64)
    _, goff, _, _, _ = cpu.conv3d_backward(gout, x, off, None, w, False)
    xz = F.pad(x, (0, 0, 0, 0, 0, 1))
    assert close(goff[:, 0], (xz[:, 0, 1:] - xz[:, 0, :-1]))
    xy = F.pad(x, (0, 0, 0, 1))
    assert close(goff[:, 1], (xy[:, 0, :, 1:] - xy[:, 0, :, :-1]))
    xx = F.pad(x, (0, 1))
    assert close(goff[:, 2], (xx[:, 0, :, :, 1:] - xx[:, 0, :, :, :-1]))


def test_position_minus_one_has_zero_value_but_live_derivative():
    # z == -1 exactly: the forward early-out returns 0 (dconv3d_gpu.cu:59-61) while
    # get_coordinate_weights (:708-754) still sees the corner z1 == 0.
    x = torch.randn(1, 1, 3, 3, 3, dtype=torch.float64)
    w = torch.ones(1, 1, 1, 1, 1, dtype=torch.float64)
    off = torch.zeros(1, 3, 3, 3, 3, dtype=torch.float64)
    off[:, 0, 0] = -1.0            # output slice z=0 samples z=-1
    out = cpu.conv3d_forward(x, off, None, w, None)
    assert torch.all(out[0, 0, 0] == 0)
    gout = torch.ones_like(out)
    gx, goff, _, _, _ = cpu.conv3d_backward(gout, x, off, None, w, False)
    assert close(goff[0, 0, 0], x[0, 0, 0])         # C(z1=0) - 0
    # nothing of that slice is scattered into grad_input: input slice 0 is sampled by no one,
    # slices 1 and 2 by exactly one output voxel each with weight 1
    assert torch.all(gx[0, 0, 0] == 0) and close(gx[0, 0, 1:], torch.ones(2, 3, 3, dtype=torch.float64))
    off[:, 0, 0] = -1.5
    _, goff, _, _, _ = cpu.conv3d_backward(gout, x, off, None, w, False)
    assert torch.all(goff[0, 0, 0] == 0)


# ------------------------------------------------------------- corner indices
def _corners_numpy(off, xshape, kshape, stride, padding, dilation, G):
    """Independent restatement of the index logic: floor of float(int base)+offset, early-out, gates."""
    N, _, D, H, W = xshape
    kd, kh, kw = kshape
    o = off.numpy()
    Do, Ho, Wo = o.shape[2:]
    K = kd * kh * kw
    base = np.zeros((N, G * K, Do * Ho * Wo, 3), np.int32)
    flags = np.zeros((N, G * K, Do * Ho * Wo), np.uint8)
    ft = o.dtype.type
    oz, oy, ox = np.meshgrid(np.arange(Do), np.arange(Ho), np.arange(Wo), indexing="ij")
    for n, g, i, j, l in itertools.product(range(N), range(G), range(kd), range(kh), range(kw)):
        k = (i * kh + j) * kw + l
        gk = g * K + k
        pos = []
        for ax, (oo, s, p, kk, dil) in enumerate(zip((oz, oy, ox), stride, padding, (i, j, l), dilation)):
            pos.append((oo * s - p + kk * dil).astype(o.dtype) + o[n, 3 * gk + ax])
        size = (D, H, W)
        inside = np.ones_like(pos[0], bool)
        for v, sz in zip(pos, size):
            inside &= (v > ft(-1)) & (v < ft(sz))
        fl = [np.floor(np.clip(v, -4, sz + 4)).astype(np.int32) for v, sz in zip(pos, size)]
        f = np.zeros(pos[0].shape, np.uint8)
        for c in range(8):
            ok = inside.copy()
            for ax, bit in enumerate((4, 2, 1)):
                idx = fl[ax] + (1 if c & bit else 0)
                ok &= (idx >= 0) & (idx < size[ax])
            f |= (ok.astype(np.uint8) << c)
        base[n, gk] = np.stack([a.reshape(-1) for a in fl], -1)
        flags[n, gk] = f.reshape(-1)
    return torch.from_numpy(base), torch.from_numpy(flags)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_corner_index_and_gates(dtype):
    g = torch.Generator().manual_seed(3)
    xshape, kshape = (2, 4, 4, 5, 6), (3, 3, 3)
    stride, padding, dilation, G = (1, 2, 1), (1, 1, 2), (1, 1, 2), 2
    od = tuple((d + 2 * p - (a * 2 + 1)) // s + 1 for d, s, p, a in zip(xshape[2:], stride, padding, dilation))
    off = (torch.randn(2, G * 81, *od, generator=g, dtype=torch.float64) * 2.5).to(dtype)
    # exact integers, exact -1 / size boundaries and huge values exercise every gate
    off.view(-1)[::7] = torch.round(off.view(-1)[::7])
    off.view(-1)[5::97] = 1e9
    off.view(-1)[11::101] = -1e9
    base, flags = cpu.conv3d_corners(xshape, off, (4, 4) + kshape, stride, padding, dilation, G)
    eb, ef = _corners_numpy(off, xshape, kshape, stride, padding, dilation, G)
    assert torch.equal(flags, ef)
    assert torch.equal(base, eb)
    assert 0 < int((flags == 0).sum()) < flags.numel() and int((flags == 255).sum()) > 0


# ------------------------------------------------------------------------ 1-D
def test_no_deformation_is_stock_conv1d():
    # test_deform_conv.py:236-255
    x, off, a, w, b = generate_data(1, dimensions=256, kernel_size=3, channels_in=24, channels_out=6,
                                    n_weight_groups=3)
    out = cpu.conv1d_forward(x, torch.zeros_like(off), torch.ones_like(a), w, b, groups=3)
    assert torch.allclose(out, F.conv1d(x, w, b, groups=3), atol=1e-7)


CASES_1D = [
    dict(dimensions=9),
    dict(dimensions=10, stride=3),
    dict(dimensions=9, channels_in=6, channels_out=4, n_offset_groups=2),
    dict(dimensions=9, channels_in=12, channels_out=6, n_weight_groups=3),
    dict(dimensions=9, channels_in=24, channels_out=12, n_weight_groups=6, n_offset_groups=2),
    dict(dimensions=11, stride=2, padding=3, dilation=2, kernel_size=5),
    dict(dimensions=9, bias=False),
    dict(dimensions=9, offset_scale=4.0, padding=1),
]


@pytest.mark.parametrize("case", range(len(CASES_1D)))
def test_forward_1d_against_loop_restatement(case):
    kw = dict(CASES_1D[case])
    x, off, a, w, b = generate_data(1, seed=70 + case, **kw)
    s, p, d = kw.get("stride", 1), kw.get("padding", 0), kw.get("dilation", 1)
    out = cpu.conv1d_forward(x, off, a, w, b, s, p, d, kw.get("n_weight_groups", 1), kw.get("n_offset_groups", 1))
    exp = brute.deform_conv_forward(x, off, a, w, b, s, p, d)
    assert close(out, exp), (out - exp).abs().max()


@pytest.mark.parametrize("case", range(len(CASES_1D)))
@pytest.mark.parametrize("quirks", [True, False])
def test_backward_1d_against_finite_differences(case, quirks):
    # at non-integer positions the integer-position rule is inert, so both settings must pass
    kw = dict(CASES_1D[case])
    x, off, a, w, b = generate_data(1, seed=90 + case, **kw)
    s, p, d = kw.get("stride", 1), kw.get("padding", 0), kw.get("dilation", 1)
    g, og = kw.get("n_weight_groups", 1), kw.get("n_offset_groups", 1)

    def fwd(x_, off_, a_, w_, b_):
        return cpu.conv1d_forward(x_, off_, a_, w_, b_, s, p, d, g, og)
    out = fwd(x, off, a, w, b)
    gout = torch.randn(out.shape, generator=torch.Generator().manual_seed(8), dtype=torch.float64)
    grads = cpu.conv1d_backward(gout, x, off, a, w, b is not None, s, p, d, g, og, quirks=quirks)
    _fd_check(fwd, [x, off, a, w, b], gout, grads, max_coords=150)


def test_1d_integer_position_rule():
    # dconv1d_gpu.cu:332-351 at exactly-integer positions: grad_offset uses in[x+1] - in[x-1] and
    # grad_mask is built from in[x+1]; with the rule off both are the right-sided/forward values.
    L = 6
    x = torch.randn(1, 1, L, dtype=torch.float64)
    w = torch.ones(1, 1, 1, dtype=torch.float64)
    off = torch.zeros(1, 1, L, dtype=torch.float64)
    a = torch.full((1, 1, L), 0.5, dtype=torch.float64)
    gout = torch.ones(1, 1, L, dtype=torch.float64)
    xp = F.pad(x[0, 0], (1, 1))                       # xp[i+1] = x[i]
    _, goff, gm, _, _ = cpu.conv1d_backward(gout, x, off, a, w, False, quirks=True)
    assert close(goff[0, 0], 0.5 * (xp[2:] - xp[:-2]))
    assert close(gm[0, 0], xp[2:])
    _, goff, gm, _, _ = cpu.conv1d_backward(gout, x, off, a, w, False, quirks=False)
    assert close(goff[0, 0], 0.5 * (xp[2:] - xp[1:-1]))
    assert close(gm[0, 0], x[0, 0])


# ---------------------------------------------------------------- plain depthwise conv3d (oracle/dwconv.py)
DW_CASES = [
    # C, multiplier, kernel, stride, padding, dilation
    (3, 1, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    (2, 2, (3, 3, 3), (2, 2, 2), (2, 2, 2), (2, 2, 2)),
    (4, 3, (1, 3, 2), (1, 2, 1), (0, 1, 2), (1, 1, 2)),
    (2, 1, (3, 3, 3), (2, 1, 2), (1, 1, 1), (1, 2, 1)),
]


@pytest.mark.parametrize("C,m,k,s,p,d", DW_CASES)
def test_plain_depthwise_oracle_is_torch_grouped_conv(C, m, k, s, p, d):
    """The library routine the reference's own test compares with (test_conv3d_depthwise.py:33-96): torch's grouped
    convolution and its autograd, float64 on the CPU."""
    from oracle import dwconv
    g = torch.Generator().manual_seed(C * 7 + m)
    x = torch.randn(2, C, 6, 7, 8, dtype=torch.float64, generator=g).requires_grad_(True)
    w = torch.randn(C * m, 1, *k, dtype=torch.float64, generator=g).requires_grad_(True)
    b = torch.randn(C * m, dtype=torch.float64, generator=g).requires_grad_(True)
    out = F.conv3d(x, w, b, s, p, d, groups=C)
    go = torch.randn(out.shape, dtype=torch.float64, generator=g)
    out.backward(go)
    eo = dwconv.forward(x.detach().numpy(), w.detach().numpy(), b.detach().numpy(), s, p, d)
    gx, gw, gb = dwconv.backward(go.numpy(), x.detach().numpy(), w.detach().numpy(), s, p, d)
    np.testing.assert_allclose(eo, out.detach().numpy(), rtol=0, atol=1e-12)
    np.testing.assert_allclose(gx, x.grad.numpy(), rtol=0, atol=1e-12)
    np.testing.assert_allclose(gw, w.grad.numpy(), rtol=0, atol=1e-12)
    np.testing.assert_allclose(gb, b.grad.numpy(), rtol=0, atol=1e-12)
    # without bias the forward value drops exactly the bias
    np.testing.assert_allclose(dwconv.forward(x.detach().numpy(), w.detach().numpy(), None, s, p, d),
                               F.conv3d(x, w, None, s, p, d, groups=C).detach().numpy(), rtol=0, atol=1e-12)
