"""The sampled columns of a forward call kept for its backward call (d2c_conv3d_forward_columns /
d2c_conv3d_backward_columns; in the Python layer: on by default where a description is served and grad_weight is
wanted, `_ops.config.set_keep_columns`).

The reference samples the input a second time in its backward pass (dconv3d_gpu.cu:1037-1088); keeping the columns
changes no result beyond the order of floating-point sums.  Expected values: the CPU oracle on the same bfloat16
tensors (2e-2 of the tensor's scale, like every bfloat16 check of the matrix-core kernels), and the plain calls on the
same tensors (a few units in bfloat16's last place: the two paths round the columns at the same point but add in
another order)."""
import ctypes

import pytest
import torch

import d2conv3d_amd as d2c
from d2conv3d_amd import _lib, _ops
from oracle import cpu
from _util import assert_close, rel_l2

pytestmark = pytest.mark.gpu

# name: (N, Cin, Cout, dims, groups, G, bias, mask, sigma) -- 3x3x3, stride 1, padding 1: at least 128 position tiles
# of 64 and weight groups wider than 128 output channels (the forward kernel that can write the columns), weight
# groups of an even number of 64-channel chunks (the grad-weight product over columns)
SHAPES = {
    "c128_o192_G2": (1, 128, 192, (9, 32, 32), 1, 2, True, True, 1.5),            # 256-wide output tile
    "c256_o512_G4_ragged": (1, 256, 512, (5, 41, 41), 1, 4, True, True, 2.0),     # 8405 positions: ragged last tile
    "c256_groups2_o640_nomask": (2, 256, 640, (4, 32, 33), 2, 2, False, False, 1.5),
}


# float32 only (channel chunks of 32): six chunks per weight group, which the product on three-term operands (sets of
# four chunks) does not take -- the float32 matrix instruction then
F32_SHAPES = dict(SHAPES, c192_o256_G2=(1, 192, 256, (9, 32, 32), 1, 2, True, True, 1.5))


def make(name, seed=0):
    N, Cin, Cout, dims, groups, G, bias, mask, sig = F32_SHAPES[name]
    g = torch.Generator().manual_seed(7000 + seed)
    x = torch.randn(N, Cin, *dims, generator=g).bfloat16()
    fan_in = Cin // groups * 27
    w = ((torch.rand(Cout, Cin // groups, 3, 3, 3, generator=g) * 2 - 1) / fan_in ** 0.5).bfloat16()
    b = ((torch.rand(Cout, generator=g) * 2 - 1) / fan_in ** 0.5).bfloat16() if bias else None
    off = torch.randn(N, G * 81, *dims, generator=g) * sig
    m = torch.sigmoid(torch.randn(N, G * 27, *dims, generator=g)) if mask else None
    gout = torch.randn(N, Cout, *dims, generator=g).bfloat16()
    return (x, off, m, w, b), gout, (groups, G)


def desc_of(x, w, dims, groups, G, dtype=_lib.D2C_BF16, flags=0):
    N, Cin = x.shape[:2]
    return _lib.Conv3dDesc(N, Cin, w.shape[0], *dims, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, groups, G, *dims,
                           dtype, _lib.D2C_F32, 0, 1.0, 7, flags)


def step(ts, gout, groups, G, dev):
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in ts]
    out = d2c.deform_conv3d(*ts, 1, 1, 1, groups, G)
    out.backward(gout.to(dev))
    return [out.detach()] + [t.grad if t is not None else None for t in ts]


@pytest.fixture
def keep_columns_restored():
    before = _ops.config.keep_columns()
    yield
    _ops.config.set_keep_columns(before["on"], before["max_bytes"])


@pytest.mark.parametrize("name", list(SHAPES))
def test_kept_columns_against_oracle_and_plain_calls(name, dev, keep_columns_restored):
    lib = _lib.load()
    (x, off, m, w, b), gout, (groups, G) = make(name)
    dims = SHAPES[name][3]
    desc = desc_of(x, w, dims, groups, G)
    ncol = lib.d2c_conv3d_columns_bytes(ctypes.byref(desc), None)
    rows = (x.shape[0] * dims[0] * dims[1] * dims[2] + 63) // 64 * 64
    assert ncol == x.shape[1] // 64 * 27 * rows * 64 * 2           # [chunk][tap][rows][64] bfloat16
    assert 0 < lib.d2c_conv3d_backward_columns_workspace_bytes(ctypes.byref(desc), None) \
        < lib.d2c_conv3d_backward_workspace_bytes(ctypes.byref(desc))
    f = lambda t: t.float() if t is not None else None
    e_out = cpu.conv3d_forward(f(x), off, m, f(w), f(b), 1, 1, 1, groups, G)
    eg = cpu.conv3d_backward(f(gout), f(x), off, m, f(w), b is not None, 1, 1, 1, groups, G)
    expected = [e_out] + list(eg)
    _ops.config.set_keep_columns(True)
    kept = step((x, off, m, w, b), gout, groups, G, dev)
    _ops.config.set_keep_columns(False)
    plain = step((x, off, m, w, b), gout, groups, G, dev)
    names = ("out", "grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias")
    for n, a, p, e in zip(names, kept, plain, expected):
        if a is None:
            assert p is None
            continue
        assert rel_l2(a, e) < 2e-2, (name, n, rel_l2(a, e))
        assert_close(a, e, 2e-2, 2e-2 * max(e.abs().max().item(), 1e-6), f"{name} {n} vs oracle")
        # the two paths: the same kernels for everything but grad_weight, whose columns are the forward kernel's
        # (sums over list entries and atomics come in another order from run to run: last-place flips in bfloat16)
        assert rel_l2(a, p) < (4e-3 if n == "grad_weight" else 1e-3), (name, n, rel_l2(a, p))


@pytest.mark.parametrize("name", ["c128_o192_G2", "c256_o512_G4_ragged", "c256_groups2_o640_nomask", "c192_o256_G2"])
def test_kept_columns_float32(name, dev, keep_columns_restored):
    """float32: the forward kernel keeps the interpolated values themselves (not the two-term operands its matrix
    step reads) and the grad-weight product runs over them with float32's accuracy -- on three-term bfloat16
    operands where the weight groups hold sets of four 32-channel chunks, on the float32 matrix instruction
    otherwise: against the float64 oracle grad_weight stays within 3e-6 of the tensor's scale, as on the path that
    samples again."""
    N, Cin, Cout, dims, groups, G, bias, mask, sig = F32_SHAPES[name]
    (x, off, m, w, b), gout, _ = make(name, seed=2)
    x, w, gout = x.float(), w.float(), gout.float()
    b = b.float() if b is not None else None
    dd = lambda t: t.double() if t is not None else None
    e_out = cpu.conv3d_forward(dd(x), dd(off), dd(m), dd(w), dd(b), 1, 1, 1, groups, G)
    eg = cpu.conv3d_backward(dd(gout), dd(x), dd(off), dd(m), dd(w), b is not None, 1, 1, 1, groups, G)
    expected = [e_out] + list(eg)
    _ops.config.set_keep_columns(True)
    kept = step((x, off, m, w, b), gout, groups, G, dev)
    _ops.config.set_keep_columns(False)
    plain = step((x, off, m, w, b), gout, groups, G, dev)
    names = ("out", "grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias")
    for n, a, p, e in zip(names, kept, plain, expected):
        if a is None:
            assert p is None
            continue
        d = (a.double().cpu() - e).abs() / e.abs().max()
        if n == "grad_offset":
            # (a sampling coordinate within float32 rounding of a whole number lands on the other side of it than in
            # float64, where the derivative jumps: a few entries in a million, the same ones on both paths)
            assert (d > 2e-5).sum().item() <= 1e-5 * d.numel(), (name, n, (d > 2e-5).sum().item())
        elif n in ("grad_weight", "grad_bias"):
            # (3e-6 of the tensor's scale, or what the path that samples again leaves: weight groups wider than one
            # pass of the backward kernels keep no columns, both steps then are the plain one)
            dp = ((p.double().cpu() - e).abs() / e.abs().max()).max().item()
            assert d.max().item() < max(3e-6, 1.2 * dp), (name, n, d.max().item(), dp)
        else:
            assert d.max().item() < 2e-5, (name, n, d.max().item())
        assert rel_l2(a, p) < 2e-6, (name, n, rel_l2(a, p))


def test_kept_columns_when_only_the_weights_want_a_gradient(dev, keep_columns_restored):
    (x, off, m, w, b), gout, (groups, G) = make("c128_o192_G2", seed=1)
    f = lambda t: t.float() if t is not None else None
    eg = cpu.conv3d_backward(f(gout), f(x), off, m, f(w), True, 1, 1, 1, groups, G)
    _ops.config.set_keep_columns(True)
    ts = [t.to(dev) for t in (x, off, m, w, b)]
    ts[3].requires_grad_(True)
    d2c.deform_conv3d(*ts, 1, 1, 1, groups, G).backward(gout.to(dev))
    assert all(t.grad is None for i, t in enumerate(ts) if i != 3)
    assert rel_l2(ts[3].grad, eg[3]) < 2e-2
    # (no gradient wanted at all: nothing is kept)
    with torch.no_grad():
        d2c.deform_conv3d(*[t.detach() for t in ts], 1, 1, 1, groups, G)


@pytest.mark.parametrize("mode,act", [("xyz", "elu"), ("xy", "relu_plus_one")])
def test_kept_columns_with_the_size_map_in_the_operator(mode, act, dev, keep_columns_restored):
    N, C, O, dims = 1, 128, 192, (9, 32, 32)
    g = torch.Generator().manual_seed(7100)
    x = torch.randn(N, C, *dims, generator=g).bfloat16().to(dev)
    w = ((torch.rand(O, C, 3, 3, 3, generator=g) * 2 - 1) / (C * 27) ** 0.5).bfloat16().to(dev)
    b = ((torch.rand(O, generator=g) * 2 - 1) / (C * 27) ** 0.5).bfloat16().to(dev)
    raw = (torch.randn(N, {"xyz": 3, "xy": 2}[mode], *dims, generator=g) * 1.2 + 0.5).to(dev)
    m = torch.sigmoid(torch.randn(N, 27, *dims, generator=g)).to(dev)
    gout = torch.randn(N, O, *dims, generator=g).bfloat16().to(dev)
    res = []
    for keep in (True, False):
        _ops.config.set_keep_columns(keep)
        ts = [t.clone().requires_grad_(True) for t in (x, raw, m, w, b)]
        out = _ops.deform_conv3d_sized(*ts, mode, act, 1, 1, 1)
        out.backward(gout)
        res.append([out.detach()] + [t.grad for t in ts])
    for i, (a, p) in enumerate(zip(*res)):
        assert rel_l2(a, p) < (4e-3 if i == 4 else 1e-3), (mode, i, rel_l2(a, p))


def test_column_buffer_checks(dev):
    lib = _lib.load()
    (x, off, m, w, b), gout, (groups, G) = make("c128_o192_G2")
    dims = SHAPES["c128_o192_G2"][3]
    # float32: [chunk of 32 channels][tap][rows][32] floats
    f32 = desc_of(x, w, dims, groups, G, dtype=_lib.D2C_F32)
    rows = (dims[0] * dims[1] * dims[2] + 63) // 64 * 64
    assert lib.d2c_conv3d_columns_bytes(ctypes.byref(f32), None) == x.shape[1] // 32 * 27 * rows * 32 * 4
    # descriptions that keep no columns: problems on the small-tile forward kernel
    small = desc_of(x, w, (3, 6, 9), groups, G)
    assert lib.d2c_conv3d_columns_bytes(ctypes.byref(small), None) == 0
    desc = desc_of(x, w, dims, groups, G)
    ncol = lib.d2c_conv3d_columns_bytes(ctypes.byref(desc), None)
    ts = [t.to(dev) for t in (x, off, m, w, b)]
    out = torch.empty(1, w.shape[0], *dims, dtype=torch.bfloat16, device=dev)
    nws = lib.d2c_conv3d_forward_workspace_bytes(ctypes.byref(desc))
    ws = torch.empty(nws, dtype=torch.uint8, device=dev)
    cols = torch.empty(ncol, dtype=torch.uint8, device=dev)
    p = lambda t: ctypes.c_void_p(t.data_ptr())      # (3 / 5 below: D2C_ERR_WORKSPACE / D2C_ERR_UNSUPPORTED)
    call = lambda d, c, n: lib.d2c_conv3d_forward_columns(ctypes.byref(d), None, p(ts[0]), p(ts[1]), p(ts[2]), p(ts[3]),
                                                          p(ts[4]), p(out), c, n, p(ws), nws, None)
    assert call(desc, p(cols), ncol - 1) == 3 and "column buffer" in _lib.last_error()
    assert call(desc, None, ncol) == 3
    assert call(small, p(cols), ncol) == 5 and "keeps no columns" in _lib.last_error()
    assert call(desc, p(cols), ncol) == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("cls", ["MDConv3d", "XYZSizeConditionedMDConv3d"])
def test_layers_keep_columns_with_the_deformation_tensor_read_in_place(cls, dtype, dev, keep_columns_restored):
    """The self-deforming layers hand the operator their deformation branch's output as it is (offsets and raw
    modulation in one tensor, activation in the sampler): the same step with and without kept columns."""
    from d2conv3d_amd import modules as M
    torch.manual_seed(29)
    layer = getattr(M, cls)(128, 192, 3, padding=1).to(dev)
    with torch.no_grad():
        layer.deform_params.weight.normal_(0, 0.02)
        layer.deform_params.bias.normal_(0, 0.5)
    layer = layer.to(dtype)
    x = torch.randn(1, 128, 9, 32, 32, device=dev).to(dtype)
    gout = torch.randn(1, 192, 9, 32, 32, device=dev).to(dtype)
    res = []
    for keep in (True, False):
        _ops.config.set_keep_columns(keep)
        layer.zero_grad()
        xi = x.clone().requires_grad_(True)
        layer(xi).backward(gout)
        res.append([xi.grad] + [p.grad.clone() for p in layer.parameters()])
    for i, (a, p) in enumerate(zip(*res)):
        assert rel_l2(a, p) < (5e-3 if dtype == torch.bfloat16 else 5e-6), (cls, i, rel_l2(a, p))
