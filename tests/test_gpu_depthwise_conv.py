"""GPU parity of the plain depthwise conv3d kernels (csrc/d2c_dwconv.hip) through Python -> C ABI against the
numpy oracle (oracle/dwconv.py): the reference's own test matrix (test_conv3d_depthwise.py:33-96: stride x dilation
x depth multiplier / bias x dtype), other filter shapes on the element-per-thread kernels, ragged widths, and the
error behaviour of conv_depthwise_shape_check."""
import numpy as np
import pytest
import torch
import torch.nn as nn

from d2conv3d_amd.depthwise_conv import DepthwiseConv3d, depthwise_separable_conv3d, install_as_fast_depthwise_conv3d
from oracle import dwconv

pytestmark = pytest.mark.gpu

# the reference's tolerances (test_conv3d_depthwise.py:25-28); bfloat16 results are compared relative to the
# largest value (inputs are bfloat16-rounded before the oracle sees them)
TOL = {torch.float32: 1e-5, torch.float64: 1e-10, torch.float16: 1e-2, torch.bfloat16: 2e-2}


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


def _run(dev, dtype, N, C, m, dims, k, s, p, d, bias, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(N, C, *dims, generator=g) / 2).to(dtype)
    w = (torch.randn(C * m, 1, *k, generator=g) / 3).to(dtype)
    b = (torch.randn(C * m, generator=g) / 2).to(dtype) if bias else None
    xs, ws = x.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    bs = b.to(dev).requires_grad_(True) if bias else None
    out = depthwise_separable_conv3d(xs, ws, bs, s, p, d)
    assert out.dtype == dtype
    eo = dwconv.forward(x.double().numpy(), w.double().numpy(), None if b is None else b.double().numpy(), s, p, d)
    assert tuple(out.shape) == eo.shape
    go = (torch.randn(out.shape, generator=g) / 2).to(dtype)
    out.backward(go.to(dev))
    egx, egw, egb = dwconv.backward(go.double().numpy(), x.double().numpy(), w.double().numpy(), s, p, d, bias)

    def close(got, exp, what):
        got = got.detach().double().cpu().numpy()
        tol = TOL[dtype] * (max(1.0, np.abs(exp).max()) if dtype in (torch.bfloat16, torch.float16) else
                            max(1.0, np.abs(exp).max()))
        err = np.abs(got - exp).max()
        assert err <= tol, f"{what}: max abs error {err} > {tol}"

    close(out, eo, "out")
    close(xs.grad, egx, "grad_input")
    close(ws.grad, egw, "grad_weight")
    if bias:
        close(bs.grad, egb, "grad_bias")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("stride,dilation", [(1, 1), (2, 1), (1, 2), (2, 2)])
@pytest.mark.parametrize("multiplier,bias", [(1, True), (2, False)])
def test_reference_matrix(dtype, stride, dilation, multiplier, bias, dev):
    """test_Conv3d_depthwise_naive_groups_cuda: 2 channels, 6^3 input, 3^3 filter, padding = dilation."""
    _run(dev, dtype, 2, 2, multiplier, (6, 6, 6), (3, 3, 3), (stride,) * 3, (dilation,) * 3, (dilation,) * 3, bias)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", [
    # N, C, m, dims, kernel, stride, padding, dilation, bias
    (2, 24, 1, (5, 13, 27), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), True),     # ragged width: 27 = 6 * 4 + 3
    (1, 16, 2, (4, 9, 10), (3, 3, 3), (2, 2, 1), (1, 1, 1), (1, 2, 1), True),      # blocked kernels, strides in z / y
    (1, 8, 1, (6, 8, 9), (3, 3, 3), (1, 1, 1), (0, 0, 0), (1, 1, 1), False),       # no padding
    (1, 8, 1, (6, 8, 9), (3, 3, 3), (1, 1, 1), (2, 2, 3), (1, 1, 1), True),        # padding wider than the filter
    (2, 6, 3, (5, 7, 8), (1, 3, 5), (1, 2, 2), (0, 1, 2), (1, 1, 1), True),        # other filter shape
    (1, 5, 1, (7, 6, 9), (3, 1, 2), (2, 1, 1), (1, 0, 1), (2, 1, 3), False),
    (1, 4, 1, (4, 5, 6), (1, 1, 1), (1, 1, 1), (0, 0, 0), (1, 1, 1), True),        # pointwise
    # widths that are multiples of 4 with padding 1 along W: vector loads, neighbours from adjacent lanes
    (2, 6, 1, (4, 7, 8), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), True),        # part of one tile
    (1, 4, 2, (3, 18, 56), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), True),      # the backbone's width
    (1, 3, 1, (3, 17, 72), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), False),     # two tiles along W, the second partial
    (1, 3, 1, (4, 5, 128), (3, 3, 3), (1, 1, 1), (0, 2, 1), (1, 2, 1), True),      # two full tiles; other padding in z / y
    (1, 4, 1, (5, 9, 16), (3, 3, 3), (2, 2, 1), (1, 1, 1), (1, 1, 1), True),       # strides in z / y
])
def test_shapes(dtype, case, dev):
    _run(dev, dtype, *case, seed=3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64])
def test_random_geometries(dtype, dev):
    """Seeded random sizes, filters, strides, paddings, dilations and depth multipliers against the oracle; widths
    are drawn so that the vector, the blocked and the element-per-thread kernels all get cases (D2C_RANDOM_CASES
    in the environment widens the sweep; each case is printed before it runs)."""
    import os
    rng = np.random.default_rng(4242)
    pick = lambda *v: v[int(rng.integers(len(v)))]
    for case in range(int(os.environ.get("D2C_RANDOM_CASES", "12"))):
        k = (pick(1, 3, 3), pick(1, 3, 3), pick(1, 2, 3, 3, 5))
        s = (pick(1, 1, 2), pick(1, 1, 2), pick(1, 1, 1, 2))
        d = (pick(1, 1, 2), pick(1, 1, 2), pick(1, 1, 2))
        p = tuple(int(rng.integers(0, 3)) for _ in range(3))
        dims = [int(rng.integers(dd * (kk - 1) + 1, dd * (kk - 1) + 1 + 8)) for kk, dd in zip(k, d)]
        if rng.integers(2):
            dims[2] = max(dims[2], 4 * int(rng.integers(1, 36)))      # widths that are multiples of 4, up to 140
        shape = (pick(1, 2, 3), int(rng.integers(1, 20)), pick(1, 1, 2, 3), tuple(dims), k, s, p, d,
                 bool(rng.integers(2)))
        print(f"random case {case} {dtype}: {shape}", flush=True)
        _run(dev, dtype, *shape, seed=500 + case)


def test_many_positions_per_channel(dev):
    """More items than one launch covers in one pass of its grid-stride loops, and several shares in grad_weight."""
    _run(dev, torch.float32, 1, 2, 1, (16, 64, 130), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), True, seed=5)


def test_module_is_a_conv3d_with_groups(dev):
    """DepthwiseConv3d keeps nn.Conv3d's parameters and initialisation (conv.py:7-13) and agrees with it."""
    torch.manual_seed(0)
    m = DepthwiseConv3d(8, 16, kernel_size=3, padding=1, groups=123).to(dev)
    torch.manual_seed(0)
    r = nn.Conv3d(8, 16, 3, padding=1, groups=8).to(dev)
    assert m.groups == 8 and torch.equal(m.weight, r.weight) and torch.equal(m.bias, r.bias)
    x = torch.randn(2, 8, 5, 6, 7, device=dev)
    assert torch.allclose(m(x), r(x), atol=1e-5, rtol=0)
    # an input without batch dimension (grouped_conv3d.cu:403-405)
    assert torch.allclose(depthwise_separable_conv3d(x[0], m.weight, m.bias, 1, 1, 1), r(x)[0], atol=1e-5, rtol=0)
    # non-zero padding modes pad first (conv.py:18-20)
    mc = DepthwiseConv3d(8, 8, 3, padding=1, padding_mode="replicate").to(dev)
    rc = nn.Conv3d(8, 8, 3, padding=1, groups=8, padding_mode="replicate").to(dev)
    rc.load_state_dict(mc.state_dict())
    assert torch.allclose(mc(x), rc(x), atol=1e-5, rtol=0)


def test_autocast_keeps_half(dev):
    """test_autograd_type_conversion: a half input gives a half output."""
    inp = torch.randn(2, 2, 5, 5, 5, device=dev).half()
    conv = DepthwiseConv3d(2, 2, kernel_size=3).to(dev)
    with torch.autocast("cuda", dtype=torch.float16):
        assert conv(inp).dtype == torch.float16


def test_only_wanted_gradients(dev):
    x = torch.randn(1, 4, 5, 6, 7, device=dev)
    w = torch.randn(4, 1, 3, 3, 3, device=dev, requires_grad=True)
    out = depthwise_separable_conv3d(x, w, None, 1, 1, 1)
    out.sum().backward()
    assert w.grad is not None and x.grad is None


def test_shape_checks(dev):
    x = torch.randn(1, 4, 5, 6, 7, device=dev)
    w = torch.randn(4, 1, 3, 3, 3, device=dev)
    with pytest.raises(RuntimeError, match="in_channels=1"):
        depthwise_separable_conv3d(x, torch.randn(4, 2, 3, 3, 3, device=dev), None, 1, 1, 1)
    with pytest.raises(RuntimeError, match="multiple of in channels"):
        depthwise_separable_conv3d(x, torch.randn(6, 1, 3, 3, 3, device=dev), None, 1, 1, 1)
    with pytest.raises(RuntimeError, match="Bias length"):
        depthwise_separable_conv3d(x, w, torch.randn(3, device=dev), 1, 1, 1)
    with pytest.raises(RuntimeError, match="Output size should be positive"):
        depthwise_separable_conv3d(x, torch.randn(4, 1, 7, 3, 3, device=dev), None, 1, 0, 1)
    with pytest.raises(RuntimeError, match="stride should be at least 1"):
        depthwise_separable_conv3d(x, w, None, (0, 1, 1), 1, 1)
    with pytest.raises(RuntimeError, match="GPU"):
        depthwise_separable_conv3d(x.cpu(), w.cpu(), None, 1, 1, 1)


def test_import_name_of_the_reference(dev):
    pkg = install_as_fast_depthwise_conv3d()
    from fast_depthwise_conv3d import DepthwiseConv3d as D
    import fast_depthwise_conv3d._ops as ops
    assert D is DepthwiseConv3d and ops.depthwise_separable_conv3d is depthwise_separable_conv3d and pkg.DepthwiseConv3d is D


def test_unaligned_tensors_take_the_scalar_kernels(dev):
    """Tensors that do not start on a 16-byte boundary (views into a larger buffer) give the same result."""
    g = torch.Generator().manual_seed(9)
    N, C, dims = 1, 4, (3, 6, 8)
    n = N * C * dims[0] * dims[1] * dims[2]
    buf = torch.randn(n + 1, generator=g).to(dev)
    x = buf[1:].view(N, C, *dims)                      # 4 bytes off
    w = torch.randn(C, 1, 3, 3, 3, generator=g).to(dev)
    a = depthwise_separable_conv3d(x, w, None, 1, 1, 1)
    b = depthwise_separable_conv3d(x.clone(), w, None, 1, 1, 1)
    assert x.data_ptr() % 16 != 0 and torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_full_size_against_torch_grouped_conv(dtype, dev):
    """The workload bench.py times (N=2, C=256, 8x56x56, 3^3, padding 1): too large for the numpy oracle, so the
    reference's own check is used, torch's grouped convolution and its autograd on the same tensors (float32
    arithmetic on bfloat16-rounded values for the bfloat16 case), plus grad_bias = sum of grad_out."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(1006)
    N, C, dims = 2, 256, (8, 56, 56)
    x = torch.randn(N, C, *dims, generator=g).to(dtype).to(dev)
    w = ((torch.rand(C, 1, 3, 3, 3, generator=g) * 2 - 1) / 27 ** 0.5).to(dtype).to(dev)
    b = ((torch.rand(C, generator=g) * 2 - 1) / 27 ** 0.5).to(dtype).to(dev)
    go = torch.randn(N, C, *dims, generator=g).to(dtype).to(dev)
    xs, ws, bs = (t.clone().requires_grad_(True) for t in (x, w, b))
    out = depthwise_separable_conv3d(xs, ws, bs, 1, 1, 1)
    out.backward(go)
    xr, wr, br = (t.float().clone().requires_grad_(True) for t in (x, w, b))
    ref = F.conv3d(xr, wr, br, 1, 1, 1, groups=C)
    ref.backward(go.float())
    tol = 1e-5 if dtype == torch.float32 else 2e-2

    def rel(a, e):
        return float((a.detach().float() - e.detach()).abs().max() / e.detach().abs().max())

    assert rel(out, ref) < tol and rel(xs.grad, xr.grad) < tol and rel(ws.grad, wr.grad) < tol and rel(bs.grad, br.grad) < tol
    assert rel(bs.grad, go.float().sum(dim=(0, 2, 3, 4))) < tol
