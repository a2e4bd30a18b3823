"""GPU parity at the full sizes of the measured workloads (the tensors bench.py
times, same seeds).

Where the CPU oracle finishes in seconds to tens of seconds (C1, C2, C3, C4,
C5a) the whole forward + backward is compared with it.  For every workload,
C5b included, size-independent properties are checked as well:

* zero offsets and unit mask reduce the operator to torch's stock convolution;
* the forward pass is linear in the input, and grad_input / grad_weight are its
  adjoints:  <op(x), g> = <x, grad_input(g)> = <w, grad_weight(g)> (bias excluded), evaluated at g = op(x);
* grad_bias = sum of grad_out.

float32: the literal gate (1e-4 relative / 1e-5 absolute) against the float64
oracle on the same values where float32 sums can meet it, else at most three
times the float32 oracle's own excess over it (both figures are printed per
tensor), and 1e-4 relative / 1e-5 absolute scaled by the tensor's magnitude
against the float32 oracle.  bfloat16: 2e-2 relative, over the tensor (L2) and
element-wise against the tensor's scale.
"""
import os
import sys

import pytest
import torch
import torch.nn.functional as F

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench  # noqa: E402  (workload table and seeded input generator)
import d2conv3d_amd as d2c  # noqa: E402
from oracle import cpu  # noqa: E402
from _util import assert_close, rel_l2  # noqa: E402

pytestmark = pytest.mark.gpu


def _tensors(name):
    c = bench.WORKLOADS[name]
    x, off, m, w, b, gout = bench.make_inputs(name, torch)
    if c["dt"] == "bf16":
        x, w, b, gout, off, m = (t.bfloat16() for t in (x, w, b, gout, off, m))
    return c, x, off, m, w, b, gout


def _run(c, dev, x, off, m, w, b, gout=None):
    ts = [t.to(dev).requires_grad_(gout is not None) if t is not None else None for t in (x, off, m, w, b)]
    fn = d2c.deform_conv3d if c["nd"] == 3 else d2c.deform_conv1d
    out = fn(*ts, 1, 1, 1, c["groups"], c["G"])
    if gout is None:
        return out, None
    out.backward(gout.to(dev))
    return out.detach(), [t.grad if t is not None else None for t in ts]


def relative_error_profile(actual, expected, floor=0.05):
    """(99.9th percentile, maximum) of |a - e| / |e| over the elements with |e| >= floor * max|e|: how the
    element-wise relative error of a bfloat16 result is distributed where a relative error means something."""
    a, e = actual.detach().double().cpu().flatten(), expected.double().flatten()
    keep = e.abs() >= floor * e.abs().max()
    r = ((a[keep] - e[keep]).abs() / e[keep].abs())
    k = max(1, int(round(0.999 * r.numel())))
    return r.kthvalue(k).values.item(), r.max().item(), int(keep.sum())


def literal_gate_excess(actual, exact):
    """max over the tensor of |actual - exact| / (1e-5 + 1e-4 |exact|): <= 1 means the literal float32 gate
    (1e-4 relative / 1e-5 absolute, no scaling) holds against the float64 result."""
    a, e = actual.detach().double().cpu(), exact.double()
    return ((a - e).abs() / (1e-5 + 1e-4 * e.abs())).max().item()


@pytest.mark.parametrize("name", ["c1", "c5a", "c4", "c2_f32", "c2_bf16", "c3", "c3_f32"])
def test_full_size_against_oracle(name, dev):
    c, x, off, m, w, b, gout = _tensors(name)
    f = lambda t: t.float()
    fwd, bwd = (cpu.conv3d_forward, cpu.conv3d_backward) if c["nd"] == 3 else (cpu.conv1d_forward, cpu.conv1d_backward)
    e_out = fwd(f(x), f(off), f(m), f(w), f(b), 1, 1, 1, c["groups"], c["G"])
    out, grads = _run(c, dev, x, off, m, w, b, gout if c["backward"] else None)
    names = ["grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias"]
    pairs = [("out", out, e_out)]
    if c["backward"]:
        e = bwd(f(gout), f(x), f(off), f(m), f(w), True, 1, 1, 1, c["groups"], c["G"])
        pairs += [(n, g, ee) for n, g, ee in zip(names, grads, e)]
    exact = None
    if c["dt"] == "f32":
        # the same float32 values in float64 arithmetic: what both float32 computations approximate
        dd = lambda t: t.double()
        exact = [fwd(dd(x), dd(off), dd(m), dd(w), dd(b), 1, 1, 1, c["groups"], c["G"])]
        if c["backward"]:
            exact += list(bwd(dd(gout), dd(x), dd(off), dd(m), dd(w), True, 1, 1, 1, c["groups"], c["G"]))
    for i, (n, a, ee) in enumerate(pairs):
        if c["dt"] == "f32":
            # Literal gate first, against the float64 result.  Long float32 sums (the gradients of the large
            # workloads add 10^4 - 10^5 terms) miss it whatever their order: where the float32 oracle, the
            # reference's own summation order, misses it too, the kernels may miss it by at most three times as much.
            hip, o32 = literal_gate_excess(a, exact[i]), literal_gate_excess(ee, exact[i])
            print(f"literal 1e-4/1e-5 gate, {name} {n}: kernels {hip:.3g}, float32 oracle {o32:.3g} "
                  f"(max |exact| {exact[i].abs().max().item():.3g})", flush=True)
            assert hip <= max(1.0, 3.0 * o32), (name, n, hip, o32)
            scale = max(1.0, ee.abs().max().item())
            assert_close(a, ee, 1e-4, 1e-5 * scale, f"{name} {n}")
        else:
            assert rel_l2(a, ee) < 2e-2, (name, n, rel_l2(a, ee))
            assert_close(a, ee, 2e-2, 2e-2 * ee.abs().max().item(), f"{name} {n}")
            # ... and the 2e-2 relative tolerance taken element by element wherever an element is large enough for a
            # relative error to mean something (at least 5 % of the tensor's maximum): 99.9 % of those elements
            # within it, none further off than 5e-2
            p999, worst, cnt = relative_error_profile(a, ee)
            print(f"element-wise relative error, {name} {n}: 99.9th percentile {p999:.3g}, max {worst:.3g} "
                  f"over {cnt} elements >= 5 % of max |expected|; L2 {rel_l2(a, ee):.3g}", flush=True)
            assert p999 <= 2e-2 and worst <= 5e-2, (name, n, p999, worst)


@pytest.mark.parametrize("name", ["c2_f32", "c2_bf16"])
def test_full_size_dilation_map_into_the_operator(name, dev):
    """Workload C2 the way bench.py times it: the dilation map [2, 3, 8, 30, 54] goes into the operator
    (deform_conv3d_sized), no offsets tensor exists.  Against the oracle on the expanded offsets; the expected
    gradient of the map is the transpose of the expansion (oracle/sizemap.py) applied to the oracle's grad_offset."""
    import numpy as np
    from oracle import sizemap
    c = bench.WORKLOADS[name]
    x, off, m, w, b, gout, size = bench.make_inputs(name, torch, want_size=True)
    f = lambda t: t.float()
    if c["dt"] == "bf16":
        x, w, b, gout, m, size = (t.bfloat16() for t in (x, w, b, gout, m, size))
        # the offsets the sampler forms from a bfloat16 map: the torch formulation in bfloat16
        from d2conv3d_amd.grid import offsets_from_size_map
        off = offsets_from_size_map(size, "xyz", (3, 3, 3), (1, 1, 1))
    else:
        assert np.array_equal(off.numpy(), sizemap.offsets(size.double().numpy(), "xyz").astype(np.float32))
    ts = [t.to(dev).requires_grad_(True) for t in (x, size, m, w, b)]
    out = d2c.deform_conv3d_sized(*ts, "xyz", "linear", 1, 1, 1, 1)
    out.backward(gout.to(dev))
    e_out = cpu.conv3d_forward(f(x), f(off), f(m), f(w), f(b), 1, 1, 1, 1, 1)
    e = list(cpu.conv3d_backward(f(gout), f(x), f(off), f(m), f(w), True, 1, 1, 1, 1, 1))
    e[1] = torch.from_numpy(sizemap.offsets_backward(e[1].double().numpy(), "xyz")).float()
    names = ["grad_input", "grad_size", "grad_mask", "grad_weight", "grad_bias"]
    for n, a, ee in [("out", out, e_out)] + list(zip(names, [t.grad for t in ts], e)):
        if c["dt"] == "f32":
            assert_close(a, ee, 1e-4, 1e-5 * max(1.0, ee.abs().max().item()), f"{name} {n}")
        else:
            assert rel_l2(a, ee) < 2e-2, (name, n, rel_l2(a, ee))
            assert_close(a, ee, 2e-2, 2e-2 * ee.abs().max().item(), f"{name} {n}")


def test_long_clip_backward_against_oracle(dev):
    """The long-clip volume of workload c5b (32 x 60 x 108 = 207360 positions, bfloat16, one offset group) with
    64 channels, which the oracle finishes in seconds: all five gradients, i.e. the grad-column rows, the offset /
    mask gradient and the sample lists at the full number of positions."""
    g = torch.Generator().manual_seed(1505)
    N, C, dims = 1, 64, (32, 60, 108)
    x = torch.randn(N, C, *dims, generator=g).bfloat16()
    bound = 1.0 / (C * 27) ** 0.5
    w = ((torch.rand(C, C, 3, 3, 3, generator=g) * 2 - 1) * bound).bfloat16()
    b = ((torch.rand(C, generator=g) * 2 - 1) * bound).bfloat16()
    off = torch.randn(N, 81, *dims, generator=g)
    m = torch.sigmoid(torch.randn(N, 27, *dims, generator=g))
    gout = torch.randn(N, C, *dims, generator=g).bfloat16()
    ts = [t.to(dev).requires_grad_(True) for t in (x, off, m, w, b)]
    from d2conv3d_amd import _ops
    assert _ops.conv3d_algo(ts[0], ts[1], ts[2], ts[3], (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, 1) == "mfma"
    out = d2c.deform_conv3d(*ts, 1, 1, 1, 1, 1)
    out.backward(gout.to(dev))
    f = lambda t: t.float()
    e_out = cpu.conv3d_forward(f(x), off, m, f(w), f(b), 1, 1, 1, 1, 1)
    e = cpu.conv3d_backward(f(gout), f(x), off, m, f(w), True, 1, 1, 1, 1, 1)
    for n, a, ee in [("out", out, e_out)] + list(zip(("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias"),
                                                     [t.grad for t in ts], e)):
        assert rel_l2(a, ee) < 2e-2, (n, rel_l2(a, ee))
        assert_close(a, ee, 2e-2, 2e-2 * ee.abs().max().item(), n)


@pytest.mark.parametrize("name", ["c2_bf16", "c3", "c4", "c5a", "c5b"])
def test_full_size_zero_offsets_equal_stock_convolution(name, dev):
    c, x, off, m, w, b, _ = _tensors(name)
    out, _ = _run(c, dev, x, torch.zeros_like(off), torch.ones_like(m), w, b)
    conv = F.conv3d if c["nd"] == 3 else F.conv1d
    ref = conv(x.to(dev).float(), w.to(dev).float(), b.to(dev).float(), 1, 1, 1, c["groups"])
    if c["dt"] == "f32":
        assert_close(out, ref, 1e-4, 1e-5 * max(1.0, ref.abs().max().item()), name)
    else:
        assert rel_l2(out, ref) < 1e-2, rel_l2(out, ref)


@pytest.mark.parametrize("name", ["c3", "c4", "c5a", "c5b"])
def test_full_size_linearity_and_adjoints(name, dev):
    c, x, off, m, w, b, gout = _tensors(name)
    tol = 2e-2 if c["dt"] == "bf16" else 2e-4
    g = torch.Generator().manual_seed(7)
    x2 = torch.randn(x.shape, generator=g).to(x.dtype)
    o1, _ = _run(c, dev, x, off, m, w, None)
    o2, _ = _run(c, dev, x2, off, m, w, None)
    xs = (x.float() * 0.5 + x2.float()).to(x.dtype)        # exact in bfloat16 only up to rounding of the sum
    o12, _ = _run(c, dev, xs, off, m, w, None)
    assert rel_l2(o12.float(), 0.5 * o1.float() + o2.float()) < tol
    # adjoints, with grad_out = op(x) so that the inner products are far from zero
    go = o1.detach().cpu()
    _, grads = _run(c, dev, x, off, m, w, b, go)
    gx, _, _, gw, gb = grads
    lhs = (o1.double() * o1.double()).sum().item()                      # <op(x), g>, bias excluded
    via_x = (x.to(dev).double() * gx.double()).sum().item()
    via_w = (w.to(dev).double() * gw.double()).sum().item()
    atol = (2e-3 if c["dt"] == "bf16" else 2e-5) * abs(lhs)
    assert abs(lhs - via_x) < atol, (lhs, via_x)
    assert abs(lhs - via_w) < atol, (lhs, via_w)
    e_gb = go.double().sum(dim=[0] + list(range(2, go.dim())))
    assert rel_l2(gb, e_gb) < (1e-2 if c["dt"] == "bf16" else 1e-5)


# Layer shapes of the reference's own networks on an 8-frame 480x854 clip at stride 16 (refinement block of
# network/segmentation/encoder_decoder.py:129, global-convolution bridge of network/modules/bridging.py:14-22, a
# deformable convolution without modulation, network/layers.py:103-105): (Cin, Cout, kernel, modulation, dtype)
NETWORK_LAYERS = {
    "refine_1024_256_bf16": (1024, 256, (3, 3, 3), True, torch.bfloat16),
    "bridge_2048_256_1x7x1_bf16": (2048, 256, (1, 7, 1), True, torch.bfloat16),
    "dconv_256_256_f32": (256, 256, (3, 3, 3), False, torch.float32),
}


@pytest.mark.parametrize("name", list(NETWORK_LAYERS))
def test_network_layer_shapes_against_oracle(name, dev):
    cin, cout, ks, modulated, dtype = NETWORK_LAYERS[name]
    dims, K = (8, 30, 54), ks[0] * ks[1] * ks[2]
    pad = tuple(k // 2 for k in ks)
    g = torch.Generator().manual_seed(9000 + cin)
    bound = 1.0 / (cin * K) ** 0.5
    x = torch.randn(1, cin, *dims, generator=g).to(dtype)
    w = ((torch.rand(cout, cin, *ks, generator=g) * 2 - 1) * bound).to(dtype)
    b = ((torch.rand(cout, generator=g) * 2 - 1) * bound).to(dtype)
    off = torch.randn(1, 3 * K, *dims, generator=g) * 1.5
    m = torch.sigmoid(torch.randn(1, K, *dims, generator=g)) if modulated else None
    gout = torch.randn(1, cout, *dims, generator=g).to(dtype)
    f = lambda t: t.float() if t is not None else None
    e_out = cpu.conv3d_forward(f(x), off, m, f(w), f(b), 1, pad, 1, 1, 1)
    eg = cpu.conv3d_backward(f(gout), f(x), off, m, f(w), True, 1, pad, 1, 1, 1)
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
    out = d2c.deform_conv3d(*ts, 1, pad, 1, 1, 1)
    out.backward(gout.to(dev))
    pairs = [("out", out.detach(), e_out)] + [(n, t.grad, e) for n, t, e in zip(
        ("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias"), ts, eg) if t is not None]
    for n, a, e in pairs:
        if dtype == torch.bfloat16:
            assert rel_l2(a, e) < 2e-2, (name, n, rel_l2(a, e))
            assert_close(a, e, 2e-2, 2e-2 * e.abs().max().item(), f"{name} {n}")
        else:
            # float32 against the float32 oracle: 1e-4 relative / 1e-5 absolute scaled by the tensor's magnitude
            assert_close(a, e, 1e-4, 1e-5 * max(1.0, e.abs().max().item()), f"{name} {n}")
