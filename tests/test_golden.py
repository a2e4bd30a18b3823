"""The committed fixtures of tests/golden/ (made by tests/golden/make_golden.py from the pinned oracle): the oracle
must still reproduce them (CPU), and the HIP library must match them through the Python surface (GPU), float64 on
the direct kernels and float32 within the tolerance of the operator (1e-4 relative, 1e-5 absolute)."""
import os

import numpy as np
import pytest
import torch

from _util import assert_close

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CONV3D = ["conv3d_groups", "conv3d_nomask_nobias"]


def load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: (torch.from_numpy(z[k]) if k != "geometry" else [int(v) for v in z[k]]) for k in z.files}


def _geo3(c):
    g = c["geometry"]
    return tuple(g[0:3]), tuple(g[3:6]), tuple(g[6:9]), g[9], g[10]


@pytest.mark.parametrize("name", CONV3D)
def test_oracle_reproduces_conv3d(name):
    from oracle import cpu
    c = load(name)
    s, p, d, groups, G = _geo3(c)
    out = cpu.conv3d_forward(c["x"], c["offset"], c.get("mask"), c["weight"], c.get("bias"), s, p, d, groups, G)
    grads = cpu.conv3d_backward(c["grad_out"], c["x"], c["offset"], c.get("mask"), c["weight"], "bias" in c, s, p, d, groups, G)
    assert_close(out, c["out"], 0, 1e-12, "out")
    for key, got in zip(("grad_x", "grad_offset", "grad_mask", "grad_weight", "grad_bias"), grads):
        if key in c:
            assert_close(got, c[key], 0, 1e-12, key)


def test_oracle_reproduces_conv1d():
    from oracle import cpu
    c = load("conv1d_groups")
    s, p, d, groups, G = c["geometry"]
    out = cpu.conv1d_forward(c["x"], c["offset"], c["mask"], c["weight"], c["bias"], s, p, d, groups, G)
    grads = cpu.conv1d_backward(c["grad_out"], c["x"], c["offset"], c["mask"], c["weight"], True, s, p, d, groups, G)
    assert_close(out, c["out"], 0, 1e-12, "out")
    for key, got in zip(("grad_x", "grad_offset", "grad_mask", "grad_weight", "grad_bias"), grads):
        assert_close(got, c[key], 0, 1e-12, key)


def test_size_map_and_plain_depthwise_fixtures_on_the_cpu():
    from d2conv3d_amd.grid import offsets_from_size_map
    from oracle import dwconv
    for mode in ("xyz", "xxz", "xy", "x"):
        c = load("size_map_" + mode)
        g = c["geometry"]
        size = c["size"].clone().requires_grad_(True)
        off = offsets_from_size_map(size, mode, tuple(g[0:3]), tuple(g[3:6]))
        assert_close(off, c["offsets"], 0, 1e-12, f"offsets ({mode})")
        off.backward(c["grad_offsets"])
        assert_close(size.grad, c["grad_size"], 0, 1e-12, f"grad_size ({mode})")
    c = load("dwconv3d_multiplier2")
    g = c["geometry"]
    s, p, d = tuple(g[0:3]), tuple(g[3:6]), tuple(g[6:9])
    assert_close(torch.from_numpy(dwconv.forward(c["x"].numpy(), c["weight"].numpy(), c["bias"].numpy(), s, p, d)),
                 c["out"], 0, 1e-12, "out")
    gx, gw, gb = dwconv.backward(c["grad_out"].numpy(), c["x"].numpy(), c["weight"].numpy(), s, p, d)
    for key, got in (("grad_x", gx), ("grad_weight", gw), ("grad_bias", gb)):
        assert_close(torch.from_numpy(got), c[key], 0, 1e-12, key)


# ------------------------------------------------------------------ GPU
def _on(dev, t, dtype, grad=True):
    return None if t is None else t.to(dev, dtype).requires_grad_(grad)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
@pytest.mark.parametrize("name", CONV3D)
def test_gpu_matches_conv3d_fixture(name, dtype, dev):
    import d2conv3d_amd as d2c
    c = load(name)
    s, p, d, groups, G = _geo3(c)
    ts = [_on(dev, c.get(k), dtype) for k in ("x", "offset", "mask", "weight", "bias")]
    out = d2c.deform_conv3d(*ts, s, p, d, groups, G)
    out.backward(c["grad_out"].to(dev, dtype))
    rt, at = (1e-10, 1e-11) if dtype == torch.float64 else (1e-4, 1e-5)
    assert_close(out, c["out"], rt, at, "out")
    for key, t in zip(("grad_x", "grad_offset", "grad_mask", "grad_weight", "grad_bias"), ts):
        if t is not None:
            assert_close(t.grad, c[key], rt, at * max(1.0, c[key].abs().max().item()), key)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_gpu_matches_conv1d_fixture(dtype, dev):
    import d2conv3d_amd as d2c
    c = load("conv1d_groups")
    s, p, d, groups, G = c["geometry"]
    ts = [_on(dev, c[k], dtype) for k in ("x", "offset", "mask", "weight", "bias")]
    out = d2c.deform_conv1d(*ts, s, p, d, groups, G)
    out.backward(c["grad_out"].to(dev, dtype))
    rt, at = (1e-10, 1e-11) if dtype == torch.float64 else (1e-4, 1e-5)
    assert_close(out, c["out"], rt, at, "out")
    for key, t in zip(("grad_x", "grad_offset", "grad_mask", "grad_weight", "grad_bias"), ts):
        assert_close(t.grad, c[key], rt, at * max(1.0, c[key].abs().max().item()), key)


@pytest.mark.gpu
def test_gpu_matches_size_map_and_plain_depthwise_fixtures(dev):
    from d2conv3d_amd.depthwise_conv import depthwise_separable_conv3d
    from d2conv3d_amd.grid import size_map_offsets
    for mode in ("xyz", "xxz", "xy", "x"):
        c = load("size_map_" + mode)
        g = c["geometry"]
        size = c["size"].float().to(dev).requires_grad_(True)
        got = size_map_offsets(size, mode, tuple(g[0:3]), tuple(g[3:6]), "linear")
        assert_close(got, c["offsets"], 1e-5, 1e-6, f"offsets ({mode})")
        got.backward(c["grad_offsets"].float().to(dev))
        assert_close(size.grad, c["grad_size"], 1e-5, 1e-5, f"grad_size ({mode})")
    c = load("dwconv3d_multiplier2")
    g = c["geometry"]
    s, p, d = tuple(g[0:3]), tuple(g[3:6]), tuple(g[6:9])
    for dtype, tol in ((torch.float64, 1e-11), (torch.float32, 1e-5)):
        x, w, b = (_on(dev, c[k], dtype) for k in ("x", "weight", "bias"))
        out = depthwise_separable_conv3d(x, w, b, s, p, d)
        out.backward(c["grad_out"].to(dev, dtype))
        assert_close(out, c["out"], 0, tol, "out")
        for key, t in (("grad_x", x), ("grad_weight", w), ("grad_bias", b)):
            assert_close(t.grad, c[key], 0, tol * max(1.0, c[key].abs().max().item()), key)
