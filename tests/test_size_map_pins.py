"""offsets_from_size_map (utils/grid.py:72-98, dconv_native/grid.py:62-80) pinned outside the package.

The numpy closed form of oracle/sizemap.py is first held to what the mathematics fixes -- a constant integer
size map turns the deformable convolution into torch's stock dilated convolution, for every mode -- and to its
own transpose; then the package's torch formulation (CPU) and the HIP kernels d2c_size_map_offsets_forward /
_backward (GPU) are held to the closed form on spatially varying maps, all four modes, an even kernel extent
and a non-unit dilation."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from d2conv3d_amd.grid import offsets_from_size_map
from oracle import cpu, sizemap

MODES = [("xyz", 3), ("xxz", 2), ("xy", 2), ("x", 1)]
KERNEL, DILATION = (3, 5, 2), (1, 2, 1)


def _varying(channels, seed, shape=(2, 3, 4, 5)):
    g = torch.Generator().manual_seed(seed)
    return torch.rand(shape[0], channels, *shape[1:], generator=g, dtype=torch.float64) * 3.5 + 0.5


# ---- the closed form itself -------------------------------------------------------------------------------
@pytest.mark.parametrize("mode,sizes,dil", [
    ("xyz", (2.0, 1.0, 3.0), (2, 1, 3)),
    ("xy", (3.0, 2.0), (1, 3, 2)),        # channels (y, x); z keeps dilation 1
    ("xy", (1.0, 2.0), (1, 1, 2)),
    ("xxz", (2.0, 3.0), (2, 3, 3)),       # channels (z, x); y follows x
    ("xxz", (1.0, 2.0), (1, 2, 2)),
    ("x", (2.0,), (1, 2, 2)),             # test_modules.py:48-67: size 2 == Conv3d(padding=(1,2,2), dilation=(1,2,2))
])
def test_constant_integer_size_map_is_a_dilated_convolution(mode, sizes, dil):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 3, 7, 8, 9, generator=g, dtype=torch.float64)
    w = torch.randn(4, 3, 3, 3, 3, generator=g, dtype=torch.float64)
    b = torch.randn(4, generator=g, dtype=torch.float64)
    sm = np.broadcast_to(np.asarray(sizes, dtype=np.float64).reshape(1, -1, 1, 1, 1), (2, len(sizes), 7, 8, 9))
    off = torch.from_numpy(sizemap.offsets(sm, mode, (3, 3, 3), (1, 1, 1)))
    out = cpu.conv3d_forward(x, off, None, w, b, padding=1)
    # the kernel centre stays where padding 1 puts it; the taps move out to +-dil: pad by dil for the same output size
    ref = F.conv3d(x, w, b, padding=dil, dilation=dil)
    assert torch.allclose(out, ref, rtol=1e-9, atol=1e-9)
    # and the package's torch formulation gives the same offsets
    assert torch.equal(offsets_from_size_map(torch.from_numpy(sm.copy()), mode, (3, 3, 3), (1, 1, 1)), off)


def test_closed_form_element_by_hand():
    # one element written out: mode xxz, kernel (3, 5, 2), dilation (1, 2, 1); tap (kz, ky, kx) = (2, 1, 0)
    size = _varying(2, 3).numpy()
    off = sizemap.offsets(size, "xxz", KERNEL, DILATION)
    k = (2 * 5 + 1) * 2 + 0
    z, x = size[1, 0, 2, 3, 4], size[1, 1, 2, 3, 4]
    assert off[1, 3 * k + 0, 2, 3, 4] == 1.0 * (z - 1.0)       # base_z = (-1, 0, 1)[2]
    assert off[1, 3 * k + 1, 2, 3, 4] == -2.0 * (x - 1.0)      # base_y = (-4, -2, 0, 2, 4)[1], y follows x
    assert off[1, 3 * k + 2, 2, 3, 4] == -1.0 * (x - 1.0)      # base_x = linspace(-1, 1, 2)[0]


@pytest.mark.parametrize("mode,channels", MODES)
def test_closed_form_backward_is_the_transpose(mode, channels):
    size = _varying(channels, 11).numpy()
    off = sizemap.offsets(size, mode, KERNEL, DILATION)
    rng = np.random.default_rng(3)
    go = rng.standard_normal(off.shape)
    gs = sizemap.offsets_backward(go, mode, KERNEL, DILATION)
    ds = rng.standard_normal(size.shape)
    # <J ds, go> = <ds, J^T go>; the map is affine, so J ds = offsets(size + ds) - offsets(size)
    jd = sizemap.offsets(size + ds, mode, KERNEL, DILATION) - off
    assert abs((jd * go).sum() - (ds * gs).sum()) < 1e-9 * abs((jd * go).sum())


@pytest.mark.parametrize("name", ["linear", "elu", "relu", "relu_plus_one"])
def test_size_activations(name):
    # network/layers.py:171-181 in torch
    raw = torch.linspace(-3, 3, 61, dtype=torch.float64)
    ref = {"linear": raw, "elu": F.elu(raw) + 1, "relu": F.relu(raw + 1), "relu_plus_one": F.relu(raw + 1e-3) + 1}[name]
    assert np.allclose(sizemap.activate(raw.numpy(), name), ref.numpy(), rtol=0, atol=1e-15)
    h = 1e-6
    fd = (sizemap.activate(raw.numpy() + h, name) - sizemap.activate(raw.numpy() - h, name)) / (2 * h)
    kink = np.abs(raw.numpy() + {"relu": 1.0, "relu_plus_one": 1e-3}.get(name, 10.0)) < 1e-5
    assert np.allclose(sizemap.activate_grad(raw.numpy(), name)[~kink], fd[~kink], atol=1e-6)


# ---- the package's torch formulation against the closed form (CPU) ------------------------------------------
@pytest.mark.parametrize("mode,channels", MODES)
def test_torch_formulation_matches_the_closed_form(mode, channels):
    size = _varying(channels, 7).requires_grad_(True)
    off = offsets_from_size_map(size, mode, KERNEL, DILATION)
    exp = sizemap.offsets(size.detach().numpy(), mode, KERNEL, DILATION)
    assert off.shape == exp.shape
    assert np.array_equal(off.detach().numpy(), exp)
    go = torch.randn(off.shape, generator=torch.Generator().manual_seed(8), dtype=torch.float64)
    off.backward(go)
    assert np.allclose(size.grad.numpy(), sizemap.offsets_backward(go.numpy(), mode, KERNEL, DILATION), rtol=1e-12, atol=1e-12)


def test_operator_package_call_convention_infers_the_mode():
    # dconv_native/grid.py:62-80: no mode argument, the channel count selects it
    for mode, channels in (("xyz", 3), ("xy", 2), ("x", 1)):
        size = _varying(channels, 9)
        assert np.array_equal(offsets_from_size_map(size, (3, 3, 3), (1, 1, 1)).numpy(),
                              sizemap.offsets(size.numpy(), mode, (3, 3, 3), (1, 1, 1)))


# ---- the HIP kernels against the closed form (GPU) --------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("mode,channels", MODES)
@pytest.mark.parametrize("activation", ["linear", "elu", "relu", "relu_plus_one"])
def test_hip_size_map_kernels_match_the_closed_form(mode, channels, activation, dev):
    from d2conv3d_amd.grid import size_map_offsets
    g = torch.Generator().manual_seed(17)
    raw = torch.randn(2, channels, 3, 5, 6, generator=g) * 1.5
    rawd = raw.to(dev).requires_grad_(True)
    out = size_map_offsets(rawd, mode, KERNEL, DILATION, activation)
    r64 = raw.double().numpy()
    exp = sizemap.offsets(sizemap.activate(r64, activation), mode, KERNEL, DILATION)
    assert np.allclose(out.detach().cpu().double().numpy(), exp, rtol=1e-5, atol=1e-6)
    go = torch.randn(out.shape, generator=g)
    out.backward(go.to(dev))
    eg = sizemap.offsets_backward(go.double().numpy(), mode, KERNEL, DILATION) * sizemap.activate_grad(r64, activation)
    assert np.allclose(rawd.grad.cpu().double().numpy(), eg, rtol=1e-4, atol=1e-5 * max(1.0, np.abs(eg).max()))
