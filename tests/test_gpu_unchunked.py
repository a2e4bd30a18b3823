"""bfloat16 problems whose channel counts the bfloat16 matrix-core kernels cannot chunk (64 channels per weight group
and per offset group) but the float32 ones can (32): the functional API runs them in float32 and rounds the result
(d2conv3d_amd/deform_conv.py::_float32_for_unchunked_bfloat16), instead of leaving them to the direct kernels, which
are two to three orders of magnitude slower.  Expected values: the CPU oracle on the same bfloat16 tensors."""
import ctypes

import pytest
import torch

import d2conv3d_amd as d2c
from d2conv3d_amd import _lib, _ops
from oracle import cpu
from _util import assert_close, rel_l2

pytestmark = pytest.mark.gpu

# name: (N, Cin, Cout, dims, groups, G, sigma)
SHAPES = {
    "c64_G2_32_per_offset_group": (1, 64, 64, (4, 9, 10), 1, 2, 1.5),
    "c96_one_and_a_half_chunks": (2, 96, 96, (3, 7, 8), 1, 1, 2.0),
    "c128_groups2_G4": (1, 128, 128, (3, 6, 7), 2, 4, 1.0),
}


@pytest.mark.parametrize("name", list(SHAPES))
def test_unchunked_bfloat16_runs_on_the_float32_matrix_kernels(name, dev):
    N, Cin, Cout, dims, groups, G, sig = SHAPES[name]
    g = torch.Generator().manual_seed(8100)
    x = torch.randn(N, Cin, *dims, generator=g).bfloat16()
    w = ((torch.rand(Cout, Cin // groups, 3, 3, 3, generator=g) * 2 - 1) / (Cin // groups * 27) ** 0.5).bfloat16()
    b = ((torch.rand(Cout, generator=g) * 2 - 1) * 0.1).bfloat16()
    off = torch.randn(N, G * 81, *dims, generator=g) * sig
    m = torch.sigmoid(torch.randn(N, G * 27, *dims, generator=g))
    gout = torch.randn(N, Cout, *dims, generator=g).bfloat16()
    f = lambda t: t.float()
    e_out = cpu.conv3d_forward(f(x), off, m, f(w), f(b), 1, 1, 1, groups, G)
    eg = cpu.conv3d_backward(f(gout), f(x), off, m, f(w), True, 1, 1, 1, groups, G)
    ts = [t.to(dev).requires_grad_(True) for t in (x, off, m, w, b)]
    args = (ts[0], ts[1], ts[2], ts[3], (1, 1, 1), (1, 1, 1), (1, 1, 1), groups, G)
    assert _ops.conv3d_algo(*args) == "generic" and _ops.conv3d_algo(*args, as_dtype=torch.float32) == "mfma"
    lib = _lib.load()
    lib.d2c_profile_reset()
    lib.d2c_profile_enable(1)
    try:
        out = d2c.deform_conv3d(*ts, 1, 1, 1, groups, G)
        out.backward(gout.to(dev))
        torch.cuda.synchronize()
    finally:
        lib.d2c_profile_enable(0)
    tot, cnt = ctypes.c_double(0), ctypes.c_int(0)
    lib.d2c_profile_read(_lib.PROF_FWD, ctypes.byref(tot), ctypes.byref(cnt))
    kernel = lib.d2c_profile_kernel_name(_lib.PROF_FWD).decode()
    lib.d2c_profile_reset()
    assert cnt.value >= 1 and kernel.startswith("tiled_fwd"), (cnt.value, kernel)
    assert out.dtype == torch.bfloat16 and ts[0].grad.dtype == torch.bfloat16 and ts[3].grad.dtype == torch.bfloat16
    assert_close(out, e_out, 1e-2, 1e-2 * e_out.abs().max().item(), f"{name} out")
    for n, t, e in zip(("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias"), ts, eg):
        assert rel_l2(t.grad, e) < 1e-2, (name, n, rel_l2(t.grad, e))


def test_unchunked_bfloat16_with_the_size_map_in_the_operator(dev):
    """The same for the dynamic-dilation entry (96 channels: one and a half bfloat16 chunks): equal to the two-step
    path on float32 copies of the tensors, rounded."""
    from d2conv3d_amd.deform_conv import deform_conv3d_sized
    g = torch.Generator().manual_seed(8200)
    N, C, dims = 1, 96, (3, 8, 9)
    x = torch.randn(N, C, *dims, generator=g).bfloat16().to(dev)
    w = ((torch.rand(C, C, 3, 3, 3, generator=g) * 2 - 1) / (C * 27) ** 0.5).bfloat16().to(dev)
    size = (torch.rand(N, 3, *dims, generator=g) * 2 + 0.5).to(dev)
    m = torch.sigmoid(torch.randn(N, 27, *dims, generator=g)).to(dev)
    gout = torch.randn(N, C, *dims, generator=g).bfloat16().to(dev)
    res = []
    for cast in (lambda t: t, lambda t: t.float()):
        ts = [cast(t).clone().requires_grad_(True) for t in (x, size, m, w)]
        out = deform_conv3d_sized(ts[0], ts[1], ts[2], ts[3], None, "xyz", "linear", padding=(1, 1, 1))
        out.backward(cast(gout))
        res.append([out.detach()] + [t.grad for t in ts])
    assert res[0][0].dtype == torch.bfloat16 and res[0][1].dtype == torch.bfloat16
    for i, (a, e) in enumerate(zip(*res)):
        assert rel_l2(a, e) < 4e-3, (i, rel_l2(a, e))


@pytest.mark.parametrize("dtype,cin", [(torch.float32, 48), (torch.bfloat16, 40), (torch.float32, 80)])
def test_channel_counts_off_the_chunking_are_padded_with_zero_channels(dtype, cin, dev):
    """One weight group, one offset group, a channel count that is no multiple of the chunk but fills at least half
    of its last one: input and weight get zero channels up to the next chunk and the matrix-core kernels run; results
    and gradients (of the original shapes) against the oracle."""
    N, Cout, dims = 1, 40, (3, 8, 9)
    g = torch.Generator().manual_seed(8300 + cin)
    x = torch.randn(N, cin, *dims, generator=g).to(dtype)
    w = ((torch.rand(Cout, cin, 3, 3, 3, generator=g) * 2 - 1) / (cin * 27) ** 0.5).to(dtype)
    b = ((torch.rand(Cout, generator=g) * 2 - 1) * 0.1).to(dtype)
    off = torch.randn(N, 81, *dims, generator=g) * 1.5
    m = torch.sigmoid(torch.randn(N, 27, *dims, generator=g))
    gout = torch.randn(N, Cout, *dims, generator=g).to(dtype)
    f = lambda t: t.float()
    e_out = cpu.conv3d_forward(f(x), off, m, f(w), f(b), 1, 1, 1, 1, 1)
    eg = cpu.conv3d_backward(f(gout), f(x), off, m, f(w), True, 1, 1, 1, 1, 1)
    ts = [t.to(dev).requires_grad_(True) for t in (x, off, m, w, b)]
    lib = _lib.load()
    lib.d2c_profile_reset()
    lib.d2c_profile_enable(1)
    try:
        out = d2c.deform_conv3d(*ts, 1, 1, 1, 1, 1)
        out.backward(gout.to(dev))
        torch.cuda.synchronize()
    finally:
        lib.d2c_profile_enable(0)
    tot, cnt = ctypes.c_double(0), ctypes.c_int(0)
    lib.d2c_profile_read(_lib.PROF_FWD, ctypes.byref(tot), ctypes.byref(cnt))
    kernel = lib.d2c_profile_kernel_name(_lib.PROF_FWD).decode()
    lib.d2c_profile_reset()
    assert cnt.value >= 1 and kernel.startswith("tiled_fwd"), (cnt.value, kernel)
    assert out.dtype == dtype and ts[0].grad.shape == x.shape and ts[3].grad.shape == w.shape
    tol = 1e-2 if dtype == torch.bfloat16 else 2e-5
    assert rel_l2(out, e_out) < tol
    for n, t, e in zip(("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias"), ts, eg):
        assert rel_l2(t.grad, e) < tol, (dtype, cin, n, rel_l2(t.grad, e))
