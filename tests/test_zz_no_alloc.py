"""The allocation-free forward entry point (d2c_conv3d_forward_static, include/d2conv.h) against
d2c_conv3d_forward on the same inputs, through the C ABI: two calls in a row on one GPU, the second with a
smaller input (the static workspace still holds what the first call left there), float32 within 1e-4 relative /
1e-5 absolute, bfloat16 within 2e-2 of the tensor's scale; both results are also held to the CPU oracle.
A description that needs more workspace than the static array holds must be refused."""
import ctypes

import pytest
import torch

from d2conv3d_amd import _lib
from oracle import cpu
from _util import assert_close, rel_l2

pytestmark = pytest.mark.gpu

# (N, Cin, Cout, (D, H, W), groups, G, sigma): the matrix-core kernel that shares out the steps of its last round
# (fp32 partial sums in the workspace, cleared by the library), then a small problem, then a channel-separated one
CASES = [
    (1, 64, 320, (7, 35, 34), 1, 1, 1.5),
    (2, 64, 64, (4, 6, 7), 1, 1, 1.0),
    (2, 64, 64, (4, 6, 7), 64, 1, 1.5),
]


def _inputs(case, dtype, seed):
    N, Cin, Cout, dims, groups, G, sig = case
    g = torch.Generator().manual_seed(4000 + seed)
    x = torch.randn(N, Cin, *dims, generator=g)
    fan_in = Cin // groups * 27
    w = (torch.rand(Cout, Cin // groups, 3, 3, 3, generator=g) * 2 - 1) / fan_in ** 0.5
    b = (torch.rand(Cout, generator=g) * 2 - 1) / fan_in ** 0.5
    off = torch.randn(N, G * 81, *dims, generator=g) * sig
    m = torch.sigmoid(torch.randn(N, G * 27, *dims, generator=g))
    if dtype == torch.bfloat16:
        x, w, b = x.bfloat16(), w.bfloat16(), b.bfloat16()
    return x, off, m, w, b


def _desc(case, dtype):
    N, Cin, Cout, (D, H, W), groups, G, _ = case
    dt = _lib.D2C_BF16 if dtype == torch.bfloat16 else _lib.D2C_F32
    return _lib.Conv3dDesc(N, Cin, Cout, D, H, W, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, groups, G, D, H, W,
                           dt, _lib.D2C_F32, _lib.EPILOGUE_NONE, 1.0)


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_static_workspace_forward_matches_the_workspace_entry_point(dtype, dev):
    lib = _lib.load()
    assert lib.d2c_static_workspace_bytes() == 32 << 20
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    for i, case in enumerate(CASES):
        print(f"static-workspace forward: case {i} {case} {dtype}", flush=True)
        host = _inputs(case, dtype, i)
        x, off, m, w, b = (t.to(dev) for t in host)
        desc = _desc(case, dtype)
        N, Cout, dims = case[0], case[2], case[3]
        need = lib.d2c_conv3d_forward_workspace_bytes(ctypes.byref(desc))
        assert 0 < need <= lib.d2c_static_workspace_bytes()
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        ref = torch.empty((N, Cout, *dims), dtype=dtype, device=dev)
        out = torch.full_like(ref, float("nan"))
        _lib.check(lib.d2c_conv3d_forward(ctypes.byref(desc), _p(x), _p(off), _p(m), _p(w), _p(b), _p(ref), _p(ws),
                                          need, stream), "d2c_conv3d_forward")
        _lib.check(lib.d2c_conv3d_forward_static(ctypes.byref(desc), _p(x), _p(off), _p(m), _p(w), _p(b), _p(out),
                                                 stream), "d2c_conv3d_forward_static")
        torch.cuda.synchronize(dev)
        # the call itself takes no device memory: once more (everything it could set up lazily is set up now) with
        # the free memory of the device read on both sides
        free_before = torch.cuda.mem_get_info(dev)[0]
        _lib.check(lib.d2c_conv3d_forward_static(ctypes.byref(desc), _p(x), _p(off), _p(m), _p(w), _p(b), _p(out),
                                                 stream), "d2c_conv3d_forward_static (second call)")
        torch.cuda.synchronize(dev)
        assert torch.cuda.mem_get_info(dev)[0] == free_before, "the static-workspace call changed the free device memory"
        xh, _, _, wh, bh = host
        exp = cpu.conv3d_forward(xh.float(), off.cpu(), m.cpu(), wh.float(), bh.float(), 1, 1, 1, case[4], case[5])
        if dtype == torch.float32:
            assert_close(out, ref, 1e-4, 1e-5, f"case {i}: static vs workspace entry point")
            assert_close(out, exp, 1e-4, 1e-5, f"case {i}: static vs oracle")
        else:
            scale = exp.abs().max().item()
            assert_close(out, ref, 2e-2, 2e-2 * scale, f"case {i}: static vs workspace entry point")
            assert rel_l2(out, exp) < 2e-2


def test_static_workspace_forward_refuses_what_does_not_fit(dev):
    lib = _lib.load()
    case = (2, 512, 512, (8, 30, 54), 1, 8, 2.0)     # needs 94 MB of workspace
    desc = _desc(case, torch.bfloat16)
    assert lib.d2c_conv3d_forward_workspace_bytes(ctypes.byref(desc)) > lib.d2c_static_workspace_bytes()
    t = torch.zeros(16, device=dev)                  # never read: the call returns before it launches anything
    rc = lib.d2c_conv3d_forward_static(ctypes.byref(desc), _p(t), _p(t), _p(t), _p(t), _p(t), _p(t), None)
    assert rc == 3, rc                               # D2C_ERR_WORKSPACE
    assert "static" in _lib.last_error()
