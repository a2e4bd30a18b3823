"""The Python layer's workspace: one tensor per (device, stream), grown on demand and shared by the calls on that
stream; results do not depend on it."""
import ctypes

import pytest
import torch

import d2conv3d_amd as d2c
from d2conv3d_amd import _lib, _ops
from oracle import cpu
from _util import assert_close, rel_l2
from test_gpu_tiled import make

pytestmark = pytest.mark.gpu


def _step(ts, gout, geo):
    for t in ts:
        if t is not None:
            t.grad = None
    out = d2c.deform_conv3d(*ts, *geo[:3], geo[3], geo[4])
    out.backward(gout)
    return out.detach().clone(), [t.grad.clone() for t in ts if t is not None]


def test_calls_on_a_stream_share_one_workspace(dev):
    (x, off, m, w, b), gout, geo = make("c128_G2_o96", torch.float32, seed=3)
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
    gout = gout.to(dev)
    _ops.config.set_workspace_caching(False)
    e_out, e_grads = _step(ts, gout, geo)
    assert _ops.config.cached_workspace_bytes() == {}
    _ops.config.set_workspace_caching(True)
    try:
        out1, grads1 = _step(ts, gout, geo)
        cached = _ops.config.cached_workspace_bytes()
        assert len(cached) == 1 and next(iter(cached.values())) > 0
        ptr = next(iter(_ops._WS_CACHE.values())).data_ptr()
        out2, grads2 = _step(ts, gout, geo)              # same sizes: the same tensor again
        assert _ops.config.cached_workspace_bytes() == cached
        assert next(iter(_ops._WS_CACHE.values())).data_ptr() == ptr
        # a smaller problem afterwards reuses it, a larger one grows it
        (xs, offs, ms, w_s, bs), gs, geos = make("c64_tail", torch.float32, seed=4)
        tss = [t.to(dev).requires_grad_(True) if t is not None else None for t in (xs, offs, ms, w_s, bs)]
        _step(tss, gs.to(dev), geos)
        assert next(iter(_ops.config.cached_workspace_bytes().values())) >= next(iter(cached.values()))
        out3, grads3 = _step(ts, gout, geo)
        for out, grads in ((out1, grads1), (out2, grads2), (out3, grads3)):
            assert_close(out, e_out, 1e-5, 1e-6, "out")
            for i, (g, e) in enumerate(zip(grads, e_grads)):
                # (atomics in the weight gradient: sums in another order)
                assert_close(g, e, 1e-4, 1e-5 * max(1.0, e.abs().max().item()), f"grad{i}")
        # another stream gets a workspace of its own
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            _step(ts, gout, geo)
        torch.cuda.current_stream().wait_stream(side)
        assert len(_ops.config.cached_workspace_bytes()) == 2
    finally:
        _ops.config.release_workspaces()
    assert _ops.config.cached_workspace_bytes() == {}


def test_backward_flags_of_the_description_size_the_workspace_and_choose_the_path(dev):
    """d2c_conv3d_desc::backward_flags: the workspace query and the call read the field from the description they
    get (no process-wide state involved), every setting gives the oracle's gradients, and the settings that exist
    to save memory ask for less of it."""
    lib = _lib.load()
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make("c256_G4_o128", torch.bfloat16, seed=11)
    N, Cin, D, H, W = x.shape
    Cout = w.shape[0]
    need = {}
    for name, flags in (("default", 0), ("in_place", _lib.BWD_GW_IN_PLACE), ("resample", _lib.BWD_GW_RESAMPLE),
                        ("slices2", _lib.bwd_slices(2)), ("slices4", _lib.bwd_slices(4))):
        desc = _lib.Conv3dDesc(N, Cin, Cout, D, H, W, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, groups, G, D, H, W,
                               _lib.D2C_BF16, _lib.D2C_F32, 0, 1.0, 7, flags)
        need[name] = lib.d2c_conv3d_backward_workspace_bytes(ctypes.byref(desc))
        assert need[name] > 0
    assert need["in_place"] < need["default"] and need["resample"] < need["default"]
    assert need["slices4"] < need["slices2"] < need["default"]
    bad = _lib.Conv3dDesc(N, Cin, Cout, D, H, W, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, groups, G, D, H, W,
                          _lib.D2C_BF16, _lib.D2C_F32, 0, 1.0, 7, 1 << 20)
    assert lib.d2c_conv3d_check(ctypes.byref(bad)) != 0 and "backward_flags" in _lib.last_error()
    eg = cpu.conv3d_backward(gout.float(), x.float(), off, m, w.float(), True, s, p, d, groups, G)
    _ops.config.set_workspace_caching(False)       # every call gets a workspace of exactly the size it asks for
    try:
        for kw in (dict(), dict(backward_memory="in_place"), dict(backward_memory="resample"), dict(backward_slices=2),
                   dict(backward_slices=4), dict(backward_memory="resample", backward_slices=2)):
            ts = [t.to(dev).requires_grad_(True) for t in (x, off, m, w, b)]
            d2c.deform_conv3d(*ts, s, p, d, groups, G, **kw).backward(gout.to(dev))
            for n, t, e in zip(("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias"), ts, eg):
                assert rel_l2(t.grad, e) < 2e-2, (kw, n, rel_l2(t.grad, e))
    finally:
        _ops.config.set_workspace_caching(True)
        _ops.config.release_workspaces()
