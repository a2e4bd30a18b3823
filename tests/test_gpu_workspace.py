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


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_prepared_region_gives_the_same_results(dtype, dev):
    """d2c_conv3d_forward_prepared / _backward_prepared through DeformConv3d.reuse_prepared: the channels-last
    input and the re-ordered weights kept in a buffer of the layer.  Every call must return what the plain calls
    return (the same kernels on the same operands: equal up to the order in which partial sums are added with
    atomics, i.e. a few units in the last place): the first call (nothing held yet), a second step with unchanged weights (forward weights and,
    in the backward call, input and backward weights reused), a step after the weights changed, two forward
    calls before their backward calls (the second forward call takes the buffer, so the first backward call must
    lay its input out again), and a call at another size."""
    from d2conv3d_amd.deform_conv import DeformConv3d
    torch.manual_seed(23)
    C, O, G = 128, 192, 2
    plain = DeformConv3d(C, O, 3, padding=1, offset_groups=G).to(dev, dtype)
    kept = DeformConv3d(C, O, 3, padding=1, offset_groups=G).to(dev, dtype)
    kept.load_state_dict(plain.state_dict())
    kept.reuse_prepared = True

    def data(dims, seed):
        g = torch.Generator().manual_seed(seed)
        x = torch.randn(1, C, *dims, generator=g).to(dev, dtype)
        off = (torch.randn(1, G * 81, *dims, generator=g) * 1.5).to(dev)
        m = torch.sigmoid(torch.randn(1, G * 27, *dims, generator=g)).to(dev)
        gout = torch.randn(1, O, *dims, generator=g).to(dev, dtype)
        return x, off, m, gout

    def step(layer, x, off, m, gout):
        layer.zero_grad()
        ts = [t.clone().requires_grad_(True) for t in (x, off, m)]
        y = layer(*ts)
        y.backward(gout)
        return [y.detach()] + [t.grad for t in ts] + [layer.weight.grad.clone(), layer.bias.grad.clone()]

    rtol = 2e-6 if dtype == torch.float32 else 8e-3      # (one unit in the last place of bfloat16 is 2^-8)

    def same(a, b, what):
        for i, (u, v) in enumerate(zip(a, b)):
            assert_close(u, v, rtol, rtol * max(1.0, v.abs().max().item()), f"{what} [{i}]")

    d1, d2 = data((4, 9, 10), 1), data((4, 9, 10), 2)
    same(step(kept, *d1), step(plain, *d1), "first call")
    assert kept._prepared.buf is not None and kept._prepared.buf.numel() > 0
    same(step(kept, *d2), step(plain, *d2), "second call, weights unchanged")
    with torch.no_grad():
        for layer in (plain, kept):
            layer.weight.mul_(1.5)
    same(step(kept, *d1), step(plain, *d1), "after the weights changed")
    # two forward calls, then their backward calls in reverse order
    res = {}
    for name, layer in (("kept", kept), ("plain", plain)):
        layer.zero_grad()
        ta = [t.clone().requires_grad_(True) for t in d1[:3]]
        tb = [t.clone().requires_grad_(True) for t in d2[:3]]
        ya, yb = layer(*ta), layer(*tb)
        yb.backward(d2[3])
        ya.backward(d1[3])
        res[name] = [ya.detach(), yb.detach()] + [t.grad for t in ta + tb]
    same(res["kept"], res["plain"], "two forward calls before their backward calls")
    d3 = data((3, 12, 13), 3)
    same(step(kept, *d3), step(plain, *d3), "another size")


@pytest.mark.parametrize("name", ["c128_G2_o96", "c64_stride_dil", "c64_o320_nomask", "c128_groups2_G1"])
def test_float32_backward_on_split_operands(name, dev):
    """D2C_BWD_F32_SPLIT: every backward matrix kernel of a float32 problem on two-term bfloat16 operands, like the
    forward kernels.  Against the float64 oracle: every gradient within 2e-5 of its tensor's scale (the operands
    keep 16 of float32's 24 significant bits: about 4e-6 relative in a long sum, against 1e-7 for plain float32).
    By default only the grad-column product takes such operands (grad_input, grad_offset and grad_mask then sit at
    the same 4e-6), and grad_weight / grad_bias, on float32 instructions, an order of magnitude closer."""
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make(name, torch.float32, seed=13)
    dd = lambda t: t.double() if t is not None else None
    eg = cpu.conv3d_backward(dd(gout), dd(x), dd(off), dd(m), dd(w), b is not None, s, p, d, groups, G)
    errs = {}
    # (with grad_weight from the kernel that samples again: over sampled columns, the forward call's or the backward
    # pass's own, the product keeps float32's accuracy whatever the flag says)
    before = _ops.config.keep_columns()
    _ops.config.set_keep_columns(False)
    _ops.set_grad_weight_mode("resample")
    try:
        for split in (True, False):
            ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
            d2c.deform_conv3d(*ts, s, p, d, groups, G, backward_f32_split=split).backward(gout.to(dev))
            errs[split] = []
            for n, t, e in zip(("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias"), ts, eg):
                if t is None:
                    continue
                err = ((t.grad.double().cpu() - e).abs().max() / e.abs().max()).item()
                errs[split].append(err)
                assert err < (2e-5 if (split or n in ("grad_input", "grad_offset", "grad_mask")) else 2e-6), (name, n, split, err)
    finally:
        _ops.set_grad_weight_mode("columns")
        _ops.config.set_keep_columns(before["on"], before["max_bytes"])
    assert errs[True][-2 if b is not None else -1] > errs[False][-2 if b is not None else -1]   # (grad_weight: the flag did change the arithmetic)
