"""GPU parity of the tiled kernel families (matrix-core implicit GEMM,
depthwise) against the CPU oracle, at sizes the oracle finishes in seconds.

float32: 1e-4 relative / 1e-5 absolute (scaled by the tensor's magnitude for
the gradients, which are long sums).  bfloat16: the oracle consumes the
bfloat16-rounded tensors up-cast to float32; results must agree within 2e-2
relative (L2 over the tensor, and element-wise against the tensor's scale).
"""
import pytest
import torch

import d2conv3d_amd as d2c
from d2conv3d_amd import _lib, _ops
from oracle import cpu
from _util import assert_close, rel_l2

pytestmark = pytest.mark.gpu

# name: (N, Cin, Cout, (D,H,W), k, stride, pad, dil, groups, G, bias, mask, offset_sigma)
SHAPES = {
    "c64_g1": (2, 64, 64, (4, 6, 7), 3, 1, 1, 1, 1, 1, True, True, 1.0),
    "c128_G2_o96": (1, 128, 96, (3, 6, 9), 3, 1, 1, 1, 1, 2, True, True, 2.0),
    "c128_groups2": (2, 128, 192, (3, 5, 6), 3, 1, 1, 1, 2, 2, False, True, 1.5),
    # an offset group that spans both weight groups: the grad-column kernel cannot keep such a group on chip, the
    # direct kernels compute grad_input / grad_offset / grad_mask beside the matrix-core grad_weight kernel
    "c128_groups2_G1": (1, 128, 64, (3, 5, 6), 3, 1, 1, 1, 2, 1, True, True, 1.5),
    "c64_o320_nomask": (1, 64, 320, (3, 5, 5), 3, 1, 1, 1, 1, 1, True, False, 1.0),
    "c64_o600": (1, 64, 600, (2, 5, 5), (1, 3, 3), 1, (0, 1, 1), 1, 1, 1, True, True, 1.0),
    "c64_stride_dil": (2, 64, 64, (5, 9, 8), 3, (1, 2, 1), (1, 2, 2), (1, 2, 1), 1, 1, True, True, 1.0),
    "c64_tail": (3, 64, 32, (3, 7, 7), 3, 1, 1, 1, 1, 1, True, True, 1.0),   # N*P = 441: ragged last tile
    # wide weight groups with many position tiles: the forward kernel that moves corner rows by DMA
    "c64_o320_big": (1, 64, 320, (7, 35, 34), 3, 1, 1, 1, 1, 1, True, True, 1.5),       # N*P = 8330: ragged
    "c128_groups2_o640_big": (1, 128, 640, (4, 32, 33), 3, 1, 1, 1, 2, 2, True, True, 2.0),
    "c64_o200_big": (1, 64, 200, (7, 35, 34), 3, 1, 1, 1, 1, 1, True, True, 1.5),       # 256-wide output tile
    # wide weight groups with a handful of position tiles but more than a thousand steps in all: the same kernel, every
    # work item cut into step ranges
    "c256_o320_few_tiles": (1, 256, 320, (4, 12, 16), 3, 1, 1, 1, 1, 1, True, True, 1.5),   # N*P = 768: 12 tiles
    "c512_groups2_o512_few_tiles": (2, 512, 512, (3, 8, 9), 3, 1, 1, 1, 2, 2, True, True, 1.0),   # 7 tiles x 2 groups
    # narrow weight groups with more than 160 position tiles: the same kernel, most of its output tile empty
    "c64_o96_many_tiles": (1, 64, 96, (9, 34, 35), 3, 1, 1, 1, 1, 1, True, True, 1.5),  # N*P = 10710: ragged
    "c128_groups2_o48_many_tiles": (1, 128, 48, (8, 32, 21), 3, 1, 1, 1, 2, 2, True, False, 1.0),   # 84 tiles x 2 groups
    # the same kernel's schedule: three output tiles per position tile (399 work items on 256 compute units: one
    # whole round, the rest cut into step ranges), two weight groups with few position tiles (all items cut)
    "c64_o1100_big": (1, 64, 1100, (7, 35, 35), 3, 1, 1, 1, 1, 1, True, True, 1.5),
    "c128_groups2_o1280_mid": (1, 128, 1280, (5, 41, 41), (1, 3, 3), 1, (0, 1, 1), 1, 2, 2, True, True, 1.0),
    # weight groups of two and four channel chunks (bfloat16: grad_weight as a matrix product over the sampled
    # columns, two chunks per workgroup), ragged last position tile, all 512 / some of the output channels of a pass
    "c256_G2_o512_tail": (1, 256, 512, (3, 7, 7), 3, 1, 1, 1, 1, 2, True, True, 1.5),
    "c256_groups2_G4_o384": (2, 256, 384, (3, 5, 6), 3, 1, 1, 1, 2, 4, False, False, 1.5),
    # four chunks per weight group, 200 output channels: half of the grad-weight product's wavefronts have no output
    # channels and only move column tiles; the last slice of output channels is ragged
    "c256_G1_o200": (2, 256, 200, (3, 6, 7), 3, 1, 1, 1, 1, 1, True, True, 1.5),
    # several offset groups of one or two channel chunks with 128 .. 512 output channels: the bfloat16 backward
    # pass runs slice by slice over the offset groups (test_backward_in_slices_over_the_offset_groups)
    "c256_G4_o128": (1, 256, 128, (3, 6, 7), 3, 1, 1, 1, 1, 4, True, True, 1.5),
    "c384_G6_o384_nomask": (2, 384, 384, (2, 5, 6), 3, 1, 1, 1, 1, 6, False, False, 1.5),
    "c384_G3_o384": (1, 384, 384, (3, 5, 7), 3, 1, 1, 1, 1, 3, True, True, 2.0),
    # channel-separated (groups == Cin == Cout)
    "dw64": (2, 64, 64, (4, 6, 7), 3, 1, 1, 1, 64, 1, True, True, 1.5),
    "dw96_G3_nomask": (1, 96, 96, (3, 5, 9), 3, 1, 1, 1, 96, 3, False, False, 1.0),
    "dw1100_stride": (1, 1100, 1100, (3, 6, 6), (1, 3, 3), (1, 2, 1), (0, 1, 1), 1, 1100, 1, True, True, 1.0),
    "dw32_45taps": (2, 32, 32, (3, 7, 5), (3, 5, 3), 1, (1, 2, 1), 1, 32, 2, True, True, 1.5),
}
ALGO = {k: ("depthwise" if k.startswith("dw") else "mfma") for k in SHAPES}


def make(name, dtype, seed=0):
    N, Cin, Cout, dims, k, s, p, d, groups, G, bias, mask, sig = SHAPES[name]
    t3 = lambda v: (v,) * 3 if isinstance(v, int) else tuple(v)
    k, s, p, d = t3(k), t3(s), t3(p), t3(d)
    od = tuple((n + 2 * pp - (dd * (kk - 1) + 1)) // ss + 1 for n, kk, ss, pp, dd in zip(dims, k, s, p, d))
    K = k[0] * k[1] * k[2]
    g = torch.Generator().manual_seed(1000 + seed)
    rn = lambda *sh: torch.randn(*sh, generator=g)
    x = rn(N, Cin, *dims)
    fan_in = Cin // groups * K
    w = (torch.rand(Cout, Cin // groups, *k, generator=g) * 2 - 1) / fan_in ** 0.5
    b = (torch.rand(Cout, generator=g) * 2 - 1) / fan_in ** 0.5 if bias else None
    off = rn(N, G * 3 * K, *od) * sig
    m = torch.sigmoid(rn(N, G * K, *od)) if mask else None
    gout = rn(N, Cout, *od)
    if dtype == torch.bfloat16:
        x, w, gout = x.bfloat16(), w.bfloat16(), gout.bfloat16()
        b = b.bfloat16() if b is not None else None
    return (x, off, m, w, b), gout, (s, p, d, groups, G)


def f32(t):
    return t.float() if t is not None else None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", list(SHAPES))
def test_tiled_forward_backward(name, dtype, dev):
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make(name, dtype)
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
    assert _ops.conv3d_algo(ts[0], ts[1], ts[2], ts[3], s, p, d, groups, G) == ALGO[name]
    out = d2c.deform_conv3d(*ts, s, p, d, groups, G)
    exp = cpu.conv3d_forward(f32(x), off, m, f32(w), f32(b), s, p, d, groups, G)
    eg = cpu.conv3d_backward(f32(gout), f32(x), off, m, f32(w), b is not None, s, p, d, groups, G)
    out.backward(gout.to(dev))
    names = ("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias")
    if dtype == torch.float32:
        assert_close(out, exp, 1e-4, 1e-5, "forward")
        for n, t, e in zip(names, ts, eg):
            if t is not None:
                assert_close(t.grad, e, 1e-4, 1e-5 * max(1.0, e.abs().max().item()), n)
    else:
        assert out.dtype == torch.bfloat16
        assert rel_l2(out, exp) < 2e-2, rel_l2(out, exp)
        assert_close(out, exp, 2e-2, 2e-2 * exp.abs().max().item(), "forward")
        for n, t, e in zip(names, ts, eg):
            if t is not None:
                assert t.grad.dtype == t.dtype
                assert rel_l2(t.grad, e) < 2e-2, (n, rel_l2(t.grad, e))
                assert_close(t.grad, e, 2e-2, 2e-2 * e.abs().max().item(), n)


@pytest.mark.parametrize("name", ["c128_G2_o96", "c256_G2_o512_tail", "c256_groups2_G4_o384", "c256_G1_o200"])
@pytest.mark.parametrize("wanted", ["all", "w+offset", "w"])
def test_grad_weight_from_columns_matches_resampling(name, wanted, dev):
    # bfloat16 grad_weight two ways: as a matrix product over the sampled columns that the offset / mask gradient
    # kernel writes on its way (when that kernel runs: grad_offset or grad_mask wanted), or by sampling the input
    # again in the grad-weight kernel; both against the oracle
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make(name, torch.bfloat16, seed=5)
    eg = cpu.conv3d_backward(f32(gout), f32(x), off, m, f32(w), b is not None, s, p, d, groups, G)
    got = {}
    for mode in ("columns", "in_place", "resample"):
        _ops.set_grad_weight_mode(mode)
        try:
            ts = [t.to(dev) if t is not None else None for t in (x, off, m, w, b)]
            ts[3].requires_grad_(True)
            if wanted != "w":
                ts[1].requires_grad_(True)
            if wanted == "all":
                ts[0].requires_grad_(True)
                if ts[2] is not None:
                    ts[2].requires_grad_(True)
            d2c.deform_conv3d(*ts, s, p, d, groups, G).backward(gout.to(dev))
            got[mode] = ts[3].grad
        finally:
            _ops.set_grad_weight_mode("columns")
        assert rel_l2(got[mode], eg[3]) < 2e-2, (mode, rel_l2(got[mode], eg[3]))
        assert_close(got[mode], eg[3], 2e-2, 2e-2 * eg[3].abs().max().item(), f"grad_weight ({mode})")
        if wanted != "w":
            assert rel_l2(ts[1].grad, eg[1]) < 2e-2, mode
        if wanted == "all":
            assert rel_l2(ts[0].grad, eg[0]) < 2e-2, mode
            if ts[2] is not None:
                assert rel_l2(ts[2].grad, eg[2]) < 2e-2, mode
    # the two differ by the rounding of the columns to bfloat16 at most (both round them before the product)
    assert rel_l2(got["columns"], got["resample"].float().cpu()) < 1e-2
    assert rel_l2(got["in_place"], got["columns"].float().cpu()) < 1e-3


@pytest.mark.parametrize("name", ["c64_g1", "c128_G2_o96", "c256_groups2_G4_o384", "c256_G1_o200"])
def test_float32_grad_weight_from_columns_matches_resampling(name, dev):
    # float32 grad_weight on the plain calls (the forward call's columns not kept): as a matrix product over the float
    # columns that the offset / mask gradient kernel writes -- on three-term bfloat16 operands where the weight groups
    # hold sets of four 32-channel chunks, on the float32 matrix instruction otherwise -- or by sampling again; both
    # against the float64 oracle, to 3e-6 of the tensor's scale
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make(name, torch.float32, seed=6)
    dd = lambda t: t.double() if t is not None else None
    eg = cpu.conv3d_backward(dd(gout), dd(x), dd(off), dd(m), dd(w), b is not None, s, p, d, groups, G)
    before = _ops.config.keep_columns()
    _ops.config.set_keep_columns(False)
    got = {}
    try:
        for mode in ("columns", "resample"):
            _ops.set_grad_weight_mode(mode)
            ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
            d2c.deform_conv3d(*ts, s, p, d, groups, G).backward(gout.to(dev))
            got[mode] = ts[3].grad
            err = ((got[mode].double().cpu() - eg[3]).abs().max() / eg[3].abs().max()).item()
            assert err < 3e-6, (name, mode, err)
            assert rel_l2(ts[0].grad, eg[0]) < 1e-5, (name, mode, rel_l2(ts[0].grad, eg[0]))
    finally:
        _ops.set_grad_weight_mode("columns")
        _ops.config.set_keep_columns(before["on"], before["max_bytes"])
    assert rel_l2(got["columns"], got["resample"].cpu()) < 2e-6


@pytest.mark.parametrize("name,dtype", [("c64_o600", torch.bfloat16), ("c64_o1100_big", torch.bfloat16),
                                        ("c64_o320_nomask", torch.float32), ("c64_o600", torch.float32)])
def test_wide_weight_groups_stay_on_the_list_based_backward(name, dtype, dev):
    # Weight groups wider than one pass of the grad-column product (512 bfloat16 / 256 float32 output channels): the
    # passes' rows are added up and the backward pass stays on the product-only kernel, the offset / mask gradient
    # kernel and the owner kernel (the fused kernel with its atomic scatter per pass is an order of magnitude slower
    # at layer sizes).  Which kernels ran is read from the library's own instrumentation; the values against the oracle.
    import ctypes
    lib = _lib.load()
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make(name, dtype, seed=21)
    eg = cpu.conv3d_backward(f32(gout), f32(x), off, m, f32(w), b is not None, s, p, d, groups, G)
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
    out = d2c.deform_conv3d(*ts, s, p, d, groups, G)
    lib.d2c_profile_reset()
    lib.d2c_profile_enable(1)
    try:
        out.backward(gout.to(dev))
        torch.cuda.synchronize()
    finally:
        lib.d2c_profile_enable(0)
    ran = {}
    for kid in (_lib.PROF_BWD_DATA, _lib.PROF_GX_OWNER, _lib.PROF_BWD_AUX):
        tot, cnt = ctypes.c_double(0), ctypes.c_int(0)
        lib.d2c_profile_read(kid, ctypes.byref(tot), ctypes.byref(cnt))
        ran[kid] = (cnt.value, lib.d2c_profile_kernel_name(kid).decode())
    lib.d2c_profile_reset()
    assert ran[_lib.PROF_BWD_DATA][0] >= 2 and ran[_lib.PROF_BWD_DATA][1] in ("tiled_bwd_col32_kernel", "tiled_bwd_col_kernel"), ran
    assert ran[_lib.PROF_GX_OWNER][0] >= 1 and ran[_lib.PROF_BWD_AUX][0] >= 1, ran
    tol = 2e-2 if dtype == torch.bfloat16 else 2e-5
    for n, t, e in zip(("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias"), ts, eg):
        if t is not None:
            assert rel_l2(t.grad, e) < tol, (name, n, rel_l2(t.grad, e))


@pytest.mark.parametrize("name", ["c256_G2_o512_tail", "c256_G4_o128", "c384_G6_o384_nomask", "c384_G3_o384"])
@pytest.mark.parametrize("wanted", ["all", "x", "w+offset", "x+w"])
def test_backward_in_slices_over_the_offset_groups(name, wanted, dev):
    # The bfloat16 backward pass slice by slice over the offset groups (buffers of grad-column rows and sampled columns
    # for one slice / one block of slices): every number of slices against the oracle, and against the pass over all
    # groups at once.  The cases cover slices of one and two groups, blocks of sampled columns that span two slices
    # (one chunk per group), a last slice shorter than the others, and a grad_weight that samples again (no offset /
    # mask gradient wanted) beside sliced grad_input.
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make(name, torch.bfloat16, seed=9)
    eg = cpu.conv3d_backward(f32(gout), f32(x), off, m, f32(w), b is not None, s, p, d, groups, G)
    need = {"all": (1, 1, 1, 1, 1), "x": (1, 0, 0, 0, 0), "w+offset": (0, 1, 0, 1, 0), "x+w": (1, 0, 0, 1, 1)}[wanted]
    names = ("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias")
    res = {}
    for n in (1, 2, 3, G, 0):
        _ops.set_backward_slices(n)
        try:
            ts = [t.to(dev).requires_grad_(bool(r)) if t is not None else None for t, r in zip((x, off, m, w, b), need)]
            d2c.deform_conv3d(*ts, s, p, d, groups, G).backward(gout.to(dev))
            res[n] = [t.grad if (t is not None and r) else None for t, r in zip(ts, need)]
        finally:
            _ops.set_backward_slices(0)
        for nm, a, e in zip(names, res[n], eg):
            if a is not None:
                assert rel_l2(a, e) < 2e-2, (n, nm, rel_l2(a, e))
                assert_close(a, e, 2e-2, 2e-2 * e.abs().max().item(), f"{nm} in {n} slices")
    for n in (2, 3, G, 0):
        for nm, a, e in zip(names, res[n], res[1]):
            if a is not None:
                assert rel_l2(a, e.float().cpu()) < 1e-3, (n, nm)


@pytest.mark.parametrize("name", ["c128_G2_o96", "c64_stride_dil", "c64_tail", "dw64", "dw96_G3_nomask",
                                  "dw1100_stride", "dw32_45taps"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_grad_input_by_atomics_matches_lists(name, dtype, dev):
    # the tiled and depthwise backward have two ways to build grad_input; both must agree with the oracle
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make(name, dtype, seed=7)
    eg = cpu.conv3d_backward(f32(gout), f32(x), off, m, f32(w), b is not None, s, p, d, groups, G)
    grads = {}
    for mode in ("atomics", "lists"):
        _ops.set_grad_input_mode(mode)
        try:
            ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
            d2c.deform_conv3d(*ts, s, p, d, groups, G).backward(gout.to(dev))
            grads[mode] = ts[0].grad
        finally:
            _ops.set_grad_input_mode("lists")
        if dtype == torch.float32:
            assert_close(grads[mode], eg[0], 1e-4, 1e-5 * max(1.0, eg[0].abs().max().item()), f"grad_input ({mode})")
        else:
            assert rel_l2(grads[mode], eg[0]) < 2e-2, mode


@pytest.mark.parametrize("name", ["c128_G2_o96", "c64_stride_dil", "c64_tail", "dw64", "dw96_G3_nomask"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cap", [2, 8])
@pytest.mark.parametrize("wanted", ["x", "x+aux", "all"])
def test_grad_input_when_sample_lists_overflow(name, dtype, cap, wanted, dev):
    # lists of tiny capacity: most samples take the overflow path (atomics after the owner kernel).  The samples
    # are filed by the offset / mask gradient kernel when that runs ("x+aux", "all"), else by a pass of their
    # own ("x")
    want_aux = wanted != "x"
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make(name, dtype, seed=11)
    eg = cpu.conv3d_backward(f32(gout), f32(x), off, m, f32(w), b is not None, s, p, d, groups, G)
    _ops.set_grad_input_mode(cap)
    try:
        ts = [t.to(dev) if t is not None else None for t in (x, off, m, w, b)]
        ts[0].requires_grad_(True)
        if want_aux:
            ts[1].requires_grad_(True)
            if ts[2] is not None:
                ts[2].requires_grad_(True)
        if wanted == "all":
            ts[3].requires_grad_(True)
        d2c.deform_conv3d(*ts, s, p, d, groups, G).backward(gout.to(dev))
    finally:
        _ops.set_grad_input_mode("lists")
    if dtype == torch.float32:
        assert_close(ts[0].grad, eg[0], 1e-4, 1e-5 * max(1.0, eg[0].abs().max().item()), "grad_input")
        if want_aux:
            assert_close(ts[1].grad, eg[1], 1e-4, 1e-5 * max(1.0, eg[1].abs().max().item()), "grad_offset")
        if wanted == "all":
            assert_close(ts[3].grad, eg[3], 1e-4, 1e-5 * max(1.0, eg[3].abs().max().item()), "grad_weight")
    else:
        assert rel_l2(ts[0].grad, eg[0]) < 2e-2
        if want_aux:
            assert rel_l2(ts[1].grad, eg[1]) < 2e-2


@pytest.mark.parametrize("name", ["c64_g1", "c128_G2_o96", "dw64"])
def test_integer_sampling_positions(name, dev):
    # integer offsets (the state at zero-initialised offsets), with padding: samples sit exactly on voxels and
    # exactly on the planes -1 and size, where the forward value is cut off by the early-out but the offset
    # gradient still sees the in-range corners (dconv3d_gpu.cu:48-109 against :708-864)
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make(name, torch.float32, seed=21)
    g = torch.Generator().manual_seed(21)
    ints = torch.randint(-2, 3, off.shape, generator=g).to(off.dtype)
    keep = torch.rand(off.shape, generator=g) < 0.25            # a quarter of the offsets stay real-valued
    off = torch.where(keep, off, ints)
    off[:, : off.shape[1] // 3] = 0.0                             # and a third of the taps sit on their own voxel
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
    out = d2c.deform_conv3d(*ts, s, p, d, groups, G)
    exp = cpu.conv3d_forward(x, off, m, w, b, s, p, d, groups, G)
    eg = cpu.conv3d_backward(gout, x, off, m, w, b is not None, s, p, d, groups, G)
    out.backward(gout.to(dev))
    assert_close(out, exp, 1e-4, 1e-5, "forward")
    for n, t, e in zip(("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias"), ts, eg):
        if t is not None:
            assert_close(t.grad, e, 1e-4, 1e-5 * max(1.0, e.abs().max().item()), n)


def test_tiled_matches_generic_family(dev):
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make("c128_G2_o96", torch.float32, seed=3)
    ts = [t.to(dev) if t is not None else None for t in (x, off, m, w, b)]
    out = d2c.deform_conv3d(*ts, s, p, d, groups, G)
    _ops.set_algo_override("generic")
    try:
        ref = d2c.deform_conv3d(*ts, s, p, d, groups, G)
    finally:
        _ops.set_algo_override(None)
    assert_close(out, ref, 1e-4, 1e-5, "tiled vs generic")


def test_bfloat16_offsets_and_masks_in_bfloat16(dev):
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make("c64_g1", torch.bfloat16, seed=4)
    off, m = off.bfloat16(), m.bfloat16()
    ts = [t.to(dev).requires_grad_(True) for t in (x, off, m, w, b)]
    out = d2c.deform_conv3d(*ts, s, p, d, groups, G)
    exp = cpu.conv3d_forward(f32(x), f32(off), f32(m), f32(w), f32(b), s, p, d, groups, G)
    assert rel_l2(out, exp) < 2e-2
    out.backward(gout.to(dev))
    eg = cpu.conv3d_backward(f32(gout), f32(x), f32(off), f32(m), f32(w), True, s, p, d, groups, G)
    for t, e in zip(ts, eg):
        assert t.grad.dtype == torch.bfloat16 and rel_l2(t.grad, e) < 2e-2


# ------------------------------------------------------------------ 1-D operator on the tiled kernels
SHAPES_1D = {
    # name: (N, Cin, Cout, L, k, stride, pad, dil, groups, G, bias, mask, sigma)
    "l64_c64": (4, 64, 64, 64, 3, 1, 1, 1, 1, 1, True, True, 1.5),
    "l40_c128_G2_o96": (2, 128, 96, 40, 5, 1, 2, 1, 1, 2, True, True, 2.0),
    "l50_groups2_stride": (2, 128, 128, 50, 3, 2, 1, 2, 2, 2, False, False, 1.0),
}


def make1d(name, dtype, seed=0):
    N, Cin, Cout, L, k, s, p, d, groups, G, bias, mask, sig = SHAPES_1D[name]
    Lo = (L + 2 * p - (d * (k - 1) + 1)) // s + 1
    g = torch.Generator().manual_seed(2000 + seed)
    x = torch.randn(N, Cin, L, generator=g)
    w = (torch.rand(Cout, Cin // groups, k, generator=g) * 2 - 1) / (Cin // groups * k) ** 0.5
    b = (torch.rand(Cout, generator=g) * 2 - 1) / (Cin // groups * k) ** 0.5 if bias else None
    off = torch.randn(N, G * k, Lo, generator=g) * sig
    m = torch.sigmoid(torch.randn(N, G * k, Lo, generator=g)) if mask else None
    gout = torch.randn(N, Cout, Lo, generator=g)
    if dtype == torch.bfloat16:
        x, w, gout = x.bfloat16(), w.bfloat16(), gout.bfloat16()
        b = b.bfloat16() if b is not None else None
    return (x, off, m, w, b), gout, (s, p, d, groups, G)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", list(SHAPES_1D))
def test_tiled_conv1d_forward_backward(name, dtype, dev):
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make1d(name, dtype)
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
    assert _ops.conv1d_algo(ts[0], ts[1], ts[2], ts[3], s, p, d, groups, G) == "mfma"
    out = d2c.deform_conv1d(*ts, s, p, d, groups, G)
    exp = cpu.conv1d_forward(f32(x), off, m, f32(w), f32(b), s, p, d, groups, G)
    eg = cpu.conv1d_backward(f32(gout), f32(x), off, m, f32(w), b is not None, s, p, d, groups, G)
    out.backward(gout.to(dev))
    names = ("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias")
    if dtype == torch.float32:
        assert_close(out, exp, 1e-4, 1e-5, "forward")
        for n, t, e in zip(names, ts, eg):
            if t is not None:
                assert_close(t.grad, e, 1e-4, 1e-5 * max(1.0, e.abs().max().item()), n)
    else:
        assert rel_l2(out, exp) < 2e-2
        for n, t, e in zip(names, ts, eg):
            if t is not None:
                assert rel_l2(t.grad, e) < 2e-2, (n, rel_l2(t.grad, e))


@pytest.mark.parametrize("quirks", [True, False])
def test_tiled_conv1d_integer_positions(quirks, dev):
    # integer sampling positions (the state at zero-initialised offsets): dconv1d_gpu.cu:332-351
    g = torch.Generator().manual_seed(5)
    N, C, L = 2, 32, 16
    x = torch.randn(N, C, L, generator=g)
    w = torch.randn(C, C, 3, generator=g) / 10
    off = torch.zeros(N, 3, L)
    off[:, 1, ::2] = 2.0          # a mix of integer offsets; some land outside the signal
    off[:, 2, 1::3] = -3.0
    off[1, 0, :] = torch.randn(L, generator=g)   # and non-integer ones
    m = torch.sigmoid(torch.randn(N, 3, L, generator=g))
    gout = torch.randn(N, C, L, generator=g)
    eg = cpu.conv1d_backward(gout, x, off, m, w, False, 1, 1, 1, 1, 1, quirks=quirks)
    ts = [t.to(dev).requires_grad_(True) for t in (x, off, m, w)]
    assert _ops.conv1d_algo(ts[0], ts[1], ts[2], ts[3], 1, 1, 1, 1, 1) == "mfma"
    out = _ops.deform_conv1d(ts[0], ts[1], ts[2], ts[3], None, 1, 1, 1, 1, 1, reference_quirks=quirks)
    out.backward(gout.to(dev))
    for n, t, e in zip(("grad_input", "grad_offset", "grad_mask", "grad_weight"), ts, eg):
        assert_close(t.grad, e, 1e-4, 1e-5 * max(1.0, e.abs().max().item()), f"{n} quirks={quirks}")


def _random_case(rng, depthwise):
    """A random geometry that the matrix-core (or channel-separated) kernels accept."""
    pick = lambda *v: v[int(rng.integers(len(v)))]
    k = (pick(1, 3), pick(1, 3), pick(2, 3))
    s = (pick(1, 2), pick(1, 1, 2), pick(1, 1, 2))
    d = (pick(1, 2), pick(1, 1, 2), pick(1, 2))
    p = tuple(int(rng.integers(0, 3)) for _ in range(3))
    dims = tuple(int(rng.integers(dd * (kk - 1) + 1 + 1, dd * (kk - 1) + 1 + 9)) for kk, dd in zip(k, d))
    N = pick(1, 2, 3)
    if depthwise:
        G = pick(1, 2, 4)
        C = G * 4 * int(rng.integers(1, 70))
        return N, C, C, dims, k, s, p, d, C, G, bool(rng.integers(2)), bool(rng.integers(2)), float(pick(0.5, 1.5, 3.0))
    groups = pick(1, 1, 2)
    G = pick(1, groups, 2 * groups)                    # fewer, as many or more offset groups than weight groups
    unit = 64 * max(G, groups)                         # channels per weight group and per offset group: multiples of 64
    Cin = unit * pick(1, 2) if groups == 1 else unit
    m = G * groups // (2 if G % 2 == 0 and groups % 2 == 0 else 1)   # Cout: a multiple of groups and of the offset groups
    Cout = m * int(rng.integers(1, 300 // m + 1))
    return N, Cin, Cout, dims, k, s, p, d, groups, G, bool(rng.integers(2)), bool(rng.integers(2)), float(pick(0.5, 1.5, 3.0))


def _check_against_oracle(res, exp, dtype, shape, family):
    """Forward value and gradients of one kernel family against the oracle's: float32 1e-4 relative / 1e-5
    absolute (the absolute part scaled by the tensor's magnitude: the gradients are long sums), bfloat16 2e-2 of
    the tensor's scale."""
    for i, (a, e) in enumerate(zip(res, exp)):
        scale = max(1.0, e.abs().max().item())
        err = (a.cpu().float() - e).abs()
        bound = (1e-5 * scale + 1e-4 * e.abs()) if dtype == torch.float32 else torch.full_like(e, 2e-2 * scale)
        assert bool((err <= bound).all()), (shape, family, i, err.max().item(), scale)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("depthwise", [False, True])
def test_random_geometries_against_the_oracle(depthwise, dtype, dev):
    """Seeded random shapes, strides, paddings, dilations, weight / offset groups and offset scales: the matrix-core
    / channel-separated kernels AND the direct kernels (one thread per element), each against the CPU oracle on
    the same tensors, forward and all gradients.  D2C_RANDOM_CASES in the environment widens the sweep (10 by
    default); each case is printed before it runs."""
    import os
    import numpy as np
    rng = np.random.default_rng(20240 + int(depthwise))
    for case in range(int(os.environ.get("D2C_RANDOM_CASES", "10"))):
        shape = _random_case(rng, depthwise)
        print(f"random case {case} depthwise={depthwise} {dtype}: {shape}", flush=True)
        SHAPES["_random"] = shape
        try:
            (x, off, m, w, b), gout, (s, p, d, groups, G) = make("_random", dtype, seed=100 + case)
        finally:
            del SHAPES["_random"]
        e_out = cpu.conv3d_forward(f32(x), off, m, f32(w), f32(b), s, p, d, groups, G)
        eg = cpu.conv3d_backward(f32(gout), f32(x), off, m, f32(w), b is not None, s, p, d, groups, G)
        exp = [e_out] + [e for e in eg if e is not None]
        for family in (None, "generic"):
            ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
            _ops.set_algo_override(family)
            try:
                if family is None:
                    assert _ops.conv3d_algo(ts[0], ts[1], ts[2], ts[3], s, p, d, groups, G) == \
                        ("depthwise" if depthwise else "mfma"), shape
                out = d2c.deform_conv3d(*ts, s, p, d, groups, G)
                out.backward(gout.to(dev))
            finally:
                _ops.set_algo_override(None)
            res = [out.detach().float()] + [t.grad.float() for t in ts if t is not None]
            _check_against_oracle(res, exp, dtype, shape, family or "tiled")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_random_geometries_1d_against_the_oracle(dtype, dev):
    """The 1-D operator on seeded random lengths, kernel sizes, strides, paddings, dilations and groups: matrix-core
    kernels and direct kernels, each against the CPU oracle on the same tensors, forward and all gradients
    (D2C_RANDOM_CASES widens the sweep)."""
    import os
    import numpy as np
    rng = np.random.default_rng(777)
    pick = lambda *v: v[int(rng.integers(len(v)))]
    for case in range(int(os.environ.get("D2C_RANDOM_CASES", "10"))):
        k, st, d = pick(1, 2, 3, 5), pick(1, 1, 2, 3), pick(1, 1, 2, 3)
        pad = int(rng.integers(0, 4))
        L = int(rng.integers(d * (k - 1) + 2, d * (k - 1) + 90))
        groups = pick(1, 1, 2)
        G = groups * pick(1, 2)
        Cin = 64 * G * pick(1, 2) if groups == 1 else 64 * G
        Cout = G * int(rng.integers(1, 300 // G + 1))
        shape = (pick(1, 2, 5), Cin, Cout, L, k, st, pad, d, groups, G, bool(rng.integers(2)), bool(rng.integers(2)),
                 float(pick(0.5, 1.5, 3.0)))
        print(f"random 1-D case {case} {dtype}: {shape}", flush=True)
        SHAPES_1D["_random"] = shape
        try:
            (x, off, m, w, b), gout, (s, p, d, groups, G) = make1d("_random", dtype, seed=300 + case)
        finally:
            del SHAPES_1D["_random"]
        e_out = cpu.conv1d_forward(f32(x), off, m, f32(w), f32(b), s, p, d, groups, G)
        eg = cpu.conv1d_backward(f32(gout), f32(x), off, m, f32(w), b is not None, s, p, d, groups, G)
        exp = [e_out] + [e for e in eg if e is not None]
        for family in (None, "generic"):
            ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
            _ops.set_algo_override(family)
            try:
                if family is None:
                    assert _ops.conv1d_algo(ts[0], ts[1], ts[2], ts[3], s, p, d, groups, G) == "mfma", shape
                out = d2c.deform_conv1d(*ts, s, p, d, groups, G)
                out.backward(gout.to(dev))
            finally:
                _ops.set_algo_override(None)
            res = [out.detach().float()] + [t.grad.float() for t in ts if t is not None]
            _check_against_oracle(res, exp, dtype, shape, family or "tiled")
