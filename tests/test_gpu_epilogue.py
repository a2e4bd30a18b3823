"""The activation fused into the forward kernels' store (descriptor fields `epilogue`, `epilogue_scale`): every
kernel family that writes the output -- direct, register-gather matrix-core (with and without shared-out steps),
DMA-gather matrix-core incl. its shared-out last round, channel-separated -- against the unfused operator followed
by torch's relu, forward and all gradients; and the module-level folding of (D2Conv, ReLU | ScaledReLU) pairs, the
`_conv` blocks of network/modules/refinement.py:38-43."""
import ctypes

import pytest
import torch
import torch.nn as nn

import d2conv3d_amd as d2c
from d2conv3d_amd import _lib, _ops, modules, util
from oracle import cpu
from test_gpu_tiled import SHAPES, make

pytestmark = pytest.mark.gpu

CASES = [
    # shape, forced family (None: the default choice), expected family
    ("c64_g1", None, "mfma"),                    # few tiles: steps shared out, fp32 tiles finished by a second kernel
    ("c64_tail", None, "mfma"),
    ("c128_groups2", None, "mfma"),
    ("c64_o320_big", None, "mfma"),              # DMA-gather kernel, 512-wide tiles, ragged last tile
    ("c64_o200_big", None, "mfma"),              # DMA-gather kernel, 256-wide tiles
    ("c64_o1100_big", None, "mfma"),             # its whole rounds and its shared-out round
    ("dw64", None, "depthwise"),
    ("dw1100_stride", None, "depthwise"),
    ("c64_g1", "generic", "generic"),
    ("c128_G2_o96", "generic", "generic"),
]


def _run(case, dtype, dev, scale, fused):
    name, family, _ = case
    (x, off, m, w, b), gout, (s, p, d, groups, G) = make(name, dtype, seed=7)
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
    _ops.set_algo_override(family)
    try:
        if fused:
            out = d2c.deform_conv3d(*ts, s, p, d, groups, G, output_relu=scale)
        else:
            out = torch.relu(d2c.deform_conv3d(*ts, s, p, d, groups, G)) * scale
        out.backward(gout.to(dev))
    finally:
        _ops.set_algo_override(None)
    return [out.detach()] + [t.grad for t in ts if t is not None]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", CASES, ids=[f"{c[0]}-{c[2]}" for c in CASES])
def test_fused_relu_equals_relu_after_the_operator(case, dtype, dev):
    name, family, expect = case
    (x, off, m, w, b), _, (s, p, d, groups, G) = make(name, dtype, seed=7)
    if family is None:
        assert _ops.conv3d_algo(x.to(dev), off.to(dev), None if m is None else m.to(dev), w.to(dev),
                                s, p, d, groups, G) == expect
    # scale 1: the same values (up to the order of the atomic sums where steps are shared out), the same masked
    # gradient going into the same backward kernels
    got, want = _run(case, dtype, dev, 1.0, True), _run(case, dtype, dev, 1.0, False)
    assert (got[0] == 0).any() and (got[0] > 0).any() and not (got[0] < 0).any()
    for i, (a, e) in enumerate(zip(got, want)):
        scale = max(1.0, e.float().abs().max().item())
        tol = (1e-6 if i == 0 else 1e-5) if dtype == torch.float32 else 2e-2
        assert (a.float() - e.float()).abs().max().item() <= tol * scale
    # ScaledReLU: fused is rounded once, the unfused bfloat16 result twice
    got, want = _run(case, dtype, dev, util.SCALED_RELU, True), _run(case, dtype, dev, util.SCALED_RELU, False)
    for a, e in zip(got, want):
        scale = max(1.0, e.float().abs().max().item())
        assert (a.float() - e.float()).abs().max().item() <= (1e-5 if dtype == torch.float32 else 2e-2) * scale


def test_fused_relu_against_the_oracle(dev):
    (x, off, m, w, b), _, (s, p, d, groups, G) = make("c64_tail", torch.float32, seed=3)
    want = torch.relu(cpu.conv3d_forward(x, off, m, w, b, s, p, d, groups, G)) * util.SCALED_RELU
    got = d2c.deform_conv3d(x.to(dev), off.to(dev), m.to(dev), w.to(dev), b.to(dev), s, p, d, groups, G,
                            output_relu=util.SCALED_RELU)
    assert (got.cpu() - want).abs().max().item() <= 1e-4 * max(1.0, want.abs().max().item())


class ScaledReLU(nn.Module):      # same name and function as network/layers.py:414-419
    def forward(self, x):
        return torch.relu(x) * 1.71285855


@pytest.mark.parametrize("act", [nn.ReLU, ScaledReLU, nn.Tanh])
def test_fold_activation_into_the_layer(act, dev):
    torch.manual_seed(11)
    def block():
        return nn.Sequential(modules.MDConv3d(64, 64, 3, padding=1, init="random"), act(), nn.GroupNorm(8, 64))
    ref = nn.Sequential(block(), block()).to(dev)
    for blk in ref:
        nn.init.normal_(blk[0].deform_params.weight, std=0.05)
    import copy
    fused = copy.deepcopy(ref)
    n = util.fuse_output_activation(fused)
    assert n == (0 if act is nn.Tanh else 2)
    assert list(fused.state_dict()) == list(ref.state_dict())
    if n:
        assert isinstance(fused[0][1], nn.Identity) and fused[0][0].deform_conv.output_relu_scale > 0
        assert util.fuse_output_activation(fused) == 0      # nothing left to fold
    x = torch.randn(1, 64, 4, 9, 10, device=dev)
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    ya, yb = ref(xa), fused(xb)
    # (the two differ by the order of atomic sums in the kernels; two GroupNorms amplify that to ~1e-5)
    close = lambda a, b, tol: (a - b).abs().max().item() <= tol * max(1.0, b.abs().max().item())
    assert close(ya, yb, 1e-4)
    ya.square().mean().backward()
    yb.square().mean().backward()
    assert close(xa.grad, xb.grad, 1e-3)
    for (k, pa), (_, pb) in zip(ref.named_parameters(), fused.named_parameters()):
        assert close(pa.grad, pb.grad, 1e-3), k


def test_descriptor_is_checked(dev):
    lib = _lib.load()
    desc = _lib.Conv3dDesc(1, 64, 64, 4, 5, 6, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 4, 5, 6, 0, 0, 7, 1.0)
    assert lib.d2c_conv3d_check(ctypes.byref(desc)) != 0 and b"epilogue" in lib.d2c_last_error()
    desc.epilogue, desc.epilogue_scale = _lib.EPILOGUE_RELU, float("nan")
    assert lib.d2c_conv3d_check(ctypes.byref(desc)) != 0 and b"epilogue_scale" in lib.d2c_last_error()
    desc.epilogue_scale = 1.5
    assert lib.d2c_conv3d_check(ctypes.byref(desc)) == 0
