"""Seeded sweep of the matrix-core 3-D operator against the CPU oracle over shapes drawn around the rules that pick
its kernels: wide weight groups on a handful of position tiles, narrow weight groups on many tiles, float32 weight
groups of one to several passes of the grad-column product, problems small enough for the split owner kernel, several
weight groups.  Forward and all five gradients, float32 and bfloat16, to the tolerances of test_gpu_tiled.py.
"""
import random

import pytest
import torch

import d2conv3d_amd as d2c
from d2conv3d_amd import _ops
from oracle import cpu
from _util import assert_close, rel_l2

pytestmark = pytest.mark.gpu

KINDS = ["few_tiles_wide", "narrow_many", "f32_passes", "small_owner", "groups"]


def draw(kind, rnd):
    G = 1
    groups = 1
    if kind == "few_tiles_wide":
        cin, cout = rnd.choice([128, 256, 320]), rnd.choice([160, 256, 320, 520])
        dims = (rnd.randint(2, 4), rnd.randint(6, 12), rnd.randint(8, 16))
        G = rnd.choice([1, 2])
    elif kind == "narrow_many":
        cin, cout = rnd.choice([64, 128]), rnd.choice([24, 64, 108, 128])
        dims = (rnd.randint(6, 9), rnd.randint(30, 36), rnd.randint(34, 40))
    elif kind == "f32_passes":
        cin, cout = rnd.choice([64, 128]), rnd.choice([100, 128, 230, 256, 384, 512])
        dims = (rnd.randint(2, 4), rnd.randint(5, 9), rnd.randint(6, 12))
        G = rnd.choice([1, 2])
    elif kind == "small_owner":
        cin, cout = rnd.choice([64, 128, 192]), rnd.choice([64, 128])
        dims = (rnd.randint(1, 5), rnd.randint(3, 9), rnd.randint(3, 11))
    else:
        cin, cout = 256, rnd.choice([256, 384, 768])
        dims = (rnd.randint(2, 4), rnd.randint(6, 10), rnd.randint(6, 12))
        groups, G = 2, rnd.choice([2, 4])
    if cin % (64 * G):
        G = 1
    k = rnd.choice([(3, 3, 3), (3, 3, 3), (1, 3, 3), (3, 1, 1)])
    p = tuple(v // 2 for v in k)
    return dict(N=rnd.randint(1, 2), cin=cin, cout=cout, dims=dims, k=k, p=p, groups=groups, G=G,
                bias=rnd.random() < 0.5, mask=rnd.random() < 0.7, sigma=rnd.choice([0.5, 1.5, 2.5]))


def tensors(c, dtype, seed):
    g = torch.Generator().manual_seed(7000 + seed)
    rn = lambda *sh: torch.randn(*sh, generator=g)
    K = c["k"][0] * c["k"][1] * c["k"][2]
    x = rn(c["N"], c["cin"], *c["dims"])
    fan_in = c["cin"] // c["groups"] * K
    w = (torch.rand(c["cout"], c["cin"] // c["groups"], *c["k"], generator=g) * 2 - 1) / fan_in ** 0.5
    b = (torch.rand(c["cout"], generator=g) * 2 - 1) / fan_in ** 0.5 if c["bias"] else None
    off = rn(c["N"], c["G"] * 3 * K, *c["dims"]) * c["sigma"]          # stride 1, "same" padding: output = input extent
    m = torch.sigmoid(rn(c["N"], c["G"] * K, *c["dims"])) if c["mask"] else None
    gout = rn(c["N"], c["cout"], *c["dims"])
    if dtype == torch.bfloat16:
        x, w, gout = x.bfloat16(), w.bfloat16(), gout.bfloat16()
        b = b.bfloat16() if b is not None else None
    return x, off, m, w, b, gout


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("seed", range(4))
def test_random_shapes_against_oracle(seed, kind, dtype, dev):
    c = draw(kind, random.Random(f"{kind}-{seed}"))
    x, off, m, w, b, gout = tensors(c, dtype, seed)
    f32 = lambda t: t.float() if t is not None else None
    s, p, d = (1, 1, 1), c["p"], (1, 1, 1)
    ts = [t.to(dev).requires_grad_(True) if t is not None else None for t in (x, off, m, w, b)]
    assert _ops.conv3d_algo(ts[0], ts[1], ts[2], ts[3], s, p, d, c["groups"], c["G"]) == "mfma", c
    out = d2c.deform_conv3d(*ts, s, p, d, c["groups"], c["G"])
    out.backward(gout.to(dev))
    exp = cpu.conv3d_forward(f32(x), off, m, f32(w), f32(b), s, p, d, c["groups"], c["G"])
    eg = cpu.conv3d_backward(f32(gout), f32(x), off, m, f32(w), b is not None, s, p, d, c["groups"], c["G"])
    names = ("grad_input", "grad_offset", "grad_mask", "grad_weight", "grad_bias")
    if dtype == torch.float32:
        assert_close(out, exp, 1e-4, 1e-5, f"forward {c}")
        for n, t, e in zip(names, ts, eg):
            if t is not None:
                assert_close(t.grad, e, 1e-4, 1e-5 * max(1.0, e.abs().max().item()), f"{n} {c}")
    else:
        assert rel_l2(out, exp) < 2e-2, (c, rel_l2(out, exp))
        for n, t, e in zip(names, ts, eg):
            if t is not None:
                assert rel_l2(t.grad, e) < 2e-2, (n, c, rel_l2(t.grad, e))
                assert_close(t.grad, e, 2e-2, 2e-2 * e.abs().max().item(), f"{n} {c}")
