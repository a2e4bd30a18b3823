"""Writes the regression fixtures of this directory (`python tests/golden/make_golden.py` from the repository root).

The reference keeps no stored vectors for this operator (its tests compare with loops and with torch's own
convolution), so these are not the reference's outputs: they are small seeded cases computed by the CPU oracle
(oracle/) after it has been pinned against those known answers (tests/test_oracle_pinning.py), kept as data so that
a later change of the oracle or of the kernels that moves any value shows up in tests/test_golden.py.  Each file
holds the inputs and the expected forward value and gradients in float64.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
sys.path.insert(0, os.path.join(HERE, ".."))

from oracle import cpu, dwconv, sizemap  # noqa: E402

CASES_3D = {
    # name: (N, Cin, Cout, dims, kernel, stride, padding, dilation, groups, offset groups, mask, bias, offset scale)
    "conv3d_groups": (1, 4, 6, (3, 4, 5), (2, 3, 2), (1, 2, 1), (1, 0, 1), (1, 1, 2), 2, 2, True, True, 1.5),
    "conv3d_nomask_nobias": (2, 2, 2, (3, 3, 4), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, 1, False, False, 2.5),
}


def case_3d(name):
    N, Cin, Cout, dims, k, s, p, d, groups, G, mask, bias, scale = CASES_3D[name]
    g = torch.Generator().manual_seed(sum(map(ord, name)))
    od = tuple((n + 2 * pp - (dd * (kk - 1) + 1)) // ss + 1 for n, kk, ss, pp, dd in zip(dims, k, s, p, d))
    K = k[0] * k[1] * k[2]
    rn = lambda *sh: torch.randn(*sh, generator=g, dtype=torch.float64)
    x, w = rn(N, Cin, *dims), rn(Cout, Cin // groups, *k) / 3
    b = rn(Cout) if bias else None
    off = rn(N, G * 3 * K, *od) * scale
    off.view(-1)[::5] = torch.round(off.view(-1)[::5])          # integer positions: the one-sided derivatives
    off.view(-1)[3::17] += 40.0                                   # far outside the volume
    m = torch.sigmoid(rn(N, G * K, *od)) if mask else None
    gout = rn(N, Cout, *od)
    out = cpu.conv3d_forward(x, off, m, w, b, s, p, d, groups, G)
    grads = cpu.conv3d_backward(gout, x, off, m, w, bias, s, p, d, groups, G)
    return dict(x=x, offset=off, mask=m, weight=w, bias=b, grad_out=gout, out=out,
                grad_x=grads[0], grad_offset=grads[1], grad_mask=grads[2], grad_weight=grads[3], grad_bias=grads[4],
                geometry=np.array([*s, *p, *d, groups, G]))


def case_1d():
    g = torch.Generator().manual_seed(51)
    rn = lambda *sh: torch.randn(*sh, generator=g, dtype=torch.float64)
    N, Cin, Cout, L, k, s, p, d, groups, G = 2, 4, 4, 9, 3, 1, 1, 1, 2, 2
    Lo = (L + 2 * p - (d * (k - 1) + 1)) // s + 1
    x, w, b = rn(N, Cin, L), rn(Cout, Cin // groups, k) / 2, rn(Cout)
    off = rn(N, G * k, Lo) * 1.5
    off.view(-1)[::4] = torch.round(off.view(-1)[::4])
    m = torch.sigmoid(rn(N, G * k, Lo))
    gout = rn(N, Cout, Lo)
    out = cpu.conv1d_forward(x, off, m, w, b, s, p, d, groups, G)
    grads = cpu.conv1d_backward(gout, x, off, m, w, True, s, p, d, groups, G)
    return dict(x=x, offset=off, mask=m, weight=w, bias=b, grad_out=gout, out=out,
                grad_x=grads[0], grad_offset=grads[1], grad_mask=grads[2], grad_weight=grads[3], grad_bias=grads[4],
                geometry=np.array([s, p, d, groups, G]))


def case_size_map(mode, channels, kernel, dilation, seed):
    # from the numpy closed form of oracle/sizemap.py (pinned by tests/test_size_map_pins.py), not from the package
    g = torch.Generator().manual_seed(seed)
    size = torch.rand(2, channels, 2, 3, 4, generator=g, dtype=torch.float64) * 3.5 + 0.5
    go = torch.randn(2, 3 * kernel[0] * kernel[1] * kernel[2], 2, 3, 4, generator=g, dtype=torch.float64)
    return dict(size=size, offsets=sizemap.offsets(size.numpy(), mode, kernel, dilation), grad_offsets=go,
                grad_size=sizemap.offsets_backward(go.numpy(), mode, kernel, dilation),
                geometry=np.array([*kernel, *dilation]))


def case_dwconv():
    g = torch.Generator().manual_seed(91)
    rn = lambda *sh: torch.randn(*sh, generator=g, dtype=torch.float64)
    x, w, b = rn(2, 3, 4, 5, 8), rn(6, 1, 3, 3, 3) / 3, rn(6)
    s, p, d = (1, 2, 1), (1, 1, 1), (1, 1, 1)
    out = dwconv.forward(x.numpy(), w.numpy(), b.numpy(), s, p, d)
    gout = rn(*out.shape)
    gx, gw, gb = dwconv.backward(gout.numpy(), x.numpy(), w.numpy(), s, p, d)
    return dict(x=x, weight=w, bias=b, grad_out=gout, out=out, grad_x=gx, grad_weight=gw, grad_bias=gb,
                geometry=np.array([*s, *p, *d]))


def save(name, case):
    arrays = {k: (v.numpy() if isinstance(v, torch.Tensor) else np.asarray(v)) for k, v in case.items() if v is not None}
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
    print(name, {k: v.shape for k, v in arrays.items()})


if __name__ == "__main__":
    for name in CASES_3D:
        save(name, case_3d(name))
    save("conv1d_groups", case_1d())
    save("size_map_xyz", case_size_map("xyz", 3, (3, 3, 3), (1, 2, 1), 77))
    save("size_map_xxz", case_size_map("xxz", 2, (3, 5, 2), (1, 2, 1), 78))
    save("size_map_xy", case_size_map("xy", 2, (3, 3, 3), (1, 1, 1), 79))
    save("size_map_x", case_size_map("x", 1, (1, 3, 3), (1, 1, 2), 80))
    save("dwconv3d_multiplier2", case_dwconv())
