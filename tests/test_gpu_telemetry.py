"""The sampler alone (d2c_conv3d_sample) and the offset histogram (d2c_conv3d_offset_histogram).

Expected values of the sampler: (i) the CPU oracle, made to return single sampled values by a one-hot weight (its
forward pass with out channel (g, k) = the sample of input channel g at tap k); (ii) torch's grid_sample on a
zero-padded copy in float64, the routine the reference's modulation loss calls for this (loss/region.py:97-125).
Expected histogram: numpy on the same values."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from d2conv3d_amd import util
from oracle import cpu
from _util import assert_close

pytestmark = pytest.mark.gpu


def _one_hot_oracle(src, off, ks, stride, pad, dil, G):
    """[N, G*K, Do, Ho, Wo]: the sample of the one-channel `src` at tap (g, k), from the oracle's forward pass."""
    K = ks[0] * ks[1] * ks[2]
    x = src.expand(-1, G, -1, -1, -1).contiguous()
    w = torch.zeros(G * K, G, *ks, dtype=src.dtype)
    for g in range(G):
        for k in range(K):
            w[g * K + k, g].view(-1)[k] = 1.0
    return cpu.conv3d_forward(x, off, None, w, None, stride, pad, dil, 1, G)


@pytest.mark.parametrize("case", [
    ((2, 1, (5, 8, 9)), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, 1.5),
    ((1, 1, (4, 7, 6)), (3, 3, 3), (1, 2, 1), (1, 1, 1), (1, 1, 2), 2, 3.0),     # stride, dilation, two offset groups
    ((1, 1, (3, 5, 5)), (1, 3, 3), (1, 1, 1), (0, 1, 1), (1, 1, 1), 1, 6.0),     # most taps outside the volume
])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_sampler_alone_against_oracle_and_grid_sample(case, dtype, dev):
    (N, Cs, dims), ks, stride, pad, dil, G, sig = case
    g = torch.Generator().manual_seed(71)
    K = ks[0] * ks[1] * ks[2]
    od = tuple((n + 2 * p - (d * (k - 1) + 1)) // s + 1 for n, k, s, p, d in zip(dims, ks, stride, pad, dil))
    src = torch.rand(N, Cs, *dims, generator=g, dtype=torch.float64).to(dtype)
    off = (torch.randn(N, G * 3 * K, *od, generator=g, dtype=torch.float64) * sig).to(dtype)
    off.view(N, G * K, 3, *od)[:, ::5] = off.view(N, G * K, 3, *od)[:, ::5].round()       # some exactly on voxels
    out = util.sample_at_taps(src.to(dev), off.to(dev), ks, stride, pad, dil, G)
    assert out.shape == (N, G * K * Cs, *od)
    e = _one_hot_oracle(src, off, ks, stride, pad, dil, G)
    tol = 1e-6 if dtype == torch.float32 else 1e-12
    assert_close(out, e, tol, tol, "sample vs oracle")
    # grid_sample on the zero-padded tensor: positions in (x, y, z) order, align_corners=True on the padded extent
    o = off.double().view(N, G, K, 3, *od)
    kz, ky, kx = torch.meshgrid(*(torch.arange(k, dtype=torch.float64) for k in ks), indexing="ij")
    base = [torch.arange(n, dtype=torch.float64) * s - p for n, s, p in zip(od, stride, pad)]
    pos = []
    for ax, (kk, dd) in enumerate(zip((kz, ky, kx), dil)):
        shape = [1, 1, 1]
        shape[ax] = od[ax]
        pos.append(kk.reshape(1, 1, K, 1, 1, 1) * dd + base[ax].view(1, 1, 1, *shape) + o[:, :, :, ax])
    padded = F.pad(src.double(), (1, 1, 1, 1, 1, 1))
    norm = [2 * (pz + 1) / (n + 1) - 1 for pz, n in zip(pos, dims)]
    grid = torch.stack([norm[2], norm[1], norm[0]], dim=-1).view(N, G * K * od[0], od[1], od[2], 3)
    gs = F.grid_sample(padded, grid, mode="bilinear", padding_mode="zeros", align_corners=True)
    gs = gs.view(N, Cs, G * K, *od).transpose(1, 2).reshape(N, G * K * Cs, *od)
    # (at a position of exactly `size` the operator's early-out returns 0 and grid_sample reads the padding with
    # weight 1: the same value)
    assert_close(out, gs, 1e-5 if dtype == torch.float32 else 1e-10, 1e-6 if dtype == torch.float32 else 1e-10,
                 "sample vs grid_sample on the padded tensor")


def test_sampler_alone_bfloat16_and_several_channels(dev):
    g = torch.Generator().manual_seed(72)
    src = torch.rand(2, 3, 4, 6, 7, generator=g).bfloat16()
    off = torch.randn(2, 81, 4, 6, 7, generator=g) * 1.5
    out = util.sample_at_taps(src.to(dev), off.to(dev))
    assert out.dtype == torch.bfloat16 and out.shape == (2, 27 * 3, 4, 6, 7)
    for c in range(3):
        e = _one_hot_oracle(src[:, c:c + 1].float(), off, (3, 3, 3), 1, 1, 1, 1)
        assert_close(out[:, c::3], e, 1e-2, 1e-2, f"channel {c}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64])
def test_offset_histogram_against_numpy(dtype, dev):
    g = torch.Generator().manual_seed(73)
    G, K = 2, 27
    off = (torch.randn(2, G * 3 * K, 3, 5, 6, generator=g, dtype=torch.float64) * 3.0).to(dtype)
    off.view(-1)[::97] = 4.0           # values on a bin edge and on the upper limit
    off.view(-1)[::89] = -4.0
    off.view(-1)[5] = float("nan")
    bins, lo, hi = 16, -4.0, 4.0
    hist = util.offset_histogram(off.to(dev), (3, 3, 3), G, bins, (lo, hi)).cpu()
    assert hist.shape == (3, bins + 2) and hist.dtype == torch.int64
    v = off.float().view(2, G * K, 3, -1).numpy()            # the kernel bins the float32 value
    for ax in range(3):
        a = v[:, :, ax].ravel()
        below = int((a < lo).sum())
        above = int((~(a < hi)).sum())
        idx = np.floor((a[(a >= lo) & (a < hi)] - np.float32(lo)) * np.float32(bins / (hi - lo))).astype(np.int64)
        e = np.bincount(np.minimum(idx, bins - 1), minlength=bins)
        assert hist[ax, 0].item() == below and hist[ax, -1].item() == above
        assert hist[ax, 1:-1].tolist() == e.tolist()
    assert int(hist.sum()) == off.numel()
