"""Shared helpers of the test-suite: seeded inputs shaped like the reference's
generate_data (ops/dconv-native/test/test_deform_conv.py:57-124) and tolerance
comparisons."""
from functools import reduce

import torch
from torch.nn.modules.utils import _single, _triple


def prod(t):
    return reduce(lambda a, b: a * b, t, 1)


def out_dims(dims, ks, stride, padding, dilation):
    return tuple((d + 2 * p - (a * (k - 1) + 1)) // s + 1
                 for d, k, s, p, a in zip(dims, ks, stride, padding, dilation))


def generate_data(nd, batch_size=2, channels_in=3, channels_out=2, dimensions=5, kernel_size=3, stride=1,
                  padding=0, dilation=1, n_offset_groups=1, n_weight_groups=1, bias=True,
                  dtype=torch.float64, seed=0, offset_scale=1.0):
    _t = _single if nd == 1 else _triple
    dimensions, kernel_size, stride, padding, dilation = (_t(v) for v in
                                                          (dimensions, kernel_size, stride, padding, dilation))
    od = out_dims(dimensions, kernel_size, stride, padding, dilation)
    g = torch.Generator().manual_seed(seed)
    K = prod(kernel_size)

    def rn(*shape):
        return torch.randn(*shape, generator=g, dtype=torch.float64).to(dtype)
    data = rn(batch_size, channels_in, *dimensions)
    offset = rn(batch_size, n_offset_groups * nd * K, *od) * offset_scale
    alpha = rn(batch_size, n_offset_groups * K, *od)
    weight = rn(channels_out, channels_in // n_weight_groups, *kernel_size)
    b = rn(channels_out) if bias else None
    return data, offset, alpha, weight, b


def assert_close(actual, expected, rtol, atol, what=""):
    actual = actual.detach().double().cpu()
    expected = expected.detach().double().cpu()
    assert actual.shape == expected.shape, f"{what}: shape {tuple(actual.shape)} vs {tuple(expected.shape)}"
    diff = (actual - expected).abs()
    bound = atol + rtol * expected.abs()
    bad = diff > bound
    assert not bool(bad.any()), (
        f"{what}: {int(bad.sum())}/{bad.numel()} elements off; max abs diff {diff.max().item():.3e}, "
        f"max |expected| {expected.abs().max().item():.3e}")


def rel_l2(actual, expected):
    a, e = actual.detach().double().cpu(), expected.detach().double().cpu()
    return ((a - e).norm() / e.norm().clamp_min(1e-30)).item()


def to_dev(dev, *ts):
    return tuple(t.to(dev) if t is not None else None for t in ts)
