"""TEST INFRASTRUCTURE ONLY: the dynamic-dilation offset expansion of the reference restated
tap by tap in numpy, independent of the package's torch formulation.

    offsets_from_size_map   utils/grid.py:72-98, ops/dconv-native/src/dconv_native/grid.py:62-80
    get_kernel_grid         utils/grid.py:21-25 / grid.py:21-25
    _apply_size_activation  network/layers.py:171-181

Closed form (one scalar statement per output element):

    off[n, ((kz*kh + ky)*kw + kx)*3 + a, d, h, w] = base_a[k_a] * (size3[n, a, d, h, w] - 1)
    base_a = linspace(-dil_a*(k_a//2), +dil_a*(k_a//2), k_a)
    size3  = the size map with the axes its mode does not predict set to one:
             "xyz": (z, y, x);  "xxz": (z, x, x) from channels (z, x);  "xy": (1, y, x);  "x": (1, s, s)

Pinned (tests/test_size_map_pins.py) by what the mathematics fixes: a constant integer size map makes the
deformable convolution a stock dilated convolution (torch's F.conv3d) for every mode, which fails for a wrong
axis order, a wrong channel-to-axis mapping, a wrong sign or a dropped "- 1"; the backward map is the transpose
of the forward map (checked as an adjoint identity and by central differences).
"""
import numpy as np

MODES = {"xyz": (0, 1, 2), "xxz": (0, 1, 1), "xy": (None, 0, 1), "x": (None, 0, 0)}   # size channel of axis z, y, x


def kernel_axis(k, dil):
    """linspace(-dil*(k//2), dil*(k//2), k) as float64 (utils/grid.py:21-25)."""
    h = dil * (k // 2)
    if k == 1:
        return np.array([-float(h)])        # torch.linspace(a, b, 1) returns the start point
    return np.array([-h + i * (2.0 * h) / (k - 1) for i in range(k)], dtype=np.float64)


def activate(raw, name):
    """network/layers.py:171-181."""
    raw = np.asarray(raw, dtype=np.float64)
    if name == "linear":
        return raw
    if name == "elu":
        return np.where(raw > 0, raw, np.expm1(np.minimum(raw, 0))) + 1.0
    if name == "relu":
        return np.maximum(raw + 1.0, 0.0)
    if name == "relu_plus_one":
        return np.maximum(raw + 1e-3, 0.0) + 1.0
    raise ValueError(name)


def activate_grad(raw, name):
    raw = np.asarray(raw, dtype=np.float64)
    if name == "linear":
        return np.ones_like(raw)
    if name == "elu":
        return np.where(raw > 0, 1.0, np.exp(np.minimum(raw, 0)))
    if name == "relu":
        return (raw + 1.0 > 0).astype(np.float64)
    if name == "relu_plus_one":
        return (raw + 1e-3 > 0).astype(np.float64)
    raise ValueError(name)


def offsets(size, mode, kernel=(3, 3, 3), dilation=(1, 1, 1)):
    """size [N, C_mode, D, H, W] (after the size activation) -> offsets [N, 3*K, D, H, W], float64."""
    size = np.asarray(size, dtype=np.float64)
    chan = MODES[mode]
    assert size.shape[1] == len({c for c in chan if c is not None}), (mode, size.shape)
    n = size.shape[0]
    sp = size.shape[2:]
    kd, kh, kw = kernel
    base = [kernel_axis(k, d) for k, d in zip(kernel, dilation)]
    out = np.zeros((n, 3 * kd * kh * kw) + sp, dtype=np.float64)
    for kz in range(kd):
        for ky in range(kh):
            for kx in range(kw):
                k = (kz * kh + ky) * kw + kx
                for a, ka in enumerate((kz, ky, kx)):
                    s = size[:, chan[a]] if chan[a] is not None else np.ones((n,) + sp)
                    out[:, 3 * k + a] = base[a][ka] * (s - 1.0)
    return out


def offsets_backward(grad_offsets, mode, kernel=(3, 3, 3), dilation=(1, 1, 1)):
    """Transpose of `offsets`: grad_offsets [N, 3*K, D, H, W] -> grad_size [N, C_mode, D, H, W]."""
    grad_offsets = np.asarray(grad_offsets, dtype=np.float64)
    chan = MODES[mode]
    nch = len({c for c in chan if c is not None})
    n = grad_offsets.shape[0]
    sp = grad_offsets.shape[2:]
    kd, kh, kw = kernel
    base = [kernel_axis(k, d) for k, d in zip(kernel, dilation)]
    out = np.zeros((n, nch) + sp, dtype=np.float64)
    for kz in range(kd):
        for ky in range(kh):
            for kx in range(kw):
                k = (kz * kh + ky) * kw + kx
                for a, ka in enumerate((kz, ky, kx)):
                    if chan[a] is not None:
                        out[:, chan[a]] += base[a][ka] * grad_offsets[:, 3 * k + a]
    return out
