"""TEST INFRASTRUCTURE ONLY: CPU restatement (numpy, float64) of the reference's plain depthwise conv3d
(ops/fast-depthwise-conv3d/csrc/grouped_conv3d.cu), used to check the HIP kernels; never part of the product path.

Pinned in tests/test_oracle_pinning.py against torch's own grouped convolution and its autograd on the CPU (the
reference's test compares with exactly that, test/test_conv3d_depthwise.py:33-96).

    forward      conv_depthwise3d_cuda_kernel                  (:25-92)
    grad_input   conv_depthwise3d_cuda_backward_input_kernel   (:97-175)
    grad_weight  conv_depthwise3d_cuda_backward_weight_kernel  (:178-276)
    grad_bias    grad_output.sum over samples and positions    (:660-662)
"""
import numpy as np


def _geometry(x, w, stride, padding, dilation):
    N, C, D, H, W = x.shape
    Cout, one, kd, kh, kw = w.shape
    assert one == 1 and Cout % C == 0
    out = tuple((n + 2 * p - (d * (k - 1) + 1)) // s + 1
                for n, p, d, k, s in zip((D, H, W), padding, dilation, (kd, kh, kw), stride))
    return N, C, Cout, (D, H, W), (kd, kh, kw), out


def _padded(x, padding):
    pd, ph, pw = padding
    return np.pad(x, ((0, 0), (0, 0), (pd, pd), (ph, ph), (pw, pw)))


def _tap_view(xp, k, stride, dilation, out):
    """x[n, c, o*s - p + k*d] for all output positions o, read from the zero-padded input."""
    sl = tuple(slice(k[a] * dilation[a], k[a] * dilation[a] + (out[a] - 1) * stride[a] + 1, stride[a]) for a in range(3))
    return xp[(slice(None), slice(None)) + sl]


def forward(x, w, bias, stride, padding, dilation):
    """out[n, co, o] = bias[co] + sum_k w[co, 0, k] * x[n, co // m, o*s - p + k*d]  (zero outside the volume), :58-90."""
    x, w = np.asarray(x, np.float64), np.asarray(w, np.float64)
    N, C, Cout, _, ks, out = _geometry(x, w, stride, padding, dilation)
    m = Cout // C
    xp = np.repeat(_padded(x, padding), m, axis=1)          # channel co reads input channel co // m
    res = np.zeros((N, Cout) + out)
    for kz in range(ks[0]):
        for ky in range(ks[1]):
            for kx in range(ks[2]):
                res += w[None, :, 0, kz, ky, kx, None, None, None] * _tap_view(xp, (kz, ky, kx), stride, dilation, out)
    if bias is not None:
        res += np.asarray(bias, np.float64)[None, :, None, None, None]
    return res


def backward(grad_out, x, w, stride, padding, dilation, has_bias=True):
    """(grad_input, grad_weight, grad_bias): the adjoints of `forward`, tap by tap."""
    g, x, w = np.asarray(grad_out, np.float64), np.asarray(x, np.float64), np.asarray(w, np.float64)
    N, C, Cout, dims, ks, out = _geometry(x, w, stride, padding, dilation)
    m = Cout // C
    xp = np.repeat(_padded(x, padding), m, axis=1)
    gxp = np.zeros_like(xp)                                  # per output channel, on the padded volume
    gw = np.zeros_like(w)
    for kz in range(ks[0]):
        for ky in range(ks[1]):
            for kx in range(ks[2]):
                k = (kz, ky, kx)
                gw[:, 0, kz, ky, kx] = (g * _tap_view(xp, k, stride, dilation, out)).sum(axis=(0, 2, 3, 4))
                _tap_view(gxp, k, stride, dilation, out)[...] += w[None, :, 0, kz, ky, kx, None, None, None] * g
    pd, ph, pw = padding
    gx = gxp[:, :, pd:pd + dims[0], ph:ph + dims[1], pw:pw + dims[2]]
    gx = gx.reshape(N, C, m, *dims).sum(axis=2)              # the m output channels of an input channel
    gb = g.sum(axis=(0, 2, 3, 4)) if has_bias else None
    return gx, gw, gb
