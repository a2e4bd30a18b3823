"""TEST INFRASTRUCTURE ONLY: loop-by-loop forward of the deformable convolution.

An independent restatement of the brute-force checker that the reference's own
test-suite uses (ops/dconv-native/test/test_deform_conv.py: linear_interpolate
:18-28, trilinear_interpolate :31-54, expected_fn :127-191): float64 scalars,
one term of the sum at a time.  It shares no code with the C oracle and exists
to pin it on inputs of a few hundred elements; it is far too slow for more.
"""
from itertools import product
from math import floor

import torch


def _interp(data, pos):
    """Multilinear sample of `data` (nd tensor) at real position `pos`; corners
    outside the volume contribute nothing (test_deform_conv.py:18-54)."""
    lo = [int(floor(float(v))) for v in pos]
    val = 0.0
    for corner in product((0, 1), repeat=len(pos)):
        idx = tuple(l + c for l, c in zip(lo, corner))
        if all(0 <= i < n for i, n in zip(idx, data.shape)):
            wgt = 1.0
            for v, l, c in zip(pos, lo, corner):
                # weight of the low corner is (hi - v), of the high corner (v - lo)
                wgt *= abs((l + 1 - c) - float(v))
            val += wgt * float(data[idx])
    return val


def _tup(v, n):
    return (int(v),) * n if isinstance(v, int) else tuple(int(a) for a in v)


def deform_conv_forward(x, offset, mask, weight, bias=None, stride=1, padding=0, dilation=1):
    """expected_fn of the reference tests (test_deform_conv.py:127-191) for 1-D
    and 3-D inputs; group counts are inferred from the shapes as there."""
    nd = x.dim() - 2
    stride, padding, dilation = (_tup(v, nd) for v in (stride, padding, dilation))
    ks = tuple(weight.shape[2:])
    dims = tuple(x.shape[2:])
    K = 1
    for k in ks:
        K *= k
    nb, cin = x.shape[:2]
    cout = weight.shape[0]
    out_dims = tuple((d + 2 * p - (a * (k - 1) + 1)) // s + 1
                     for d, k, s, p, a in zip(dims, ks, stride, padding, dilation))
    n_off_grp = offset.shape[1] // (nd * K)
    cin_wg = weight.shape[1]
    n_wg = cin // cin_wg
    cout_wg = cout // n_wg
    cin_og = cin // n_off_grp
    xd, od, wd = x.double(), offset.double(), weight.double()
    md = mask.double() if mask is not None else None
    out = torch.zeros(nb, cout, *out_dims, dtype=torch.float64)
    for b in range(nb):
        for co in range(cout):
            wg = co // cout_wg
            for oi in product(*(range(d) for d in out_dims)):
                acc = 0.0
                for ki in product(*(range(k) for k in ks)):
                    kflat = 0
                    for n, i in zip(ks, ki):
                        kflat = kflat * n + i
                    for c in range(cin_wg):
                        ci = wg * cin_wg + c
                        og = ci // cin_og
                        a_idx = og * K + kflat
                        pos = tuple(
                            s * l - p + a * dl + float(od[(b, nd * a_idx + ax) + oi])
                            for ax, (s, l, p, a, dl) in enumerate(zip(stride, oi, padding, dilation, ki)))
                        m = float(md[(b, a_idx) + oi]) if md is not None else 1.0
                        acc += m * float(wd[(co, c) + ki]) * _interp(xd[b, ci], pos)
                out[(b, co) + oi] = acc
    if bias is not None:
        out += bias.double().view(1, cout, *(1,) * nd)
    return out
