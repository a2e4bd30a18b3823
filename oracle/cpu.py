"""TEST INFRASTRUCTURE ONLY: ctypes front end of the C oracle (libd2c_oracle.so).

Takes and returns contiguous torch CPU tensors of dtype float32 or float64 in
the reference's layouts (see d2c_oracle.h).  bfloat16 cases are checked by
feeding the bfloat16-rounded values up-cast to float32.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libd2c_oracle.so")
_lib = None


class Conv3dDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in (
        "N", "Cin", "Cout", "D", "H", "W", "kd", "kh", "kw", "sd", "sh", "sw",
        "pd", "ph", "pw", "dd", "dh", "dw", "groups", "offset_groups", "Do", "Ho", "Wo")]


class Conv1dDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in (
        "N", "Cin", "Cout", "L", "k", "s", "p", "d", "groups", "offset_groups", "Lo")]


def build(force=False):
    """Compile the oracle with the Makefile beside this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        _lib.oracle_output_size.restype = ctypes.c_int
        _lib.oracle_num_threads.restype = ctypes.c_int
    return _lib


def num_threads():
    return lib().oracle_num_threads()


def output_size(n, k, s, p, d):
    """dconv_gpu_common.h:13-15 (C integer division)."""
    return lib().oracle_output_size(int(n), int(k), int(s), int(p), int(d))


def _t3(v):
    return (v, v, v) if isinstance(v, int) else tuple(int(a) for a in v)


def _sfx(t):
    if t.dtype == torch.float32:
        return "f32"
    if t.dtype == torch.float64:
        return "f64"
    raise TypeError(f"oracle handles float32/float64, got {t.dtype}")


def _p(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _c(t, ref):
    if t is None:
        return None
    assert t.device.type == "cpu"
    return t.detach().to(ref.dtype).contiguous()


def desc3d(x, weight, stride, padding, dilation, groups, offset_groups):
    s, p, d = _t3(stride), _t3(padding), _t3(dilation)
    N, Cin, D, H, W = x.shape
    Cout, _, kd, kh, kw = weight.shape
    Do = output_size(D, kd, s[0], p[0], d[0])
    Ho = output_size(H, kh, s[1], p[1], d[1])
    Wo = output_size(W, kw, s[2], p[2], d[2])
    return Conv3dDesc(N, Cin, Cout, D, H, W, kd, kh, kw, *s, *p, *d, groups, offset_groups, Do, Ho, Wo)


def conv3d_forward(x, offset, mask, weight, bias=None, stride=1, padding=0, dilation=1,
                   groups=1, offset_groups=1):
    x = _c(x, x)
    offset, mask, weight, bias = (_c(t, x) for t in (offset, mask, weight, bias))
    q = desc3d(x, weight, stride, padding, dilation, groups, offset_groups)
    out = torch.empty(q.N, q.Cout, q.Do, q.Ho, q.Wo, dtype=x.dtype)
    fn = getattr(lib(), "oracle_conv3d_forward_" + _sfx(x))
    rc = fn(_p(x), _p(offset), _p(mask), _p(weight), _p(bias), _p(out), ctypes.byref(q))
    assert rc == 0
    return out


def conv3d_backward(gout, x, offset, mask, weight, has_bias=True, stride=1, padding=0, dilation=1,
                    groups=1, offset_groups=1):
    """Returns (gx, goff, gmask or None, gw, gb or None)."""
    x = _c(x, x)
    gout, offset, mask, weight = (_c(t, x) for t in (gout, offset, mask, weight))
    q = desc3d(x, weight, stride, padding, dilation, groups, offset_groups)
    gx = torch.empty_like(x)
    goff = torch.empty_like(offset)
    gmask = torch.empty_like(mask) if mask is not None else None
    gw = torch.empty_like(weight)
    gb = torch.empty(q.Cout, dtype=x.dtype) if has_bias else None
    fn = getattr(lib(), "oracle_conv3d_backward_" + _sfx(x))
    rc = fn(_p(gout), _p(x), _p(offset), _p(mask), _p(weight), _p(gx), _p(goff), _p(gmask),
            _p(gw), _p(gb), ctypes.byref(q))
    assert rc == 0
    return gx, goff, gmask, gw, gb


def conv3d_corners(x_shape, offset, weight_shape, stride=1, padding=0, dilation=1, offset_groups=1):
    """Per (n, g, k, p): int32 floor(z, y, x) and the uint8 live-corner flags of the forward pass."""
    offset = offset.detach().contiguous()
    x = torch.empty(x_shape, dtype=offset.dtype, device="meta")
    w = torch.empty(weight_shape, dtype=offset.dtype, device="meta")
    q = desc3d(x, w, stride, padding, dilation, 1, offset_groups)
    K = q.kd * q.kh * q.kw
    P = q.Do * q.Ho * q.Wo
    base = torch.empty(q.N, offset_groups * K, P, 3, dtype=torch.int32)
    flags = torch.empty(q.N, offset_groups * K, P, dtype=torch.uint8)
    fn = getattr(lib(), "oracle_conv3d_corners_" + _sfx(offset))
    rc = fn(_p(offset), ctypes.byref(q), _p(base), _p(flags))
    assert rc == 0
    return base, flags


def desc1d(x, weight, stride, padding, dilation, groups, offset_groups):
    N, Cin, L = x.shape
    Cout, _, k = weight.shape
    Lo = output_size(L, k, stride, padding, dilation)
    return Conv1dDesc(N, Cin, Cout, L, k, stride, padding, dilation, groups, offset_groups, Lo)


def _one(v):
    return int(v[0]) if isinstance(v, (tuple, list)) else int(v)


def conv1d_forward(x, offset, mask, weight, bias=None, stride=1, padding=0, dilation=1,
                   groups=1, offset_groups=1):
    x = _c(x, x)
    offset, mask, weight, bias = (_c(t, x) for t in (offset, mask, weight, bias))
    q = desc1d(x, weight, _one(stride), _one(padding), _one(dilation), groups, offset_groups)
    out = torch.empty(q.N, q.Cout, q.Lo, dtype=x.dtype)
    fn = getattr(lib(), "oracle_conv1d_forward_" + _sfx(x))
    rc = fn(_p(x), _p(offset), _p(mask), _p(weight), _p(bias), _p(out), ctypes.byref(q))
    assert rc == 0
    return out


def conv1d_backward(gout, x, offset, mask, weight, has_bias=True, stride=1, padding=0, dilation=1,
                    groups=1, offset_groups=1, quirks=True):
    x = _c(x, x)
    gout, offset, mask, weight = (_c(t, x) for t in (gout, offset, mask, weight))
    q = desc1d(x, weight, _one(stride), _one(padding), _one(dilation), groups, offset_groups)
    gx = torch.empty_like(x)
    goff = torch.empty_like(offset)
    gmask = torch.empty_like(mask) if mask is not None else None
    gw = torch.empty_like(weight)
    gb = torch.empty(q.Cout, dtype=x.dtype) if has_bias else None
    fn = getattr(lib(), "oracle_conv1d_backward_" + _sfx(x))
    rc = fn(_p(gout), _p(x), _p(offset), _p(mask), _p(weight), _p(gx), _p(goff), _p(gmask),
            _p(gw), _p(gb), ctypes.byref(q), ctypes.c_int(1 if quirks else 0))
    assert rc == 0
    return gx, goff, gmask, gw, gb
