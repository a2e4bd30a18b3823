"""Plain depthwise conv3d on the HIP library: the Python surface of the
reference's `fast_depthwise_conv3d` package (ops/fast-depthwise-conv3d), which
its backbone and refinement modules use in place of `nn.Conv3d(groups=C)`
(network/backbone/resnet.py:12-16,110; network/modules/refinement.py:18-22).

    depthwise_separable_conv3d(input, weight, bias, stride, padding, dilation)
        <- `_ops.depthwise_separable_conv3d` (csrc/python_bindings.cpp:5,
           csrc/grouped_conv3d.h:108-118; autograd node :29-106)
    DepthwiseConv3d  <- src/fast_depthwise_conv3d/conv.py:7-22
"""
import ctypes

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.nn.modules.utils import _triple

from . import _lib
from ._ops import _DT, _ptr, _stream


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _describe(input, weight, bias, stride, padding, dilation, grad_output=None):
    """conv_depthwise_shape_check (csrc/grouped_conv3d.cu:279-345) and the device / output-size checks of
    conv_depthwise3d_cuda (:392-411), with the reference's messages."""
    for name, v in (("stride", stride), ("padding", padding), ("dilation", dilation)):
        _check(len(v) == 3, f"{name} length should be 3, but got {len(v)}")
    _check(weight is not None, "Weight must be defined.")
    _check(input.dim() in (4, 5), f"Input dimension should be 4D or 5D, got {input.dim()}D")
    _check(weight.dim() == 5, f"Weight dimension should be 5D, got {weight.dim()}D")
    _check(weight.size(1) == 1, f"Depthwise weight should have in_channels=1, got {weight.size(1)}")
    C = input.size(-4)
    _check(weight.size(0) % C == 0,
           f"Depthwise out channels should be a multiple of in channels, got {weight.size(0)} and {C}")
    for i in range(3):
        _check(stride[i] >= 1, f"stride should be at least 1, got {tuple(stride)}")
        _check(padding[i] >= 0, f"padding should be non-negative, got {tuple(padding)}")
        _check(dilation[i] >= 1, f"dilation should be at least 1, got {tuple(dilation)}")
    if bias is not None:
        _check(bias.dim() == 1, f"Bias should be 1D tensor, got {bias.dim()}D")
        _check(bias.size(0) == weight.size(0),
               f"Bias length should be equal to out_channels, got {bias.size(0)} and {weight.size(0)}")
    _check(input.device == weight.device, "expects input and weight tensors to be on the same device.")
    if bias is not None:
        _check(input.device == bias.device, "expects input and bias tensors to be on the same device.")
    if not input.is_cuda:
        raise RuntimeError("depthwise_separable_conv3d: tensors must be on the GPU (this build has no CPU path)")
    if input.dtype not in _DT:
        raise RuntimeError(f"depthwise_separable_conv3d: unsupported dtype {input.dtype}")
    _check(weight.dtype == input.dtype and (bias is None or bias.dtype == input.dtype),
           "expects input, weight and bias of one dtype")
    dims = input.shape[-3:]
    ks = weight.shape[2:]
    out = [(dims[i] + 2 * padding[i] - (dilation[i] * (ks[i] - 1) + 1)) // stride[i] + 1 for i in range(3)]
    for i in range(3):
        _check(out[i] > 0, f"Output size should be positive, got {out[i]} at dim {i + 2}")
    N = input.size(0) if input.dim() == 5 else 1
    if grad_output is not None:
        want = (N, weight.size(0), *out)
        _check(tuple(grad_output.shape[-5:]) == want or tuple(grad_output.shape) == want[1:],
               f"Expect grad_output to be of same shape as output, got {tuple(grad_output.shape)} and {want}")
    return _lib.DwConv3dDesc(N, C, weight.size(0), *dims, *ks, *stride, *padding, *dilation, *out, _DT[input.dtype]), out


class _DepthwiseConv3dFunction(torch.autograd.Function):
    """DepthwiseConv3dFunction (csrc/grouped_conv3d.h:29-106); gradients are computed only where wanted
    (the reference passes `requires_grad` of input, weight and bias as its output mask, :84)."""

    @staticmethod
    def forward(ctx, input, weight, bias, stride, padding, dilation):
        stride, padding, dilation = tuple(stride), tuple(padding), tuple(dilation)
        desc, out_dims = _describe(input, weight, bias, stride, padding, dilation)
        lib = _lib.load()
        x, w = input.contiguous(), weight.contiguous()
        b = bias.contiguous() if bias is not None else None
        out = torch.empty((desc.N, desc.Cout, *out_dims), dtype=x.dtype, device=x.device)
        with torch.cuda.device(x.device):
            rc = lib.d2c_dwconv3d_forward(ctypes.byref(desc), _ptr(x), _ptr(w), _ptr(b), _ptr(out), _stream(x.device))
        _lib.check(rc, "depthwise_separable_conv3d")
        ctx.save_for_backward(x, w)
        ctx.geometry = (stride, padding, dilation, bias is not None, input.dim() == 4)
        return out[0] if input.dim() == 4 else out

    @staticmethod
    def backward(ctx, grad_output):
        x, w = ctx.saved_tensors
        stride, padding, dilation, has_bias, unbatched = ctx.geometry
        desc, _ = _describe(x, w, None, stride, padding, dilation, grad_output)
        lib = _lib.load()
        g = grad_output.contiguous()
        want_x, want_w, want_b = ctx.needs_input_grad[0], ctx.needs_input_grad[1], has_bias and ctx.needs_input_grad[2]
        gx = torch.empty_like(x) if want_x else None
        gw = torch.empty_like(w) if want_w else None
        gb = torch.empty(desc.Cout, dtype=x.dtype, device=x.device) if want_b else None
        nws = lib.d2c_dwconv3d_backward_workspace_bytes(ctypes.byref(desc)) if (want_w or want_b) else 0
        ws = torch.empty(max(nws, 256), dtype=torch.uint8, device=x.device)
        with torch.cuda.device(x.device):
            rc = lib.d2c_dwconv3d_backward(ctypes.byref(desc), _ptr(g), _ptr(x), _ptr(w), _ptr(gx), _ptr(gw), _ptr(gb),
                                           _ptr(ws), nws, _stream(x.device))
        _lib.check(rc, "depthwise_separable_conv3d backward")
        return gx, gw, gb, None, None, None


def depthwise_separable_conv3d(input, weight, bias, stride, padding, dilation):
    """`_ops.depthwise_separable_conv3d` (csrc/grouped_conv3d.h:108-118).  float32, float64 and bfloat16 run as
    they are (sums in float32 / float64); float16, which the reference computes in half with float sums
    (csrc/grouped_conv3d.cu:419), is computed in float32 and returned as float16."""
    stride, padding, dilation = _triple(stride), _triple(padding), _triple(dilation)
    if input.dtype == torch.float16:
        out = _DepthwiseConv3dFunction.apply(input.float(), weight.float(), None if bias is None else bias.float(),
                                             stride, padding, dilation)
        return out.half()
    return _DepthwiseConv3dFunction.apply(input, weight, bias, stride, padding, dilation)


class DepthwiseConv3d(nn.Conv3d):
    """src/fast_depthwise_conv3d/conv.py:7-22: an `nn.Conv3d` with groups = in_channels (the `groups` argument
    is accepted and ignored, as there) whose forward pass runs the depthwise kernels."""

    def __init__(self, in_channels, out_channels, kernel_size=1, stride=1, padding=0, dilation=1, groups=None,
                 bias=True, padding_mode="zeros"):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, in_channels, bias,
                         padding_mode)

    def forward(self, input):
        weight = self.weight.to(dtype=input.dtype)
        bias = None if self.bias is None else self.bias.to(dtype=input.dtype)
        if self.padding_mode != "zeros":
            return depthwise_separable_conv3d(
                F.pad(input, self._reversed_padding_repeated_twice, mode=self.padding_mode), weight, bias,
                self.stride, (0, 0, 0), self.dilation)
        return depthwise_separable_conv3d(input, weight, bias, self.stride, self.padding, self.dilation)


def install_as_fast_depthwise_conv3d():
    """Registers this module under the reference's import name, so that
    `from fast_depthwise_conv3d import DepthwiseConv3d` (network/backbone/resnet.py:12) resolves here."""
    import sys
    import types
    pkg = types.ModuleType("fast_depthwise_conv3d")
    pkg.DepthwiseConv3d = DepthwiseConv3d
    ops = types.ModuleType("fast_depthwise_conv3d._ops")
    ops.depthwise_separable_conv3d = depthwise_separable_conv3d
    pkg._ops = ops
    sys.modules.setdefault("fast_depthwise_conv3d", pkg)
    sys.modules.setdefault("fast_depthwise_conv3d._ops", ops)
    return sys.modules["fast_depthwise_conv3d"]
