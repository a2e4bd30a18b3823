"""Counterpart of the reference's native module `dconv_native._ops`
(ops/dconv-native/csrc/ops/dconv.cpp:6-12): `deform_conv1d`, `deform_conv3d`
with the flat argument lists of dconv1d.h:161-172 / dconv3d.h:188-205, and the
`config` sub-namespace.  Autograd lives here (torch.autograd.Function) and the
arithmetic in the C-ABI HIP library.
"""
import ctypes
import types

import torch
from torch.autograd.function import once_differentiable

from . import _lib

_DT = {torch.float32: _lib.D2C_F32, torch.float64: _lib.D2C_F64, torch.bfloat16: _lib.D2C_BF16}


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _stream(dev):
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


# One workspace tensor per (device, stream), grown when a call needs more and handed to every call on that stream:
# the kernels of a stream run one after the other, so they can share it, and a training step does not allocate (and
# hold in the caching allocator, beside whatever else is cached) its largest workspace anew per layer call.  Calls
# recorded into a HIP graph take a tensor of their own from the graph's pool, as any other tensor made under capture.
_WS_CACHE = {}
_WS_CACHE_ON = [True]


def _workspace(nbytes, dev):
    if nbytes == 0:
        return None
    if not _WS_CACHE_ON[0] or torch.cuda.is_current_stream_capturing():
        return torch.empty(nbytes, dtype=torch.uint8, device=dev)
    dev = torch.device(dev)
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    key = (index, torch.cuda.current_stream(dev).cuda_stream)
    ws = _WS_CACHE.get(key)
    if ws is None or ws.numel() < nbytes:
        _WS_CACHE.pop(key, None)      # (the old one goes back to the allocator before the new one is asked for)
        ws = None
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        _WS_CACHE[key] = ws
    return ws


def _release_workspaces():
    """Drops the cached workspace tensors (they return to torch's caching allocator)."""
    _WS_CACHE.clear()


def _set_workspace_caching(on):
    _WS_CACHE_ON[0] = bool(on)
    if not on:
        _WS_CACHE.clear()


def _workspace_bytes_cached():
    return {k: v.numel() for k, v in _WS_CACHE.items()}


def _check_common(nd, input, offset, alpha, weight, bias, groups, offset_groups):
    """SANITY_CHECK_DCONV_INPUTS / _GROUPS of dconv_gpu_common.h:17-43."""
    def req(cond, msg):
        if not cond:
            raise RuntimeError(f"deform_conv{nd}d: {msg}")
    for name, t in (("input", input), ("offset", offset), ("weight", weight)):
        req(isinstance(t, torch.Tensor), f"{name} must be a Tensor")
        req(t.dim() == nd + 2, f"{name}.ndimension() == {nd + 2} failed (got {t.dim()})")
    if alpha is not None:
        req(alpha.dim() == nd + 2, f"alpha.ndimension() == {nd + 2} failed (got {alpha.dim()})")
    if bias is not None:
        req(bias.dim() == 1, "bias.ndimension() == 1 failed")
    for name, t in (("input", input), ("offset", offset), ("alpha", alpha), ("weight", weight), ("bias", bias)):
        if t is not None:
            req(t.is_cuda, f"{name}.device().is_cuda() failed: this operator has GPU kernels only")
            req(t.device == input.device, f"{name} is on {t.device}, input on {input.device}")
    req(offset.size(0) == input.size(0), "offset.size(0) == input.size(0) failed")
    if alpha is not None:
        req(alpha.size(0) == input.size(0), "alpha.size(0) == input.size(0) failed")
    req(groups > 0 and offset_groups > 0, "group counts must be positive")
    K = 1
    for k in weight.shape[2:]:
        K *= k
    req(weight.size(1) * groups == input.size(1), "weight.size(1) * n_weight_groups == input.size(1) failed")
    req(weight.size(0) % groups == 0, "weight.size(0) % n_weight_groups == 0 failed")
    req(weight.size(0) % offset_groups == 0, "weight.size(0) % n_offset_groups == 0 failed")
    req(input.size(1) % offset_groups == 0, "input.size(1) % n_offset_groups == 0 failed")
    req(offset.size(1) == offset_groups * nd * K,
        f"offset.size(1) == n_offset_groups * {nd} * num_kernel_points failed "
        f"(got {offset.size(1)}, expected {offset_groups * nd * K})")
    if alpha is not None:
        req(alpha.size(1) == offset_groups * K,
            f"alpha.size(1) == n_offset_groups * num_kernel_points failed "
            f"(got {alpha.size(1)}, expected {offset_groups * K})")
        req(tuple(alpha.shape[2:]) == tuple(offset.shape[2:]),
            f"mask output dims do not match computed dims. Got: {tuple(alpha.shape[2:])} "
            f"but expected: {tuple(offset.shape[2:])}")
    if bias is not None:
        req(bias.size(0) == weight.size(0), "bias.size(0) == weight.size(0) failed")


def _unify(input, offset, alpha, weight, bias):
    """Element types handed to the library: x/weight/bias share `dtype`;
    offset/mask share `aux_dtype` (= dtype, or float32 next to bfloat16 data)."""
    dt = input.dtype
    if dt not in _DT:
        raise RuntimeError(f"deform_conv: unsupported input dtype {dt}")
    weight = weight.to(dt)
    bias = bias.to(dt) if bias is not None else None
    if dt == torch.bfloat16:
        adt = torch.bfloat16 if (offset.dtype == torch.bfloat16 and
                                 (alpha is None or alpha.dtype == torch.bfloat16)) else torch.float32
    else:
        adt = dt
    offset = offset.to(adt)
    alpha = alpha.to(adt) if alpha is not None else None
    return input, offset, alpha, weight, bias


class PreparedRegion:
    """What a layer keeps between calls for the matrix-core kernels (d2c_conv3d_*_prepared): the channels-last copy of
    the last input and the weights in the kernels' operand orders, in one device buffer, with the bookkeeping that
    says which parts still belong to the tensors of the next call.  One per layer; not shared between layers."""

    def __init__(self):
        self.buf = None
        self.input_token = 0          # bumped by every forward call: the buffer holds the copy of that call's input
        self.fwd_weights = None       # (data_ptr, version, shape) of the weight tensor whose forward operand is held
        self.bwd_weights = None

    def buffer(self, nbytes, dev):
        if self.buf is None or self.buf.numel() < nbytes or self.buf.device != dev:
            self.buf = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            self.fwd_weights = self.bwd_weights = None
            self.input_token += 1
        return self.buf

    @staticmethod
    def key(t):
        return (t.data_ptr(), t._version, tuple(t.shape), t.dtype)


# The sampled columns of a forward call kept for its backward call (d2c_conv3d_forward_columns): taps x the size of
# the input, held from the forward to the backward pass of a step, in exchange for the backward pass's second
# sampling pass.  On where the description is served, grad_weight is wanted and the buffer stays under the limit.
_KEEP_COLUMNS = {"on": True, "max_bytes": 4 << 30}


def _set_keep_columns(on=True, max_bytes=None):
    _KEEP_COLUMNS["on"] = bool(on)
    if max_bytes is not None:
        _KEEP_COLUMNS["max_bytes"] = int(max_bytes)


def _columns_for(lib, desc, sdesc, weight_grad_wanted, dev):
    if not (_KEEP_COLUMNS["on"] and weight_grad_wanted):
        return None
    n = lib.d2c_conv3d_columns_bytes(ctypes.byref(desc), ctypes.byref(sdesc) if sdesc is not None else None)
    if n == 0 or n > _KEEP_COLUMNS["max_bytes"]:
        return None
    try:
        return torch.empty(n, dtype=torch.uint8, device=dev)
    except torch.cuda.OutOfMemoryError:
        return None      # (no room to keep them: the backward pass samples again)


class _DeformConv3dFunction(torch.autograd.Function):
    """DeformConv3dFunction of dconv3d.h:70-186.  `relu_scale` > 0 (not in the reference) makes the forward
    kernels store relu_scale * max(out, 0) -- the activation that follows the convolution, fused into their last
    step; the backward pass then starts from grad_out * relu_scale where the stored output is positive."""

    @staticmethod
    def forward(ctx, input, offset, alpha, weight, bias, sd, sh, sw, pd, ph, pw, dd, dh, dw, groups, offset_groups,
                relu_scale=0.0, want_stats=False, offset_axes=7, backward_flags=0, prepared=None):
        lib = _lib.load()
        input, offset, weight = input.contiguous(), offset.contiguous(), weight.contiguous()
        alpha = alpha.contiguous() if alpha is not None else None
        bias = bias.contiguous() if bias is not None else None
        N, Cin, D, H, W = input.shape
        Cout, _, kd, kh, kw = weight.shape
        Do, Ho, Wo = offset.shape[2:]
        desc = _lib.Conv3dDesc(N, Cin, Cout, D, H, W, kd, kh, kw, sd, sh, sw, pd, ph, pw, dd, dh, dw,
                               groups, offset_groups, Do, Ho, Wo, _DT[input.dtype], _DT[offset.dtype],
                               _lib.EPILOGUE_RELU if relu_scale > 0 else _lib.EPILOGUE_NONE, float(relu_scale) or 1.0,
                               int(offset_axes), int(backward_flags))
        _lib.check(lib.d2c_conv3d_check(ctypes.byref(desc)), "deform_conv3d")
        dev = input.device
        out = torch.empty((N, Cout, Do, Ho, Wo), dtype=input.dtype, device=dev)
        stats = torch.empty((N, Cout, 2), dtype=torch.float32, device=dev) if want_stats else None
        with torch.cuda.device(dev):
            nb = (lib.d2c_conv3d_forward_stats_workspace_bytes(ctypes.byref(desc), None) if want_stats
                  else lib.d2c_conv3d_forward_workspace_bytes(ctypes.byref(desc)))
            ws = _workspace(nb, dev)
            npre = lib.d2c_conv3d_prepared_bytes(ctypes.byref(desc)) if (prepared is not None and not want_stats) else 0
            ctx.prepared = None
            columns = None
            if want_stats:
                rc = lib.d2c_conv3d_forward_stats(ctypes.byref(desc), None, _ptr(input), _ptr(offset), _ptr(alpha),
                                                  _ptr(weight), _ptr(bias), _ptr(out), _ptr(stats), _ptr(ws), nb,
                                                  _stream(dev))
            elif npre:
                # the layer's prepared region: forward weights kept while the weight tensor is the same, the input's
                # channels-last copy left there for the backward call of this forward call
                buf = prepared.buffer(npre, dev)
                wkey = PreparedRegion.key(weight)
                reuse = _lib.REUSE_FORWARD_WEIGHTS if prepared.fwd_weights == wkey else 0
                rc = lib.d2c_conv3d_forward_prepared(ctypes.byref(desc), _ptr(input), _ptr(offset), _ptr(alpha),
                                                     _ptr(weight), _ptr(bias), _ptr(out), _ptr(buf), buf.numel(), reuse,
                                                     _ptr(ws), nb, _stream(dev))
                prepared.fwd_weights = wkey
                prepared.input_token += 1
                ctx.prepared, ctx.input_token = prepared, prepared.input_token
            else:
                columns = _columns_for(lib, desc, None, ctx.needs_input_grad[3], dev)
                if columns is not None:
                    rc = lib.d2c_conv3d_forward_columns(ctypes.byref(desc), None, _ptr(input), _ptr(offset), _ptr(alpha),
                                                        _ptr(weight), _ptr(bias), _ptr(out), _ptr(columns),
                                                        columns.numel(), _ptr(ws), nb, _stream(dev))
                else:
                    rc = lib.d2c_conv3d_forward(ctypes.byref(desc), _ptr(input), _ptr(offset), _ptr(alpha),
                                                _ptr(weight), _ptr(bias), _ptr(out), _ptr(ws), nb, _stream(dev))
        _lib.check(rc, "deform_conv3d forward")
        ctx.save_for_backward(input, offset, alpha, weight, bias, out if relu_scale > 0 else None, columns)
        ctx.desc = desc
        ctx.relu_scale = float(relu_scale)
        if want_stats:
            ctx.mark_non_differentiable(stats)
            return out, stats
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out, _grad_stats=None):
        lib = _lib.load()
        input, offset, alpha, weight, bias, out, columns = ctx.saved_tensors
        desc = ctx.desc
        dev = input.device
        grad_out = grad_out.contiguous().to(input.dtype)
        if out is not None:    # gradient with respect to the value before the fused activation
            grad_out = torch.where(out > 0, grad_out * ctx.relu_scale, torch.zeros_like(grad_out))
        need = ctx.needs_input_grad
        gx = torch.empty_like(input) if need[0] else None
        goff = torch.empty_like(offset) if need[1] else None
        galpha = torch.empty_like(alpha) if (alpha is not None and need[2]) else None
        gw = torch.empty_like(weight) if need[3] else None
        gb = torch.empty_like(bias) if (bias is not None and need[4]) else None
        prepared = getattr(ctx, "prepared", None)
        with torch.cuda.device(dev):
            nb = (lib.d2c_conv3d_backward_columns_workspace_bytes(ctypes.byref(desc), None) if columns is not None
                  else lib.d2c_conv3d_backward_workspace_bytes(ctypes.byref(desc)))
            ws = _workspace(nb, dev)
            if columns is not None:
                # (the columns the forward call of this step kept: no second sampling pass)
                rc = lib.d2c_conv3d_backward_columns(ctypes.byref(desc), None, _ptr(grad_out), _ptr(input), _ptr(offset),
                                                     _ptr(alpha), _ptr(weight), _ptr(columns), columns.numel(),
                                                     _ptr(gx), _ptr(goff), _ptr(galpha), _ptr(gw), _ptr(gb), _ptr(ws),
                                                     nb, _stream(dev))
            elif prepared is not None and prepared.buf is not None:
                # (the region still holds this call's input unless another forward call has used it since)
                wkey = PreparedRegion.key(weight)
                reuse = (_lib.REUSE_INPUT if prepared.input_token == ctx.input_token else 0) | \
                        (_lib.REUSE_BACKWARD_WEIGHTS if prepared.bwd_weights == wkey else 0)
                rc = lib.d2c_conv3d_backward_prepared(ctypes.byref(desc), _ptr(grad_out), _ptr(input), _ptr(offset),
                                                      _ptr(alpha), _ptr(weight), _ptr(gx), _ptr(goff), _ptr(galpha),
                                                      _ptr(gw), _ptr(gb), _ptr(prepared.buf), prepared.buf.numel(), reuse,
                                                      _ptr(ws), nb, _stream(dev))
                prepared.bwd_weights = wkey
                if not reuse & _lib.REUSE_INPUT:
                    prepared.input_token += 1          # (the region now holds THIS input's copy, nobody's token)
            else:
                rc = lib.d2c_conv3d_backward(ctypes.byref(desc), _ptr(grad_out), _ptr(input), _ptr(offset), _ptr(alpha),
                                             _ptr(weight), _ptr(gx), _ptr(goff), _ptr(galpha), _ptr(gw), _ptr(gb),
                                             _ptr(ws), nb, _stream(dev))
        _lib.check(rc, "deform_conv3d backward")
        return (gx, goff, galpha, gw, gb) + (None,) * 16


def deform_conv3d(input, offset, alpha, weight, bias, stride_d, stride_h, stride_w, pad_d, pad_h, pad_w,
                  dilation_d, dilation_h, dilation_w, groups, offset_groups, relu_scale=0.0, want_stats=False,
                  offset_axes=7, backward_flags=0, prepared=None):
    """deform_conv3d of dconv3d.h:188-226; `alpha` and `bias` may be None.  `relu_scale` > 0 fuses
    relu_scale * relu(.) into the store of the output (see _DeformConv3dFunction).  `want_stats` also returns the
    float32 [N, Cout, 2] sums and sums of squares of the stored output per (sample, channel), added up by the
    forward kernels where they store (the statistics a GroupNorm behind the convolution needs).  `offset_axes`: mask
    of the axes (1 z, 2 y, 4 x) the offsets displace along; the others are taken as zero and their gradient
    channels come back zero (matrix-core kernels only, see conv3d_algo).  `backward_flags`: the description's field
    of that name (_lib.BWD_GW_* | _lib.bwd_slices(n)): how the backward pass trades workspace for time.  `prepared`: a
    PreparedRegion kept by the calling layer (see DeformConv3d.reuse_prepared)."""
    _check_common(3, input, offset, alpha, weight, bias, groups, offset_groups)
    input, offset, alpha, weight, bias = _unify(input, offset, alpha, weight, bias)
    return _DeformConv3dFunction.apply(
        input, offset, alpha, weight, bias, int(stride_d), int(stride_h), int(stride_w),
        int(pad_d), int(pad_h), int(pad_w), int(dilation_d), int(dilation_h), int(dilation_w),
        int(groups), int(offset_groups), float(relu_scale), bool(want_stats), int(offset_axes), int(backward_flags),
        prepared)


class _DeformConv3dSizedFunction(torch.autograd.Function):
    """The deformable convolution of the size-conditioned layers (network/layers.py:184-313) with the predicted size
    map as its input: size activation, expansion to tap offsets (utils/grid.py:72-98) and the operator itself in
    d2c_conv3d_sized_forward / _backward.  No offsets tensor and no gradient of one exist where the matrix-core
    kernels serve the call."""

    @staticmethod
    def forward(ctx, input, size_raw, alpha, weight, bias, mode, activation, stride, padding, dilation, groups,
                relu_scale=0.0, want_stats=False):
        from .grid import size_map_desc
        lib = _lib.load()
        input, size_raw, weight = input.contiguous(), size_raw.contiguous(), weight.contiguous()
        alpha = alpha.contiguous() if alpha is not None else None
        bias = bias.contiguous() if bias is not None else None
        N, Cin, D, H, W = input.shape
        Cout, _, kd, kh, kw = weight.shape
        Do, Ho, Wo = size_raw.shape[2:]
        desc = _lib.Conv3dDesc(N, Cin, Cout, D, H, W, kd, kh, kw, *stride, *padding, *dilation, groups, 1, Do, Ho, Wo,
                               _DT[input.dtype], _DT[size_raw.dtype],
                               _lib.EPILOGUE_RELU if relu_scale > 0 else _lib.EPILOGUE_NONE, float(relu_scale) or 1.0)
        sdesc = size_map_desc(size_raw, mode, (kd, kh, kw), dilation, activation)
        _lib.check(lib.d2c_conv3d_check(ctypes.byref(desc)), "deform_conv3d_sized")
        dev = input.device
        out = torch.empty((N, Cout, Do, Ho, Wo), dtype=input.dtype, device=dev)
        stats = torch.empty((N, Cout, 2), dtype=torch.float32, device=dev) if want_stats else None
        with torch.cuda.device(dev):
            nb = (lib.d2c_conv3d_forward_stats_workspace_bytes(ctypes.byref(desc), ctypes.byref(sdesc)) if want_stats
                  else lib.d2c_conv3d_sized_forward_workspace_bytes(ctypes.byref(desc), ctypes.byref(sdesc)))
            ws = _workspace(nb, dev)
            columns = None
            if want_stats:
                rc = lib.d2c_conv3d_forward_stats(ctypes.byref(desc), ctypes.byref(sdesc), _ptr(input), _ptr(size_raw),
                                                  _ptr(alpha), _ptr(weight), _ptr(bias), _ptr(out), _ptr(stats),
                                                  _ptr(ws), nb, _stream(dev))
            else:
                columns = _columns_for(lib, desc, sdesc, ctx.needs_input_grad[3], dev)
                if columns is not None:
                    rc = lib.d2c_conv3d_forward_columns(ctypes.byref(desc), ctypes.byref(sdesc), _ptr(input),
                                                        _ptr(size_raw), _ptr(alpha), _ptr(weight), _ptr(bias), _ptr(out),
                                                        _ptr(columns), columns.numel(), _ptr(ws), nb, _stream(dev))
                else:
                    rc = lib.d2c_conv3d_sized_forward(ctypes.byref(desc), ctypes.byref(sdesc), _ptr(input),
                                                      _ptr(size_raw), _ptr(alpha), _ptr(weight), _ptr(bias), _ptr(out),
                                                      _ptr(ws), nb, _stream(dev))
        _lib.check(rc, "deform_conv3d_sized forward")
        ctx.save_for_backward(input, size_raw, alpha, weight, bias, out if relu_scale > 0 else None, columns)
        ctx.desc, ctx.sdesc = desc, sdesc
        ctx.relu_scale = float(relu_scale)
        if want_stats:
            ctx.mark_non_differentiable(stats)
            return out, stats
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out, _grad_stats=None):
        lib = _lib.load()
        input, size_raw, alpha, weight, bias, out, columns = ctx.saved_tensors
        desc, sdesc = ctx.desc, ctx.sdesc
        dev = input.device
        grad_out = grad_out.contiguous().to(input.dtype)
        if out is not None:    # gradient with respect to the value before the fused activation
            grad_out = torch.where(out > 0, grad_out * ctx.relu_scale, torch.zeros_like(grad_out))
        need = ctx.needs_input_grad
        gx = torch.empty_like(input) if need[0] else None
        gsize = torch.empty_like(size_raw) if need[1] else None
        galpha = torch.empty_like(alpha) if (alpha is not None and need[2]) else None
        gw = torch.empty_like(weight) if need[3] else None
        gb = torch.empty_like(bias) if (bias is not None and need[4]) else None
        with torch.cuda.device(dev):
            if columns is not None:
                nb = lib.d2c_conv3d_backward_columns_workspace_bytes(ctypes.byref(desc), ctypes.byref(sdesc))
                ws = _workspace(nb, dev)
                rc = lib.d2c_conv3d_backward_columns(ctypes.byref(desc), ctypes.byref(sdesc), _ptr(grad_out), _ptr(input),
                                                     _ptr(size_raw), _ptr(alpha), _ptr(weight), _ptr(columns),
                                                     columns.numel(), _ptr(gx), _ptr(gsize), _ptr(galpha), _ptr(gw),
                                                     _ptr(gb), _ptr(ws), nb, _stream(dev))
            else:
                nb = lib.d2c_conv3d_sized_backward_workspace_bytes(ctypes.byref(desc), ctypes.byref(sdesc))
                ws = _workspace(nb, dev)
                rc = lib.d2c_conv3d_sized_backward(ctypes.byref(desc), ctypes.byref(sdesc), _ptr(grad_out), _ptr(input),
                                                   _ptr(size_raw), _ptr(alpha), _ptr(weight), _ptr(gx), _ptr(gsize),
                                                   _ptr(galpha), _ptr(gw), _ptr(gb), _ptr(ws), nb, _stream(dev))
        _lib.check(rc, "deform_conv3d_sized backward")
        return (gx, gsize, galpha, gw, gb) + (None,) * 8


def deform_conv3d_sized(input, size_raw, alpha, weight, bias, mode, activation, stride, padding, dilation, groups=1,
                        relu_scale=0.0, want_stats=False):
    """Deformable convolution whose tap offsets follow from a predicted size map:
    deform_conv3d(input, offsets_from_size_map(size_activation(size_raw), mode, kernel, dilation), alpha, ...)
    of network/layers.py:184-313 as one operator.  `size_raw` [N, 3|2|2|1, Do, Ho, Wo] for mode xyz|xxz|xy|x."""
    from torch.nn.modules.utils import _triple
    stride, padding, dilation = (tuple(int(v) for v in _triple(t)) for t in (stride, padding, dilation))
    mode = mode.lower()
    want_c = {"xyz": 3, "xxz": 2, "xy": 2, "x": 1}[mode]
    K = weight.shape[2] * weight.shape[3] * weight.shape[4]
    if size_raw.dim() != 5 or size_raw.shape[1] != want_c:
        raise RuntimeError(f"deform_conv3d_sized: mode '{mode}' wants {want_c} size channels, got {tuple(size_raw.shape)}")
    if not size_raw.is_cuda or size_raw.device != input.device:
        raise RuntimeError("deform_conv3d_sized: size_raw must be on the input's GPU")
    # the operator's own checks, with (a view shaped like) the offsets tensor the size map stands for
    stand_in = size_raw.new_empty(1).expand((size_raw.shape[0], 3 * K) + tuple(size_raw.shape[2:]))
    _check_common(3, input, stand_in, alpha, weight, bias, groups, 1)
    input, size_raw, alpha, weight, bias = _unify(input, size_raw, alpha, weight, bias)
    return _DeformConv3dSizedFunction.apply(input, size_raw, alpha, weight, bias, mode, activation, stride, padding,
                                            dilation, int(groups), float(relu_scale), bool(want_stats))


def _ptr_at(t, channel):
    """Device pointer of t[:, channel] of a contiguous [N, C, *spatial] tensor (first sample)."""
    per_channel = 1
    for d in t.shape[2:]:
        per_channel *= d
    return ctypes.c_void_p(t.data_ptr() + channel * per_channel * t.element_size())


class _DeformConv3dPackedFunction(torch.autograd.Function):
    """The operator fed by the output of the layer's deformation branch as it is (network/layers.py:107-132,
    :233-313): `deformation` [N, lead + G*K, Do, Ho, Wo] holds the offsets (lead = 3*G*K channels) or the raw size map
    (lead = 1 | 2 | 3 channels, `mode` given) in front of the raw modulation values.  The kernels read both parts
    inside that tensor (description field deform_channels) and apply the modulation activation where they read a
    mask value (mask_activation); the backward pass writes one gradient tensor of the same shape, the modulation
    part with respect to the raw values.  No split copies and no activation kernels in either direction."""

    @staticmethod
    def forward(ctx, input, deformation, weight, bias, lead, mask_act, mode, size_activation, stride, padding,
                dilation, groups, offset_groups, relu_scale, want_stats, offset_axes, backward_flags):
        lib = _lib.load()
        input, deformation, weight = input.contiguous(), deformation.contiguous(), weight.contiguous()
        bias = bias.contiguous() if bias is not None else None
        N, Cin, D, H, W = input.shape
        Cout, _, kd, kh, kw = weight.shape
        Ctot = deformation.shape[1]
        Do, Ho, Wo = deformation.shape[2:]
        desc = _lib.Conv3dDesc(N, Cin, Cout, D, H, W, kd, kh, kw, *stride, *padding, *dilation, groups, offset_groups,
                               Do, Ho, Wo, _DT[input.dtype], _DT[deformation.dtype],
                               _lib.EPILOGUE_RELU if relu_scale > 0 else _lib.EPILOGUE_NONE, float(relu_scale) or 1.0,
                               int(offset_axes), int(backward_flags), Ctot, int(mask_act))
        sdesc = None
        if mode is not None:
            from .grid import size_map_desc
            sdesc = size_map_desc(deformation, mode, (kd, kh, kw), dilation, size_activation)
        sref = ctypes.byref(sdesc) if sdesc is not None else None
        _lib.check(lib.d2c_conv3d_check(ctypes.byref(desc)), "deform_conv3d_packed")
        dev = input.device
        out = torch.empty((N, Cout, Do, Ho, Wo), dtype=input.dtype, device=dev)
        stats = torch.empty((N, Cout, 2), dtype=torch.float32, device=dev) if want_stats else None
        p_off, p_mask = _ptr_at(deformation, 0), _ptr_at(deformation, lead)
        columns = None
        with torch.cuda.device(dev):
            if not want_stats:
                columns = _columns_for(lib, desc, sdesc, ctx.needs_input_grad[2], dev)
            if columns is not None:
                nb = (lib.d2c_conv3d_sized_forward_workspace_bytes(ctypes.byref(desc), sref) if sdesc is not None
                      else lib.d2c_conv3d_forward_workspace_bytes(ctypes.byref(desc)))
                ws = _workspace(nb, dev)
                rc = lib.d2c_conv3d_forward_columns(ctypes.byref(desc), sref, _ptr(input), p_off, p_mask, _ptr(weight),
                                                    _ptr(bias), _ptr(out), _ptr(columns), columns.numel(), _ptr(ws), nb,
                                                    _stream(dev))
            elif want_stats:
                nb = lib.d2c_conv3d_forward_stats_workspace_bytes(ctypes.byref(desc), sref)
                ws = _workspace(nb, dev)
                rc = lib.d2c_conv3d_forward_stats(ctypes.byref(desc), sref, _ptr(input), p_off, p_mask, _ptr(weight),
                                                  _ptr(bias), _ptr(out), _ptr(stats), _ptr(ws), nb, _stream(dev))
            elif sdesc is not None:
                nb = lib.d2c_conv3d_sized_forward_workspace_bytes(ctypes.byref(desc), sref)
                ws = _workspace(nb, dev)
                rc = lib.d2c_conv3d_sized_forward(ctypes.byref(desc), sref, _ptr(input), p_off, p_mask, _ptr(weight),
                                                  _ptr(bias), _ptr(out), _ptr(ws), nb, _stream(dev))
            else:
                nb = lib.d2c_conv3d_forward_workspace_bytes(ctypes.byref(desc))
                ws = _workspace(nb, dev)
                rc = lib.d2c_conv3d_forward(ctypes.byref(desc), _ptr(input), p_off, p_mask, _ptr(weight), _ptr(bias),
                                            _ptr(out), _ptr(ws), nb, _stream(dev))
        _lib.check(rc, "deform_conv3d_packed forward")
        ctx.save_for_backward(input, deformation, weight, bias, out if relu_scale > 0 else None, columns)
        ctx.desc, ctx.sdesc, ctx.lead = desc, sdesc, lead
        ctx.relu_scale = float(relu_scale)
        if want_stats:
            ctx.mark_non_differentiable(stats)
            return out, stats
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out, _grad_stats=None):
        lib = _lib.load()
        input, deformation, weight, bias, out, columns = ctx.saved_tensors
        desc, sdesc = ctx.desc, ctx.sdesc
        dev = input.device
        grad_out = grad_out.contiguous().to(input.dtype)
        if out is not None:
            grad_out = torch.where(out > 0, grad_out * ctx.relu_scale, torch.zeros_like(grad_out))
        need = ctx.needs_input_grad
        gx = torch.empty_like(input) if need[0] else None
        gdef = torch.empty_like(deformation) if need[1] else None
        gw = torch.empty_like(weight) if need[2] else None
        gb = torch.empty_like(bias) if (bias is not None and need[3]) else None
        p_off, p_mask = _ptr_at(deformation, 0), _ptr_at(deformation, ctx.lead)
        g_off = _ptr_at(gdef, 0) if gdef is not None else ctypes.c_void_p(0)
        g_mask = _ptr_at(gdef, ctx.lead) if gdef is not None else ctypes.c_void_p(0)
        with torch.cuda.device(dev):
            if columns is not None:
                sref = ctypes.byref(sdesc) if sdesc is not None else None
                nb = lib.d2c_conv3d_backward_columns_workspace_bytes(ctypes.byref(desc), sref)
                ws = _workspace(nb, dev)
                rc = lib.d2c_conv3d_backward_columns(ctypes.byref(desc), sref, _ptr(grad_out), _ptr(input), p_off, p_mask,
                                                     _ptr(weight), _ptr(columns), columns.numel(), _ptr(gx), g_off, g_mask,
                                                     _ptr(gw), _ptr(gb), _ptr(ws), nb, _stream(dev))
            elif sdesc is not None:
                nb = lib.d2c_conv3d_sized_backward_workspace_bytes(ctypes.byref(desc), ctypes.byref(sdesc))
                ws = _workspace(nb, dev)
                rc = lib.d2c_conv3d_sized_backward(ctypes.byref(desc), ctypes.byref(sdesc), _ptr(grad_out), _ptr(input),
                                                   p_off, p_mask, _ptr(weight), _ptr(gx), g_off, g_mask, _ptr(gw),
                                                   _ptr(gb), _ptr(ws), nb, _stream(dev))
            else:
                nb = lib.d2c_conv3d_backward_workspace_bytes(ctypes.byref(desc))
                ws = _workspace(nb, dev)
                rc = lib.d2c_conv3d_backward(ctypes.byref(desc), _ptr(grad_out), _ptr(input), p_off, p_mask,
                                             _ptr(weight), _ptr(gx), g_off, g_mask, _ptr(gw), _ptr(gb), _ptr(ws), nb,
                                             _stream(dev))
        _lib.check(rc, "deform_conv3d_packed backward")
        return (gx, gdef, gw, gb) + (None,) * 13


def deform_conv3d_packed_supported(input, deformation, weight, lead, mask_activation, mode, size_activation, stride,
                                   padding, dilation, groups, offset_groups, offset_axes=7):
    """Whether the kernels take the deformation tensor as it is for these arguments (matrix-core family, both
    directions); where not, the caller splits it and applies the activation itself."""
    if (not input.is_cuda or input.dtype not in (torch.float32, torch.bfloat16) or deformation.device != input.device
            or mask_activation not in _lib.MASK_ACTIVATIONS):
        return False
    lib = _lib.load()
    adt = deformation.dtype if (deformation.dtype == input.dtype or
                                (input.dtype == torch.bfloat16 and deformation.dtype == torch.float32)) else None
    if adt is None:
        return False
    N, Cin, D, H, W = input.shape
    Cout, _, kd, kh, kw = weight.shape
    Do, Ho, Wo = deformation.shape[2:]
    desc = _lib.Conv3dDesc(N, Cin, Cout, D, H, W, kd, kh, kw, *stride, *padding, *dilation, groups, offset_groups,
                           Do, Ho, Wo, _DT[input.dtype], _DT[adt], _lib.EPILOGUE_NONE, 1.0, int(offset_axes), 0,
                           deformation.shape[1], _lib.MASK_ACTIVATIONS[mask_activation])
    sdesc = None
    if mode is not None:
        from .grid import size_map_desc
        sdesc = size_map_desc(deformation, mode, (kd, kh, kw), dilation, size_activation)
    with torch.cuda.device(input.device):
        return bool(lib.d2c_conv3d_packed_supported(ctypes.byref(desc), ctypes.byref(sdesc) if sdesc is not None else None))


def deform_conv3d_packed(input, deformation, weight, bias, lead, mask_activation, stride, padding, dilation, groups,
                         offset_groups, mode=None, size_activation="linear", relu_scale=0.0, want_stats=False,
                         offset_axes=7, backward_flags=0):
    """deform_conv3d / deform_conv3d_sized on the un-split output of the deformation branch: see
    _DeformConv3dPackedFunction.  `lead`: channels in front of the modulation values (3*G*K offsets, or the size
    map's 1 | 2 | 3 with `mode`); `mask_activation`: "sigmoid" | "relu" | "tanh" | "linear"."""
    K = weight.shape[2] * weight.shape[3] * weight.shape[4]
    GK = offset_groups * K
    if deformation.dim() != 5 or deformation.shape[1] != lead + GK:
        raise RuntimeError(f"deform_conv3d_packed: deformation must have {lead} + {GK} channels, got {tuple(deformation.shape)}")
    if mode is None and lead != 3 * GK:
        raise RuntimeError(f"deform_conv3d_packed: {3 * GK} offset channels expected in front of the modulation, got {lead}")
    stand_in = deformation.new_empty(1)
    _check_common(3, input, stand_in.expand((deformation.shape[0], 3 * GK) + tuple(deformation.shape[2:])),
                  stand_in.expand((deformation.shape[0], GK) + tuple(deformation.shape[2:])), weight, bias, groups,
                  offset_groups)
    weight = weight.to(input.dtype)
    bias = bias.to(input.dtype) if bias is not None else None
    if not (deformation.dtype == input.dtype or (input.dtype == torch.bfloat16 and deformation.dtype == torch.float32)):
        deformation = deformation.to(torch.float32 if input.dtype == torch.bfloat16 else input.dtype)
    return _DeformConv3dPackedFunction.apply(
        input, deformation, weight, bias, int(lead), _lib.MASK_ACTIVATIONS[mask_activation], mode, size_activation,
        tuple(int(v) for v in stride), tuple(int(v) for v in padding), tuple(int(v) for v in dilation), int(groups),
        int(offset_groups), float(relu_scale), bool(want_stats), int(offset_axes), int(backward_flags))


class _GroupNormFromStats(torch.autograd.Function):
    """torch.nn.functional.group_norm on the output of a convolution whose forward kernels already added up the
    per-(sample, channel) sums (d2c_conv3d_forward_stats): d2c_group_norm_forward / _backward."""

    @staticmethod
    def forward(ctx, x, stats, weight, bias, groups, eps):
        lib = _lib.load()
        x = x.contiguous()
        N, C = x.shape[:2]
        P = x[0, 0].numel()
        desc = _lib.GroupNormDesc(N, C, P, groups, _DT[x.dtype], eps)
        weight = weight.to(x.dtype).contiguous() if weight is not None else None
        bias = bias.to(x.dtype).contiguous() if bias is not None else None
        y = torch.empty_like(x)
        with torch.cuda.device(x.device):
            rc = lib.d2c_group_norm_forward(ctypes.byref(desc), _ptr(x), _ptr(stats), _ptr(weight), _ptr(bias), _ptr(y),
                                            _stream(x.device))
        _lib.check(rc, "group_norm forward")
        ctx.save_for_backward(x, stats, weight)
        ctx.desc = desc
        ctx.has_affine = (weight is not None, bias is not None)
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_y):
        lib = _lib.load()
        x, stats, weight = ctx.saved_tensors
        desc = ctx.desc
        grad_y = grad_y.contiguous().to(x.dtype)
        need = ctx.needs_input_grad
        gx = torch.empty_like(x) if need[0] else None
        gw = torch.empty(desc.C, dtype=x.dtype, device=x.device) if (ctx.has_affine[0] and need[2]) else None
        gb = torch.empty(desc.C, dtype=x.dtype, device=x.device) if (ctx.has_affine[1] and need[3]) else None
        with torch.cuda.device(x.device):
            nb = lib.d2c_group_norm_backward_workspace_bytes(ctypes.byref(desc))
            ws = _workspace(nb, x.device)
            rc = lib.d2c_group_norm_backward(ctypes.byref(desc), _ptr(grad_y), _ptr(x), _ptr(stats), _ptr(weight),
                                             _ptr(gx), _ptr(gw), _ptr(gb), _ptr(ws), nb, _stream(x.device))
        _lib.check(rc, "group_norm backward")
        return gx, None, gw, gb, None, None


def group_norm_from_stats(x, stats, weight, bias, groups, eps=1e-5):
    """GroupNorm of `x` [N, C, *spatial] (CUDA, float32 or bfloat16) from `stats` [N, C, 2] = per (sample, channel)
    sum and sum of squares of x in float32, as the convolutions return them with want_stats."""
    if not x.is_cuda or x.dtype not in (torch.float32, torch.bfloat16):
        raise RuntimeError("group_norm_from_stats: CUDA float32 / bfloat16 tensors only")
    if stats.shape != (x.shape[0], x.shape[1], 2) or stats.dtype != torch.float32 or stats.device != x.device:
        raise RuntimeError(f"group_norm_from_stats: stats must be float32 [N, C, 2] on the input's GPU, got {tuple(stats.shape)}")
    if x.shape[1] % groups != 0:
        raise RuntimeError("group_norm_from_stats: groups must divide the channel count")
    return _GroupNormFromStats.apply(x, stats.contiguous(), weight, bias, int(groups), float(eps))


def channel_stats(x):
    """float32 [N, C, 2]: per (sample, channel) sum and sum of squares of x (d2c_channel_stats)."""
    lib = _lib.load()
    x = x.contiguous()
    N, C = x.shape[:2]
    desc = _lib.GroupNormDesc(N, C, x[0, 0].numel(), 1, _DT[x.dtype], 0.0)
    stats = torch.empty((N, C, 2), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        rc = lib.d2c_channel_stats(ctypes.byref(desc), _ptr(x), _ptr(stats), _stream(x.device))
    _lib.check(rc, "channel_stats")
    return stats


class _DeformConv1dFunction(torch.autograd.Function):
    """DeformConv1dFunction of dconv1d.h:69-159."""

    @staticmethod
    def forward(ctx, input, offset, alpha, weight, bias, stride, pad, dilation, groups, offset_groups, quirks):
        lib = _lib.load()
        input, offset, weight = input.contiguous(), offset.contiguous(), weight.contiguous()
        alpha = alpha.contiguous() if alpha is not None else None
        bias = bias.contiguous() if bias is not None else None
        N, Cin, L = input.shape
        Cout, _, k = weight.shape
        Lo = offset.shape[2]
        desc = _lib.Conv1dDesc(N, Cin, Cout, L, k, stride, pad, dilation, groups, offset_groups, Lo,
                               _DT[input.dtype], _DT[offset.dtype], 1 if quirks else 0)
        _lib.check(lib.d2c_conv1d_check(ctypes.byref(desc)), "deform_conv1d")
        dev = input.device
        out = torch.empty((N, Cout, Lo), dtype=input.dtype, device=dev)
        with torch.cuda.device(dev):
            nb = lib.d2c_conv1d_forward_workspace_bytes(ctypes.byref(desc))
            ws = _workspace(nb, dev)
            rc = lib.d2c_conv1d_forward(ctypes.byref(desc), _ptr(input), _ptr(offset), _ptr(alpha), _ptr(weight),
                                        _ptr(bias), _ptr(out), _ptr(ws), nb, _stream(dev))
        _lib.check(rc, "deform_conv1d forward")
        ctx.save_for_backward(input, offset, alpha, weight, bias)
        ctx.desc = desc
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out):
        lib = _lib.load()
        input, offset, alpha, weight, bias = ctx.saved_tensors
        desc = ctx.desc
        dev = input.device
        grad_out = grad_out.contiguous().to(input.dtype)
        need = ctx.needs_input_grad
        gx = torch.empty_like(input) if need[0] else None
        goff = torch.empty_like(offset) if need[1] else None
        galpha = torch.empty_like(alpha) if (alpha is not None and need[2]) else None
        gw = torch.empty_like(weight) if need[3] else None
        gb = torch.empty_like(bias) if (bias is not None and need[4]) else None
        with torch.cuda.device(dev):
            nb = lib.d2c_conv1d_backward_workspace_bytes(ctypes.byref(desc))
            ws = _workspace(nb, dev)
            rc = lib.d2c_conv1d_backward(ctypes.byref(desc), _ptr(grad_out), _ptr(input), _ptr(offset), _ptr(alpha),
                                         _ptr(weight), _ptr(gx), _ptr(goff), _ptr(galpha), _ptr(gw), _ptr(gb),
                                         _ptr(ws), nb, _stream(dev))
        _lib.check(rc, "deform_conv1d backward")
        return (gx, goff, galpha, gw, gb) + (None,) * 6


def _one(v):
    return int(v[0]) if isinstance(v, (tuple, list)) else int(v)


def deform_conv1d(input, offset, alpha, weight, bias, stride, pad, dilation, groups, offset_groups,
                  reference_quirks=True):
    """deform_conv1d of dconv1d.h:161-187.  Unlike the reference binding, which
    takes plain ints and defined tensors only, 1-tuples for stride / pad /
    dilation and None for `alpha` / `bias` are accepted (DeformConv1d.forward,
    deform_conv.py:168-172, passes exactly those)."""
    _check_common(1, input, offset, alpha, weight, bias, groups, offset_groups)
    input, offset, alpha, weight, bias = _unify(input, offset, alpha, weight, bias)
    return _DeformConv1dFunction.apply(
        input, offset, alpha, weight, bias, _one(stride), _one(pad), _one(dilation),
        int(groups), int(offset_groups), bool(reference_quirks))


def _get_max_intermediate_elements():
    return int(_lib.load().d2c_get_max_intermediate_elements())


def _set_max_intermediate_elements(m):
    _lib.load().d2c_set_max_intermediate_elements(int(m))


# dconv.cpp:9-11.  Kept for interface parity: no column buffer is ever
# materialised here, so the limit changes nothing.
config = types.SimpleNamespace(
    get_max_intermediate_elements=_get_max_intermediate_elements,
    set_max_intermediate_elements=_set_max_intermediate_elements,
    # not in the reference: the workspace tensors this layer keeps per (device, stream)
    release_workspaces=_release_workspaces,
    set_workspace_caching=_set_workspace_caching,
    cached_workspace_bytes=_workspace_bytes_cached,
    # not in the reference: whether forward calls keep their sampled columns for the backward call (and up to what size)
    set_keep_columns=_set_keep_columns,
    keep_columns=lambda: dict(_KEEP_COLUMNS),
)


def conv3d_corner_index(input_shape, offset, kernel_size, stride=(1, 1, 1), padding=(0, 0, 0),
                        dilation=(1, 1, 1), offset_groups=1):
    """Debug output of the sampler: per (n, g*K+k, p) the int32 floor of the
    sampling position and the uint8 set of corners the forward pass reads."""
    lib = _lib.load()
    offset = offset.contiguous()
    if offset.dtype == torch.bfloat16:
        offset = offset.float()
    N, Cin, D, H, W = input_shape
    kd, kh, kw = kernel_size
    Do, Ho, Wo = offset.shape[2:]
    dt = _DT[offset.dtype]
    desc = _lib.Conv3dDesc(N, Cin, Cin, D, H, W, kd, kh, kw, *stride, *padding, *dilation,
                           1, offset_groups, Do, Ho, Wo, dt, dt)
    K = kd * kh * kw
    base = torch.empty((N, offset_groups * K, Do * Ho * Wo, 3), dtype=torch.int32, device=offset.device)
    flags = torch.empty((N, offset_groups * K, Do * Ho * Wo), dtype=torch.uint8, device=offset.device)
    with torch.cuda.device(offset.device):
        rc = lib.d2c_conv3d_corner_index(ctypes.byref(desc), _ptr(offset), _ptr(base), _ptr(flags),
                                         _stream(offset.device))
    _lib.check(rc, "conv3d_corner_index")
    return base, flags


def conv3d_sample(src, offset, kernel_size, stride=(1, 1, 1), padding=(0, 0, 0), dilation=(1, 1, 1), offset_groups=1):
    """`src` [N, Cs, D, H, W] read at every sampling point of an offset field [N, G*3*K, Do, Ho, Wo] with the forward
    pass's trilinear rule (d2c_conv3d_sample): [N, G*K*Cs, Do, Ho, Wo], channel (g*K + k)*Cs + c."""
    lib = _lib.load()
    if not src.is_cuda or src.dtype not in _DT or offset.device != src.device:
        raise RuntimeError("conv3d_sample: CUDA tensors of float32 / float64 / bfloat16 on one device")
    src, offset = src.contiguous(), offset.contiguous()
    if src.dtype == torch.bfloat16:
        offset = offset.to(torch.bfloat16 if offset.dtype == torch.bfloat16 else torch.float32)
    else:
        offset = offset.to(src.dtype)
    N, Cs, D, H, W = src.shape
    kd, kh, kw = kernel_size
    K = kd * kh * kw
    Do, Ho, Wo = offset.shape[2:]
    if offset.shape[0] != N or offset.shape[1] != offset_groups * 3 * K:
        raise RuntimeError(f"conv3d_sample: offset must be [N, {offset_groups * 3 * K}, ...], got {tuple(offset.shape)}")
    G = offset_groups
    desc = _lib.Conv3dDesc(N, G, G, D, H, W, kd, kh, kw, *stride, *padding, *dilation, 1, G, Do, Ho, Wo,
                           _DT[src.dtype], _DT[offset.dtype])
    out = torch.empty((N, G * K * Cs, Do, Ho, Wo), dtype=src.dtype, device=src.device)
    with torch.cuda.device(src.device):
        rc = lib.d2c_conv3d_sample(ctypes.byref(desc), Cs, _ptr(src), _ptr(offset), _ptr(out), _stream(src.device))
    _lib.check(rc, "conv3d_sample")
    return out


def conv3d_offset_histogram(offset, kernel_size, offset_groups=1, bins=64, lo=-8.0, hi=8.0):
    """int64 [3, bins + 2]: per axis (z, y, x) the histogram of an offset field [N, G*3*K, Do, Ho, Wo] over `bins`
    equal-width bins of [lo, hi), with the counts below lo in column 0 and at or above hi in the last column
    (d2c_conv3d_offset_histogram)."""
    lib = _lib.load()
    offset = offset.contiguous()
    if not offset.is_cuda or offset.dtype not in _DT:
        raise RuntimeError("conv3d_offset_histogram: a CUDA tensor of float32 / float64 / bfloat16")
    kd, kh, kw = kernel_size
    N = offset.shape[0]
    Do, Ho, Wo = offset.shape[2:]
    G = offset_groups
    if offset.shape[1] != G * 3 * kd * kh * kw:
        raise RuntimeError(f"conv3d_offset_histogram: offset must be [N, {G * 3 * kd * kh * kw}, ...], got {tuple(offset.shape)}")
    dt = _DT[offset.dtype]
    # (only the offsets' own shape matters; any input volume with this output size passes the check)
    desc = _lib.Conv3dDesc(N, G, G, Do, Ho, Wo, 1, 1, 1, 1, 1, 1, 0, 0, 0, 1, 1, 1, 1, G, Do, Ho, Wo,
                           dt if dt != _lib.D2C_BF16 else _lib.D2C_BF16, dt)
    desc.kd, desc.kh, desc.kw = kd, kh, kw
    desc.pd, desc.ph, desc.pw = kd // 2, kh // 2, kw // 2
    desc.D, desc.H, desc.W = Do + (kd - 1) - 2 * (kd // 2), Ho + (kh - 1) - 2 * (kh // 2), Wo + (kw - 1) - 2 * (kw // 2)
    hist = torch.empty((3, bins + 2), dtype=torch.int64, device=offset.device)
    with torch.cuda.device(offset.device):
        rc = lib.d2c_conv3d_offset_histogram(ctypes.byref(desc), _ptr(offset), float(lo), float(hi), int(bins),
                                             _ptr(hist), _stream(offset.device))
    _lib.check(rc, "conv3d_offset_histogram")
    return hist


def conv3d_algo(input, offset, alpha, weight, stride=(1, 1, 1), padding=(0, 0, 0), dilation=(1, 1, 1),
                groups=1, offset_groups=1, offset_axes=7, as_dtype=None):
    """Name of the kernel family ("generic", "mfma", "depthwise") these arguments are served by; "invalid" when
    none takes them (a partial `offset_axes` on a shape the matrix-core kernels do not serve in both directions).
    `as_dtype`: answer for tensors of this element type instead of the ones given (no tensor is converted)."""
    lib = _lib.load()
    dt = input.dtype if as_dtype is None else as_dtype
    if dt not in _DT:
        raise RuntimeError(f"deform_conv: unsupported input dtype {dt}")
    adt = dt
    if dt == torch.bfloat16 and not (offset.dtype == torch.bfloat16 and (alpha is None or alpha.dtype == torch.bfloat16)):
        adt = torch.float32
    N, Cin, D, H, W = input.shape
    Cout, _, kd, kh, kw = weight.shape
    Do, Ho, Wo = offset.shape[2:]
    desc = _lib.Conv3dDesc(N, Cin, Cout, D, H, W, kd, kh, kw, *stride, *padding, *dilation,
                           groups, offset_groups, Do, Ho, Wo, _DT[dt], _DT[adt],
                           _lib.EPILOGUE_NONE, 1.0, int(offset_axes))
    return _lib.ALGO_NAMES.get(lib.d2c_conv3d_algo(ctypes.byref(desc)), "invalid")


def conv1d_algo(input, offset, alpha, weight, stride=1, padding=0, dilation=1, groups=1, offset_groups=1):
    """Name of the kernel family ("generic" or "mfma") that serves these 1-D arguments."""
    lib = _lib.load()
    input, offset, alpha, weight, _ = _unify(input, offset, alpha, weight, None)
    N, Cin, L = input.shape
    Cout, _, k = weight.shape
    desc = _lib.Conv1dDesc(N, Cin, Cout, L, k, _one(stride), _one(padding), _one(dilation), groups, offset_groups,
                           offset.shape[2], _DT[input.dtype], _DT[offset.dtype], 1)
    return _lib.ALGO_NAMES.get(lib.d2c_conv1d_algo(ctypes.byref(desc)), "invalid")


def set_algo_override(name):
    """Test hook: force "generic" / "mfma" / "depthwise", or None for the default choice."""
    code = {None: _lib.ALGO_AUTO, "auto": _lib.ALGO_AUTO, "generic": _lib.ALGO_GENERIC,
            "mfma": _lib.ALGO_MFMA, "depthwise": _lib.ALGO_DEPTHWISE}[name]
    _lib.load().d2c_set_algo_override(code)


def set_grad_weight_mode(mode):
    """Test hook for the matrix-core kernels: "columns" (default; grad_weight as a matrix product over the sampled
    columns that the offset / mask gradient kernel writes), "in_place" (bfloat16: the same, the columns written over
    the grad-column rows: no buffer of their own, grad_input taken from the rows first; float32 problems sample
    again) or "resample" (the grad-weight kernel samples the input again)."""
    _lib.load().d2c_set_grad_weight_mode(mode if isinstance(mode, int)
                                         else {"columns": 1, "in_place": 2, "resample": 0}[mode])


def set_backward_slices(n):
    """Test hook: number of slices over the offset groups that the matrix-core backward pass of bfloat16 problems
    runs in (0: the library's choice, 1: one pass over all groups)."""
    _lib.load().d2c_set_backward_slices(int(n))


def set_grad_input_mode(mode):
    """Test hook: "lists" (default; grad_input gathered from per-voxel sample lists, every element
    written once), "atomics" (scatter with fp32 atomics like the reference), or an int n >= 2: lists of
    at most n samples per voxel, the rest taking the overflow path."""
    _lib.load().d2c_set_grad_input_mode(mode if isinstance(mode, int) else {"lists": 1, "atomics": 0}[mode])
