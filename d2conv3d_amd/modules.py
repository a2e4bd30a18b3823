"""Self-deforming layers: a zero-initialised Conv3d predicts offsets (and
modulation) for a DeformConv3d with the same geometry.  Mirrors
ops/dconv-native/src/dconv_native/modules.py and the application's superset of
it in network/layers.py:18-313 (norm on the deformation input, `init`,
`size_activation`, the XXZ variant, activation checkpointing).

Constructor arguments follow network/layers.py:27-30; the operator package's
shorter list (modules.py:17-19) is its prefix, and a `deform_param_op` given in
the position of `init` is recognised as such.
"""
import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.nn.modules.utils import _triple
from torch.utils.checkpoint import checkpoint

from .deform_conv import DeformConv3d, deform_conv3d_sized
from .grid import offsets_from_size_map, size_map_offsets


def _apply_size_activation(activation_mode, size_map):
    # network/layers.py:171-181
    if activation_mode == "elu":
        return F.elu(size_map) + 1
    if activation_mode == "relu":
        return F.relu(size_map + 1)
    if activation_mode == "relu_plus_one":
        return F.relu(size_map + 1e-3) + 1
    if activation_mode == "linear":
        return size_map
    raise ValueError(f"Unexpected size activation mode '{activation_mode}'")


_ZERO_OFFSETS = {}


def _zero_offsets(device, n, channels, dims):
    """A float32 tensor of zeros [n, channels, *dims] on `device`, kept for the next call of that shape (a handful of
    shapes at most: the layers of a network at the sizes of its feature maps)."""
    key = (device, n, channels, tuple(dims))
    t = _ZERO_OFFSETS.get(key)
    if t is None:
        if len(_ZERO_OFFSETS) >= 16:
            _ZERO_OFFSETS.clear()
        t = _ZERO_OFFSETS[key] = torch.zeros(n, channels, *dims, device=device)
    return t


def release_zero_offsets():
    """Frees the zero tensors that _branch_conv keeps per feature-map shape (81 x positions floats each)."""
    _ZERO_OFFSETS.clear()


def _branch_conv(layer, x):
    """The deformation branch of a layer: its stock convolution `deform_params` (network/layers.py:66-68).  Where that
    is a plain nn.Conv3d whose shape the matrix-core kernels serve, it is evaluated by the deformable operator at
    all-zero offsets without modulation -- the same convolution (sampling points on the voxels, zero padding outside
    the volume), on this library's kernels instead of the vendor library's im2col + GEMM + col2im: 1.3 - 2.3 times
    faster forward + backward at the reference networks' layer sizes (1024 -> 108 channels, 8x30x54, bfloat16: 2.5
    against 3.6 ms; 256 -> 108, 8x60x107, float32: 4.7 against 10.8 ms).  `layer.branch_on_operator`: True (default) does
    so for bfloat16, where the two convolutions differ by less than either differs from a float64 run of the layer;
    "all" also for float32, where the forward kernel's two-term bfloat16 operands move the predicted offsets by a few
    1e-6 of their size -- enough to put one sampling point in 10^4 .. 10^5 on the other side of a voxel boundary, where
    grad_offset jumps (the layer's grad_input then agrees with a float64 run to 2e-3 instead of 4e-6 in relative
    L2); False keeps the stock call.  Parameters, state dict and initialisation are those of the nn.Conv3d either way."""
    conv = layer.deform_params
    wanted = layer.branch_on_operator
    if (wanted and (x.dtype == torch.bfloat16 or wanted == "all") and type(conv) is nn.Conv3d and x.is_cuda and x.dim() == 5
            and x.dtype in (torch.bfloat16, torch.float32) and conv.weight.dtype == x.dtype and conv.groups == 1
            and conv.padding_mode == "zeros" and not isinstance(conv.padding, str)):
        from . import _ops
        from .deform_conv import deform_conv3d
        k, s, p, d = conv.kernel_size, conv.stride, conv.padding, conv.dilation
        dims = tuple((x.shape[2 + i] + 2 * p[i] - d[i] * (k[i] - 1) - 1) // s[i] + 1 for i in range(3))
        if min(dims) > 0:
            off0 = _zero_offsets(x.device, x.shape[0], 3 * k[0] * k[1] * k[2], dims)
            if _ops.conv3d_algo(x, off0, None, conv.weight, s, p, d, 1, 1) == "mfma":
                return deform_conv3d(x, off0, None, conv.weight, conv.bias, s, p, d, 1, 1)
    return conv(x)


class _DConvBase(nn.Module):
    # (not in the reference: see _branch_conv)
    branch_on_operator = True
    _activations = {
        "sigmoid": torch.sigmoid,
        "relu": torch.relu,
        "tanh": torch.tanh,
        "linear": lambda x: x,
        "none": lambda x: x,
    }
    # network/layers.py:99 wraps the deformation branch in torch.utils.checkpoint;
    # the operator package (modules.py:62-64) does not.  Same numbers either way.
    checkpoint_deformation = False

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, offset_groups=1, bias=True, activation="sigmoid", init="zero",
                 norm_type="none", norm_groups=1, size_activation="elu", deform_param_op=nn.Conv3d):
        super().__init__()
        if not isinstance(init, str):  # modules.py:17-19: 11th positional is deform_param_op
            deform_param_op, init = init, "zero"
        kernel_size = _triple(kernel_size)
        self.num_kernel_points = kernel_size[0] * kernel_size[1] * kernel_size[2]
        self.offset_groups = offset_groups
        self.groups = groups
        self.size_activation = size_activation

        if norm_type not in ("BatchNorm", "GroupNorm", "none"):
            raise ValueError(f"Unexpected norm_type: '{norm_type}'")
        if norm_type == "GroupNorm":
            self.norm = nn.GroupNorm(norm_groups, in_channels)
        elif norm_type == "BatchNorm":
            self.norm = nn.BatchNorm3d(in_channels)
        else:
            self.norm = None

        # construction order deform_params -> deform_conv keeps the RNG stream of the reference
        if isinstance(deform_param_op, nn.Module):
            self.deform_params = deform_param_op
        else:
            self.deform_params = deform_param_op(in_channels, self._deform_channels(), kernel_size,
                                                 stride, padding, dilation, 1, bias)
        self.deform_conv = DeformConv3d(in_channels, out_channels, kernel_size, stride, padding,
                                        dilation, groups, offset_groups, bias)
        self.activation = self._activations[activation] if isinstance(activation, str) else activation
        # (a named activation can run inside the sampler, see _packed_forward)
        self._activation_name = {"none": "linear"}.get(activation, activation) if isinstance(activation, str) else None
        if not isinstance(deform_param_op, nn.Module):
            self._init_deform_params(activation, init)

    def _init_deform_params(self, activation, init):
        # network/layers.py:79-86
        if init == "zero":
            nn.init.zeros_(self.deform_params.weight)
            if self.deform_params.bias is not None:
                nn.init.zeros_(self.deform_params.bias)
        else:
            raise ValueError(f"init scheme {init} not supported")

    def _deform_channels(self):
        return 3 * self.offset_groups * self.num_kernel_points

    def _get_deformation(self, input):
        return _branch_conv(self, input), None

    def forward(self, input):
        deform_input = input if self.norm is None else self.norm(input)
        if self.checkpoint_deformation and torch.is_grad_enabled():
            deformation = checkpoint(self._get_deformation, deform_input, use_reentrant=False)
        else:
            deformation = self._get_deformation(deform_input)
        return self.deform_conv(input, *deformation)


class DConv3d(_DConvBase):
    pass


def _deformation_tensor(layer, input):
    deform_input = input if layer.norm is None else layer.norm(input)
    if layer.checkpoint_deformation and torch.is_grad_enabled():
        return checkpoint(lambda t: _branch_conv(layer, t), deform_input, use_reentrant=False)
    return _branch_conv(layer, deform_input)


def _packed_forward(layer, input, deformation, lead, mode=None, offset_axes=7):
    """The operator on the un-split output of the deformation branch (`lead` channels of offsets or of the raw size
    map, then the raw modulation values): the kernels read both parts where they lie and apply the modulation
    activation themselves; no split copies, no activation kernel, one gradient tensor coming back.  Returns None
    where the matrix-core kernels do not serve the call (the caller then splits and activates as the reference does)."""
    from . import _ops
    dc = layer.deform_conv
    name = layer._activation_name
    if name is None or not _ops.deform_conv3d_packed_supported(input, deformation, dc.weight, lead, name, mode,
                                                             layer.size_activation, dc.stride, dc.padding, dc.dilation,
                                                             dc.groups, dc.offset_groups, offset_axes):
        return None
    from . import _lib
    flags = {"default": _lib.BWD_GW_DEFAULT, "columns": _lib.BWD_GW_COLUMNS, "in_place": _lib.BWD_GW_IN_PLACE,
             "resample": _lib.BWD_GW_RESAMPLE}[dc.backward_memory] | _lib.bwd_slices(dc.backward_slices)
    out = _ops.deform_conv3d_packed(input, deformation, dc.weight, dc.bias, lead, name, dc.stride, dc.padding,
                                    dc.dilation, dc.groups, dc.offset_groups, mode, layer.size_activation,
                                    float(dc.output_relu_scale) if dc.output_relu_scale else 0.0, dc.keep_output_stats,
                                    offset_axes, flags)
    if dc.keep_output_stats:
        out, dc.last_output_stats = out
    return out


def _may_fuse(layer, input):
    return (layer.fused_deformation is True and layer._activation_name is not None and input.is_cuda
            and input.dtype in (torch.float32, torch.bfloat16))


class MDConv3d(_DConvBase):
    # True: the deformation branch's output goes to the operator as it is where the kernels take it (see
    # _packed_forward); False: split + activation in front of the operator, as the reference does
    fused_deformation = True

    def forward(self, input):
        if not _may_fuse(self, input):
            return super().forward(input)
        deformation = _deformation_tensor(self, input)
        out = _packed_forward(self, input, deformation, self.offset_channels)
        if out is not None:
            return out
        offset, alpha = torch.split(deformation, [self.offset_channels, self.alpha_channels], dim=1)
        return self.deform_conv(input, offset, self.activation(alpha))

    def _deform_channels(self):
        self.offset_channels = 3 * self.offset_groups * self.num_kernel_points
        self.alpha_channels = self.offset_groups * self.num_kernel_points
        return self.offset_channels + self.alpha_channels

    def _get_deformation(self, input):
        deformation = _branch_conv(self, input)
        offset, alpha = torch.split(deformation, [self.offset_channels, self.alpha_channels], dim=1)
        return offset, self.activation(alpha)

    def _init_deform_params(self, activation, init):
        # network/layers.py:122-132
        if init == "zero":
            nn.init.zeros_(self.deform_params.weight)
        elif init == "random":
            with torch.no_grad():
                if activation == "sigmoid" or activation == "tanh":
                    nn.init.xavier_normal_(self.deform_params.weight[self.offset_channels:])
                else:
                    nn.init.kaiming_normal_(self.deform_params.weight[self.offset_channels:])
        if self.deform_params.bias is not None:
            nn.init.zeros_(self.deform_params.bias)


def _fixed_axes_in_kernel(layer, input, offsets, alpha):
    """Whether the operator itself can hold the offsets of some axes at zero (descriptor field offset_axes: the
    matrix-core kernels then skip those offset channels and the corners that get weight zero) instead of the
    reference's overwrite of a cloned offsets tensor."""
    if not layer.fixed_axes_in_kernel or not input.is_cuda or input.dtype not in (torch.float32, torch.bfloat16):
        return False
    from . import _ops
    dc = layer.deform_conv
    return _ops.conv3d_algo(input, offsets, alpha, dc.weight, dc.stride, dc.padding, dc.dilation, dc.groups,
                            dc.offset_groups, offset_axes=layer._offset_axes) == "mfma"


class _AxesMixin:
    """dconv_native/modules.py:87-120: the Spatial layers do not displace along the temporal axis (offset channels
    0, 3, 6, ... zero), the Temporal layers displace along it only."""
    _offset_axes = 7              # 1 z | 2 y | 4 x
    fixed_axes_in_kernel = True

    def forward(self, input):
        if isinstance(self, MDConv3d) and self.fixed_axes_in_kernel and _may_fuse(self, input):
            deformation = _deformation_tensor(self, input)
            out = _packed_forward(self, input, deformation, self.offset_channels, offset_axes=self._offset_axes)
            if out is not None:
                return out
            offsets, alpha = torch.split(deformation, [self.offset_channels, self.alpha_channels], dim=1)
            alpha = self.activation(alpha)
        else:
            deform_input = input if self.norm is None else self.norm(input)
            if self.checkpoint_deformation and torch.is_grad_enabled():
                offsets, alpha = checkpoint(super()._get_deformation, deform_input, use_reentrant=False)
            else:
                offsets, alpha = super()._get_deformation(deform_input)
        if _fixed_axes_in_kernel(self, input, offsets, alpha):
            return self.deform_conv(input, offsets, alpha, offset_axes=self._offset_axes)
        offsets = offsets.clone()
        for a in range(3):
            if not (self._offset_axes >> a) & 1:
                offsets[:, a::3] = 0
        return self.deform_conv(input, offsets, alpha)

    def _get_deformation(self, input):
        offsets, alpha = super()._get_deformation(input)
        offsets = offsets.clone()
        for a in range(3):
            if not (self._offset_axes >> a) & 1:
                offsets[:, a::3] = 0
        return offsets, alpha


class _SpatialMixin(_AxesMixin):
    _offset_axes = 6


class _TemporalMixin(_AxesMixin):
    _offset_axes = 1


class SpatialDConv3d(_SpatialMixin, DConv3d):
    pass


class SpatialMDConv3d(_SpatialMixin, MDConv3d):
    pass


class TemporalDConv3d(_TemporalMixin, DConv3d):
    pass


class TemporalMDConv3d(_TemporalMixin, MDConv3d):
    pass


def _sized_forward(layer, input):
    """forward() of the size-conditioned layers with `fused_deformation = True` (the default) on CUDA tensors: the
    predicted size map goes to the operator as it is (deform_conv3d_sized); no [N, 3K, ...] offsets tensor and no
    autograd graph of its expansion exist.  Returns None where that does not apply (CPU tensors, float64)."""
    if layer.fused_deformation is not True or not input.is_cuda or input.dtype == torch.float64:
        return None
    if isinstance(layer, MDConv3d) and _may_fuse(layer, input):
        # the size map and the raw modulation values where the deformation branch wrote them
        deformation = _deformation_tensor(layer, input)
        out = _packed_forward(layer, input, deformation, layer._size_channels, layer._mode)
        if out is not None:
            return out
        size_raw, alpha = torch.split(deformation, [layer._size_channels, layer.alpha_channels], dim=1)
        alpha = layer.activation(alpha)
        dc = layer.deform_conv
        out = deform_conv3d_sized(input, size_raw, alpha, dc.weight, dc.bias, layer._mode, layer.size_activation,
                                  dc.stride, dc.padding, dc.dilation, dc.groups, output_relu=dc.output_relu_scale,
                                  output_stats=dc.keep_output_stats)
        if dc.keep_output_stats:
            out, dc.last_output_stats = out
        return out
    deform_input = input if layer.norm is None else layer.norm(input)
    if layer.checkpoint_deformation and torch.is_grad_enabled():
        size_raw, alpha = checkpoint(layer._get_size_and_alpha, deform_input, use_reentrant=False)
    else:
        size_raw, alpha = layer._get_size_and_alpha(deform_input)
    dc = layer.deform_conv
    out = deform_conv3d_sized(input, size_raw, alpha, dc.weight, dc.bias, layer._mode, layer.size_activation,
                              dc.stride, dc.padding, dc.dilation, dc.groups, output_relu=dc.output_relu_scale,
                              output_stats=dc.keep_output_stats)
    if dc.keep_output_stats:
        out, dc.last_output_stats = out
    return out


def _size_offsets(layer, size_raw):
    """Size activation + offsets_from_size_map as tensors: one library kernel each way for CUDA float32 / bfloat16
    tensors (`fused_deformation = "expand"`), the reference's torch formulation otherwise."""
    if layer.fused_deformation and size_raw.is_cuda and size_raw.dtype in (torch.float32, torch.bfloat16):
        return size_map_offsets(size_raw, layer._mode, layer.deform_conv.kernel_size, layer.deform_conv.dilation,
                                layer.size_activation)
    return offsets_from_size_map(_apply_size_activation(layer.size_activation, size_raw), layer._mode,
                                 layer.deform_conv.kernel_size, layer.deform_conv.dilation)


class _SizeConditionedD(DConv3d):
    """modules.py:123-159 / network/layers.py:184-230: the deformation branch
    predicts a dilation ("size") per location and axis subset; offsets follow
    from offsets_from_size_map.  Emits 3*K offset channels, i.e. offset_groups=1."""
    _size_channels = 1
    _mode = "x"
    fused_deformation = True

    def _deform_channels(self):
        self.offset_channels = self._size_channels
        return self.offset_channels

    def _get_deformation(self, input):
        return _size_offsets(self, _branch_conv(self, input)), None

    def _get_size_and_alpha(self, input):
        return _branch_conv(self, input), None

    def forward(self, input):
        out = _sized_forward(self, input)
        return out if out is not None else super().forward(input)


class _SizeConditionedMD(MDConv3d):
    """modules.py:162-219 / network/layers.py:233-313."""
    _size_channels = 1
    _mode = "x"
    fused_deformation = True

    def _deform_channels(self):
        self.alpha_channels = self.offset_groups * self.num_kernel_points
        self.offset_channels = self._size_channels
        return self.offset_channels + self.alpha_channels

    def _get_deformation(self, input):
        deformation = _branch_conv(self, input)
        size_map, alpha = torch.split(deformation, [self._size_channels, self.alpha_channels], dim=1)
        return _size_offsets(self, size_map), self.activation(alpha)

    def _get_size_and_alpha(self, input):
        deformation = _branch_conv(self, input)
        size_map, alpha = torch.split(deformation, [self._size_channels, self.alpha_channels], dim=1)
        return size_map, self.activation(alpha)

    def forward(self, input):
        out = _sized_forward(self, input)
        return out if out is not None else super().forward(input)


class SizeConditionedDConv3d(_SizeConditionedD):
    _size_channels, _mode = 1, "x"


class XYSizeConditionedDConv3d(_SizeConditionedD):
    _size_channels, _mode = 2, "xy"


class XXZSizeConditionedDConv3d(_SizeConditionedD):
    _size_channels, _mode = 2, "xxz"


class XYZSizeConditionedDConv3d(_SizeConditionedD):
    _size_channels, _mode = 3, "xyz"


class SizeConditionedMDConv3d(_SizeConditionedMD):
    _size_channels, _mode = 1, "x"


class XYSizeConditionedMDConv3d(_SizeConditionedMD):
    _size_channels, _mode = 2, "xy"


class XXZSizeConditionedMDConv3d(_SizeConditionedMD):
    _size_channels, _mode = 2, "xxz"


class XYZSizeConditionedMDConv3d(_SizeConditionedMD):
    _size_channels, _mode = 3, "xyz"


__all__ = [
    "DConv3d", "MDConv3d", "SpatialDConv3d", "SpatialMDConv3d", "TemporalDConv3d", "TemporalMDConv3d",
    "SizeConditionedDConv3d", "XYSizeConditionedDConv3d", "XXZSizeConditionedDConv3d",
    "XYZSizeConditionedDConv3d", "SizeConditionedMDConv3d", "XYSizeConditionedMDConv3d",
    "XXZSizeConditionedMDConv3d", "XYZSizeConditionedMDConv3d",
]
