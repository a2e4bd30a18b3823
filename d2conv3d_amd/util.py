"""nn.Conv3d -> deformable layer replacement, mirroring
ops/dconv-native/src/dconv_native/util.py and utils/replace.py:11-82.
"""
import torch
import torch.nn as nn

from .modules import *  # noqa: F401,F403  (the reference's util.py re-exports the layer classes)
from . import modules as _m


def replace_module(replacement_func, replaced_cls, module, **kwargs):
    """util.py:4-21: depth-first replacement; returns (module, number of replacements)."""
    n_conversions = 0
    module_output = module
    if isinstance(module, replaced_cls):
        module_output = replacement_func(module, **kwargs)
        n_conversions += 1 if module_output is not module else 0
    for name, child in module.named_children():
        converted, conversions = replace_module(replacement_func, replaced_cls, child, **kwargs)
        module_output.add_module(name, converted)
        n_conversions += conversions
    return module_output, n_conversions


# util.py:24-37 and utils/replace.py:30-47 (union of both name tables)
_dconv_versions = {
    "DCNv1": _m.DConv3d,
    "DCNv2": _m.MDConv3d,
    "SpatialDCNv1": _m.SpatialDConv3d,
    "SpatialDCNv2": _m.SpatialMDConv3d,
    "TemporalDCNv1": _m.TemporalDConv3d,
    "TemporalDCNv2": _m.TemporalMDConv3d,
    "ConditionedDCNv1": _m.SizeConditionedDConv3d,
    "SizeConditionedDCNv1": _m.SizeConditionedDConv3d,
    "XYConditionedDCNv1": _m.XYSizeConditionedDConv3d,
    "XYSizeConditionedDCNv1": _m.XYSizeConditionedDConv3d,
    "XXZConditionedDCNv1": _m.XXZSizeConditionedDConv3d,
    "XYZConditionedDCNv1": _m.XYZSizeConditionedDConv3d,
    "XYZSizeConditionedDCNv1": _m.XYZSizeConditionedDConv3d,
    "ConditionedDCNv2": _m.SizeConditionedMDConv3d,
    "SizeConditionedDCNv2": _m.SizeConditionedMDConv3d,
    "XYConditionedDCNv2": _m.XYSizeConditionedMDConv3d,
    "XYSizeConditionedDCNv2": _m.XYSizeConditionedMDConv3d,
    "XXZConditionedDCNv2": _m.XXZSizeConditionedMDConv3d,
    "XYZConditionedDCNv2": _m.XYZSizeConditionedMDConv3d,
    "XYZSizeConditionedDCNv2": _m.XYZSizeConditionedMDConv3d,
}


def dconv_replace_layer(conv_module, **kwargs):
    """utils/replace.py:48-78: 1x1x1 kernels are kept unless `replace_1x1_kernels`;
    weight and bias of the convolution are carried over."""
    if not kwargs.get("replace_1x1_kernels") and conv_module.kernel_size == (1, 1, 1):
        return conv_module
    DC = _dconv_versions[kwargs["version"]]
    dconv = DC(
        conv_module.in_channels, conv_module.out_channels, conv_module.kernel_size,
        conv_module.stride, conv_module.padding, conv_module.dilation, conv_module.groups,
        kwargs.get("offset_groups", 1), conv_module.bias is not None,
        kwargs.get("activation", "sigmoid"), kwargs.get("init", "zero"),
        kwargs.get("norm_type", "none"), kwargs.get("norm_groups", 1),
        kwargs.get("size_activation", "elu"),
    )
    dconv.deform_conv.weight.data = conv_module.weight.data.detach()
    if conv_module.bias is not None:
        dconv.deform_conv.bias.data = conv_module.bias.data.detach()
    return dconv


def add_deformable_conv(module, **kwargs):
    """util.py:62-63."""
    return replace_module(dconv_replace_layer, nn.Conv3d, module, **kwargs)


SCALED_RELU = 1.71285855    # network/layers.py:409-411


def fuse_output_activation(module):
    """Folds the activation that follows a deformable convolution into the convolution's forward kernels: in
    every nn.Sequential under `module` a D2Conv layer directly followed by nn.ReLU or by a ScaledReLU
    (network/layers.py:414-419; recognised by its class name) -- the `_conv` blocks of the reference's
    refinement modules, network/modules/refinement.py:38-43 -- keeps its place, the activation becomes
    nn.Identity and the layer's DeformConv3d stores scale * relu(out) itself.  Returns the number of fused pairs.
    State-dict keys do not change (neither activation has parameters)."""
    fused = 0
    for seq in [m for m in module.modules() if isinstance(m, nn.Sequential)]:
        names = list(seq._modules)
        for a, b in zip(names, names[1:]):
            conv, act = seq._modules[a], seq._modules[b]
            if not isinstance(conv, _m._DConvBase) or conv.deform_conv.output_relu_scale is not None:
                continue
            if isinstance(act, nn.ReLU):
                scale = 1.0
            elif type(act).__name__ == "ScaledReLU":
                scale = SCALED_RELU
            else:
                continue
            conv.deform_conv.output_relu_scale = scale
            seq._modules[b] = nn.Identity()
            fused += 1
    return fused


class ConvActGroupNorm(nn.Sequential):
    """Sequential(deformable convolution, ReLU | ScaledReLU | Identity, GroupNorm) -- the `_conv` block of the
    reference's refinement modules (network/modules/refinement.py:38-43) -- run as two kernels' worth of passes:
    the convolution applies the activation where it stores its output and adds up the per-channel sums on the
    way, and the normalisation is one pass over the output from those sums (no statistics pass).  Children keep
    their places and names, so state-dict keys do not change.  CPU / float64 inputs take the plain sequence."""

    def forward(self, input):
        conv, act, norm = self[0], self[1], self[2]
        dc = conv.deform_conv
        if not input.is_cuda or input.dtype == torch.float64:
            return norm(act(conv(input)))
        from . import _ops
        dc.keep_output_stats = True
        try:
            out = conv(input)            # the activation is folded into the convolution (output_relu_scale)
            stats = dc.last_output_stats
        finally:
            dc.keep_output_stats = False
            dc.last_output_stats = None
        return _ops.group_norm_from_stats(out, stats, norm.weight, norm.bias, norm.num_groups, norm.eps)


def fuse_conv_act_norm(module):
    """Turns every nn.Sequential of exactly (D2Conv layer, nn.ReLU | ScaledReLU | nn.Identity, nn.GroupNorm) under
    `module` into a ConvActGroupNorm (in place: same children, same state-dict keys).  Returns their number."""
    fused = 0
    fuse_output_activation(module)
    for parent in list(module.modules()):
        for name, seq in list(parent.named_children()):
            if type(seq) is not nn.Sequential or len(seq) != 3:
                continue
            conv, act, norm = seq[0], seq[1], seq[2]
            if not (isinstance(conv, _m._DConvBase) and isinstance(norm, nn.GroupNorm)):
                continue
            if not (isinstance(act, nn.Identity) and conv.deform_conv.output_relu_scale is not None):
                continue
            block = ConvActGroupNorm()
            for n, child in seq.named_children():
                block.add_module(n, child)
            setattr(parent, name, block)
            fused += 1
    return fused


def tap_statistics(input_shape, offset, kernel_size, stride=(1, 1, 1), padding=(0, 0, 0), dilation=(1, 1, 1),
                   offset_groups=1):
    """How much of an offset field samples outside the volume: the debug output the reference's trainer expects
    from a `tools.hooks.oob_tracking` hook that its repository does not contain (trainer.py:99-101).

    Counts come from the sampler's own bookkeeping (the set of corners the forward pass reads per tap,
    dconv3d_gpu.cu:59-86), so they are exact for the kernel that runs.  Returns a dict:
      taps            number of (sample, offset group, tap, position) sampling points
      dead            fraction whose value is 0 by the early-out (no corner read)
      partial         fraction read with at least one corner outside the volume
      corners_read    fraction of all 8 * taps corner values that are read
    """
    import torch
    from . import _ops
    _, flags = _ops.conv3d_corner_index(tuple(input_shape), offset, tuple(kernel_size), tuple(stride), tuple(padding),
                                        tuple(dilation), offset_groups)
    n = flags.numel()
    f = flags.to(torch.int32)
    dead = int((f == 0).sum())
    full = int((f == 255).sum())
    bits = sum(((f >> c) & 1).sum() for c in range(8))
    return {"taps": n, "dead": dead / n, "partial": (n - dead - full) / n, "corners_read": int(bits) / (8.0 * n)}


def offset_histogram(offset, kernel_size=(3, 3, 3), offset_groups=1, bins=64, value_range=(-8.0, 8.0)):
    """Histogram of an offset field per axis (z, y, x): int64 [3, bins + 2] with the counts below / at or above
    `value_range` in the first / last column.  With tap_statistics, the debug output that the reference's trainer
    expects from its missing `tools.hooks.oob_tracking` hook (trainer.py:99-101)."""
    from . import _ops
    return _ops.conv3d_offset_histogram(offset, tuple(kernel_size), offset_groups, bins, value_range[0], value_range[1])


def sample_at_taps(src, offset, kernel_size=(3, 3, 3), stride=(1, 1, 1), padding=(1, 1, 1), dilation=(1, 1, 1),
                   offset_groups=1):
    """`src` [N, Cs, D, H, W] read at every sampling point of the offset field, [N, G*K*Cs, Do, Ho, Wo]: what the
    reference's modulation loss gets from grid_sample on a zero-padded ground-truth mask (loss/region.py:97-125),
    with the sampler's own rules."""
    from . import _ops
    return _ops.conv3d_sample(src, offset, tuple(kernel_size), tuple(stride), tuple(padding), tuple(dilation),
                              offset_groups)
