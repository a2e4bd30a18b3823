"""MI355X-native D2Conv3D operator path: modulated deformable conv3d,
dynamic-dilation conv3d and deformable conv1d, forward and backward, as
hand-written HIP kernels for gfx950 behind the Python surface of the
reference's `dconv_native` package (ops/dconv-native/src/dconv_native).
"""
from .deform_conv import deform_conv1d, deform_conv3d, deform_conv3d_sized
from .deform_conv import DeformConv1d, DeformConv3d, DeformConvNd
from .modules import (
    DConv3d, MDConv3d, SpatialDConv3d, SpatialMDConv3d, TemporalDConv3d, TemporalMDConv3d,
    SizeConditionedDConv3d, SizeConditionedMDConv3d,
    XYSizeConditionedDConv3d, XYSizeConditionedMDConv3d,
    XXZSizeConditionedDConv3d, XXZSizeConditionedMDConv3d,
    XYZSizeConditionedDConv3d, XYZSizeConditionedMDConv3d,
)
from .grid import offsets_from_size_map
from .util import add_deformable_conv
from .depthwise_conv import DepthwiseConv3d, depthwise_separable_conv3d, install_as_fast_depthwise_conv3d

__all__ = [
    "deform_conv1d", "deform_conv3d", "deform_conv3d_sized", "DeformConv1d", "DeformConv3d", "DeformConvNd",
    "DConv3d", "MDConv3d", "SpatialDConv3d", "SpatialMDConv3d", "TemporalDConv3d", "TemporalMDConv3d",
    "SizeConditionedDConv3d", "SizeConditionedMDConv3d",
    "XYSizeConditionedDConv3d", "XYSizeConditionedMDConv3d",
    "XXZSizeConditionedDConv3d", "XXZSizeConditionedMDConv3d",
    "XYZSizeConditionedDConv3d", "XYZSizeConditionedMDConv3d",
    "offsets_from_size_map", "add_deformable_conv", "install_as_dconv_native",
    "DepthwiseConv3d", "depthwise_separable_conv3d", "install_as_fast_depthwise_conv3d",
]


def install_as_dconv_native():
    """Registers this package under the reference's import name, so that
    `from dconv_native import DeformConv3d` (network/layers.py:9,
    network/modules/bridging.py:5) and `from dconv_native.deform_conv import
    DeformConvNd` (loss/util.py:4) resolve here without touching those files."""
    import sys
    from . import _ops, deform_conv, grid, modules, util
    me = sys.modules[__name__]
    sys.modules.setdefault("dconv_native", me)
    for name, mod in (("_ops", _ops), ("deform_conv", deform_conv), ("grid", grid),
                      ("modules", modules), ("util", util)):
        sys.modules.setdefault("dconv_native." + name, mod)
    return me
