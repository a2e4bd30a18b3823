"""ctypes binding of libd2conv.so, the C-ABI HIP library (include/d2conv.h).

There is no fallback: if the library has not been built, or a call fails, an
exception is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libd2conv.so")

D2C_F32, D2C_F64, D2C_BF16 = 0, 1, 2
ALGO_AUTO, ALGO_GENERIC, ALGO_MFMA, ALGO_DEPTHWISE = 0, 1, 2, 3
PROF_FWD, PROF_BWD_DATA, PROF_BWD_WEIGHT, PROF_PACK, PROF_GX_OWNER, PROF_BWD_AUX = 0, 1, 2, 3, 4, 5
ALGO_NAMES = {ALGO_GENERIC: "generic", ALGO_MFMA: "mfma", ALGO_DEPTHWISE: "depthwise"}

# every symbol that include/d2conv.h declares
EXPORTS = (
    "d2c_output_size", "d2c_conv3d_check", "d2c_conv3d_algo", "d2c_conv3d_packed_supported",
    "d2c_conv3d_forward_workspace_bytes", "d2c_conv3d_backward_workspace_bytes",
    "d2c_conv3d_forward", "d2c_conv3d_backward", "d2c_conv3d_forward_static", "d2c_static_workspace_bytes",
    "d2c_conv3d_prepared_bytes", "d2c_conv3d_forward_prepared", "d2c_conv3d_backward_prepared",
    "d2c_conv3d_columns_bytes", "d2c_conv3d_forward_columns", "d2c_conv3d_backward_columns_workspace_bytes",
    "d2c_conv3d_backward_columns",
    "d2c_conv1d_check", "d2c_conv1d_algo", "d2c_conv1d_forward_workspace_bytes", "d2c_conv1d_backward_workspace_bytes",
    "d2c_conv1d_forward", "d2c_conv1d_backward", "d2c_conv3d_corner_index", "d2c_conv3d_sample",
    "d2c_conv3d_offset_histogram",
    "d2c_get_max_intermediate_elements", "d2c_set_max_intermediate_elements",
    "d2c_set_algo_override", "d2c_set_grad_input_mode", "d2c_set_grad_weight_mode", "d2c_set_backward_slices", "d2c_last_error", "d2c_version",
    "d2c_profile_enable", "d2c_profile_reset", "d2c_profile_read", "d2c_profile_kernel_name",
    "d2c_size_map_offsets_forward", "d2c_size_map_offsets_backward",
    "d2c_conv3d_sized_forward_workspace_bytes", "d2c_conv3d_sized_backward_workspace_bytes",
    "d2c_conv3d_sized_forward", "d2c_conv3d_sized_backward",
    "d2c_conv3d_forward_stats_workspace_bytes", "d2c_conv3d_forward_stats", "d2c_channel_stats",
    "d2c_group_norm_forward", "d2c_group_norm_backward_workspace_bytes", "d2c_group_norm_backward",
    "d2c_dwconv3d_check", "d2c_dwconv3d_backward_workspace_bytes", "d2c_dwconv3d_forward", "d2c_dwconv3d_backward",
)


class Conv3dDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "N", "Cin", "Cout", "D", "H", "W", "kd", "kh", "kw", "sd", "sh", "sw",
        "pd", "ph", "pw", "dd", "dh", "dw", "groups", "offset_groups", "Do", "Ho", "Wo",
        "dtype", "aux_dtype", "epilogue")] + [("epilogue_scale", ctypes.c_float), ("offset_axes", ctypes.c_int32),
                                               ("backward_flags", ctypes.c_int32), ("deform_channels", ctypes.c_int32),
                                               ("mask_activation", ctypes.c_int32)]


MASK_ACTIVATIONS = {"none": 0, "linear": 0, "sigmoid": 1, "relu": 2, "tanh": 3}


# d2c_conv3d_desc::backward_flags
BWD_GW_DEFAULT, BWD_GW_COLUMNS, BWD_GW_IN_PLACE, BWD_GW_RESAMPLE = 0, 1, 2, 3
BWD_F32_SPLIT = 0x10000


def bwd_slices(n):
    return (int(n) & 0xff) << 8


EPILOGUE_NONE, EPILOGUE_RELU = 0, 1
REUSE_INPUT, REUSE_FORWARD_WEIGHTS, REUSE_BACKWARD_WEIGHTS = 1, 2, 4


SIZE_MAX_K = 16
SIZE_MODES = {"xyz": 0, "xxz": 1, "xy": 2, "x": 3}
SIZE_ACTIVATIONS = {"linear": 0, "elu": 1, "relu": 2, "relu_plus_one": 3}


class SizeMapDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("N", "P", "kd", "kh", "kw", "mode", "activation", "dtype")] + [
        (n, ctypes.c_float * SIZE_MAX_K) for n in ("base_z", "base_y", "base_x")]


class GroupNormDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("N", "C", "P", "groups", "dtype")] + [("eps", ctypes.c_float)]


class DwConv3dDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "N", "C", "Cout", "D", "H", "W", "kd", "kh", "kw", "sd", "sh", "sw",
        "pd", "ph", "pw", "dd", "dh", "dw", "Do", "Ho", "Wo", "dtype")]


class Conv1dDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "N", "Cin", "Cout", "L", "k", "s", "p", "d", "groups", "offset_groups", "Lo",
        "dtype", "aux_dtype", "reference_quirks")]


_lib = None


def load():
    """Returns the loaded library; raises if it was never built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP library has not been built "
            "(run `python -m d2conv3d_amd.build`); there is no fallback path")
    lib = ctypes.CDLL(LIB_PATH)
    vp, sz, i32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int32
    p3, p1 = ctypes.POINTER(Conv3dDesc), ctypes.POINTER(Conv1dDesc)
    lib.d2c_output_size.restype = i32
    lib.d2c_output_size.argtypes = [i32] * 5
    lib.d2c_last_error.restype = ctypes.c_char_p
    lib.d2c_version.restype = ctypes.c_int
    lib.d2c_get_max_intermediate_elements.restype = ctypes.c_uint64
    lib.d2c_set_max_intermediate_elements.argtypes = [ctypes.c_uint64]
    lib.d2c_set_max_intermediate_elements.restype = None
    lib.d2c_set_algo_override.argtypes = [ctypes.c_int]
    lib.d2c_set_algo_override.restype = None
    for name, p in (("conv3d", p3), ("conv1d", p1)):
        getattr(lib, f"d2c_{name}_check").argtypes = [p]
        getattr(lib, f"d2c_{name}_check").restype = ctypes.c_int
        for d in ("forward", "backward"):
            f = getattr(lib, f"d2c_{name}_{d}_workspace_bytes")
            f.argtypes, f.restype = [p], sz
        f = getattr(lib, f"d2c_{name}_forward")
        f.argtypes, f.restype = [p] + [vp] * 7 + [sz, vp], ctypes.c_int
        f = getattr(lib, f"d2c_{name}_backward")
        f.argtypes, f.restype = [p] + [vp] * 11 + [sz, vp], ctypes.c_int
    lib.d2c_conv3d_algo.argtypes, lib.d2c_conv3d_algo.restype = [p3], ctypes.c_int
    lib.d2c_conv3d_packed_supported.argtypes = [p3, ctypes.POINTER(SizeMapDesc)]
    lib.d2c_conv3d_packed_supported.restype = ctypes.c_int
    lib.d2c_conv3d_forward_static.argtypes, lib.d2c_conv3d_forward_static.restype = [p3] + [vp] * 7, ctypes.c_int
    lib.d2c_static_workspace_bytes.argtypes, lib.d2c_static_workspace_bytes.restype = [], sz
    lib.d2c_conv3d_prepared_bytes.argtypes, lib.d2c_conv3d_prepared_bytes.restype = [p3], sz
    lib.d2c_conv3d_forward_prepared.argtypes = [p3] + [vp] * 6 + [vp, sz, i32, vp, sz, vp]
    lib.d2c_conv3d_forward_prepared.restype = ctypes.c_int
    lib.d2c_conv3d_backward_prepared.argtypes = [p3] + [vp] * 10 + [vp, sz, i32, vp, sz, vp]
    lib.d2c_conv3d_backward_prepared.restype = ctypes.c_int
    # (the second argument: a pointer to a size-map description, or None)
    lib.d2c_conv3d_columns_bytes.argtypes, lib.d2c_conv3d_columns_bytes.restype = [p3, vp], sz
    lib.d2c_conv3d_backward_columns_workspace_bytes.argtypes = [p3, vp]
    lib.d2c_conv3d_backward_columns_workspace_bytes.restype = sz
    lib.d2c_conv3d_forward_columns.argtypes = [p3, vp] + [vp] * 6 + [vp, sz, vp, sz, vp]
    lib.d2c_conv3d_forward_columns.restype = ctypes.c_int
    lib.d2c_conv3d_backward_columns.argtypes = [p3, vp] + [vp] * 5 + [vp, sz] + [vp] * 5 + [vp, sz, vp]
    lib.d2c_conv3d_backward_columns.restype = ctypes.c_int
    lib.d2c_conv1d_algo.argtypes, lib.d2c_conv1d_algo.restype = [p1], ctypes.c_int
    lib.d2c_conv3d_corner_index.argtypes = [p3, vp, vp, vp, vp]
    lib.d2c_conv3d_corner_index.restype = ctypes.c_int
    lib.d2c_conv3d_sample.argtypes, lib.d2c_conv3d_sample.restype = [p3, i32, vp, vp, vp, vp], ctypes.c_int
    lib.d2c_conv3d_offset_histogram.argtypes = [p3, vp, ctypes.c_float, ctypes.c_float, i32, vp, vp]
    lib.d2c_conv3d_offset_histogram.restype = ctypes.c_int
    lib.d2c_set_grad_input_mode.argtypes, lib.d2c_set_grad_input_mode.restype = [ctypes.c_int], None
    lib.d2c_set_grad_weight_mode.argtypes, lib.d2c_set_grad_weight_mode.restype = [ctypes.c_int], None
    lib.d2c_set_backward_slices.argtypes, lib.d2c_set_backward_slices.restype = [ctypes.c_int], None
    psm = ctypes.POINTER(SizeMapDesc)
    lib.d2c_size_map_offsets_forward.argtypes, lib.d2c_size_map_offsets_forward.restype = [psm, vp, vp, vp], ctypes.c_int
    lib.d2c_size_map_offsets_backward.argtypes, lib.d2c_size_map_offsets_backward.restype = [psm, vp, vp, vp, vp], ctypes.c_int
    for d in ("forward", "backward"):
        f = getattr(lib, f"d2c_conv3d_sized_{d}_workspace_bytes")
        f.argtypes, f.restype = [p3, psm], sz
    lib.d2c_conv3d_sized_forward.argtypes, lib.d2c_conv3d_sized_forward.restype = [p3, psm] + [vp] * 7 + [sz, vp], ctypes.c_int
    lib.d2c_conv3d_sized_backward.argtypes, lib.d2c_conv3d_sized_backward.restype = [p3, psm] + [vp] * 11 + [sz, vp], ctypes.c_int
    pgn = ctypes.POINTER(GroupNormDesc)
    lib.d2c_conv3d_forward_stats_workspace_bytes.argtypes = [p3, psm]
    lib.d2c_conv3d_forward_stats_workspace_bytes.restype = sz
    lib.d2c_conv3d_forward_stats.argtypes, lib.d2c_conv3d_forward_stats.restype = [p3, psm] + [vp] * 8 + [sz, vp], ctypes.c_int
    lib.d2c_channel_stats.argtypes, lib.d2c_channel_stats.restype = [pgn, vp, vp, vp], ctypes.c_int
    lib.d2c_group_norm_forward.argtypes, lib.d2c_group_norm_forward.restype = [pgn] + [vp] * 6, ctypes.c_int
    lib.d2c_group_norm_backward_workspace_bytes.argtypes = [pgn]
    lib.d2c_group_norm_backward_workspace_bytes.restype = sz
    lib.d2c_group_norm_backward.argtypes, lib.d2c_group_norm_backward.restype = [pgn] + [vp] * 8 + [sz, vp], ctypes.c_int
    pdw = ctypes.POINTER(DwConv3dDesc)
    lib.d2c_dwconv3d_check.argtypes, lib.d2c_dwconv3d_check.restype = [pdw], ctypes.c_int
    lib.d2c_dwconv3d_backward_workspace_bytes.argtypes = [pdw]
    lib.d2c_dwconv3d_backward_workspace_bytes.restype = sz
    lib.d2c_dwconv3d_forward.argtypes, lib.d2c_dwconv3d_forward.restype = [pdw] + [vp] * 5, ctypes.c_int
    lib.d2c_dwconv3d_backward.argtypes, lib.d2c_dwconv3d_backward.restype = [pdw] + [vp] * 7 + [sz, vp], ctypes.c_int
    lib.d2c_profile_enable.argtypes, lib.d2c_profile_enable.restype = [ctypes.c_int], None
    lib.d2c_profile_reset.argtypes, lib.d2c_profile_reset.restype = [], None
    lib.d2c_profile_read.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_int)]
    lib.d2c_profile_read.restype = ctypes.c_int
    lib.d2c_profile_kernel_name.argtypes, lib.d2c_profile_kernel_name.restype = [ctypes.c_int], ctypes.c_char_p
    _lib = lib
    return lib


def last_error():
    return load().d2c_last_error().decode("utf-8", "replace")


def check(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what}: {last_error()} (code {rc})")
