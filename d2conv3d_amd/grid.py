"""Kernel-grid helpers and the dynamic-dilation offset expansion, mirroring
ops/dconv-native/src/dconv_native/grid.py and the application's utils/grid.py.
"""
import torch
from torch.nn.modules.utils import _triple


def grid_like(tensor):
    """grid.py:8-18: integer grid [n_spatial, D_1, ..., D_n] over the spatial dims of `tensor`."""
    axes = [torch.arange(0, d, device=tensor.device) for d in tensor.shape[2:]]
    return torch.stack(torch.meshgrid(axes, indexing="ij"))


def get_kernel_grid(kernel_shape, dilation, device="cpu"):
    """grid.py:21-25: [3, kz, ky, kx] tap coordinates relative to the kernel centre,
    linspace(-d*(k//2), d*(k//2), k) per axis."""
    axes = [torch.linspace(-d * (k // 2), d * (k // 2), k, device=device)
            for d, k in zip(dilation, kernel_shape)]
    return torch.stack(torch.meshgrid(axes, indexing="ij"))


def get_convolution_grid(input_shape, kernel_shape, stride, padding, dilation, device="cpu"):
    """grid.py:28-32: centre position of every kernel application."""
    axes = [torch.arange(a * (k // 2) - p, d - a * (k // 2) + p, s, device=device)
            for d, k, s, p, a in zip(input_shape, kernel_shape, stride, padding, dilation)]
    return torch.stack(torch.meshgrid(axes, indexing="ij"))


@torch.no_grad()
def construct_3d_kernel_grid(input_size, kernel_size=3, stride=1, pad=1, dilation=1, device="cpu"):
    """grid.py:35-59: input coordinates touched by each tap, [(K), 3, D, H, W]."""
    kernel_size, stride, pad, dilation = _triple(kernel_size), _triple(stride), _triple(pad), _triple(dilation)
    kernel_grid = get_kernel_grid(kernel_size, dilation, device)            # [3, kz, ky, kx]
    position_grid = get_convolution_grid(input_size, kernel_size, stride, pad, dilation, device)
    kernel_grid = kernel_grid.reshape(3, -1).t().reshape(-1, 3, 1, 1, 1)    # [(kz ky kx), 3, 1, 1, 1]
    return kernel_grid + position_grid


def _inflate_size_map(size_map, mode):
    ones = torch.ones_like(size_map[:, :1])
    c = size_map.shape[1]
    if mode is None:
        # grid.py:66-76 of the operator package: the channel count selects the mode
        mode = {3: "xyz", 2: "xy", 1: "x"}.get(c)
        if mode is None:
            raise ValueError(f"size_map should have 1, 2, or 3 channels, but has {c}")
    mode = mode.lower()
    if mode == "xyz":
        assert c == 3
        return size_map
    if mode == "xxz":
        assert c == 2
        z, x = torch.split(size_map, [1, 1], dim=1)
        return torch.cat([z, x, x], dim=1)
    if mode == "xy":
        assert c == 2
        return torch.cat([ones, size_map], dim=1)
    if mode == "x":
        assert c == 1
        return torch.cat([ones, size_map, size_map], dim=1)
    raise ValueError(f"Unknown offset mode '{mode}'")


def offsets_from_size_map(size_map, *args, **kwargs):
    """Per-location, per-axis dilation -> tap offsets:

        off[n, ((kz*kh+ky)*kw+kx)*3 + a, d, h, w] = base_a(k_a) * (size[n, a, d, h, w] - 1)

    Both call conventions of the reference are accepted:
      offsets_from_size_map(size_map, kernel_shape=(3,3,3), dilation=(1,1,1))        (grid.py:62-80)
      offsets_from_size_map(size_map, mode, kernel_shape=(3,3,3), dilation=(1,1,1))  (utils/grid.py:72-98)
    """
    args = list(args)
    mode = kwargs.pop("mode", None)
    if args and isinstance(args[0], str):
        mode = args.pop(0)
    kernel_shape = kwargs.pop("kernel_shape", args.pop(0) if args else (3, 3, 3))
    dilation = kwargs.pop("dilation", args.pop(0) if args else (1, 1, 1))
    if args or kwargs:
        raise TypeError("offsets_from_size_map: unexpected arguments")
    kernel_shape, dilation = _triple(kernel_shape), _triple(dilation)
    base = get_kernel_grid(kernel_shape, dilation, size_map.device).to(size_map.dtype)  # [3, kz, ky, kx]
    base = base.permute(1, 2, 3, 0).reshape(1, -1, 3, 1, 1, 1)                           # [1, K, 3, 1, 1, 1]
    size3 = _inflate_size_map(size_map, mode)                                           # [n, 3, d, h, w]
    offsets = base * (size3.unsqueeze(1) - 1)                                           # [n, K, 3, d, h, w]
    n, _, d, h, w = size3.shape
    return offsets.reshape(n, -1, d, h, w)


class _SizeMapOffsets(torch.autograd.Function):
    """Size activation + offsets_from_size_map as one library kernel each way
    (d2c_size_map_offsets_forward / _backward)."""

    @staticmethod
    def forward(ctx, size_raw, desc):
        import ctypes
        from . import _lib
        lib = _lib.load()
        size_raw = size_raw.contiguous()
        n = size_raw.shape[0]
        K = desc.kd * desc.kh * desc.kw
        out = torch.empty((n, 3 * K) + tuple(size_raw.shape[2:]), dtype=size_raw.dtype, device=size_raw.device)
        with torch.cuda.device(size_raw.device):
            st = ctypes.c_void_p(torch.cuda.current_stream(size_raw.device).cuda_stream)
            _lib.check(lib.d2c_size_map_offsets_forward(ctypes.byref(desc), ctypes.c_void_p(size_raw.data_ptr()),
                                                        ctypes.c_void_p(out.data_ptr()), st), "size_map_offsets")
        ctx.save_for_backward(size_raw)
        ctx.desc = desc
        return out

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_out):
        import ctypes
        from . import _lib
        lib = _lib.load()
        (size_raw,) = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        grad = torch.empty_like(size_raw)
        with torch.cuda.device(size_raw.device):
            st = ctypes.c_void_p(torch.cuda.current_stream(size_raw.device).cuda_stream)
            _lib.check(lib.d2c_size_map_offsets_backward(ctypes.byref(ctx.desc), ctypes.c_void_p(size_raw.data_ptr()),
                                                         ctypes.c_void_p(grad_out.data_ptr()),
                                                         ctypes.c_void_p(grad.data_ptr()), st), "size_map_offsets backward")
        return grad, None


def size_map_offsets(size_raw, mode, kernel_shape=(3, 3, 3), dilation=(1, 1, 1), activation="linear"):
    """offsets_from_size_map(size_activation(size_raw), mode, kernel_shape, dilation) in one kernel:
    the deformation producer of the size-conditioned layers (network/layers.py:171-181 and
    utils/grid.py:72-98) without the intermediate tensors and autograd nodes of the torch
    formulation.  CUDA tensors, float32 or bfloat16; `size_raw` is the prediction BEFORE
    the size activation.  Same values as the torch formulation (bit for bit in float32 except
    for the exponential of the ELU)."""
    from . import _lib
    if not size_raw.is_cuda:
        raise RuntimeError("size_map_offsets: CUDA tensors only (use offsets_from_size_map for CPU tensors)")
    if size_raw.dtype not in (torch.float32, torch.bfloat16):
        raise RuntimeError("size_map_offsets: float32 or bfloat16 only")
    mode = mode.lower()
    kernel_shape, dilation = _triple(kernel_shape), _triple(dilation)
    want_c = {"xyz": 3, "xxz": 2, "xy": 2, "x": 1}[mode]
    if size_raw.dim() < 3 or size_raw.shape[1] != want_c:
        raise RuntimeError(f"size_map_offsets: mode '{mode}' wants {want_c} size channels, got {tuple(size_raw.shape)}")
    if max(kernel_shape) > _lib.SIZE_MAX_K:
        raise RuntimeError(f"size_map_offsets: kernel extents up to {_lib.SIZE_MAX_K}")
    return _SizeMapOffsets.apply(size_raw, size_map_desc(size_raw, mode, kernel_shape, dilation, activation))


def size_map_desc(size_raw, mode, kernel_shape, dilation, activation):
    """The d2c_size_map_desc of a raw size map [N, channels(mode), *spatial] (or of a tensor that holds the map in its
    leading channels: only the batch size, the spatial shape and the element type are read)."""
    from . import _lib
    desc = _lib.SizeMapDesc()
    desc.N = size_raw.shape[0]
    desc.P = 1
    for d in size_raw.shape[2:]:
        desc.P *= int(d)
    desc.kd, desc.kh, desc.kw = kernel_shape
    desc.mode, desc.activation = _lib.SIZE_MODES[mode.lower()], _lib.SIZE_ACTIVATIONS[activation]
    desc.dtype = _lib.D2C_BF16 if size_raw.dtype == torch.bfloat16 else _lib.D2C_F32
    for name, d, k in zip(("base_z", "base_y", "base_x"), dilation, kernel_shape):
        arr = getattr(desc, name)
        for i, v in enumerate(_kernel_axis(d, k)):
            arr[i] = v
    return desc


_AXIS_CACHE = {}


def _kernel_axis(d, k):
    """linspace(-d*(k//2), d*(k//2), k) exactly as get_kernel_grid computes it, as Python floats."""
    key = (d, k)
    if key not in _AXIS_CACHE:
        _AXIS_CACHE[key] = torch.linspace(-d * (k // 2), d * (k // 2), k).tolist()
    return _AXIS_CACHE[key]
