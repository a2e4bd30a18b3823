"""CPU checks of the drop-in boundary: the C-ABI library loads and exports
every symbol the header declares, the host-side argument checks behave like
the reference's, and the Python surface has the reference's names."""
import ctypes
import os
import re

import pytest
import torch

import d2conv3d_amd as d2c
from d2conv3d_amd import _lib, _ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    header = open(os.path.join(ROOT, "include", "d2conv.h")).read()
    declared = set(re.findall(r"\b(d2c_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found in the header"
    assert declared == set(_lib.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), f"{name} not exported"
    assert lib.d2c_version() >= 1


def test_output_size_formula():
    lib = _lib.load()
    # get_output_size, dconv_gpu_common.h:13-15
    for (n, k, s, p, d) in [(5, 3, 1, 0, 1), (7, 3, 2, 1, 1), (7, 3, 1, 2, 2), (32, 3, 1, 1, 1), (2, 3, 1, 1, 1)]:
        assert lib.d2c_output_size(n, k, s, p, d) == (n + 2 * p - (d * (k - 1) + 1)) // s + 1


def _desc(**kw):
    base = dict(N=2, Cin=4, Cout=6, D=5, H=5, W=5, kd=3, kh=3, kw=3, sd=1, sh=1, sw=1, pd=0, ph=0, pw=0,
                dd=1, dh=1, dw=1, groups=1, offset_groups=1, Do=3, Ho=3, Wo=3, dtype=0, aux_dtype=0)
    base.update(kw)
    return _lib.Conv3dDesc(**base)


def test_conv3d_check_accepts_and_rejects():
    lib = _lib.load()
    assert lib.d2c_conv3d_check(ctypes.byref(_desc())) == 0
    rc = lib.d2c_conv3d_check(ctypes.byref(_desc(Do=4)))
    assert rc != 0
    # message of dconv3d_gpu.cu:514-519
    assert "offset output dims do not match computed dims" in _lib.last_error()
    assert "(4, 3, 3)" in _lib.last_error() and "(3, 3, 3)" in _lib.last_error()
    assert lib.d2c_conv3d_check(ctypes.byref(_desc(groups=3))) != 0        # Cin % groups
    assert lib.d2c_conv3d_check(ctypes.byref(_desc(offset_groups=4))) != 0  # Cout % offset_groups
    assert lib.d2c_conv3d_check(ctypes.byref(_desc(sd=0))) != 0
    assert lib.d2c_conv3d_check(ctypes.byref(_desc(pd=-1))) != 0
    assert lib.d2c_conv3d_check(ctypes.byref(_desc(D=2, Do=0))) != 0        # non-positive output
    assert lib.d2c_conv3d_check(ctypes.byref(_desc(dtype=7))) != 0
    assert lib.d2c_conv3d_check(ctypes.byref(_desc(dtype=0, aux_dtype=2))) != 0
    assert lib.d2c_conv3d_check(ctypes.byref(_desc(dtype=2, aux_dtype=0))) == 0
    # the forward epilogue: none, or a ReLU with a positive finite scale
    assert lib.d2c_conv3d_check(ctypes.byref(_desc(epilogue=_lib.EPILOGUE_RELU, epilogue_scale=1.71285855))) == 0
    assert lib.d2c_conv3d_check(ctypes.byref(_desc(epilogue=5, epilogue_scale=1.0))) != 0
    assert "unknown epilogue" in _lib.last_error()
    assert lib.d2c_conv3d_check(ctypes.byref(_desc(epilogue=_lib.EPILOGUE_RELU, epilogue_scale=0.0))) != 0
    assert lib.d2c_conv3d_check(ctypes.byref(_desc(epilogue=_lib.EPILOGUE_RELU, epilogue_scale=float("inf")))) != 0


def test_workspace_queries_run_without_gpu():
    lib = _lib.load()
    q = _desc()
    assert lib.d2c_conv3d_forward_workspace_bytes(ctypes.byref(q)) >= 0
    assert lib.d2c_conv3d_backward_workspace_bytes(ctypes.byref(q)) >= 0
    assert lib.d2c_conv3d_algo(ctypes.byref(q)) in (_lib.ALGO_GENERIC, _lib.ALGO_MFMA, _lib.ALGO_DEPTHWISE)


def test_max_intermediate_elements_knob():
    # dconv3d_gpu.cu:12-14, dconv.cpp:9-11
    assert _ops.config.get_max_intermediate_elements() == 1 << 32
    _ops.config.set_max_intermediate_elements(1234)
    assert _ops.config.get_max_intermediate_elements() == 1234
    _ops.config.set_max_intermediate_elements(1 << 32)


def test_cpu_tensors_are_rejected_loudly():
    x = torch.randn(1, 2, 4, 4, 4)
    off = torch.zeros(1, 81, 2, 2, 2)
    w = torch.randn(2, 2, 3, 3, 3)
    with pytest.raises(RuntimeError, match="is_cuda"):
        d2c.deform_conv3d(x, off, None, w)


def test_python_shape_checks():
    x = torch.randn(1, 2, 4, 4, 4, device="meta")
    w = torch.randn(2, 2, 3, 3, 3, device="meta")
    with pytest.raises(RuntimeError):
        _ops._check_common(3, x, torch.zeros(1, 80, 2, 2, 2, device="meta"), None, w, None, 1, 1)
    with pytest.raises(RuntimeError):
        _ops._check_common(3, x, torch.zeros(2, 81, 2, 2, 2, device="meta"), None, w, None, 1, 1)
    with pytest.raises(RuntimeError):
        _ops._check_common(3, x, torch.zeros(1, 81, 2, 2, 2, device="meta"),
                           torch.zeros(1, 26, 2, 2, 2, device="meta"), w, None, 1, 1)


def test_surface_names_of_the_reference():
    # ops/dconv-native/src/dconv_native/__init__.py:1-10 and the app's imports
    for name in ("deform_conv1d", "deform_conv3d", "DeformConv1d", "DeformConv3d", "DConv3d", "MDConv3d",
                 "SizeConditionedDConv3d", "SizeConditionedMDConv3d"):
        assert hasattr(d2c, name)
    d2c.install_as_dconv_native()
    from dconv_native import DeformConv3d  # noqa: F401
    from dconv_native.deform_conv import DeformConvNd  # noqa: F401
    from dconv_native.util import add_deformable_conv  # noqa: F401
    import dconv_native._ops as ops
    assert callable(ops.deform_conv3d) and callable(ops.deform_conv1d)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()


def test_plain_depthwise_boundary_without_gpu():
    """d2c_dwconv3d_check mirrors conv_depthwise_shape_check (grouped_conv3d.cu:279-345); the Python surface
    carries the reference's names (src/fast_depthwise_conv3d/__init__.py, conv.py:7-22) and rejects CPU tensors."""
    import ctypes
    lib = _lib.load()

    def desc(**kw):
        f = dict(N=2, C=4, Cout=8, D=6, H=7, W=8, kd=3, kh=3, kw=3, sd=1, sh=1, sw=1, pd=1, ph=1, pw=1, dd=1, dh=1, dw=1,
                 Do=6, Ho=7, Wo=8, dtype=_lib.D2C_F32)
        f.update(kw)
        return _lib.DwConv3dDesc(*(f[n] for n, _ in _lib.DwConv3dDesc._fields_))

    assert lib.d2c_dwconv3d_check(ctypes.byref(desc())) == 0
    assert lib.d2c_dwconv3d_backward_workspace_bytes(ctypes.byref(desc())) >= 8 * 28 * 4
    for bad, text in ((dict(Cout=6), "multiple of in channels"), (dict(sd=0), "stride should be at least 1"),
                      (dict(pw=-1), "padding should be non-negative"), (dict(dh=0), "dilation should be at least 1"),
                      (dict(D=2, pd=0, Do=0), "Output size should be positive"), (dict(Wo=9), "does not match"),
                      (dict(dtype=7), "dtype")):
        assert lib.d2c_dwconv3d_check(ctypes.byref(desc(**bad))) != 0
        assert text in _lib.last_error()
    assert lib.d2c_dwconv3d_backward_workspace_bytes(ctypes.byref(desc(Cout=6))) == 0

    m = d2c.DepthwiseConv3d(4, 8, kernel_size=3, padding=1, groups=99)
    assert isinstance(m, torch.nn.Conv3d) and m.groups == 4 and tuple(m.weight.shape) == (8, 1, 3, 3, 3)
    with pytest.raises(RuntimeError, match="GPU"):
        m(torch.randn(1, 4, 5, 5, 5))
    with pytest.raises(RuntimeError, match="in_channels=1"):
        d2c.depthwise_separable_conv3d(torch.randn(1, 4, 5, 5, 5), torch.randn(4, 2, 3, 3, 3), None, 1, 1, 1)
    d2c.install_as_fast_depthwise_conv3d()
    from fast_depthwise_conv3d import DepthwiseConv3d  # noqa: F401
    import fast_depthwise_conv3d._ops as ops
    assert callable(ops.depthwise_separable_conv3d)
