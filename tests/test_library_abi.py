"""CPU-side checks of the drop-in boundary: the shared library loads, exports every symbol the public header
declares, reports errors by status code, and the Python binding refuses bad tensors like the reference's does."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "norm_dist_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ndist_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_the_twelve_entry_points():
    names = declared_functions()
    for n in ["norm_dist_forward", "norm_dist_forward_with_max", "norm_dist_backward_input",
              "norm_dist_backward_input_weight", "inf_dist_forward", "inf_dist_forward_nograd",
              "inf_dist_backward_input", "inf_dist_backward_input_weight", "bound_inf_dist_forward",
              "bound_inf_dist_forward_nograd", "bound_inf_dist_backward_input",
              "bound_inf_dist_backward_input_weight"]:
        assert "ndist_" + n in names


def test_library_exports_every_declared_symbol():
    from core import _C
    lib = ctypes.CDLL(_C.LIBRARY_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), name
    assert _C.version() >= 10000
    lib.ndist_status_string.restype = ctypes.c_char_p
    assert b"NULL" in lib.ndist_status_string(1)


def test_argument_validation_returns_status_without_touching_a_device():
    from core import _C
    lib = ctypes.CDLL(_C.LIBRARY_PATH)
    f = lib.ndist_inf_dist_forward_nograd
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_void_p] * 2 + [ctypes.c_int] * 5 + [ctypes.c_void_p] * 2
    assert f(None, None, 1, 1, 1, 1, 1, None, None) == 1          # null pointers
    dummy = ctypes.c_void_p(16)
    assert f(dummy, dummy, 0, 4, 4, 1, 1, dummy, None) == 2        # empty batch
    assert f(dummy, dummy, 2, 4, 6, 4, 1, dummy, None) == 2        # CI not divisible by G
    g = lib.ndist_norm_dist_forward
    g.restype = ctypes.c_int
    g.argtypes = [ctypes.c_void_p] * 2 + [ctypes.c_int] * 5 + [ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p]
    assert g(dummy, dummy, 2, 4, 4, 1, 1, dummy, 0.0, None) == 3   # p must be positive
    assert g(dummy, dummy, 2, 4, 4, 1, 1, dummy, float("inf"), None) == 3


def test_tail_entry_points_validate_their_arguments():
    from core import _C
    lib = ctypes.CDLL(_C.LIBRARY_PATH)
    dummy = ctypes.c_void_p(16)
    m = lib.ndist_margin_forward
    m.restype = ctypes.c_int
    m.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 2 + [ctypes.c_float] + [ctypes.c_void_p] * 2
    assert m(None, None, None, dummy, 4, 10, 0.1, dummy, None) == 1       # neither x nor both bounds
    assert m(None, dummy, None, dummy, 4, 10, 0.1, dummy, None) == 1      # one bound alone
    assert m(dummy, None, None, None, 4, 10, 0.1, dummy, None) == 1       # no targets
    assert m(dummy, None, None, dummy, 0, 10, 0.1, dummy, None) == 2      # empty batch
    assert m(dummy, None, None, dummy, 4, 10, 0.0, dummy, None) == 2      # the margin divides by 2 eps
    h = lib.ndist_hinge_forward
    h.restype = ctypes.c_int
    h.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 2 + [ctypes.c_float] + [ctypes.c_void_p] * 3
    assert h(None, 4, 10, 0.25, dummy, dummy, None) == 1
    assert h(dummy, 4, 0, 0.25, dummy, dummy, None) == 2


def test_binding_rejects_cpu_and_non_contiguous_tensors():
    from core import _C
    x = torch.zeros(2, 4, 1)
    w = torch.zeros(3, 4)
    out = torch.zeros(2, 3, 1)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _C.inf_dist_forward_nograd(x, w, out, 1)


def test_operator_rejects_non_positive_p_and_shape_mismatch():
    from core.norm_dist import NormDistF
    x = torch.zeros(2, 4, 1)
    with pytest.raises(AssertionError):
        NormDistF.apply(x, torch.zeros(3, 5), 1, 2.0, False, None)
    with pytest.raises(NotImplementedError):
        NormDistF.apply(x, torch.zeros(3, 4), 1, -1.0, False, None)


def test_unfold_geometry_and_validation():
    from core import _C
    geo, (oh, ow) = _C.unfold_geometry((2, 3, 9, 7), (3, 2), 1, (1, 0), (2, 1))
    ref = torch.nn.functional.unfold(torch.zeros(2, 3, 9, 7), (3, 2), 1, (1, 0), (2, 1))
    assert ref.shape == (2, 3 * 3 * 2, oh * ow)
    lib = ctypes.CDLL(_C.LIBRARY_PATH)
    f = lib.ndist_unfold_forward
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_void_p] + [ctypes.c_int] * 12 + [ctypes.c_void_p] * 2
    dummy = ctypes.c_void_p(16)
    assert f(None, 1, 1, 4, 4, 3, 3, 1, 1, 1, 1, 1, 1, dummy, None) == 1
    assert f(dummy, 1, 1, 4, 4, 3, 3, 1, 1, 1, 1, 0, 1, dummy, None) == 2    # stride 0
    assert f(dummy, 1, 1, 2, 2, 5, 5, 1, 1, 0, 0, 1, 1, dummy, None) == 2    # window larger than the padded image


def test_extension_module_exports_the_reference_names():
    # the compiled PyTorch binding (csrc/binding/norm_dist_ext.cpp) imports without a GPU and carries the twelve
    # functions of the reference's extension (core/cuda/norm_dist.cpp:191-204) plus this library's additions
    from core import _C
    assert _C.BINDING == "ext", "norm_dist_hip_ext.so has not been built"
    E = _C._ext
    for n in ["norm_dist_forward", "norm_dist_forward_with_max", "norm_dist_backward_input",
              "norm_dist_backward_input_weight", "inf_dist_forward", "inf_dist_forward_nograd",
              "inf_dist_backward_input", "inf_dist_backward_input_weight", "bound_inf_dist_forward",
              "bound_inf_dist_forward_nograd", "bound_inf_dist_backward_input",
              "bound_inf_dist_backward_input_weight", "norm_dist_backward_input_weight_noalloc", "unfold_forward",
              "unfold_backward", "conv_inf_dist_forward", "conv_bound_inf_dist_backward_input_weight"]:
        assert callable(getattr(E, n)), n
    assert E.version() == _C.version()
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        E.norm_dist_forward(torch.zeros(2, 4, 1), torch.zeros(3, 4), torch.zeros(2, 3, 1), 1, 2.0)
