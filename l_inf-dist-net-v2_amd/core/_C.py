"""Binding of libnorm_dist_hip.so: the twelve kernel entry points under the names, argument orders and checks of the
reference's extension module (core/cuda/norm_dist.cpp:40-204), taking torch tensors.

Two routes lead to the same C ABI.  The PyTorch C++ extension `norm_dist_hip_ext` (csrc/binding/norm_dist_ext.cpp,
built next to the library) is used when it is there: it validates the tensors, makes their device current and
launches on PyTorch's current stream from compiled code.  Without it (or with NORM_DIST_BINDING=ctypes) the same
calls go through ctypes from this file, with the same checks written in Python.  Either way, importing this module
fails loudly when the library itself has not been built: there is no fallback implementation of the kernels.
Each call validates its tensors the way the reference's CHECK_INPUT does (device + contiguity, core/cuda/norm_dist.cpp:8-10)
plus dtype, derives (B, CO, CI, HW) exactly as the reference does, and launches on torch's current stream of the
tensors' device.
"""
import ctypes
import os
import re
import sys

import torch

# NORM_DIST_HIP_LIBRARY overrides the location of the shared library (e.g. a build made elsewhere)
_LIB_PATH = os.environ.get("NORM_DIST_HIP_LIBRARY") or os.path.join(
    os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "lib", "libnorm_dist_hip.so")
if not os.path.exists(_LIB_PATH):
    raise ImportError(
        "libnorm_dist_hip.so is not built (expected at %s); run `make -C %s`" %
        (_LIB_PATH, os.path.join(os.path.dirname(os.path.dirname(_LIB_PATH)), "csrc")))
_lib = ctypes.CDLL(_LIB_PATH)
LIBRARY_PATH = _LIB_PATH

# The compiled binding, when it has been built (it links against the library above, same directory).
_ext = None
EXTENSION_PATH = os.path.join(os.path.dirname(_LIB_PATH), "norm_dist_hip_ext.so")
if os.environ.get("NORM_DIST_BINDING", "ext") != "ctypes" and os.path.exists(EXTENSION_PATH):
    import importlib.util
    try:
        _spec = importlib.util.spec_from_file_location("norm_dist_hip_ext", EXTENSION_PATH)
        _ext = importlib.util.module_from_spec(_spec)
        _spec.loader.exec_module(_ext)
        sys.modules.setdefault("norm_dist_hip_ext", _ext)
    except ImportError as _exc:  # built against another torch: the ctypes route serves the same C ABI
        import warnings
        warnings.warn("norm_dist_hip_ext could not be loaded (%s); using the ctypes binding" % _exc)
        _ext = None
BINDING = "ext" if _ext is not None else "ctypes"

_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float


def _sig(name, *argtypes):
    fn = getattr(_lib, name)
    fn.argtypes = list(argtypes)
    fn.restype = ctypes.c_int
    return fn


_lib.ndist_status_string.restype = ctypes.c_char_p
_lib.ndist_status_string.argtypes = [ctypes.c_int]
_lib.ndist_last_hip_error.restype = ctypes.c_int
_lib.ndist_version.restype = ctypes.c_int
_lib.ndist_set_profiling.argtypes = [ctypes.c_int]
_lib.ndist_set_profiling.restype = None
_lib.ndist_set_skip_mode.argtypes = [ctypes.c_int, ctypes.c_int]
_lib.ndist_set_skip_mode.restype = None
_lib.ndist_set_hot_mode.argtypes = [ctypes.c_int]
_lib.ndist_set_hot_mode.restype = None
_lib.ndist_set_scaled_mode.argtypes = [ctypes.c_int]
_lib.ndist_set_scaled_mode.restype = None
_lib.ndist_get_modes.argtypes = [ctypes.POINTER(ctypes.c_int)] * 4
_lib.ndist_get_modes.restype = None
_lib.ndist_release_scratch.argtypes = []
_lib.ndist_release_scratch.restype = ctypes.c_int
_lib.ndist_last_kernel_ms.argtypes = [ctypes.POINTER(ctypes.c_float)]
_lib.ndist_last_kernel_ms.restype = ctypes.c_int
_lib.ndist_scratch_counters.argtypes = [ctypes.POINTER(ctypes.c_long), ctypes.POINTER(ctypes.c_long)]
_lib.ndist_scratch_counters.restype = None
_lib.ndist_noalloc_scratch_bytes.argtypes = []
_lib.ndist_noalloc_scratch_bytes.restype = ctypes.c_size_t
_lib.ndist_noalloc_prepare.argtypes = []
_lib.ndist_noalloc_prepare.restype = ctypes.c_int

_DIMS = (_I, _I, _I, _I, _I)
_norm_fwd = _sig("ndist_norm_dist_forward", _P, _P, *_DIMS, _P, _F, _P)
_norm_fwd_max = _sig("ndist_norm_dist_forward_with_max", _P, _P, _P, *_DIMS, _P, _F, _P)
_norm_bwd_x = _sig("ndist_norm_dist_backward_input", _P, _P, _P, _P, *_DIMS, _P, _F, _P)
_norm_bwd_xw = _sig("ndist_norm_dist_backward_input_weight", _P, _P, _P, _P, *_DIMS, _P, _P, _F, _P)
_norm_bwd_xw_noalloc = _sig("ndist_norm_dist_backward_input_weight_noalloc", _P, _P, _P, _P, *_DIMS, _P, _P, _F, _P)
_inf_fwd_ng = _sig("ndist_inf_dist_forward_nograd", _P, _P, *_DIMS, _P, _P)
_inf_fwd = _sig("ndist_inf_dist_forward", _P, _P, *_DIMS, _P, _P, _P)
_inf_bwd_x = _sig("ndist_inf_dist_backward_input", _P, _P, *_DIMS, _P, _P)
_inf_bwd_xw = _sig("ndist_inf_dist_backward_input_weight", _P, _P, *_DIMS, _P, _P, _P)
_bnd_fwd_ng = _sig("ndist_bound_inf_dist_forward_nograd", _P, _P, _P, *_DIMS, _P, _P, _P)
_bnd_fwd = _sig("ndist_bound_inf_dist_forward", _P, _P, _P, *_DIMS, _P, _P, _P, _P, _P)
_bnd_bwd_x = _sig("ndist_bound_inf_dist_backward_input", _P, _P, _P, _P, *_DIMS, _P, _P, _P)
_bnd_bwd_xw = _sig("ndist_bound_inf_dist_backward_input_weight", _P, _P, _P, _P, *_DIMS, _P, _P, _P, _P)
_joint_ng = _sig("ndist_inf_and_bound_forward_nograd", _P, _P, _P, _P, *_DIMS, _P, _P, _P, _P)
_joint = _sig("ndist_inf_and_bound_forward", _P, _P, _P, _P, *_DIMS, _P, _P, _P, _P, _P, _P, _P)
_ms_fwd = _sig("ndist_mean_shift_forward", _P, _P, _P, _I, _I, _I, _I, _F, _P, _P, _P, _P, _P, _P, _P, _P)
_lib.ndist_weight_cache_bytes.argtypes = [_I, _I, _I]
_lib.ndist_weight_cache_bytes.restype = ctypes.c_longlong
_wcache_prepare = _sig("ndist_weight_cache_prepare", _P, _I, _I, _I, _P, _P)
_inf_ng_cached = _sig("ndist_inf_dist_forward_nograd_cached", _P, _P, _P, _I, _I, _I, _I, _I, _P, _P)
_joint_ng_cached = _sig("ndist_inf_and_bound_forward_nograd_cached", _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _P, _P, _P)
_margin_fwd = _sig("ndist_margin_forward", _P, _P, _P, _P, _I, _I, _F, _P, _P)
_margin_bwd = _sig("ndist_margin_backward", _P, _P, _I, _I, _F, _P, _P, _P, _P)
_hinge_fwd = _sig("ndist_hinge_forward", _P, _I, _I, _F, _P, _P, _P)
_hinge_bwd = _sig("ndist_hinge_backward", _P, _P, _P, _I, _I, _F, _P, _P)
_ms_bwd = _sig("ndist_mean_shift_backward", _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P)
_unfold_fwd = _sig("ndist_unfold_forward", _P, *([_I] * 12), _P, _P)
_unfold_bwd = _sig("ndist_unfold_backward", _P, *([_I] * 12), _P, _P)
_conv_inf_ng = _sig("ndist_conv_inf_dist_forward_nograd", _P, _P, *([_I] * 14), _P, _P)
_conv_bnd_ng = _sig("ndist_conv_bound_inf_dist_forward_nograd", _P, _P, _P, *([_I] * 14), _P, _P, _P)
_conv_inf_fwd = _sig("ndist_conv_inf_dist_forward", _P, _P, *([_I] * 14), _P, _P, _P)
_conv_bnd_fwd = _sig("ndist_conv_bound_inf_dist_forward", _P, _P, _P, *([_I] * 14), _P, _P, _P, _P, _P)
_conv_norm_fwd = _sig("ndist_conv_norm_dist_forward", _P, _P, *([_I] * 14), _P, _F, _P)
_conv_norm_bwd_x = _sig("ndist_conv_norm_dist_backward_input", _P, _P, _P, _P, *([_I] * 14), _P, _F, _P)
_conv_norm_bwd_xw = _sig("ndist_conv_norm_dist_backward_input_weight", _P, _P, _P, _P, *([_I] * 14), _P, _P, _F, _P)
_conv_inf_bwd_x = _sig("ndist_conv_inf_dist_backward_input", _P, _P, *([_I] * 14), _P, _P)
_conv_inf_bwd_xw = _sig("ndist_conv_inf_dist_backward_input_weight", _P, _P, *([_I] * 14), _P, _P, _P)
_conv_bnd_bwd_x = _sig("ndist_conv_bound_inf_dist_backward_input", _P, _P, _P, _P, *([_I] * 14), _P, _P, _P)
_conv_bnd_bwd_xw = _sig("ndist_conv_bound_inf_dist_backward_input_weight", _P, _P, _P, _P, *([_I] * 14), _P, _P, _P, _P)


# status codes of the library (include/norm_dist_hip.h)
ERR_CAPTURE = 6
ERR_TOO_LARGE = 7


class NormDistError(RuntimeError):
    """A library call returned a non-zero status; `status` holds the code."""

    def __init__(self, message, status):
        super().__init__(message)
        self.status = status


def version():
    return _lib.ndist_version()


def scratch_counters():
    """(hipMalloc calls, hipFree calls) the library has made for its scratch arenas since it was loaded."""
    m, f = ctypes.c_long(0), ctypes.c_long(0)
    _lib.ndist_scratch_counters(ctypes.byref(m), ctypes.byref(f))
    return m.value, f.value


def noalloc_scratch_bytes():
    """Size of the fixed scratch array behind norm_dist_backward_input_weight_noalloc."""
    return int(_lib.ndist_noalloc_scratch_bytes())


def set_profiling(enable):
    """Measurement aid: bracket the dominant kernel of every following call with HIP events."""
    _lib.ndist_set_profiling(1 if enable else 0)


def set_skip_mode(skip=-1, bounds=-1):
    """Tuning / test aid: -1 lets the device-side probes choose the large-p kernel variants (default), 0 / 1 forces
    the pair-skipping variants off / on; `bounds` likewise for the two skipping variants of the backward.  Like the
    two settings below it belongs to the calling host thread: the entry points this thread calls afterwards follow
    it, other threads (autograd's backward threads among them) do not."""
    _lib.ndist_set_skip_mode(int(skip), int(bounds))


def set_hot_mode(mode=-1):
    """Tuning / test aid for the p = inf forward through hot k-tiles: -1 the device-side counts decide (default),
    0 never, 1 always the cheaper side, 2 always by the rows of x, 3 always by the rows of w."""
    _lib.ndist_set_hot_mode(int(mode))


def set_scaled_mode(mode=-1):
    """Tuning / test aid for the one-pass normalised forward (10 < p <= 48, fully connected layout): -1 from 2e7
    pairs on (default), 0 never, 1 whenever the layout allows."""
    _lib.ndist_set_scaled_mode(int(mode))


def get_modes():
    """(skip, bounds, hot, scaled) as the calling thread has them (see set_skip_mode, set_hot_mode, set_scaled_mode)."""
    v = [ctypes.c_int(-9) for _ in range(4)]
    _lib.ndist_get_modes(*(ctypes.byref(c) for c in v))
    return tuple(c.value for c in v)


def release_scratch():
    """Frees the temporary device memory the library keeps per (device, stream) between calls (waits for the device)."""
    rc = _lib.ndist_release_scratch()
    if rc != 0:
        raise RuntimeError("ndist_release_scratch failed (status %d)" % rc)


def last_kernel_ms():
    """Duration of the most recent bracketed kernel launched from this thread (waits for it)."""
    ms = ctypes.c_float(0.0)
    rc = _lib.ndist_last_kernel_ms(ctypes.byref(ms))
    if rc != 0:
        raise RuntimeError("no kernel timing recorded (status %d)" % rc)
    return ms.value


def _check(dtype, **tensors):
    dev = None
    for name, t in tensors.items():
        if not t.is_cuda:
            raise RuntimeError("%s must be a CUDA tensor" % name)  # same wording as the reference's CHECK_CUDA
        if not t.is_contiguous():
            raise RuntimeError("%s must be contiguous" % name)
        want = dtype.get(name, torch.float32)
        if t.dtype != want:
            raise RuntimeError("%s must have dtype %s, got %s" % (name, want, t.dtype))
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError("%s is on %s, expected %s" % (name, t.device, dev))
    return dev


def _agree(B, CO, CI, G, HW, **tensors):
    """Shape agreement of one operator call, by argument name: input-like tensors are [B, CI, HW], output-like ones
    (outputs, their gradients, arg-max codes) [B, CO, HW], weights [CO, CI / G].  The kernels index every tensor from
    these five numbers alone, so a tensor of another size would be read or written out of bounds."""
    if G <= 0 or CI % G or CO % G:
        raise RuntimeError("groups (%d) must divide the %d input and the %d output features" % (G, CI, CO))
    for name, t in tensors.items():
        if name == "cache":
            continue
        base = name[5:] if name.startswith("grad_") else name
        if base.startswith("input"):
            want = (B, CI, HW)
        elif base.startswith("weight"):
            want = (CO, CI // G)
        else:
            want = (B, CO, HW)
        if tuple(t.shape) != want:
            raise RuntimeError("%s must be %s, got %s" % (name, list(want), list(t.shape)))


def _run(fn, dev, *args, stream=None):
    with torch.cuda.device(dev):
        if stream is None:
            stream = torch.cuda.current_stream(dev).cuda_stream
        rc = fn(*args, stream)
    if rc != 0:
        raise NormDistError("%s failed: %s (hip error %d)" % (
            fn.__name__, _lib.ndist_status_string(rc).decode(), _lib.ndist_last_hip_error()), rc)


def _p(t):
    return t.data_ptr()


_STATUS_RE = re.compile(r"\(status (\d+),")


def _ext_call(fn, *args):
    """Call into the compiled binding; its errors carry the library's status code in their text."""
    try:
        fn(*args)
    except RuntimeError as e:
        m = _STATUS_RE.search(str(e))
        if m:
            raise NormDistError(str(e).split("\n")[0], int(m.group(1))) from None
        raise


def _geo8(geo):
    return list(geo[4:12])


_INT = {"pos": torch.int32, "posL": torch.int32, "posU": torch.int32}


def norm_dist_forward(input, weight, output, G, p):
    if _ext is not None:
        return _ext_call(_ext.norm_dist_forward, input, weight, output, G, p)
    dev = _check({}, input=input, weight=weight, output=output)
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _agree(B, CO, CI, G, HW, input=input, weight=weight, output=output)
    _run(_norm_fwd, dev, _p(input), _p(weight), B, CO, CI, G, HW, _p(output), p)


def norm_dist_forward_with_max(input, weight, max_output, output, G, p):
    if _ext is not None:
        return _ext_call(_ext.norm_dist_forward_with_max, input, weight, max_output, output, G, p)
    dev = _check({}, input=input, weight=weight, max_output=max_output, output=output)
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _agree(B, CO, CI, G, HW, input=input, weight=weight, max_output=max_output, output=output)
    _run(_norm_fwd_max, dev, _p(input), _p(weight), _p(max_output), B, CO, CI, G, HW, _p(output), p)


def norm_dist_backward_input(grad_output, input, weight, output, grad_input, G, p):
    if _ext is not None:
        return _ext_call(_ext.norm_dist_backward_input, grad_output, input, weight, output, grad_input, G, p)
    dev = _check({}, grad_output=grad_output, input=input, weight=weight, output=output, grad_input=grad_input)
    B, CO, CI, HW = grad_output.size(0), output.size(1), input.size(1), input.size(2)
    _agree(B, CO, CI, G, HW, grad_output=grad_output, input=input, weight=weight, output=output, grad_input=grad_input)
    _run(_norm_bwd_x, dev, _p(grad_output), _p(input), _p(weight), _p(output), B, CO, CI, G, HW, _p(grad_input), p)


def norm_dist_backward_input_weight(grad_output, input, weight, output, grad_input, grad_weight, G, p):
    if _ext is not None:
        return _ext_call(_ext.norm_dist_backward_input_weight, grad_output, input, weight, output, grad_input, grad_weight, G, p)
    dev = _check({}, grad_output=grad_output, input=input, weight=weight, output=output, grad_input=grad_input,
                 grad_weight=grad_weight)
    B, CO, CI, HW = grad_output.size(0), output.size(1), input.size(1), input.size(2)
    _agree(B, CO, CI, G, HW, grad_output=grad_output, input=input, weight=weight, output=output, grad_input=grad_input, grad_weight=grad_weight)
    _run(_norm_bwd_xw, dev, _p(grad_output), _p(input), _p(weight), _p(output), B, CO, CI, G, HW,
         _p(grad_input), _p(grad_weight), p)


def norm_dist_backward_input_weight_noalloc(grad_output, input, weight, output, grad_input, grad_weight, G, p,
                                            stream=None):
    """norm_dist_backward_input_weight without any allocation inside the library (scratch from a fixed device array);
    no counterpart in the reference.  `stream`: a raw hipStream_t to launch on instead of torch's current stream."""
    if _ext is not None and stream is None:
        return _ext_call(_ext.norm_dist_backward_input_weight_noalloc, grad_output, input, weight, output, grad_input,
                         grad_weight, G, p)
    dev = _check({}, grad_output=grad_output, input=input, weight=weight, output=output, grad_input=grad_input,
                 grad_weight=grad_weight)
    B, CO, CI, HW = grad_output.size(0), output.size(1), input.size(1), input.size(2)
    _agree(B, CO, CI, G, HW, grad_output=grad_output, input=input, weight=weight, output=output, grad_input=grad_input, grad_weight=grad_weight)
    _run(_norm_bwd_xw_noalloc, dev, _p(grad_output), _p(input), _p(weight), _p(output), B, CO, CI, G, HW,
         _p(grad_input), _p(grad_weight), p, stream=stream)


def inf_dist_forward(input, weight, output, pos, G):
    if _ext is not None:
        return _ext_call(_ext.inf_dist_forward, input, weight, output, pos, G)
    dev = _check(_INT, input=input, weight=weight, output=output, pos=pos)
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _agree(B, CO, CI, G, HW, input=input, weight=weight, output=output, pos=pos)
    _run(_inf_fwd, dev, _p(input), _p(weight), B, CO, CI, G, HW, _p(output), _p(pos))


def inf_dist_forward_nograd(input, weight, output, G):
    if _ext is not None:
        return _ext_call(_ext.inf_dist_forward_nograd, input, weight, output, G)
    dev = _check({}, input=input, weight=weight, output=output)
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _agree(B, CO, CI, G, HW, input=input, weight=weight, output=output)
    _run(_inf_fwd_ng, dev, _p(input), _p(weight), B, CO, CI, G, HW, _p(output))


def inf_dist_backward_input(grad_output, pos, grad_input, G):
    if _ext is not None:
        return _ext_call(_ext.inf_dist_backward_input, grad_output, pos, grad_input, G)
    dev = _check(_INT, grad_output=grad_output, pos=pos, grad_input=grad_input)
    B, CO, CI, HW = grad_output.size(0), grad_output.size(1), grad_input.size(1), grad_input.size(2)
    _agree(B, CO, CI, G, HW, grad_output=grad_output, pos=pos, grad_input=grad_input)
    _run(_inf_bwd_x, dev, _p(grad_output), _p(pos), B, CO, CI, G, HW, _p(grad_input))


def inf_dist_backward_input_weight(grad_output, pos, grad_input, grad_weight, G):
    if _ext is not None:
        return _ext_call(_ext.inf_dist_backward_input_weight, grad_output, pos, grad_input, grad_weight, G)
    dev = _check(_INT, grad_output=grad_output, pos=pos, grad_input=grad_input, grad_weight=grad_weight)
    B, CO, CI, HW = grad_output.size(0), grad_output.size(1), grad_weight.size(1) * G, grad_output.size(2)
    _agree(B, CO, CI, G, HW, grad_output=grad_output, pos=pos, grad_input=grad_input, grad_weight=grad_weight)
    _run(_inf_bwd_xw, dev, _p(grad_output), _p(pos), B, CO, CI, G, HW, _p(grad_input), _p(grad_weight))


def bound_inf_dist_forward_nograd(inputL, inputU, weight, outputL, outputU, G):
    if _ext is not None:
        return _ext_call(_ext.bound_inf_dist_forward_nograd, inputL, inputU, weight, outputL, outputU, G)
    dev = _check({}, inputL=inputL, inputU=inputU, weight=weight, outputL=outputL, outputU=outputU)
    B, CO, CI, HW = inputL.size(0), outputL.size(1), inputL.size(1), inputL.size(2)
    _agree(B, CO, CI, G, HW, inputL=inputL, inputU=inputU, weight=weight, outputL=outputL, outputU=outputU)
    _run(_bnd_fwd_ng, dev, _p(inputL), _p(inputU), _p(weight), B, CO, CI, G, HW, _p(outputL), _p(outputU))


def bound_inf_dist_forward(inputL, inputU, weight, outputL, outputU, posL, posU, G):
    if _ext is not None:
        return _ext_call(_ext.bound_inf_dist_forward, inputL, inputU, weight, outputL, outputU, posL, posU, G)
    dev = _check(_INT, inputL=inputL, inputU=inputU, weight=weight, outputL=outputL, outputU=outputU,
                 posL=posL, posU=posU)
    B, CO, CI, HW = inputL.size(0), outputL.size(1), inputL.size(1), inputL.size(2)
    _agree(B, CO, CI, G, HW, inputL=inputL, inputU=inputU, weight=weight, outputL=outputL, outputU=outputU, posL=posL, posU=posU)
    _run(_bnd_fwd, dev, _p(inputL), _p(inputU), _p(weight), B, CO, CI, G, HW, _p(outputL), _p(outputU),
         _p(posL), _p(posU))


def bound_inf_dist_backward_input(grad_outputL, grad_outputU, posL, posU, grad_inputL, grad_inputU, G):
    if _ext is not None:
        return _ext_call(_ext.bound_inf_dist_backward_input, grad_outputL, grad_outputU, posL, posU, grad_inputL, grad_inputU, G)
    dev = _check(_INT, grad_outputL=grad_outputL, grad_outputU=grad_outputU, posL=posL, posU=posU,
                 grad_inputL=grad_inputL, grad_inputU=grad_inputU)
    B, CO, CI, HW = grad_outputL.size(0), grad_outputL.size(1), grad_inputL.size(1), grad_inputL.size(2)
    _agree(B, CO, CI, G, HW, grad_outputL=grad_outputL, grad_outputU=grad_outputU, posL=posL, posU=posU, grad_inputL=grad_inputL, grad_inputU=grad_inputU)
    _run(_bnd_bwd_x, dev, _p(grad_outputL), _p(grad_outputU), _p(posL), _p(posU), B, CO, CI, G, HW,
         _p(grad_inputL), _p(grad_inputU))


def bound_inf_dist_backward_input_weight(grad_outputL, grad_outputU, posL, posU, grad_inputL, grad_inputU,
                                         grad_weight, G):
    if _ext is not None:
        return _ext_call(_ext.bound_inf_dist_backward_input_weight, grad_outputL, grad_outputU, posL, posU, grad_inputL, grad_inputU, grad_weight, G)
    dev = _check(_INT, grad_outputL=grad_outputL, grad_outputU=grad_outputU, posL=posL, posU=posU,
                 grad_inputL=grad_inputL, grad_inputU=grad_inputU, grad_weight=grad_weight)
    B, CO, CI, HW = grad_outputL.size(0), grad_outputL.size(1), grad_weight.size(1) * G, grad_outputL.size(2)
    _agree(B, CO, CI, G, HW, grad_outputL=grad_outputL, grad_outputU=grad_outputU, posL=posL, posU=posU, grad_inputL=grad_inputL, grad_inputU=grad_inputU, grad_weight=grad_weight)
    _run(_bnd_bwd_xw, dev, _p(grad_outputL), _p(grad_outputU), _p(posL), _p(posU), B, CO, CI, G, HW,
         _p(grad_inputL), _p(grad_inputU), _p(grad_weight))


def inf_and_bound_forward_nograd(input, inputL, inputU, weight, output, outputL, outputU, G):
    """inf_dist_forward_nograd(input) and bound_inf_dist_forward_nograd(inputL, inputU) against the same weights in one
    call: the two calls a layer makes under certification (reference: core/modules/norm_dist.py:30-34), with the
    pre-pass over the weights shared."""
    if _ext is not None:
        return _ext_call(_ext.inf_and_bound_forward_nograd, input, inputL, inputU, weight, output, outputL, outputU, G)
    dev = _check({}, input=input, inputL=inputL, inputU=inputU, weight=weight, output=output, outputL=outputL,
                 outputU=outputU)
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _agree(B, CO, CI, G, HW, input=input, inputL=inputL, inputU=inputU, weight=weight, output=output, outputL=outputL, outputU=outputU)
    _run(_joint_ng, dev, _p(input), _p(inputL), _p(inputU), _p(weight), B, CO, CI, G, HW, _p(output), _p(outputL),
         _p(outputU))


def weight_cache(weight, G):
    """The p = inf forwards' pre-pass over the weights (row maxima, their positions, 32-wide tile maxima) as a device
    buffer to pass to the *_cached forwards while the weights stay as they are: evaluation, certification, serving.
    (No counterpart in the reference; ctypes on either binding.)"""
    dev = _check({}, weight=weight)
    CO, CIg = weight.shape
    nbytes = _lib.ndist_weight_cache_bytes(CO, CIg * G, G)
    if nbytes <= 0:
        raise NormDistError("ndist_weight_cache_bytes: bad shape", 2)
    cache = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=weight.device)
    _run(_wcache_prepare, dev, _p(weight), CO, CIg * G, G, _p(cache))
    return cache


def inf_dist_forward_nograd_cached(input, weight, cache, output, G):
    dev = _check({}, input=input, weight=weight, cache=cache, output=output)
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _agree(B, CO, CI, G, HW, input=input, weight=weight, cache=cache, output=output)
    _run(_inf_ng_cached, dev, _p(input), _p(weight), _p(cache), B, CO, CI, G, HW, _p(output))


def inf_and_bound_forward_nograd_cached(input, inputL, inputU, weight, cache, output, outputL, outputU, G):
    dev = _check({}, input=input, inputL=inputL, inputU=inputU, weight=weight, cache=cache, output=output,
                 outputL=outputL, outputU=outputU)
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _agree(B, CO, CI, G, HW, input=input, inputL=inputL, inputU=inputU, weight=weight, cache=cache, output=output, outputL=outputL, outputU=outputU)
    _run(_joint_ng_cached, dev, _p(input), _p(inputL), _p(inputU), _p(weight), _p(cache), B, CO, CI, G, HW, _p(output),
         _p(outputL), _p(outputU))


def inf_and_bound_forward(input, inputL, inputU, weight, output, pos, outputL, outputU, posL, posU, G):
    """The same with the arg-max codes of all three reductions (inf_dist_forward + bound_inf_dist_forward)."""
    if _ext is not None:
        return _ext_call(_ext.inf_and_bound_forward, input, inputL, inputU, weight, output, pos, outputL, outputU, posL,
                         posU, G)
    dev = _check(_INT, input=input, inputL=inputL, inputU=inputU, weight=weight, output=output, pos=pos,
                 outputL=outputL, outputU=outputU, posL=posL, posU=posU)
    B, CO, CI, HW = input.size(0), output.size(1), input.size(1), input.size(2)
    _agree(B, CO, CI, G, HW, input=input, inputL=inputL, inputU=inputU, weight=weight, output=output, pos=pos, outputL=outputL, outputU=outputU, posL=posL, posU=posU)
    _run(_joint, dev, _p(input), _p(inputL), _p(inputU), _p(weight), B, CO, CI, G, HW, _p(output), _p(pos), _p(outputL),
         _p(outputU), _p(posL), _p(posU))


def _po(t):
    return None if t is None else t.data_ptr()


def _check_some(**tensors):
    return _check({}, **{k: v for k, v in tensors.items() if v is not None})


def mean_shift_forward(x, lower, upper, training, momentum, running_mean, bias1, bias2, mean_out, y, y_lower, y_upper):
    """Mean shift + bias of a distance layer in one call (no kernel of its own in the reference, which writes it in
    torch primitives: core/modules/basic_modules.py:121-132, core/modules/norm_dist.py:35-38).  Tensors [B, C, HW];
    absent ones are None.  y* = t* - mean[c] + bias1[c] + bias2[c] with mean the batch mean of x (training; also
    written to mean_out and folded into running_mean) or running_mean (evaluation)."""
    lead = x if x is not None else (lower if lower is not None else upper)
    B, C, HW = lead.shape
    if _ext is not None:
        return _ext_call(_ext.mean_shift_forward, x, lower, upper, B, C, HW, bool(training), float(momentum), running_mean,
                         bias1, bias2, mean_out, y, y_lower, y_upper)
    dev = _check_some(x=x, lower=lower, upper=upper, running_mean=running_mean, bias1=bias1, bias2=bias2,
                      mean_out=mean_out, y=y, y_lower=y_lower, y_upper=y_upper)
    _run(_ms_fwd, dev, _po(x), _po(lower), _po(upper), B, C, HW, 1 if training else 0, float(momentum), _po(running_mean),
         _po(bias1), _po(bias2), _po(mean_out), _po(y), _po(y_lower), _po(y_upper))


def mean_shift_backward(grad_y, grad_y_lower, grad_y_upper, training, grad_x, colsum_out, mean_scratch):
    """Backward of mean_shift_forward: colsum_out[c] = sum over (b, hw) of the given gradients (the bias gradient);
    training: grad_x = grad_y - colsum / (B HW).  The bounds' gradients pass through unchanged."""
    lead = grad_y if grad_y is not None else (grad_y_lower if grad_y_lower is not None else grad_y_upper)
    B, C, HW = lead.shape
    if _ext is not None:
        return _ext_call(_ext.mean_shift_backward, grad_y, grad_y_lower, grad_y_upper, B, C, HW, bool(training), grad_x,
                         colsum_out, mean_scratch)
    dev = _check_some(grad_y=grad_y, grad_y_lower=grad_y_lower, grad_y_upper=grad_y_upper, grad_x=grad_x,
                      colsum_out=colsum_out, mean_scratch=mean_scratch)
    _run(_ms_bwd, dev, _po(grad_y), _po(grad_y_lower), _po(grad_y_upper), B, C, HW, 1 if training else 0, _po(grad_x),
         _po(colsum_out), _po(mean_scratch))


_TAIL = {"targets": torch.int64, "argmax": torch.int32}


def margin_forward(x, lower, upper, targets, eps, margin):
    """Worst-case margins of the logits -x (ell_inf_models.py:41-46): margin[b, c] = (upper[b, t_b] - lower[b, c]) /
    (2 eps), 0 at c = t_b; lower / upper None: x -/+ eps.  (These four go through the C ABI with ctypes on either
    binding: a handful of launches per step.)"""
    dev = _check(_TAIL, **{k: v for k, v in dict(x=x, lower=lower, upper=upper, targets=targets, margin=margin).items()
                           if v is not None})
    B, C = margin.shape
    _run(_margin_fwd, dev, _po(x), _po(lower), _po(upper), _p(targets), B, C, float(eps), _p(margin))


def margin_backward(grad_margin, targets, eps, grad_x, grad_lower, grad_upper):
    dev = _check(_TAIL, **{k: v for k, v in dict(grad_margin=grad_margin, targets=targets, grad_x=grad_x,
                                                   grad_lower=grad_lower, grad_upper=grad_upper).items() if v is not None})
    B, C = grad_margin.shape
    _run(_margin_bwd, dev, _p(grad_margin), _p(targets), B, C, float(eps), _po(grad_x), _po(grad_lower), _po(grad_upper))


def hinge_forward(margin, mix, loss, argmax):
    """loss[0] = (1 - mix) * mean_b max_c relu(margin) + mix * mean relu(margin) (main.py:304-310)."""
    dev = _check(_TAIL, margin=margin, loss=loss, argmax=argmax)
    B, C = margin.shape
    _run(_hinge_fwd, dev, _p(margin), B, C, float(mix), _p(loss), _p(argmax))


def hinge_backward(margin, argmax, grad_loss, mix, grad_margin):
    dev = _check(_TAIL, margin=margin, argmax=argmax, grad_loss=grad_loss, grad_margin=grad_margin)
    B, C = margin.shape
    _run(_hinge_bwd, dev, _p(margin), _p(argmax), _p(grad_loss), B, C, float(mix), _p(grad_margin))


def _pair(v):
    return (int(v), int(v)) if isinstance(v, int) else (int(v[0]), int(v[1]))


def unfold_geometry(size, kernel_size, dilation, padding, stride):
    """(B, C, H, W, kh, kw, dh, dw, ph, pw, sh, sw) and the output size (OH, OW) of torch.nn.functional.unfold."""
    B, C, H, W = size
    (kh, kw), (dh, dw), (ph, pw), (sh, sw) = _pair(kernel_size), _pair(dilation), _pair(padding), _pair(stride)
    OH = (H + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    OW = (W + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    return (B, C, H, W, kh, kw, dh, dw, ph, pw, sh, sw), (OH, OW)


def unfold_forward(input, output, kernel_size, dilation, padding, stride):
    """input [B, C, H, W] -> output [B, C*kh*kw, OH*OW]; no counterpart in the reference's extension (it calls
    torch.nn.functional.unfold, core/modules/norm_dist.py:93-102)."""
    dev = _check({}, input=input, output=output)
    geo, (OH, OW) = unfold_geometry(input.shape, kernel_size, dilation, padding, stride)
    if tuple(output.shape) != (geo[0], geo[1] * geo[4] * geo[5], OH * OW):
        raise RuntimeError("output has shape %s, expected %s" % (tuple(output.shape), (geo[0], geo[1] * geo[4] * geo[5], OH * OW)))
    if _ext is not None:
        return _ext_call(_ext.unfold_forward, input, output, _geo8(geo))
    _run(_unfold_fwd, dev, _p(input), *geo, _p(output))


def unfold_backward(grad_output, grad_input, kernel_size, dilation, padding, stride):
    """Adjoint of unfold_forward: grad_output [B, C*kh*kw, OH*OW] -> grad_input [B, C, H, W] (fully overwritten)."""
    dev = _check({}, grad_output=grad_output, grad_input=grad_input)
    geo, (OH, OW) = unfold_geometry(grad_input.shape, kernel_size, dilation, padding, stride)
    if tuple(grad_output.shape) != (geo[0], geo[1] * geo[4] * geo[5], OH * OW):
        raise RuntimeError("grad_output has shape %s, expected %s" % (tuple(grad_output.shape), (geo[0], geo[1] * geo[4] * geo[5], OH * OW)))
    if _ext is not None:
        return _ext_call(_ext.unfold_backward, grad_output, grad_input, _geo8(geo))
    _run(_unfold_bwd, dev, _p(grad_output), *geo, _p(grad_input))


def _conv_args(input, weight, output, G, kernel_size, dilation, padding, stride):
    (B, C, H, W, kh, kw, dh, dw, ph, pw, sh, sw), (OH, OW) = unfold_geometry(input.shape, kernel_size, dilation, padding,
                                                                                stride)
    CO = weight.size(0)
    if C % G != 0 or tuple(weight.shape) != (CO, C // G * kh * kw):
        raise RuntimeError("weight has shape %s, expected %s" % (tuple(weight.shape), (CO, C // G * kh * kw)))
    if tuple(output.shape) != (B, CO, OH * OW):
        raise RuntimeError("output has shape %s, expected %s" % (tuple(output.shape), (B, CO, OH * OW)))
    return (B, C, H, W, CO, G, kh, kw, dh, dw, ph, pw, sh, sw)


def conv_inf_dist_forward_nograd(input, weight, output, G, kernel_size, dilation, padding, stride):
    """unfold + inf_dist_forward_nograd in one kernel: input [B, C, H, W] -> output [B, CO, OH*OW], the unfolded
    tensor is never written (the reference materialises it, core/modules/norm_dist.py:93-102)."""
    dev = _check({}, input=input, weight=weight, output=output)
    args = _conv_args(input, weight, output, G, kernel_size, dilation, padding, stride)
    if _ext is not None:
        return _ext_call(_ext.conv_inf_dist_forward_nograd, input, weight, output, G, list(args[6:14]))
    _run(_conv_inf_ng, dev, _p(input), _p(weight), *args, _p(output))


def conv_bound_inf_dist_forward_nograd(inputL, inputU, weight, outputL, outputU, G, kernel_size, dilation, padding,
                                       stride):
    """unfold of both bounds + bound_inf_dist_forward_nograd in one kernel."""
    dev = _check({}, inputL=inputL, inputU=inputU, weight=weight, outputL=outputL, outputU=outputU)
    if inputL.shape != inputU.shape or outputL.shape != outputU.shape:
        raise RuntimeError("lower and upper tensors must have the same shape")
    args = _conv_args(inputL, weight, outputL, G, kernel_size, dilation, padding, stride)
    if _ext is not None:
        return _ext_call(_ext.conv_bound_inf_dist_forward_nograd, inputL, inputU, weight, outputL, outputU, G,
                         list(args[6:14]))
    _run(_conv_bnd_ng, dev, _p(inputL), _p(inputU), _p(weight), *args, _p(outputL), _p(outputU))


def conv_norm_dist_forward(input, weight, output, G, p, kernel_size, dilation, padding, stride):
    """unfold + norm_dist_forward in one kernel for finite p: input [B, C, H, W] -> output [B, CO, OH*OW]."""
    dev = _check({}, input=input, weight=weight, output=output)
    args = _conv_args(input, weight, output, G, kernel_size, dilation, padding, stride)
    if _ext is not None:
        return _ext_call(_ext.conv_norm_dist_forward, input, weight, output, G, float(p), list(args[6:14]))
    _run(_conv_norm_fwd, dev, _p(input), _p(weight), *args, _p(output), float(p))


def conv_norm_dist_backward_input(grad_output, input, weight, output, grad_input, G, p, kernel_size, dilation, padding,
                                  stride):
    """Finite-p backward on images: grad_input [B, C, H, W] (the adjoint of the patch extraction applied)."""
    dev = _check({}, grad_output=grad_output, input=input, weight=weight, output=output, grad_input=grad_input)
    args = _conv_args(input, weight, output, G, kernel_size, dilation, padding, stride)
    if grad_output.shape != output.shape or grad_input.shape != input.shape:
        raise RuntimeError("gradients must have the shapes of output and input")
    if _ext is not None:
        return _ext_call(_ext.conv_norm_dist_backward_input, grad_output, input, weight, output, grad_input, G, float(p),
                         list(args[6:14]))
    _run(_conv_norm_bwd_x, dev, _p(grad_output), _p(input), _p(weight), _p(output), *args, _p(grad_input), float(p))


def conv_norm_dist_backward_input_weight(grad_output, input, weight, output, grad_input, grad_weight, G, p, kernel_size,
                                         dilation, padding, stride):
    dev = _check({}, grad_output=grad_output, input=input, weight=weight, output=output, grad_input=grad_input,
                 grad_weight=grad_weight)
    args = _conv_args(input, weight, output, G, kernel_size, dilation, padding, stride)
    if grad_output.shape != output.shape or grad_input.shape != input.shape or grad_weight.shape != weight.shape:
        raise RuntimeError("gradients must have the shapes of output, input and weight")
    if _ext is not None:
        return _ext_call(_ext.conv_norm_dist_backward_input_weight, grad_output, input, weight, output, grad_input,
                         grad_weight, G, float(p), list(args[6:14]))
    _run(_conv_norm_bwd_xw, dev, _p(grad_output), _p(input), _p(weight), _p(output), *args, _p(grad_input),
         _p(grad_weight), float(p))


def conv_inf_dist_forward(input, weight, output, pos, G, kernel_size, dilation, padding, stride):
    """unfold + inf_dist_forward in one kernel pair: values and arg-max codes of the unfolded problem."""
    dev = _check(_INT, input=input, weight=weight, output=output, pos=pos)
    args = _conv_args(input, weight, output, G, kernel_size, dilation, padding, stride)
    if pos.shape != output.shape:
        raise RuntimeError("pos must have the shape of output")
    if _ext is not None:
        return _ext_call(_ext.conv_inf_dist_forward, input, weight, output, pos, G, list(args[6:14]))
    _run(_conv_inf_fwd, dev, _p(input), _p(weight), *args, _p(output), _p(pos))


def conv_bound_inf_dist_forward(inputL, inputU, weight, outputL, outputU, posL, posU, G, kernel_size, dilation, padding,
                                stride):
    dev = _check(_INT, inputL=inputL, inputU=inputU, weight=weight, outputL=outputL, outputU=outputU, posL=posL,
                 posU=posU)
    if inputL.shape != inputU.shape or not (outputL.shape == outputU.shape == posL.shape == posU.shape):
        raise RuntimeError("lower and upper tensors must have the same shape")
    args = _conv_args(inputL, weight, outputL, G, kernel_size, dilation, padding, stride)
    if _ext is not None:
        return _ext_call(_ext.conv_bound_inf_dist_forward, inputL, inputU, weight, outputL, outputU, posL, posU, G,
                         list(args[6:14]))
    _run(_conv_bnd_fwd, dev, _p(inputL), _p(inputU), _p(weight), *args, _p(outputL), _p(outputU), _p(posL), _p(posU))


def _conv_backward_args(grad_output, grad_input, weight_shape, G, kernel_size, dilation, padding, stride):
    (B, C, H, W, kh, kw, dh, dw, ph, pw, sh, sw), (OH, OW) = unfold_geometry(grad_input.shape, kernel_size, dilation,
                                                                                padding, stride)
    CO = weight_shape[0]
    if C % G != 0 or tuple(weight_shape) != (CO, C // G * kh * kw):
        raise RuntimeError("weight has shape %s, expected %s" % (tuple(weight_shape), (CO, C // G * kh * kw)))
    if tuple(grad_output.shape) != (B, CO, OH * OW):
        raise RuntimeError("grad_output has shape %s, expected %s" % (tuple(grad_output.shape), (B, CO, OH * OW)))
    return (B, C, H, W, CO, G, kh, kw, dh, dw, ph, pw, sh, sw)


def conv_inf_dist_backward_input(grad_output, pos, grad_input, weight_shape, G, kernel_size, dilation, padding, stride):
    """inf_dist_backward_input followed by the adjoint of the patch extraction: grad_input is [B, C, H, W]."""
    dev = _check(_INT, grad_output=grad_output, pos=pos, grad_input=grad_input)
    args = _conv_backward_args(grad_output, grad_input, weight_shape, G, kernel_size, dilation, padding, stride)
    if _ext is not None:
        return _ext_call(_ext.conv_inf_dist_backward_input, grad_output, pos, grad_input, args[4], G, list(args[6:14]))
    _run(_conv_inf_bwd_x, dev, _p(grad_output), _p(pos), *args, _p(grad_input))


def conv_inf_dist_backward_input_weight(grad_output, pos, grad_input, grad_weight, G, kernel_size, dilation, padding,
                                        stride):
    dev = _check(_INT, grad_output=grad_output, pos=pos, grad_input=grad_input, grad_weight=grad_weight)
    args = _conv_backward_args(grad_output, grad_input, grad_weight.shape, G, kernel_size, dilation, padding, stride)
    if _ext is not None:
        return _ext_call(_ext.conv_inf_dist_backward_input_weight, grad_output, pos, grad_input, grad_weight, G,
                         list(args[6:14]))
    _run(_conv_inf_bwd_xw, dev, _p(grad_output), _p(pos), *args, _p(grad_input), _p(grad_weight))


def conv_bound_inf_dist_backward_input(grad_outputL, grad_outputU, posL, posU, grad_inputL, grad_inputU, weight_shape, G,
                                       kernel_size, dilation, padding, stride):
    dev = _check(_INT, grad_outputL=grad_outputL, grad_outputU=grad_outputU, posL=posL, posU=posU,
                 grad_inputL=grad_inputL, grad_inputU=grad_inputU)
    args = _conv_backward_args(grad_outputL, grad_inputL, weight_shape, G, kernel_size, dilation, padding, stride)
    if _ext is not None:
        return _ext_call(_ext.conv_bound_inf_dist_backward_input, grad_outputL, grad_outputU, posL, posU, grad_inputL,
                         grad_inputU, args[4], G, list(args[6:14]))
    _run(_conv_bnd_bwd_x, dev, _p(grad_outputL), _p(grad_outputU), _p(posL), _p(posU), *args, _p(grad_inputL),
         _p(grad_inputU))


def conv_bound_inf_dist_backward_input_weight(grad_outputL, grad_outputU, posL, posU, grad_inputL, grad_inputU,
                                              grad_weight, G, kernel_size, dilation, padding, stride):
    dev = _check(_INT, grad_outputL=grad_outputL, grad_outputU=grad_outputU, posL=posL, posU=posU,
                 grad_inputL=grad_inputL, grad_inputU=grad_inputU, grad_weight=grad_weight)
    args = _conv_backward_args(grad_outputL, grad_inputL, grad_weight.shape, G, kernel_size, dilation, padding, stride)
    if _ext is not None:
        return _ext_call(_ext.conv_bound_inf_dist_backward_input_weight, grad_outputL, grad_outputU, posL, posU,
                         grad_inputL, grad_inputU, grad_weight, G, list(args[6:14]))
    _run(_conv_bnd_bwd_xw, dev, _p(grad_outputL), _p(grad_outputU), _p(posL), _p(posU), *args, _p(grad_inputL),
         _p(grad_inputU), _p(grad_weight))
