"""Tensor-level front end of libboxconv_hip.so (C ABI in include/boxconv.h).

The four functions mirror the reference's pybind11 module ``box_convolution_cpp_cuda``
(reference src/bind.cpp:29-34) in names, argument order, argument meaning and error messages
(reference src/box_convolution_interface.cpp:19-34,153-170, src/integral_image_interface.cpp:9).
PyTorch is used only for device memory and the current stream; all arithmetic happens in the HIP
kernels. There is no CPU implementation here: tensors that are not on a HIP device, or a missing
library, raise ``RuntimeError``.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libboxconv_hip.so"
LIB_PATH = os.path.join(_HERE, LIB_NAME)

ABI_VERSION = 4

_lib = None

_vp, _i, _i64, _sz, _f, _d = (ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t,
                              ctypes.c_float, ctypes.c_double)

# name -> (restype, argtypes); kept in step with include/boxconv.h
_SIGNATURES = {
    "boxconv_abi_version": (_i, []),
    "boxconv_last_error": (ctypes.c_char_p, []),
    "boxconv_reload_env": (None, []),
    "boxconv_profile_arm": (_i, [ctypes.c_char_p]),
    "boxconv_profile_arm_every": (_i, [ctypes.c_char_p, _i]),
    "boxconv_profile_collect": (_i, [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_int)]),
    "boxconv_probe_copy_bands": (_i, [_vp, _vp, _i64, _i, _i, _i, _i, _vp]),
    "boxconv_probe_grad_input_pattern": (_i, [_vp, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _vp]),
    "boxconv_integral_image_workspace_bytes": (_sz, [_i64, _i, _i]),
    "boxconv_backward_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _i, _i, _i]),
}
for _s in ("f32", "f64"):
    _SIGNATURES["boxconv_integral_image_" + _s] = (_i, [_vp, _vp, _i64, _i, _i, _vp, _sz, _vp])
    _SIGNATURES["boxconv_forward_" + _s] = (_i, [_vp] * 6 + [_i] * 7 + [_vp])
    _SIGNATURES["boxconv_backward_" + _s] = (
        _i, [_vp] * 7 + [_f, _f, _i, _i] + [_vp] * 5 + [_i] * 5 + [_vp, _sz, _vp])
    _SIGNATURES["boxconv_clip_parameters_" + _s] = (_i, [_vp] * 4 + [_i] + [_d] * 4 + [_i, _vp])
    _SIGNATURES["boxconv_clip_reparametrize_" + _s] = (_i, [_vp] * 5 + [_i] + [_d] * 4 + [_i, _vp])
    _SIGNATURES["boxconv_training_forward_" + _s] = (
        _i, [_vp] * 8 + [_i] * 5 + [_d] * 4 + [_i, _i] + [_vp, _sz, _vp])
    _SIGNATURES["boxconv_inference_forward_" + _s] = (
        _i, [_vp] * 8 + [_i] * 5 + [_d] * 2 + [_i, _i] + [_vp, _sz, _vp])

_SIGNATURES["boxconv_backward_half_f32"] = (
    _i, [_vp] * 6 + [_i, _f, _f, _i, _i] + [_vp] * 5 + [_i] * 5 + [_vp, _sz, _vp])
_SIGNATURES["boxconv_training_forward_half_f32"] = (
    _i, [_vp, _i] + [_vp] * 7 + [_i] * 5 + [_d] * 4 + [_i, _i, _i] + [_vp, _sz, _vp])
_SIGNATURES["boxconv_integral_image_static_f32"] = (_i, [_vp, _vp, _i64, _i, _i, _vp])
_SIGNATURES["boxconv_integral_image_int"] = (_i, [_vp, _vp, _i, _i64, _i, _i, _vp])
_SIGNATURES["boxconv_integral_image_half_f32"] = (_i, [_vp, _i, _vp, _i64, _i, _i, _vp, _sz, _vp])
_SIGNATURES["boxconv_forward_fused_f32"] = (_i, [_vp] * 6 + [_i] + [_vp] * 3 + [_i] * 8 + [_vp])

EXPORTED_SYMBOLS = tuple(sorted(_SIGNATURES))

# element type codes BOXCONV_F32 / BOXCONV_F16 / BOXCONV_BF16 (include/boxconv.h)
_FUSED_OUTPUT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}

_SUFFIX = {torch.float32: "f32", torch.float64: "f64"}
# element type codes BOXCONV_U8 .. BOXCONV_I64
_INT_DTYPE = {torch.uint8: 16, torch.int8: 17, torch.int16: 18, torch.int32: 19, torch.int64: 20}


def load():
    """Load libboxconv_hip.so once. Raises RuntimeError if it was never built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.isfile(LIB_PATH):
        raise RuntimeError(
            "box_convolution: %s is missing; build it with "
            "`python box-convolutions_amd/build.py` (needs hipcc). There is no CPU fallback."
            % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.boxconv_abi_version() != ABI_VERSION:
        raise RuntimeError("box_convolution: %s has ABI version %d, expected %d"
                           % (LIB_PATH, lib.boxconv_abi_version(), ABI_VERSION))
    _lib = lib
    return lib


GLUE_NAME = "_boxconv_glue"
GLUE_PATH = os.path.join(_HERE, GLUE_NAME + ".so")
_glue = None          # the module, or False once loading was tried without success


def glue():
    """The C++ autograd node of the training step (csrc/torch_glue.cpp), or None where that
    extension was not built: an optional fast path for the HOST side of a step (checks,
    allocations, autograd callbacks in C++ instead of Python). It calls the same entry points of
    libboxconv_hip.so, handed over here as addresses, so results do not depend on it; set
    BOXCONV_PYTHON_GLUE=1 to keep it out."""
    global _glue
    if _glue is None:
        _glue = False
        if os.path.isfile(GLUE_PATH) and os.environ.get("BOXCONV_PYTHON_GLUE") != "1":
            import importlib.util
            import warnings
            lib = load()
            try:
                spec = importlib.util.spec_from_file_location(GLUE_NAME, GLUE_PATH)
                module = importlib.util.module_from_spec(spec)
                spec.loader.exec_module(module)
            except (ImportError, OSError) as exc:      # e.g. built against another torch
                warnings.warn("box_convolution: %s could not be loaded (%s); the training step keeps "
                              "its Python glue (same kernels, more host time per step)" % (GLUE_PATH, exc))
                return None
            module.init(*[ctypes.cast(getattr(lib, name), ctypes.c_void_p).value for name in (
                "boxconv_training_forward_f32", "boxconv_training_forward_f64",
                "boxconv_inference_forward_f32", "boxconv_inference_forward_f64", "boxconv_backward_f32",
                "boxconv_backward_f64", "boxconv_training_forward_half_f32", "boxconv_backward_half_f32",
                "boxconv_integral_image_workspace_bytes", "boxconv_backward_workspace_bytes",
                "boxconv_last_error")])
            _glue = module
    return _glue or None


def training_step(input, x_min, x_max, y_min, y_max, reparametrization_h, reparametrization_w,
                  max_input_h, max_input_w, normalize, exact, clip=True):
    """``BoxConv2d.forward`` through the C++ autograd node. ``clip`` (training mode): clips the
    stored parameters in place first; without it (eval mode) they are only read. Returns the
    output; its backward gives the five gradients. Same native calls as
    ``BoxConvolutionFunction`` (with ``clip_to`` in training mode). Requires ``glue()``."""
    # (the backward runs on the autograd engine's thread for input's device, which makes that
    # device current itself)
    with _on_device(input.device):
        return _glue.training_step(
            input, x_min, x_max, y_min, y_max, float(reparametrization_h), float(reparametrization_w),
            float(max_input_h), float(max_input_w), bool(normalize), bool(exact), bool(clip),
            _stream(input.device) or 0, torch.cuda.is_current_stream_capturing())


def _check(rc, what):
    if rc != 0:
        msg = load().boxconv_last_error().decode("utf-8", "replace")
        raise RuntimeError("box_convolution: %s failed (code %d): %s" % (what, rc, msg))


def _suffix(t, what):
    try:
        return _SUFFIX[t.dtype]
    except KeyError:
        raise RuntimeError("box_convolution: %s must be float32 or float64, got %s"
                           % (what, t.dtype)) from None


def _require_device(t, what):
    if not t.is_cuda:
        raise RuntimeError(
            "box_convolution: %s is on '%s'; this build runs on AMD GPUs only (no CPU path)"
            % (what, t.device))


def _stream(device):
    """The current stream of `device` as a raw hipStream_t (an integer; 0 is the null stream,
    which the C ABI takes as NULL)."""
    index = device.index
    if index is None:
        index = torch.cuda.current_device()
    return torch._C._cuda_getCurrentRawStream(index) or None


class _on_device:
    """``with _on_device(dev):`` makes `dev` the current device for the native call; it does
    nothing when it already is (the usual case, and ``torch.cuda.device`` costs microseconds)."""
    __slots__ = ("guard",)

    def __init__(self, device):
        index = device.index
        self.guard = (torch.cuda.device(index)
                      if index is not None and index != torch.cuda.current_device() else None)

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            return self.guard.__exit__(*exc)
        return False


def _ptr(t):
    """Device address as an integer (ctypes converts it to void*), None for a null pointer."""
    return None if t is None else t.data_ptr()


# Scratch memory of the native calls. Every call needs it only until its own kernels have run, and
# calls on one stream run in order, so one buffer per (device, stream), grown on demand, serves
# them all: a training step then allocates no scratch (at the headline size the backward's is
# 537 MB). While a stream is being captured into a graph the buffer comes from the allocator as
# usual (the capture's own pool), because a cached buffer may be replaced, and so freed, by a
# later, larger call while the graph still points at it.
_workspaces = {}


def _workspace(nbytes, device, stream):
    if nbytes == 0:
        return None
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(nbytes, dtype=torch.uint8, device=device)
    key = (device.index, stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        _workspaces.pop(key, None)
        ws = None                       # released before the larger one is requested
        ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def release_workspaces():
    """Drop the cached scratch buffers (they are re-created on demand)."""
    _workspaces.clear()
    if _glue:
        _glue.release_workspaces()


# workspace sizes by call signature: the C ABI's *_workspace_bytes functions are pure
_workspace_bytes = {}


def _integral_workspace_bytes(lib, planes, h, w):
    key = (planes, h, w)
    n = _workspace_bytes.get(key)
    if n is None:
        n = _workspace_bytes[key] = lib.boxconv_integral_image_workspace_bytes(planes, h, w)
    return n


def _backward_workspace_bytes(lib, B, C, F, h, w, elem, want_input, want_params):
    key = (B, C, F, h, w, elem, want_input, want_params)
    n = _workspace_bytes.get(key)
    if n is None:
        n = _workspace_bytes[key] = lib.boxconv_backward_workspace_bytes(
            B, C, F, h, w, elem, int(want_input), int(want_params))
    return n


_MAX_WIDENING_WIDTH = 2048     # widest row boxconv_integral_image_half_f32 reads directly
_MAX_STREAM_WIDTH = 4096       # widest row boxconv_backward_half_f32 reads directly


def half_rows_read_directly(h, w):
    """Whether the integral image kernels read float16 / bfloat16 planes of h x w themselves
    (otherwise the tensor is converted to float32 first)."""
    return w <= _MAX_WIDENING_WIDTH and (h + 1) * (w + 1) * 4 < 2 ** 31


def integral_image(input):
    """``integral_image(Tensor) -> Tensor`` (reference src/integral_image_interface.cpp:8-27).

    A float16 / bfloat16 input gives a float32 integral image (sums carried in double, as for
    float32 input); the reference would integrate it in half precision."""
    if input.dim() < 2:
        raise RuntimeError("integral image input must have >=2 dimensions")
    _require_device(input, "integral image input")
    if input.dtype in _INT_DTYPE:
        return _integral_image_int(input)
    half = input.dtype in (torch.float16, torch.bfloat16)
    h, w = input.shape[-2:]
    if half and not half_rows_read_directly(h, w):
        input, half = input.float(), False
    sfx = "half_f32" if half else _suffix(input, "integral image input")
    lib = load()
    input = input.contiguous()
    out_shape = tuple(input.shape[:-2]) + (h + 1, w + 1)
    output = torch.empty(out_shape, dtype=torch.float32 if half else input.dtype, device=input.device)
    if h == 0 or w == 0:
        return output.zero_()
    planes = input.numel() // (h * w)
    with _on_device(input.device):
        nbytes = _integral_workspace_bytes(lib, planes, h, w)
        stream = _stream(input.device)
        ws = _workspace(nbytes, input.device, stream)
        if half:
            rc = lib.boxconv_integral_image_half_f32(
                _ptr(input), _FUSED_OUTPUT[input.dtype], _ptr(output), planes, h, w, _ptr(ws), nbytes,
                stream)
        else:
            rc = getattr(lib, "boxconv_integral_image_" + sfx)(
                _ptr(input), _ptr(output), planes, h, w, _ptr(ws), nbytes, stream)
    _check(rc, "integral_image")
    return output


def _integral_image_int(input):
    """Integer tensors (the reference's CPU function takes every ATen type,
    src/integral_image.cpp:14): exact sums, stored modulo 2^bits in the input's own type."""
    lib = load()
    input = input.contiguous()
    h, w = input.shape[-2:]
    output = torch.empty(tuple(input.shape[:-2]) + (h + 1, w + 1), dtype=input.dtype, device=input.device)
    if h == 0 or w == 0:
        return output.zero_()
    planes = input.numel() // (h * w)
    with _on_device(input.device):
        rc = lib.boxconv_integral_image_int(_ptr(input), _ptr(output), _INT_DTYPE[input.dtype], planes,
                                            h, w, _stream(input.device))
    _check(rc, "integral_image")
    return output


def _check_params(x_min, x_max, y_min, y_max, in_planes, prefix):
    if not (x_min.dim() == 2 and x_max.dim() == 2 and y_min.dim() == 2 and y_max.dim() == 2):
        raise RuntimeError(prefix + "all parameters must have 2 dimensions")
    if not (x_min.size(0) == x_max.size(0) == y_min.size(0) == y_max.size(0) == in_planes):
        raise RuntimeError(
            prefix + "all parameters must have as many rows as there are input channels")
    if not (x_min.size(1) == x_max.size(1) == y_min.size(1) == y_max.size(1)):
        raise RuntimeError(prefix + "all parameters must have equal number of columns")


def _same_kind(params, like, what):
    out = []
    for p in params:
        if p.device != like.device:
            raise RuntimeError("BoxConv2d: input and parameters are on different devices")
        if p.dtype != like.dtype:
            raise RuntimeError("box_convolution: %s and parameters have different dtypes (%s, %s)"
                               % (what, like.dtype, p.dtype))
        out.append(p if p.is_contiguous() else p.contiguous())    # (only the address is used)
    return out


def box_convolution_forward(input_integrated, x_min, x_max, y_min, y_max, normalize, exact):
    """Reference src/box_convolution_interface.cpp:13-139. Parameters are in real pixel units.

    Returns ``[B, C*F, h, w]``."""
    if input_integrated.device != x_min.device:
        raise RuntimeError("BoxConv2d: input and parameters are on different devices")
    _require_device(input_integrated, "input")
    if input_integrated.dim() != 4:
        raise RuntimeError("BoxConv2d: input must have 4 dimensions")
    sfx = _suffix(input_integrated, "input")
    _check_params(x_min, x_max, y_min, y_max, input_integrated.size(1), "BoxConv2d: ")
    lib = load()
    input_integrated = input_integrated.contiguous()
    x_min, x_max, y_min, y_max = _same_kind((x_min, x_max, y_min, y_max), input_integrated, "input")
    B, C, h1, w1 = input_integrated.shape
    F = x_min.size(1)
    h, w = h1 - 1, w1 - 1
    if h < 1 or w < 1:
        raise RuntimeError("BoxConv2d: integral image must be at least 2x2")
    output = torch.empty((B, C * F, h, w), dtype=input_integrated.dtype,
                         device=input_integrated.device)
    if output.numel() == 0:
        return output
    with _on_device(input_integrated.device):
        rc = getattr(lib, "boxconv_forward_" + sfx)(
            _ptr(input_integrated), _ptr(x_min), _ptr(x_max), _ptr(y_min), _ptr(y_max),
            _ptr(output), B, C, F, h, w, int(bool(normalize)), int(bool(exact)),
            _stream(output.device))
    _check(rc, "box_convolution_forward")
    return output


def box_convolution_forward_fused(input_integrated, x_min, x_max, y_min, y_max, normalize, exact,
                                  output_dtype=torch.float32, channel_scale=None,
                                  channel_shift=None, residual=None, relu=False):
    """Forward box sums from a float32 integral image, written as ``output_dtype`` (float32,
    float16 or bfloat16), with an optional tail fused into the store:
    ``y = S * channel_scale[ch] + channel_shift[ch] + residual``, then ``relu`` (the tail of the
    reference's BottleneckBoxConv in eval mode, examples/Cityscapes/models/ENet.py:290-304).
    Parameters are in real pixel units, float32. Inference only: nothing here is differentiable.

    Returns ``[B, C*F, h, w]`` of ``output_dtype``."""
    if input_integrated.device != x_min.device:
        raise RuntimeError("BoxConv2d: input and parameters are on different devices")
    _require_device(input_integrated, "input")
    if input_integrated.dim() != 4:
        raise RuntimeError("BoxConv2d: input must have 4 dimensions")
    if input_integrated.dtype != torch.float32:
        raise RuntimeError("box_convolution: the fused forward takes a float32 integral image, got %s"
                           % input_integrated.dtype)
    if output_dtype not in _FUSED_OUTPUT:
        raise RuntimeError("box_convolution: the fused forward writes float32, float16 or bfloat16, "
                           "not %s" % output_dtype)
    _check_params(x_min, x_max, y_min, y_max, input_integrated.size(1), "BoxConv2d: ")
    lib = load()
    input_integrated = input_integrated.contiguous()
    x_min, x_max, y_min, y_max = _same_kind((x_min, x_max, y_min, y_max), input_integrated, "input")
    B, C, h1, w1 = input_integrated.shape
    F = x_min.size(1)
    h, w = h1 - 1, w1 - 1
    if h < 1 or w < 1:
        raise RuntimeError("BoxConv2d: integral image must be at least 2x2")
    dev = input_integrated.device
    per_channel = []
    for name, t in (("channel_scale", channel_scale), ("channel_shift", channel_shift)):
        if t is not None:
            if t.device != dev or t.numel() != C * F:
                raise RuntimeError("box_convolution: %s must hold %d values on %s" % (name, C * F, dev))
            t = t.detach().to(torch.float32).contiguous()
        per_channel.append(t)
    if residual is not None:
        if residual.device != dev or tuple(residual.shape) != (B, C * F, h, w):
            raise RuntimeError("box_convolution: residual must have the shape of the output, "
                               "%s, on %s" % ((B, C * F, h, w), dev))
        residual = residual.detach().to(output_dtype).contiguous()
    output = torch.empty((B, C * F, h, w), dtype=output_dtype, device=dev)
    if output.numel() == 0:
        return output
    with _on_device(dev):
        rc = lib.boxconv_forward_fused_f32(
            _ptr(input_integrated), _ptr(x_min), _ptr(x_max), _ptr(y_min), _ptr(y_max),
            _ptr(output), _FUSED_OUTPUT[output_dtype], _ptr(residual), _ptr(per_channel[0]),
            _ptr(per_channel[1]), int(bool(relu)), B, C, F, h, w, int(bool(normalize)),
            int(bool(exact)), _stream(dev))
    _check(rc, "box_convolution_forward_fused")
    return output


def box_convolution_backward(input_integrated, x_min, x_max, y_min, y_max, grad_output, output,
                             reparametrization_h, reparametrization_w, normalize, exact,
                             input_needs_grad, x_min_needs_grad, x_max_needs_grad,
                             y_min_needs_grad, y_max_needs_grad):
    """Reference src/box_convolution_interface.cpp:141-395.

    Returns ``[grad_input, grad_x_min, grad_x_max, grad_y_min, grad_y_max]`` with ``None`` for a
    gradient that was not requested. ``output`` (the saved forward result) may be ``None``."""
    _require_device(grad_output, "grad_output")
    if grad_output.dim() != 4:
        raise RuntimeError("grad_output for box_convolution must have 4 dimensions")
    if input_integrated.dim() != 4:
        raise RuntimeError("BoxConv2d: input must have 4 dimensions")
    B, C, h1, w1 = input_integrated.shape
    h, w = h1 - 1, w1 - 1
    _check_params(x_min, x_max, y_min, y_max, C, "all box conv parameters: ")
    F = x_min.size(1)
    if tuple(grad_output.shape) != (B, C * F, h, w):
        raise RuntimeError("box_convolution: sizes of grad_output and input_integrated don't match")
    half = grad_output.dtype in _FUSED_OUTPUT and grad_output.dtype != torch.float32
    if half:
        # float16 / bfloat16 grad_output with the float32 integral image the forward saved: read
        # directly by the kernels (grad_input comes back in the same half type, the parameter
        # gradients in float32); rows too wide for that go through float32 copies
        if input_integrated.dtype != torch.float32:
            raise RuntimeError("box_convolution: half-precision grad_output needs a float32 "
                               "input_integrated, got %s" % input_integrated.dtype)
        if w > _MAX_STREAM_WIDTH or (h + 1) * (w + 1) * 4 >= 2 ** 31:
            grads = box_convolution_backward(
                input_integrated, x_min, x_max, y_min, y_max, grad_output.float(), output,
                reparametrization_h, reparametrization_w, normalize, exact, input_needs_grad,
                x_min_needs_grad, x_max_needs_grad, y_min_needs_grad, y_max_needs_grad)
            if grads[0] is not None:
                grads[0] = grads[0].to(grad_output.dtype)
            return grads
        sfx = "half_f32"
    else:
        sfx = _suffix(grad_output, "grad_output")
        if input_integrated.dtype != grad_output.dtype:
            raise RuntimeError("box_convolution: grad_output and input_integrated differ in device or dtype")
    if input_integrated.device != grad_output.device:
        raise RuntimeError("box_convolution: grad_output and input_integrated differ in device or dtype")
    lib = load()
    grad_output = grad_output.contiguous()
    input_integrated = input_integrated.contiguous()
    x_min, x_max, y_min, y_max = _same_kind((x_min, x_max, y_min, y_max), input_integrated, "input_integrated")
    dev, dt = grad_output.device, input_integrated.dtype
    needs_p = (x_min_needs_grad, x_max_needs_grad, y_min_needs_grad, y_max_needs_grad)

    grad_input = None
    if input_needs_grad:
        grad_input = (torch.empty if F > 0 else torch.zeros)((B, C, h, w), dtype=grad_output.dtype, device=dev)
    if all(needs_p):
        grads = list(torch.empty((4, C, F), dtype=dt, device=dev).unbind(0))    # one allocation
    else:
        grads = [torch.empty((C, F), dtype=dt, device=dev) if n else None for n in needs_p]
    want_input = input_needs_grad and grad_input.numel() > 0 and F > 0
    want_params = any(needs_p) and C * F > 0
    if want_input or want_params:
        with _on_device(dev):
            nbytes = _backward_workspace_bytes(lib, B, C, F, h, w, input_integrated.element_size(),
                                               want_input, want_params)
            stream = _stream(dev)
            ws = _workspace(nbytes, dev, stream)
            if half:
                rc = lib.boxconv_backward_half_f32(
                    _ptr(input_integrated), _ptr(x_min), _ptr(x_max), _ptr(y_min), _ptr(y_max),
                    _ptr(grad_output), _FUSED_OUTPUT[grad_output.dtype],
                    float(reparametrization_h), float(reparametrization_w), int(bool(normalize)),
                    int(bool(exact)), _ptr(grad_input) if want_input else None,
                    *[_ptr(g) if want_params else None for g in grads],
                    B, C, F, h, w, _ptr(ws), nbytes, stream)
            else:
                rc = getattr(lib, "boxconv_backward_" + sfx)(
                    _ptr(input_integrated), _ptr(x_min), _ptr(x_max), _ptr(y_min), _ptr(y_max),
                    _ptr(grad_output), _ptr(output) if output is not None and output.numel() else None,
                    float(reparametrization_h), float(reparametrization_w), int(bool(normalize)),
                    int(bool(exact)), _ptr(grad_input) if want_input else None,
                    *[_ptr(g) if want_params else None for g in grads],
                    B, C, F, h, w, _ptr(ws), nbytes, stream)
        _check(rc, "box_convolution_backward")
    return [grad_input] + grads


def clip_parameters(x_min, x_max, y_min, y_max, reparametrization_h, reparametrization_w,
                    max_input_h, max_input_w, exact):
    """In place on the stored parameters (reference src/box_convolution_interface.cpp:397-415).

    Parameters that live in host memory are clipped by the same HIP kernel through a device copy,
    so that ``BoxConv2d(...).eval()`` works before the module is moved to the GPU."""
    if not x_min.is_contiguous():
        raise RuntimeError("x_min must be contiguous")
    params = (x_min, x_max, y_min, y_max)
    for p in params[1:]:
        if (p.shape != x_min.shape or p.dtype != x_min.dtype or p.device != x_min.device
                or not p.is_contiguous()):
            raise RuntimeError("box_convolution: clip_parameters needs four contiguous tensors of "
                               "one shape, dtype and device")
    if x_min.dtype in (torch.float16, torch.bfloat16):
        # half-precision parameters (module.half()): clipped in float32, as the kernel's
        # arithmetic is double anyway, and rounded back once
        with torch.no_grad():
            staged = [p.detach().float() for p in params]
            clip_parameters(*staged, reparametrization_h, reparametrization_w, max_input_h,
                            max_input_w, exact)
            for p, s in zip(params, staged):
                p.detach().copy_(s)
        return
    sfx = _suffix(x_min, "parameters")
    n = x_min.numel()
    if n == 0:
        return
    lib = load()
    if not x_min.is_cuda:
        if not torch.cuda.is_available():
            raise RuntimeError("box_convolution: parameters are on '%s' and no AMD GPU is "
                               "available; there is no CPU path" % x_min.device)
        with torch.no_grad():
            staged = [p.detach().to("cuda") for p in params]
            clip_parameters(*staged, reparametrization_h, reparametrization_w, max_input_h,
                            max_input_w, exact)
            for p, s in zip(params, staged):
                p.detach().copy_(s)
        return
    with _on_device(x_min.device):
        rc = getattr(lib, "boxconv_clip_parameters_" + sfx)(
            _ptr(x_min), _ptr(x_max), _ptr(y_min), _ptr(y_max), n,
            float(reparametrization_h), float(reparametrization_w), float(max_input_h),
            float(max_input_w), int(bool(exact)), _stream(x_min.device))
    _check(rc, "clip_parameters")


def clip_reparametrize(x_min, x_max, y_min, y_max, reparametrization_h, reparametrization_w,
                       max_input_h, max_input_w, exact):
    """``clip_parameters`` followed by ``reparametrize(..., inverse=True)`` in one launch: clips the
    stored parameters in place and returns the four clipped tensors in real pixel units (new
    tensors, views of one allocation). Device tensors only."""
    params = (x_min, x_max, y_min, y_max)
    for p in params:
        if (not p.is_cuda or p.shape != x_min.shape or p.dtype != x_min.dtype
                or p.device != x_min.device or not p.is_contiguous()):
            raise RuntimeError("box_convolution: clip_reparametrize needs four contiguous device "
                               "tensors of one shape, dtype and device")
    sfx = _suffix(x_min, "parameters")
    n = x_min.numel()
    real = torch.empty((4,) + tuple(x_min.shape), dtype=x_min.dtype, device=x_min.device)
    if n > 0:
        lib = load()
        with _on_device(x_min.device):
            rc = getattr(lib, "boxconv_clip_reparametrize_" + sfx)(
                _ptr(x_min), _ptr(x_max), _ptr(y_min), _ptr(y_max), _ptr(real), n,
                float(reparametrization_h), float(reparametrization_w), float(max_input_h),
                float(max_input_w), int(bool(exact)), _stream(x_min.device))
        _check(rc, "clip_reparametrize")
    return real[0], real[1], real[2], real[3]


def training_forward(input, x_min, x_max, y_min, y_max, reparametrization_h, reparametrization_w,
                     max_input_h, max_input_w, normalize, exact):
    """``BoxConv2d.forward`` in training mode as one native call (reference
    box_convolution_module.py:203-214, box_convolution_function.py:41-46): clips the stored
    parameters in place, converts them to real pixel units, integrates the input and samples the
    boxes. Returns ``(input_integrated, output, (x_min, x_max, y_min, y_max) in real units)``."""
    _require_device(input, "input")
    if input.dim() != 4:
        raise RuntimeError("BoxConv2d: input must have 4 dimensions")
    params = (x_min, x_max, y_min, y_max)
    for p in params:
        if p.device != input.device:
            raise RuntimeError("BoxConv2d: input and parameters are on different devices")
        if p.dtype != input.dtype:
            raise RuntimeError("box_convolution: input and parameters have different dtypes (%s, %s)"
                               % (input.dtype, p.dtype))
        if not p.is_contiguous():
            raise RuntimeError("box_convolution: parameters must be contiguous to be clipped in place")
    sfx = _suffix(input, "input")
    _check_params(x_min, x_max, y_min, y_max, input.size(1), "BoxConv2d: ")
    lib = load()
    input = input.contiguous()
    B, C, h, w = input.shape
    F = x_min.size(1)
    if h < 1 or w < 1:
        raise RuntimeError("BoxConv2d: input must be at least 1x1")
    dev = input.device
    integrated = torch.empty((B, C, h + 1, w + 1), dtype=input.dtype, device=dev)
    output = torch.empty((B, C * F, h, w), dtype=input.dtype, device=dev)
    real = torch.empty((4, C, F), dtype=input.dtype, device=dev)
    with _on_device(dev):
        nbytes = _integral_workspace_bytes(lib, B * C, h, w)
        stream = _stream(dev)
        ws = _workspace(nbytes, dev, stream)
        rc = getattr(lib, "boxconv_training_forward_" + sfx)(
            _ptr(input), _ptr(x_min), _ptr(x_max), _ptr(y_min), _ptr(y_max), _ptr(real),
            _ptr(integrated), _ptr(output), B, C, F, h, w,
            float(reparametrization_h), float(reparametrization_w), float(max_input_h),
            float(max_input_w), int(bool(normalize)), int(bool(exact)), _ptr(ws), nbytes,
            stream)
    _check(rc, "training_forward")
    return integrated, output, real.unbind(0)


KERNEL_NAMES = ("band_colsum", "band_prefix", "band_scan", "forward_rows", "grad_output_stream",
                "grad_input_cols", "param_grad_finalize", "fill_zero", "fill_marker", "clip",
                "forward_gather", "grad_input_gather", "grad_params_gather", "int_row_prefix",
                "int_col_prefix")


def reload_switches():
    """Make the library read its BOXCONV_* environment switches again (it reads them once, at
    first use). For tests that change a switch inside a running process."""
    load().boxconv_reload_env()
    _workspace_bytes.clear()        # the switches decide which kernels run, hence how much scratch


def profile_arm(kernel_name, every=1):
    """Bracket later launches of `kernel_name` with HIP events, one launch in `every` (None
    disarms)."""
    _check(load().boxconv_profile_arm_every(kernel_name.encode() if kernel_name else None, every),
           "profile_arm")


def probe_copy_bands(src, dst, rows_per_group, rows_in_flight):
    """Plain copy of `src` [planes, h, w] into rows 1..h of `dst` [planes, h+1, w] with the access
    pattern of the backward's streaming pass (a measurement yardstick, see include/boxconv.h)."""
    planes, h, w = src.shape
    if (src.dtype != torch.float32 or dst.dtype != torch.float32 or not src.is_cuda or not dst.is_cuda
            or tuple(dst.shape) != (planes, h + 1, w) or not src.is_contiguous() or not dst.is_contiguous()):
        raise RuntimeError("probe_copy_bands: contiguous float32 device tensors [planes,h,w] -> [planes,h+1,w]")
    _check(load().boxconv_probe_copy_bands(_ptr(src), _ptr(dst), planes, h, w, rows_per_group,
                                           rows_in_flight, _stream(src.device)), "probe_copy_bands")


def probe_grad_input_pattern(column_workspace, out, x_lo, x_hi, mode):
    """The grad-input pass's loads and stores without its arithmetic (a measurement yardstick, see
    include/boxconv.h): column_workspace [planes, F, h+1, 1024] float32, out [planes, h, 1024],
    x_lo / x_hi [C, F] int32 row offsets of the two runs."""
    planes, F, h1, w = column_workspace.shape
    C = x_lo.shape[0]
    ok = (w == 1024 and tuple(out.shape) == (planes, h1 - 1, w) and tuple(x_lo.shape) == (C, F)
          and tuple(x_hi.shape) == (C, F) and x_lo.dtype == torch.int32 and x_hi.dtype == torch.int32
          and column_workspace.dtype == torch.float32 and out.dtype == torch.float32
          and all(t.is_cuda and t.is_contiguous() for t in (column_workspace, out, x_lo, x_hi)))
    if not ok:
        raise RuntimeError("probe_grad_input_pattern: float32 [planes,F,h+1,1024] -> [planes,h,1024], int32 [C,F] offsets")
    _check(load().boxconv_probe_grad_input_pattern(_ptr(column_workspace), _ptr(out), _ptr(x_lo), _ptr(x_hi), planes,
                                                   C, F, h1 - 1, mode, _stream(out.device)), "probe_grad_input_pattern")


def profile_collect():
    """(summed kernel milliseconds, launches) since profile_arm; waits for the kernels."""
    total, count = ctypes.c_double(0.0), ctypes.c_int(0)
    _check(load().boxconv_profile_collect(ctypes.byref(total), ctypes.byref(count)),
           "profile_collect")
    return total.value, count.value
