"""ctypes front end of the CPU checkers. TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Two libraries export the same entry points under different prefixes:

* ``oracle/libboxconv_oracle.so`` (prefix ``oracle_``): the plain C++ restatement of the
  reference's CPU path (``oracle/boxconv_oracle.cpp``), built anywhere ``g++`` exists.
* ``oracle/_ref/libboxconv_ref.so`` (prefix ``ref_``): the reference's own CPU kernels compiled
  from ``/root/reference/src`` (``oracle/ref_driver.cpp``); exists only where it was built.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg import this
module. All arrays are numpy, C-contiguous, float32 or float64, on the host.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_LIB = os.path.join(_HERE, "libboxconv_oracle.so")
REF_LIB = os.path.join(_HERE, "_ref", "libboxconv_ref.so")

_SUFFIX = {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64"}
# the integral image alone also takes the integer types (src/integral_image.cpp:14)
_INT_SUFFIX = {np.dtype(np.uint8): "u8", np.dtype(np.int8): "i8", np.dtype(np.int16): "i16",
               np.dtype(np.int32): "i32", np.dtype(np.int64): "i64"}


def build(with_reference=True):
    """Compile the checkers (make). The reference build is attempted only if its sources exist."""
    subprocess.check_call(["make", "-C", _HERE, "-s"])
    if with_reference and os.path.isfile("/root/reference/src/box_convolution.cpp"):
        subprocess.check_call(["make", "-C", _HERE, "-s", "ref"])


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype=None):
    a = np.ascontiguousarray(a, dtype=dtype)
    if a.dtype not in _SUFFIX:
        raise TypeError("checker supports float32 and float64 only, got %s" % a.dtype)
    return a


class CpuChecker:
    """One loaded checker library. ``kind`` is 'port' (restatement) or 'reference'."""

    def __init__(self, path, prefix, kind):
        if prefix == "ref_":
            import torch  # noqa: F401  (libtorch_cpu must be resident before the library loads)
        self.lib = ctypes.CDLL(path)
        self.prefix = prefix
        self.kind = kind
        self.path = path

    def _fn(self, name, dtype):
        return getattr(self.lib, "%s%s_%s" % (self.prefix, name, _SUFFIX[np.dtype(dtype)]))

    # -- the four functions of the reference's native module (src/bind.cpp:29-34) --------------
    def integral_image(self, x):
        x = np.ascontiguousarray(x)
        if x.dtype in _INT_SUFFIX:
            h, w = x.shape[-2:]
            planes = x.size // (h * w) if x.size else 0
            out = np.empty(x.shape[:-2] + (h + 1, w + 1), dtype=x.dtype)
            getattr(self.lib, "%sintegral_image_%s" % (self.prefix, _INT_SUFFIX[x.dtype]))(
                _ptr(x), _ptr(out), ctypes.c_int64(planes), h, w)
            return out
        x = _c(x)
        h, w = x.shape[-2:]
        planes = x.size // (h * w) if x.size else 0
        out = np.empty(x.shape[:-2] + (h + 1, w + 1), dtype=x.dtype)
        self._fn("integral_image", x.dtype)(_ptr(x), _ptr(out), ctypes.c_int64(planes), h, w)
        return out

    def box_forward(self, integ, xmin, xmax, ymin, ymax, normalize, exact):
        integ = _c(integ)
        dt = integ.dtype
        B, C, h1, w1 = integ.shape
        h, w = h1 - 1, w1 - 1
        xmin, xmax, ymin, ymax = (_c(p, dt) for p in (xmin, xmax, ymin, ymax))
        F = xmin.shape[1]
        assert xmin.shape == (C, F)
        out = np.empty((B, C * F, h, w), dtype=dt)
        self._fn("box_forward", dt)(_ptr(integ), _ptr(xmin), _ptr(xmax), _ptr(ymin), _ptr(ymax),
                                    _ptr(out), B, C, F, h, w, int(normalize), int(exact))
        return out

    def box_backward(self, integ, xmin, xmax, ymin, ymax, grad_out, output, reparam_h, reparam_w,
                     normalize, exact, needs=(True,) * 5):
        integ = _c(integ)
        dt = integ.dtype
        B, C, h1, w1 = integ.shape
        h, w = h1 - 1, w1 - 1
        xmin, xmax, ymin, ymax = (_c(p, dt) for p in (xmin, xmax, ymin, ymax))
        F = xmin.shape[1]
        grad_out = _c(grad_out, dt)
        assert grad_out.shape == (B, C * F, h, w)
        if normalize:
            output = _c(output, dt)
            assert output.shape == grad_out.shape
        else:
            output = None
        needs_arr = (ctypes.c_int * 5)(*[int(bool(n)) for n in needs])
        gin = np.zeros((B, C, h, w), dtype=dt) if needs[0] else None
        gp = [np.zeros((C, F), dtype=dt) if needs[1 + k] else None for k in range(4)]
        self._fn("box_backward", dt)(
            _ptr(integ), _ptr(xmin), _ptr(xmax), _ptr(ymin), _ptr(ymax), _ptr(grad_out),
            _ptr(output), ctypes.c_float(reparam_h), ctypes.c_float(reparam_w), int(normalize),
            int(exact), needs_arr, _ptr(gin), _ptr(gp[0]), _ptr(gp[1]), _ptr(gp[2]), _ptr(gp[3]),
            B, C, F, h, w)
        return (gin,) + tuple(gp)

    def clip_parameters(self, xmin, xmax, ymin, ymax, reparam_h, reparam_w, max_h, max_w, exact):
        """In place, like the reference (src/box_convolution_interface.cpp:397-415)."""
        for p in (xmin, xmax, ymin, ymax):
            assert p.flags.c_contiguous and p.dtype == xmin.dtype
        self._fn("clip_parameters", xmin.dtype)(
            _ptr(xmin), _ptr(xmax), _ptr(ymin), _ptr(ymax), int(xmin.size),
            ctypes.c_double(reparam_h), ctypes.c_double(reparam_w), ctypes.c_double(max_h),
            ctypes.c_double(max_w), int(exact))

    # -- finer-grained pieces, used to pin the restatement against the compiled reference ------
    def grad_input_planes(self, gint, xmin, xmax, ymin, ymax, normalize, exact):
        gint = _c(gint)
        dt = gint.dtype
        B, C, F, h1, w1 = gint.shape
        xmin, xmax, ymin, ymax = (_c(p, dt) for p in (xmin, xmax, ymin, ymax))
        tmp = np.empty((B, C, F, h1 - 1, w1 - 1), dtype=dt)
        self._fn("box_grad_input_planes", dt)(
            _ptr(gint), _ptr(xmin), _ptr(xmax), _ptr(ymin), _ptr(ymax), _ptr(tmp), B, C, F,
            h1 - 1, w1 - 1, int(normalize), int(exact))
        return tmp

    def grad_param_planes(self, integ, xmin, xmax, ymin, ymax, which, exact):
        integ = _c(integ)
        dt = integ.dtype
        B, C, h1, w1 = integ.shape
        xmin, xmax, ymin, ymax = (_c(p, dt) for p in (xmin, xmax, ymin, ymax))
        F = xmin.shape[1]
        tmp = np.empty((B, C, F, h1 - 1, w1 - 1), dtype=dt)
        self._fn("box_grad_param_planes", dt)(
            _ptr(integ), _ptr(xmin), _ptr(xmax), _ptr(ymin), _ptr(ymax), _ptr(tmp), int(which),
            B, C, F, h1 - 1, w1 - 1, int(exact))
        return tmp

    def split(self, variant, xmin, xmax, ymin, ymax, dtype=np.float32):
        p4 = np.array([xmin, xmax, ymin, ymax], dtype=dtype)
        ints = np.zeros(4, dtype=np.int32)
        fracs = np.zeros(4, dtype=dtype)
        self._fn("split", dtype)(int(variant), _ptr(p4), _ptr(ints), _ptr(fracs))
        return ints, fracs

    # -- the module-level path: what BoxConv2d.forward + backward computes ----------------------
    def module_forward(self, x, x_min, x_max, y_min, y_max, reparam_h, reparam_w, normalize,
                       exact):
        """box_convolution_function.py:32-51. Parameters are in stored (reparametrized) units.

        Returns (output, saved) where saved = (integral, real-unit parameters, output)."""
        x = _c(x)
        dt = x.dtype
        # reparametrize(inverse=True): tensor * python scalar, rounded in the tensor's dtype
        real = tuple(_c(p, dt) * dt.type(s) for p, s in
                     ((x_min, reparam_h), (x_max, reparam_h), (y_min, reparam_w),
                      (y_max, reparam_w)))
        integ = self.integral_image(x)
        out = self.box_forward(integ, *real, normalize, exact)
        return out, (integ, real, out)

    def module_backward(self, saved, grad_out, reparam_h, reparam_w, normalize, exact,
                        needs=(True,) * 5):
        integ, real, out = saved
        return self.box_backward(integ, *real, grad_out, out, reparam_h, reparam_w, normalize,
                                 exact, needs)


_cache = {}


def oracle():
    """The restatement; built on demand."""
    if "oracle" not in _cache:
        if not os.path.isfile(ORACLE_LIB):
            build(with_reference=False)
        _cache["oracle"] = CpuChecker(ORACLE_LIB, "oracle_", "port")
    return _cache["oracle"]


def reference():
    """The compiled reference kernels, or None where oracle/_ref was never built."""
    if "ref" not in _cache:
        _cache["ref"] = (CpuChecker(REF_LIB, "ref_", "reference")
                         if os.path.isfile(REF_LIB) else None)
    return _cache["ref"]
