"""The C-ABI library loads and exports every symbol include/boxconv.h declares; argument errors
are reported before anything is launched (so these calls need no GPU)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "boxconv.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(boxconv_\w+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from box_convolution import _native
    return _native.load()


def test_header_declares_the_four_reference_functions():
    names = declared_functions()
    for stem in ("integral_image", "forward", "backward", "clip_parameters"):
        for sfx in ("f32", "f64"):
            assert "boxconv_%s_%s" % (stem, sfx) in names


def test_library_exports_every_declared_symbol(lib):
    from box_convolution import _native
    names = declared_functions()
    assert names, "no declarations found in include/boxconv.h"
    for n in names:
        assert hasattr(lib, n), "libboxconv_hip.so does not export " + n
    # and the Python binding table covers exactly the header
    assert sorted(_native.EXPORTED_SYMBOLS) == names
    assert lib.boxconv_abi_version() == _native.ABI_VERSION


def test_argument_errors_are_reported_without_launching(lib):
    null = ctypes.c_void_p(None)
    rc = lib.boxconv_integral_image_f32(null, null, 1, 0, 5, null, 0, null)
    assert rc == -1 and b"invalid sizes" in lib.boxconv_last_error()
    rc = lib.boxconv_integral_image_f32(null, null, 2, 4, 5, null, 0, null)
    assert rc == -1 and b"null" in lib.boxconv_last_error()
    rc = lib.boxconv_forward_f32(null, null, null, null, null, null, 1, 1, 1, 4, 4, 1, 1, null)
    assert rc == -1
    rc = lib.boxconv_forward_f64(null, null, null, null, null, null, 1, 1, 1, 0, 4, 1, 1, null)
    assert rc == -1
    rc = lib.boxconv_forward_fused_f32(null, null, null, null, null, null, 7, null, null, null, 0,
                                       1, 1, 1, 4, 4, 1, 1, null)
    assert rc == -1 and b"output_dtype" in lib.boxconv_last_error()
    rc = lib.boxconv_forward_fused_f32(null, null, null, null, null, null, 1, null, null, null, 0,
                                       1, 1, 1, 4, 4, 1, 1, null)
    assert rc == -1 and b"null" in lib.boxconv_last_error()
    rc = lib.boxconv_integral_image_half_f32(null, 0, null, 1, 4, 4, null, 0, null)
    assert rc == -1 and b"input_dtype" in lib.boxconv_last_error()
    rc = lib.boxconv_integral_image_int(null, null, 3, 1, 4, 4, null)
    assert rc == -1 and b"BOXCONV_U8" in lib.boxconv_last_error()
    rc = lib.boxconv_integral_image_int(null, null, 19, 1, 4, 4, null)
    assert rc == -1 and b"null" in lib.boxconv_last_error()
    dummy16 = ctypes.c_void_p(256)
    rc = lib.boxconv_probe_copy_bands(dummy16, dummy16, 4, 64, 1000, 64, 2, null)     # w not a multiple of 256
    assert rc == -1 and b"copy probe" in lib.boxconv_last_error()
    rc = lib.boxconv_probe_copy_bands(dummy16, dummy16, 4, 64, 1024, 48, 2, null)     # bands do not tile h
    assert rc == -1 and b"copy probe" in lib.boxconv_last_error()
    rc = lib.boxconv_probe_copy_bands(null, null, 4, 64, 1024, 64, 2, null)
    assert rc == -1 and b"null" in lib.boxconv_last_error()
    rc = lib.boxconv_probe_grad_input_pattern(dummy16, dummy16, dummy16, dummy16, 8, 2, 3, 100, 0, null)   # h % 8
    assert rc == -1 and b"pattern probe" in lib.boxconv_last_error()
    rc = lib.boxconv_probe_grad_input_pattern(dummy16, dummy16, null, dummy16, 8, 2, 3, 104, 0, null)
    assert rc == -1 and b"null" in lib.boxconv_last_error()
    rc = lib.boxconv_integral_image_half_f32(dummy16, 1, dummy16, 1, 4, 4096, null, 0, null)
    assert rc == -3 and b"2048" in lib.boxconv_last_error()
    assert lib.boxconv_profile_arm_every(b"forward_rows", 0) == -1
    assert lib.boxconv_profile_arm_every(None, 3) == 0
    f64 = ctypes.c_double
    rc = lib.boxconv_training_forward_f32(null, null, null, null, null, null, null, null, 1, 1, 1, 4, 4,
                                          f64(8.0), f64(8.0), f64(4.0), f64(4.0), 1, 1, null, 0, null)
    assert rc == -1 and b"null parameter pointer" in lib.boxconv_last_error()
    rc = lib.boxconv_inference_forward_f32(null, null, null, null, null, null, null, null, 1, 1, 1, 4, 4,
                                           f64(8.0), f64(8.0), 1, 1, null, 0, null)
    assert rc == -1 and b"null parameter pointer" in lib.boxconv_last_error()
    rc = lib.boxconv_inference_forward_f64(dummy16, dummy16, dummy16, dummy16, dummy16, dummy16, dummy16,
                                           dummy16, 1, 1, 1, 4, 4, f64(8.0), f64(-1.0), 1, 1, null, 0, null)
    assert rc == -1 and b"positive" in lib.boxconv_last_error()
    rc = lib.boxconv_training_forward_f32(dummy16, dummy16, dummy16, dummy16, dummy16, dummy16, dummy16,
                                          dummy16, 1, 1, 1, 4, 4, f64(0.0), f64(8.0), f64(4.0), f64(4.0),
                                          1, 1, null, 0, null)
    assert rc == -1 and b"positive" in lib.boxconv_last_error()
    half_args = (dummy16,) * 7
    rc = lib.boxconv_training_forward_half_f32(dummy16, 0, *half_args, 1, 1, 1, 4, 4, f64(8.0), f64(8.0), f64(4.0),
                                               f64(4.0), 1, 1, 1, null, 0, null)
    assert rc == -1 and b"io_dtype" in lib.boxconv_last_error()
    rc = lib.boxconv_training_forward_half_f32(null, 1, *((null,) * 7), 1, 1, 1, 4, 4, f64(8.0), f64(8.0), f64(4.0),
                                               f64(4.0), 1, 1, 1, null, 0, null)
    assert rc == -1 and b"null parameter pointer" in lib.boxconv_last_error()
    rc = lib.boxconv_training_forward_half_f32(dummy16, 2, *half_args, 1, 1, 1, 4, 4096, f64(8.0), f64(8.0), f64(4.0),
                                               f64(4.0), 0, 1, 1, null, 0, null)
    assert rc == -3 and b"2048" in lib.boxconv_last_error()
    rc = lib.boxconv_training_forward_half_f32(dummy16, 1, *half_args, 2, 16, 8, 512, 1024, f64(8.0), f64(8.0),
                                               f64(512.0), f64(1024.0), 1, 1, 1, null, 0, null)
    assert rc == -2 and b"workspace" in lib.boxconv_last_error()
    # several bands and no workspace: refused before anything is launched
    rc = lib.boxconv_training_forward_f32(dummy16, dummy16, dummy16, dummy16, dummy16, dummy16, dummy16,
                                          dummy16, 2, 16, 8, 512, 1024, f64(8.0), f64(8.0), f64(512.0),
                                          f64(1024.0), 1, 1, null, 0, null)
    assert rc == -2 and b"workspace" in lib.boxconv_last_error()
    # more than 2^31-1 elements
    rc = lib.boxconv_forward_f32(null, null, null, null, null, null, 64, 64, 64, 4096, 4096, 1, 1, null)
    assert rc == -3
    # backward with nothing requested is a no-op; with a request but no workspace it is refused
    f = ctypes.c_float(1.0)
    rc = lib.boxconv_backward_f32(null, null, null, null, null, null, null, f, f, 1, 1,
                                  null, null, null, null, null, 1, 1, 1, 4, 4, null, 0, null)
    assert rc == 0
    dummy = ctypes.c_void_p(256)
    rc = lib.boxconv_backward_f32(dummy, dummy, dummy, dummy, dummy, dummy, null, f, f, 1, 1,
                                  dummy, null, null, null, null, 1, 1, 1, 4, 4, null, 0, null)
    assert rc == -2 and b"workspace" in lib.boxconv_last_error()
    rc = lib.boxconv_clip_parameters_f32(null, null, null, null, 3, 1.0, 1.0, 4.0, 4.0, 1, null)
    assert rc == -1
    rc = lib.boxconv_clip_parameters_f32(null, null, null, null, 0, 1.0, 1.0, 4.0, 4.0, 1, null)
    assert rc == 0


def test_workspace_sizes(lib):
    # one band (short planes, many of them): no scratch for the integral image
    assert lib.boxconv_integral_image_workspace_bytes(4096, 28, 28) == 0
    # several bands: (bands-1) column-sum vectors of w doubles per plane
    n = lib.boxconv_integral_image_workspace_bytes(32, 512, 1024)
    assert n > 0 and n % (32 * 1024 * 8) == 0
    full = lib.boxconv_backward_workspace_bytes(2, 16, 8, 512, 1024, 4, 1, 1)
    only_params = lib.boxconv_backward_workspace_bytes(2, 16, 8, 512, 1024, 4, 0, 1)
    only_input = lib.boxconv_backward_workspace_bytes(2, 16, 8, 512, 1024, 4, 1, 0)
    gint = 2 * 16 * 8 * 513 * 1024 * 4     # column workspace: h+1 rows of w (rounded up to 4) per (plane, filter)
    # per-box sums: five doubles per (batch item, box, row band), 256-byte granules
    assert only_params % 256 == 0 and only_params >= 2 * 16 * 8 * 5 * 8
    assert only_params % (2 * 16 * 8 * 5 * 8) == 0
    assert only_input >= gint and full == only_input + only_params
    assert lib.boxconv_backward_workspace_bytes(2, 16, 8, 512, 1024, 2, 1, 1) == 0   # bad elem size
    # the shape chooser at the width limits: float32 rows stream up to 4096 columns (column workspace
    # of h+1 rows of w rounded up to 4), float64 rows up to 2048; wider rows take the gather
    # kernels (a true integral image of (h+1)(w+1) elements)
    f32_4096 = lib.boxconv_backward_workspace_bytes(1, 1, 1, 64, 4096, 4, 1, 0)
    f32_4097 = lib.boxconv_backward_workspace_bytes(1, 1, 1, 64, 4097, 4, 1, 0)
    f64_2048 = lib.boxconv_backward_workspace_bytes(1, 1, 1, 64, 2048, 8, 1, 0)
    f64_2049 = lib.boxconv_backward_workspace_bytes(1, 1, 1, 64, 2049, 8, 1, 0)
    assert 65 * 4096 * 4 <= f32_4096 < 65 * 4097 * 4
    assert f32_4097 >= 65 * 4098 * 4
    assert 65 * 2048 * 8 <= f64_2048 < 65 * 2049 * 8
    assert f64_2049 >= 65 * 2050 * 8
