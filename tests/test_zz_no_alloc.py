"""boxconv_integral_image_static_f32: the integral image for callers that cannot pass or allocate
a workspace (its band column sums go to a fixed array in device memory). Checked bit for bit
against boxconv_integral_image_f32, which runs the same kernels on a caller-provided workspace,
on two calls in a row, the second with a smaller input (the array keeps the first call's contents).
Both are called through the C ABI with ctypes."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

STATIC_SCRATCH_BYTES = 8 << 20     # BOXCONV_STATIC_SCRATCH_BYTES in include/boxconv.h


def _stream(dev):
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def _with_workspace(lib, x):
    planes, h, w = x.shape
    out = torch.empty((planes, h + 1, w + 1), dtype=torch.float32, device=x.device)
    n = lib.boxconv_integral_image_workspace_bytes(planes, h, w)
    ws = torch.empty(max(n, 8), dtype=torch.uint8, device=x.device)
    rc = lib.boxconv_integral_image_f32(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(out.data_ptr()),
                                        planes, h, w, ctypes.c_void_p(ws.data_ptr()), n, _stream(x.device))
    assert rc == 0, lib.boxconv_last_error()
    return out, n


def _static(lib, x, out):
    planes, h, w = x.shape
    return lib.boxconv_integral_image_static_f32(ctypes.c_void_p(x.data_ptr()),
                                                 ctypes.c_void_p(out.data_ptr()), planes, h, w,
                                                 _stream(x.device))


def test_static_scratch_integral_image_matches_workspace_version(hip):
    lib = hip.load()
    dev = torch.device("cuda:0")
    gen = torch.Generator().manual_seed(4242)
    # (planes, h, w): the headline shape (single-pass kernel: hand-over words in the scratch array),
    # then smaller inputs that reuse the same words: two-pass shapes (column sums), a ragged
    # width, and one that needs no scratch at all
    shapes = [(32, 512, 1024), (6, 200, 300), (3, 96, 1024), (5, 130, 77), (4, 20, 33)]
    used = []
    for planes, h, w in shapes:
        x = torch.randn((planes, h, w), generator=gen).to(dev)
        expect, need = _with_workspace(lib, x)
        assert need <= STATIC_SCRATCH_BYTES
        used.append(need)
        got = torch.full_like(expect, float("nan"))
        rc = _static(lib, x, got)
        assert rc == 0, lib.boxconv_last_error()
        torch.cuda.synchronize()
        assert torch.equal(got, expect), "static-scratch integral image differs at %s" % ((planes, h, w),)
        # and against the definition, in float64
        ref = torch.zeros((planes, h + 1, w + 1), dtype=torch.float64, device=dev)
        ref[:, 1:, 1:] = x.double().cumsum(1).cumsum(2)
        assert torch.allclose(got.double(), ref, rtol=1e-6, atol=1e-4)
    assert used[0] > used[1] > 0, "the first two calls must both use the array, the second less of it"
    assert used[-1] == 0


def test_static_scratch_repeated_calls_and_limit(hip):
    lib = hip.load()
    dev = torch.device("cuda:0")
    x = torch.randn((8, 256, 512), generator=torch.Generator().manual_seed(7)).to(dev)
    expect, need = _with_workspace(lib, x)
    assert 0 < need <= STATIC_SCRATCH_BYTES
    for _ in range(3):                       # same stream: ordered, each call re-initialises what it reads
        got = torch.empty_like(expect)
        assert _static(lib, x, got) == 0, lib.boxconv_last_error()
    torch.cuda.synchronize()
    assert torch.equal(got, expect)
    # a shape whose column sums do not fit is refused before anything is launched
    planes, h, w = 128, 1024, 2048
    assert lib.boxconv_integral_image_workspace_bytes(planes, h, w) > STATIC_SCRATCH_BYTES
    dummy = ctypes.c_void_p(256)
    rc = lib.boxconv_integral_image_static_f32(dummy, dummy, planes, h, w, None)
    assert rc == -3 and b"scratch" in lib.boxconv_last_error()
    # argument errors as for the workspace version
    assert lib.boxconv_integral_image_static_f32(None, None, 1, 0, 5, None) == -1
    assert lib.boxconv_integral_image_static_f32(None, None, 0, 4, 5, None) == 0
