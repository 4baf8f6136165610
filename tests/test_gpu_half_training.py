"""Training in float16 / bfloat16: the backward kernels read a half-precision grad_output and write
a half-precision grad_input directly (float32 integral image, float32 and double sums, float32
parameter gradients). The reference dispatches its CUDA kernels on half tensors
(src/box_convolution_cuda_backward.cu:176,431); its CPU path, the parity target, has no half
type, so the expected values are the CPU oracle's float32 results on the same (half-rounded)
tensors, rounded to the half type on the host. Bounds: the float32 bounds of the other parity
tests (grad_input 1e-4, parameter gradients 1e-3 of the largest entry) plus one unit in the last
place of the half type for the tensor that is stored in it.
"""
import random

import numpy as np
import pytest
import torch

from box_convolution import BoxConv2d
from helpers import make_boxes, param_grad_floor

pytestmark = pytest.mark.gpu
DEV = "cuda"
HALF_ULP = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}

# B, C, F, h, w: narrow (filters shared between thread sets), several bands, full rows, three
# columns per lane, 512 threads, 1024 threads (two launches), wider than the direct path (float32
# copies)
SHAPES = [(2, 2, 5, 20, 33), (1, 2, 2, 150, 90), (1, 1, 2, 40, 1024), (1, 2, 1, 18, 1536),
          (1, 1, 2, 12, 2048), (1, 1, 1, 9, 2100), (1, 1, 2, 8, 4096), (1, 1, 1, 6, 4100),
          (1, 2, 2, 131, 256), (1, 1, 3, 70, 512),    # rows that fill one and two waves exactly
          (1, 2, 2, 128, 256), (2, 1, 3, 64, 100),    # whole power-of-two bands: interleaved workspace rows
          (1, 2, 2, 30, 960), (1, 1, 2, 20, 1920), (1, 1, 3, 25, 640)]   # consecutive columns per lane with idle lanes


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kind", ["inside", "hanging"])
@pytest.mark.parametrize("shape", SHAPES)
def test_backward_reads_and_writes_half_precision(hip, oracle, shape, kind, dtype):
    B, C, F, h, w = shape
    rng = np.random.default_rng(sum(shape) + len(kind))
    x = rng.standard_normal((B, C, h, w)).astype(np.float32)
    boxes = make_boxes(rng, C, F, h, w, kind)
    g_half = torch.from_numpy(rng.standard_normal((B, C * F, h, w)).astype(np.float32)).to(dtype)
    g32 = g_half.float().numpy()                                  # the values the kernels see
    integ_c = oracle.integral_image(x)
    integ = hip.integral_image(torch.from_numpy(x).to(DEV))
    dev_boxes = [torch.from_numpy(b).to(DEV) for b in boxes]
    for normalize, exact, needs in [(True, True, (True,) * 5), (False, True, (True, False, True, False, True)),
                                    (True, False, (True, False, False, False, False)),
                                    (True, True, (False, True, True, True, True))]:
        out_c = oracle.box_forward(integ_c, *boxes, normalize, exact)
        want = oracle.box_backward(integ_c, *boxes, g32, out_c, 3.0 * h, 2.0 * w, normalize, exact, needs)
        got = hip.box_convolution_backward(integ, *dev_boxes, g_half.to(DEV), None, 3.0 * h, 2.0 * w,
                                           normalize, exact, *needs)
        if needs[0]:
            assert got[0].dtype == dtype
            gi, ref = got[0].float().cpu().numpy(), want[0]
            gi_noise = 8 * np.finfo(np.float32).eps * np.abs(oracle.integral_image(g32)).max()
            assert np.all(np.abs(gi - ref) <= HALF_ULP[dtype] * np.abs(ref) + 1e-4 * np.abs(ref).max() + gi_noise)
        else:
            assert got[0] is None
        floor = param_grad_floor(want[1:])
        for i in range(1, 5):
            if not needs[i]:
                assert got[i] is None
                continue
            assert got[i].dtype == torch.float32
            scale = max(np.abs(want[i]).max(), floor)
            noise = np.finfo(np.float32).eps * np.abs(integ_c).max() * np.abs(g32).max() * max(3.0 * h, 2.0 * w) * np.sqrt(h * w)
            assert np.abs(got[i].cpu().numpy() - want[i]).max() <= 1e-3 * scale + noise, (normalize, exact, i)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("h,w", [(14, 60), (24, 1024)])
def test_half_grad_output_with_a_bound_one_ulp_above_an_integer(hip, oracle, h, w, dtype):
    """Rounded mode with normalisation and a lower bound one ulp above an integer: the one sum
    that is then taken again with the forward split (finalize_box) reads grad_output in its own
    half type."""
    rng = np.random.default_rng(h + w)
    B, C, F = 1, 2, 2
    x = rng.standard_normal((B, C, h, w)).astype(np.float32)
    g_half = torch.from_numpy(rng.standard_normal((B, C * F, h, w)).astype(np.float32)).to(dtype)
    g32 = g_half.float().numpy()
    just_above = np.nextafter(np.float32(-1.0), np.float32(0.0))
    boxes = (np.array([[just_above, -3.3], [np.nextafter(np.float32(-3.0), np.float32(0.0)), -0.4]], np.float32),
             np.array([[4.6, 2.2], [5.0, 3.5]], np.float32),
             np.array([[just_above, just_above], [-7.25, np.nextafter(np.float32(-2.0), np.float32(0.0))]], np.float32),
             np.array([[6.4, 9.0], [3.75, 11.5]], np.float32))
    integ_c = oracle.integral_image(x)
    out_c = oracle.box_forward(integ_c, *boxes, True, False)
    want = oracle.box_backward(integ_c, *boxes, g32, out_c, 3.0 * h, 2.0 * w, True, False, (True,) * 5)
    integ = hip.integral_image(torch.from_numpy(x).to(DEV))
    got = hip.box_convolution_backward(integ, *[torch.from_numpy(b).to(DEV) for b in boxes], g_half.to(DEV), None,
                                       3.0 * h, 2.0 * w, True, False, True, True, True, True, True)
    gi, ref = got[0].float().cpu().numpy(), want[0]
    assert np.all(np.abs(gi - ref) <= HALF_ULP[dtype] * np.abs(ref) + 1e-4 * np.abs(ref).max())
    floor = param_grad_floor(want[1:])
    for i in range(1, 5):
        assert np.abs(got[i].cpu().numpy() - want[i]).max() <= 1e-3 * max(np.abs(want[i]).max(), floor), i


def make_module(C, F, h, w, seed):
    random.seed(seed)
    return BoxConv2d(C, F, h, w).to(DEV)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_training_step_on_half_precision_input(oracle, dtype):
    C, F, h, w = 3, 4, 48, 80
    m = make_module(C, F, h, w, 11).train()
    x = torch.randn(2, C, h, w, device=DEV).to(dtype)
    go = torch.randn(2, C * F, h, w, device=DEV).to(dtype)
    xg = x.clone().requires_grad_(True)
    out = m(xg)
    assert out.dtype == dtype and out.requires_grad
    out.backward(go)
    assert xg.grad.dtype == dtype and m.x_min.grad.dtype == torch.float32
    # the oracle in float32 on the same values
    stored = [p.detach().cpu().numpy() for p in (m.x_min, m.x_max, m.y_min, m.y_max)]
    out_c, saved = oracle.module_forward(x.float().cpu().numpy(), *stored, m.reparametrization_h,
                                         m.reparametrization_w, True, True)
    grads_c = oracle.module_backward(saved, go.float().cpu().numpy(), m.reparametrization_h,
                                     m.reparametrization_w, True, True)
    u = HALF_ULP[dtype]
    assert np.all(np.abs(out.detach().float().cpu().numpy() - out_c) <= u * np.abs(out_c) + 1e-4 * np.abs(out_c).max())
    assert np.all(np.abs(xg.grad.float().cpu().numpy() - grads_c[0])
                  <= u * np.abs(grads_c[0]) + 1e-4 * np.abs(grads_c[0]).max())
    floor = param_grad_floor(grads_c[1:])
    for p, ref in zip((m.x_min, m.x_max, m.y_min, m.y_max), grads_c[1:]):
        assert np.abs(p.grad.cpu().numpy() - ref).max() <= 1e-3 * max(np.abs(ref).max(), floor)
    # a second step accumulates into .grad as for any parameter
    before = m.x_min.grad.clone()
    m(xg).backward(go)
    assert torch.allclose(m.x_min.grad, 2 * before, rtol=1e-6, atol=0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("training", [True, False])
@pytest.mark.parametrize("shape,needs", [((2, 3, 4, 40, 130), (True, True, True, True, True)),
                                         ((1, 2, 3, 64, 1024), (True, False, True, False, True)),
                                         ((2, 2, 2, 33, 2048), (False, True, True, True, True)),
                                         ((3, 1, 5, 70, 77), (True, False, False, False, False))])
def test_half_precision_step_through_the_cpp_node(dtype, training, shape, needs):
    """A float16 / bfloat16 input with float32 parameters goes through the C++ autograd node like
    a float32 one (one native call for clip, integral image and sampling, one for the backward);
    BoxConvolutionFunction is the same step in Python with the same kernels. Output, clipped
    parameters and every requested gradient agree bit for bit; under no_grad there is no graph."""
    from box_convolution import _native
    from box_convolution.box_convolution_function import BoxConvolutionFunction
    if _native.glue() is None:
        pytest.skip("the C++ glue was not built")
    B, C, F, h, w = shape
    modules = [make_module(C, F, h, w, 21) for _ in range(2)]
    modules[1].load_state_dict(modules[0].state_dict())
    torch.manual_seed(h + w)
    x0 = torch.randn(B, C, h, w, device=DEV).to(dtype)
    g = torch.randn(B, C * F, h, w, device=DEV).to(dtype)
    names = ("x_min", "x_max", "y_min", "y_max")
    results = []
    for which, m in enumerate(modules):
        with torch.no_grad():
            m.x_min.mul_(2.0)          # some boxes out of bounds: the clip has work to do (training mode only)
        for name, need in zip(names, needs[1:]):
            getattr(m, name).requires_grad_(need)
        x = x0.clone().requires_grad_(needs[0])
        m.train(training)
        if which == 0:
            out = m(x)                                                      # C++ node
            assert type(out.grad_fn).__name__ != "BoxConvolutionFunctionBackward"
        else:
            out = BoxConvolutionFunction.apply(
                x, m.x_min, m.x_max, m.y_min, m.y_max, m.reparametrization_h, m.reparametrization_w,
                m.normalize, m.exact, (m.max_input_h, m.max_input_w) if training else None)
        assert out.dtype == dtype
        out.backward(g)
        results.append((out.detach(), x.grad, [getattr(m, n).grad for n in names],
                        [getattr(m, n).detach().clone() for n in names]))
    (out_a, gx_a, gp_a, p_a), (out_b, gx_b, gp_b, p_b) = results
    assert torch.equal(out_a, out_b)
    assert (gx_a is None) == (not needs[0])
    if needs[0]:
        assert gx_a.dtype == dtype and torch.equal(gx_a, gx_b)
    for a, b, need in zip(gp_a, gp_b, needs[1:]):
        assert (a is None) == (not need) and (b is None) == (not need)
        if need:
            assert a.dtype == torch.float32 and torch.equal(a, b)
    for a, b in zip(p_a, p_b):
        assert torch.equal(a, b)
    with torch.no_grad():
        quiet = modules[0](x0)
    assert quiet.grad_fn is None and torch.equal(quiet, out_a)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_module_converted_to_half_precision(dtype):
    """module.half() / .bfloat16(): the four bounds are stored in the half type; they are clipped
    through a float32 copy, used in float32, and receive gradients of their own type."""
    C, F, h, w = 2, 3, 40, 64
    m = make_module(C, F, h, w, 4)
    ref = make_module(C, F, h, w, 4)
    m = m.to(dtype)
    with torch.no_grad():
        for p, q in zip(ref.parameters(), m.parameters()):
            p.copy_(q.float())                     # the same (half-rounded) bounds in float32
    assert m.x_min.dtype == dtype
    x = torch.randn(2, C, h, w, device=DEV).to(dtype)
    go = torch.randn(2, C * F, h, w, device=DEV).to(dtype)
    m.train()
    ref.train()
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    ya, yb = m(xa), ref(xb)
    # training mode clips: the half-precision bounds are clipped in float32 and rounded back, so
    # they may differ from the float32 module's by the rounding of the half type
    for p, q in zip(m.parameters(), ref.parameters()):
        assert torch.allclose(p.float(), q, rtol=HALF_ULP[dtype], atol=0)
    ya.backward(go)
    yb.backward(go)
    assert ya.dtype == dtype and xa.grad.dtype == dtype and m.y_max.grad.dtype == dtype
    same_boxes = all(torch.equal(p.float(), q) for p, q in zip(m.parameters(), ref.parameters()))
    if same_boxes:
        assert torch.equal(ya, yb) and torch.equal(xa.grad, xb.grad)
        for p, q in zip(m.parameters(), ref.parameters()):
            assert torch.equal(p.grad, q.grad.to(dtype))
    m.eval()                                            # clips once more, must not raise
    with torch.no_grad():
        assert m(x).dtype == dtype
