"""BoxConv2d on the GPU, tested the way the reference tests itself (box_convolution/test.py):
integral image against float64 cumulative sums, forward and grad_input against an explicit dense
box kernel run through zero-padded conv2d, parameter gradients against finite differences
(torch.autograd.gradcheck in float64) -- plus the golden vectors of the reference's CPU kernels,
multi-channel cases and the clip/eval behaviour the reference leaves untested.
"""
import math
import os
import random

import numpy as np
import pytest
import torch

from box_convolution import BoxConv2d
from box_convolution.box_convolution_function import BoxConvolutionFunction, reparametrize

pytestmark = pytest.mark.gpu
DEV = "cuda"
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.npz")


def dense_box_kernel(x_min, x_max, y_min, y_max, normalize, dtype):
    """(2*rh+1) x (2*rw+1) kernel whose entry (p, q) is the area of pixel (p, q) covered by the
    box [x_min, x_max+1) x [y_min, y_max+1) (reference test.py:60-86)."""
    rh = math.ceil(max(x_max, -x_min))
    rw = math.ceil(max(y_max, -y_min))
    rows = torch.tensor([max(0.0, min(p + 1, x_max + 1) - max(p, x_min)) for p in range(-rh, rh + 1)], dtype=dtype)
    cols = torch.tensor([max(0.0, min(q + 1, y_max + 1) - max(q, y_min)) for q in range(-rw, rw + 1)], dtype=dtype)
    k = rows[:, None] * cols[None, :]
    if normalize:
        k = k / ((x_max - x_min + 1) * (y_max - y_min + 1))
    return k


def conv2d_reference(x, real, normalize, exact):
    """Depthwise zero-padded conv2d with the dense kernels; differentiable w.r.t. x."""
    x_min, x_max, y_min, y_max = (p.detach().cpu().double() for p in real)
    if not exact:
        x_min, y_min, x_max, y_max = x_min.ceil(), y_min.ceil(), x_max.floor(), y_max.floor()
    C, F = x_min.shape
    outs = []
    for c in range(C):
        for f in range(F):
            k = dense_box_kernel(x_min[c, f].item(), x_max[c, f].item(), y_min[c, f].item(),
                                 y_max[c, f].item(), normalize, x.dtype).to(x.device)
            pad = (k.shape[0] // 2, k.shape[1] // 2)
            outs.append(torch.conv2d(x[:, c:c + 1], k[None, None], padding=pad))
    return torch.cat(outs, dim=1)


def module_with(stored, h, w, factor, normalize, exact, dtype=torch.float32):
    C, F = stored[0].shape
    m = BoxConv2d(C, F, h, w, factor).to(device=DEV, dtype=dtype)
    for name, t in zip(("x_min", "x_max", "y_min", "y_max"), stored):
        delattr(m, name)
        setattr(m, name, t)          # plain tensors instead of Parameters, as reference test.py:162-165
    m.normalize, m.exact = normalize, exact
    return m


def random_boxes(rng, C, F, h, w, exact, margin=0.012):
    """Boxes as in reference test.py:205-235: inside (-h+1, h-1), at least ~1 px (2 px when not
    exact) thick, every bound further than `margin` from a whole number."""
    def draw(lo, hi):
        while True:
            v = rng.uniform(lo, hi)
            if abs(v - round(v)) > margin:
                return v
    real = torch.empty(4, C, F, dtype=torch.float64)
    for c in range(C):
        for f in range(F):
            x0 = draw(-h + 1.05, h - (not exact) - 1.1)
            y0 = draw(-w + 1.05, w - (not exact) - 1.1)
            x1 = draw(x0 + (not exact) + 0.013, h - 1.05)
            y1 = draw(y0 + (not exact) + 0.013, w - 1.05)
            real[:, c, f] = torch.tensor([x0, x1, y0, y1])
    return real


def test_integral_image_like_reference_test():
    from box_convolution_cpp_cuda import integral_image
    rng = random.Random(1546545757)
    for _ in range(50):
        shape = (rng.randint(1, 3), rng.randint(1, 3), rng.randint(2, 10), rng.randint(2, 10))
        x = torch.rand(*shape, device=DEV)
        want = torch.zeros(shape[0], shape[1], shape[2] + 1, shape[3] + 1, dtype=torch.float64, device=DEV)
        want[..., 1:, 1:] = x.double().cumsum(-2).cumsum(-1)
        assert integral_image(x).allclose(want.float())        # default rtol/atol, reference test.py:53


def test_native_module_stand_in_on_the_gpu(oracle):
    """The four functions of `box_convolution_cpp_cuda` called the way the reference's Python layer
    calls them (box_convolution_function.py:44-46,59-62; box_convolution_module.py:203-206),
    against the CPU oracle; gradients that were not asked for come back as 0-element tensors
    (reference src/box_convolution_interface.cpp:181-183,394)."""
    import box_convolution_cpp_cuda as cpp_cuda
    from helpers import make_boxes
    rng = np.random.default_rng(31)
    B, C, F, h, w = 2, 3, 2, 21, 34
    x = rng.standard_normal((B, C, h, w)).astype(np.float32)
    g = rng.standard_normal((B, C * F, h, w)).astype(np.float32)
    boxes = make_boxes(rng, C, F, h, w, "hanging")
    dev_boxes = [torch.from_numpy(b).to(DEV) for b in boxes]
    integ = cpp_cuda.integral_image(torch.from_numpy(x).to(DEV))
    out = cpp_cuda.box_convolution_forward(integ, *dev_boxes, True, True)
    integ_c = oracle.integral_image(x)
    out_c = oracle.box_forward(integ_c, *boxes, True, True)
    assert np.abs(out.cpu().numpy() - out_c).max() <= 1e-4 * np.abs(out_c).max()
    for needs in [(True, True, True, True, True), (True, False, False, False, False),
                  (False, True, False, False, True), (False, False, True, True, False)]:
        grads = cpp_cuda.box_convolution_backward(integ, *dev_boxes, torch.from_numpy(g).to(DEV), out,
                                                  3.0, 5.0, True, True, *needs)
        grads_c = oracle.box_backward(integ_c, *boxes, g, out_c, 3.0, 5.0, True, True, needs)
        assert len(grads) == 5
        scale = max(np.abs(gc).max() for gc in grads_c[1:] if gc is not None) if any(needs[1:]) else 1.0
        for i, (got, want, need) in enumerate(zip(grads, grads_c, needs)):
            if not need:
                assert isinstance(got, torch.Tensor) and got.numel() == 0
                continue
            tol = 1e-4 * np.abs(want).max() if i == 0 else 1e-3 * max(np.abs(want).max(), 1e-2 * scale)
            assert got.shape == want.shape and np.abs(got.cpu().numpy() - want).max() <= tol, (needs, i)
    # clip_parameters: in place on the stored parameters, bit for bit as the oracle
    stored = [torch.from_numpy((b / s).astype(np.float32)).to(DEV)
              for b, s in zip(boxes, (8.0 * h, 8.0 * h, 8.0 * w, 8.0 * w))]
    host = [p.cpu().numpy().copy() for p in stored]
    assert cpp_cuda.clip_parameters(*stored, 8.0 * h, 8.0 * w, float(h), float(w), True) is None
    oracle.clip_parameters(*host, 8.0 * h, 8.0 * w, float(h), float(w), True)
    for p, q in zip(stored, host):
        assert np.array_equal(p.cpu().numpy(), q)


@pytest.mark.parametrize("seed", range(12))
def test_module_against_conv2d_like_reference_test(seed):
    rng = random.Random(1546545757 + seed)
    torch.manual_seed(seed)
    exact = rng.random() < 0.7
    C, F = rng.choice([(1, 1), (1, 1), (2, 3), (3, 2)])
    B = rng.randint(1, 2)
    h, w = rng.randint(2 + (not exact), 10), rng.randint(2 + (not exact), 10)
    factor = rng.random() * 4.5 + 0.5
    normalize = rng.choice((False, True))
    real = random_boxes(rng, C, F, h, w, exact)
    reparam_h, reparam_w = (h + 1) * factor, (w + 1) * factor
    stored = [t.float().to(DEV) for t in reparametrize(*real, reparam_h, reparam_w)]
    x = torch.rand(B, C, h, w, device=DEV, requires_grad=True)
    g = (torch.rand(B, C * F, h, w, device=DEV) < 0.15).float()

    m = module_with(stored, h + 1, w + 1, factor, normalize, exact)
    before = m.get_actual_parameters()
    out = m(x)
    for a, b in zip(before, m.get_actual_parameters()):
        assert torch.equal(a, b), "test boxes must not be altered by _clip_parameters"
    out.backward(g)
    ours_grad = x.grad.clone()
    x.grad = None

    ref = conv2d_reference(x, m.get_actual_parameters(), normalize, exact)
    ref.backward(g)
    assert out.allclose(ref, rtol=3e-5, atol=1e-5)                 # reference test.py:260
    assert ours_grad.allclose(x.grad, rtol=3e-5, atol=1e-5)        # reference test.py:267


@pytest.mark.parametrize("seed", range(6))
def test_parameter_gradients_gradcheck_float64(seed):
    rng = random.Random(99 + seed)
    torch.manual_seed(seed)
    C, F = rng.choice([(1, 1), (2, 2)])
    h, w = rng.randint(3, 8), rng.randint(3, 8)
    factor = rng.random() * 4.5 + 0.5
    normalize = rng.choice((False, True))
    real = random_boxes(rng, C, F, h, w, True)
    reparam_h, reparam_w = (h + 1) * factor, (w + 1) * factor
    stored = [t.to(DEV).requires_grad_() for t in reparametrize(*real, reparam_h, reparam_w)]
    x = torch.rand(2, C, h, w, device=DEV, dtype=torch.float64)

    def fn(x_min, x_max, y_min, y_max):
        return BoxConvolutionFunction.apply(x, x_min, x_max, y_min, y_max, reparam_h, reparam_w,
                                            normalize, True)

    assert torch.autograd.gradcheck(fn, stored, eps=0.004 / max(reparam_h, reparam_w),
                                    raise_exception=True)           # reference test.py:296-301


@pytest.mark.parametrize("case", ["inside_f32", "hanging_f32", "integer_f32", "unit_f32",
                                  "hanging_f64", "integer_f64", "tall_f32"])
def test_hip_matches_golden_vectors_of_the_reference(hip, case):
    gold = np.load(GOLDEN)
    x = torch.from_numpy(gold[case + "/x"]).to(DEV)
    g = torch.from_numpy(gold[case + "/grad_output"]).to(DEV)
    reparam_h, reparam_w = (float(v) for v in gold[case + "/reparam"])
    f32 = x.dtype == torch.float32
    tol_f, tol_p = (1e-4, 1e-3) if f32 else (1e-9, 1e-9)
    integ = hip.integral_image(x)
    want_i = gold[case + "/integral"]
    assert np.abs(integ.cpu().numpy() - want_i).max() <= (1e-6 if f32 else 1e-13) * max(1.0, np.abs(want_i).max())
    eps = np.finfo(want_i.dtype).eps
    noise = 8 * eps * float(np.abs(want_i).max())
    gnoise = 8 * eps * float(hip.integral_image(g).abs().max())
    for exact in (1, 0):
        bx = [torch.from_numpy(gold["%s/exact%d/%s" % (case, exact, n)]).to(DEV)
              for n in ("x_min", "x_max", "y_min", "y_max")]
        for normalize in (1, 0):
            tag = "%s/exact%d/norm%d" % (case, exact, normalize)
            out = hip.box_convolution_forward(integ, *bx, normalize, exact)
            back = hip.box_convolution_backward(integ, *bx, g, out, reparam_h, reparam_w, normalize,
                                                exact, True, True, True, True, True)
            want = gold[tag + "/output"]
            assert np.abs(out.cpu().numpy() - want).max() <= tol_f * np.abs(want).max() + noise, tag
            want = gold[tag + "/grad_input"]
            assert np.abs(back[0].cpu().numpy() - want).max() <= tol_f * np.abs(want).max() + gnoise, tag
            names = ("grad_x_min", "grad_x_max", "grad_y_min", "grad_y_max")
            scale = max(np.abs(gold[tag + "/" + n]).max() for n in names)
            for k, n in enumerate(names):
                want = gold[tag + "/" + n]
                assert np.abs(back[1 + k].cpu().numpy() - want).max() <= tol_p * max(np.abs(want).max(), 1e-2 * scale), (tag, n)


def test_clip_matches_golden_vectors_bit_for_bit(hip):
    gold = np.load(GOLDEN)
    for tag in ("clip_f32", "clip_f64"):
        rh, rw, mh, mw = (float(v) for v in gold[tag + "/meta"])
        for exact in (1, 0):
            p = [torch.from_numpy(gold["%s/in%d" % (tag, k)]).to(DEV) for k in range(4)]
            hip.clip_parameters(*p, rh, rw, mh, mw, exact)
            for k in range(4):
                assert np.array_equal(p[k].cpu().numpy(), gold["%s/exact%d/out%d" % (tag, exact, k)])


def test_training_forward_clips_and_eval_clips_once():
    random.seed(3)
    m = BoxConv2d(2, 3, 16, 16).to(DEV)
    with torch.no_grad():
        m.x_min.fill_(0.5)       # 64 px: far outside [-(16+1), 16-1]
        m.x_max.fill_(0.5)
    m.eval()
    assert torch.all(m.x_max * m.reparametrization_h <= 15 + 1e-3)
    assert torch.all((m.x_max - m.x_min) * m.reparametrization_h >= 0.0011 - 1e-4)
    with torch.no_grad():
        m.y_min.fill_(-1.0)
    m.train()
    x = torch.randn(1, 2, 16, 16, device=DEV)
    m(x)
    assert torch.all(m.y_min * m.reparametrization_w >= -17 - 1e-3)
    # eval-mode forward leaves the parameters alone
    m.training = False
    with torch.no_grad():
        m.y_min.fill_(-1.0)
    m(x)
    assert torch.all(m.y_min == -1.0)


def test_eval_before_moving_to_gpu_uses_the_hip_kernel():
    random.seed(4)
    m = BoxConv2d(1, 4, 12, 12)
    with torch.no_grad():
        m.x_max.copy_(m.x_min)                     # zero-thickness boxes on the host
    m.eval()
    assert m.x_min.device.type == "cpu"
    thick = (m.x_max - m.x_min) * m.reparametrization_h
    assert torch.allclose(thick, torch.full_like(thick, 1.001 - 0.9999), atol=1e-4)


def test_module_trains_end_to_end():
    random.seed(5)
    torch.manual_seed(5)
    m = BoxConv2d(3, 4, 24, 32).to(DEV)
    opt = torch.optim.SGD(m.parameters(), lr=1e-4)
    x = torch.randn(2, 3, 24, 32, device=DEV, requires_grad=True)
    target = torch.randn(2, 12, 24, 32, device=DEV)
    losses = []
    for _ in range(5):
        opt.zero_grad()
        loss = ((m(x) - target) ** 2).mean()
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert all(np.isfinite(losses)) and x.grad is not None and x.grad.shape == x.shape
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in m.parameters())


def test_training_trajectory_matches_the_cpu_twin(oracle):
    """Twenty steps of SGD with momentum on a BoxConv2d layer (GPU, the module as a user calls
    it: clip, unit conversion, integral image, sampling, backward) against the same loop on the
    host with the CPU oracle in the place of every native call (clip_parameters at the start of
    each training forward, reference box_convolution/box_convolution_module.py:203-206). Losses
    and the final parameters must agree: a difference in any gradient, in the clip or in the
    units would compound over the steps."""
    random.seed(11)
    torch.manual_seed(11)
    B, C, F, h, w = 2, 3, 4, 30, 44
    m = BoxConv2d(C, F, h, w).to(DEV)
    names = ("x_min", "x_max", "y_min", "y_max")
    twin = [getattr(m, n).detach().cpu().numpy().copy() for n in names]
    x = torch.randn(B, C, h, w)
    target = torch.randn(B, C * F, h, w) * 0.1 + x.repeat_interleave(F, dim=1) * 0.5
    lr, mom, steps = 2e-3, 0.9, 20
    opt = torch.optim.SGD(m.parameters(), lr=lr, momentum=mom)
    xg, tg = x.to(DEV), target.to(DEV)
    m.train()
    losses_gpu, losses_cpu = [], []
    velocity = [np.zeros_like(p) for p in twin]
    moved = 0.0
    start = [p.copy() for p in twin]
    for step in range(steps):
        opt.zero_grad()
        out = m(xg)
        loss = ((out - tg) ** 2).mean()
        loss.backward()
        opt.step()
        losses_gpu.append(loss.item())
        # the twin: clip in place, forward, loss, backward, the same momentum update in float32
        oracle.clip_parameters(*twin, m.reparametrization_h, m.reparametrization_w, m.max_input_h, m.max_input_w, True)
        out_c, saved = oracle.module_forward(x.numpy(), *twin, m.reparametrization_h, m.reparametrization_w, True, True)
        diff = out_c - target.numpy()
        losses_cpu.append(float((diff.astype(np.float64) ** 2).mean()))
        grad_out = (2.0 / diff.size * diff).astype(np.float32)
        grads = oracle.module_backward(saved, grad_out, m.reparametrization_h, m.reparametrization_w, True, True,
                                       (False, True, True, True, True))
        for k in range(4):
            velocity[k] = (mom * velocity[k] + grads[1 + k]).astype(np.float32) if step else grads[1 + k].copy()
            twin[k] = (twin[k] - np.float32(lr) * velocity[k]).astype(np.float32)
    for a, b in zip(losses_gpu, losses_cpu):
        assert abs(a - b) <= 1e-4 * abs(b), (losses_gpu, losses_cpu)
    for n, want, first in zip(names, twin, start):
        got = getattr(m, n).detach().cpu().numpy()
        moved = max(moved, float(np.abs(want - first).max()))
        assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max(), n
    assert moved > 1e-3, "the parameters hardly moved: the test would not notice a wrong gradient"
    assert losses_gpu[-1] < losses_gpu[0]


def test_noncontiguous_input_and_dtype_errors(hip):
    x = torch.randn(2, 2, 9, 20, device=DEV)[..., ::2]
    assert not x.is_contiguous()
    assert torch.equal(hip.integral_image(x), hip.integral_image(x.contiguous()))
    with pytest.raises(RuntimeError, match="float32 or float64"):
        hip.integral_image(torch.zeros(1, 4, 4, device=DEV, dtype=torch.bool))
    # (float16 / bfloat16 inputs are integrated into float32: test_gpu_fused_forward.py; integer
    # tensors in their own type: test_gpu_parity.py)
    z = torch.zeros(2, 1, device=DEV)
    with pytest.raises(RuntimeError, match="as many rows"):
        hip.box_convolution_forward(torch.zeros(1, 3, 5, 5, device=DEV), z, z, z, z, True, True)
    with pytest.raises(RuntimeError, match="different devices"):
        hip.box_convolution_forward(torch.zeros(1, 2, 5, 5, device=DEV), z.cpu(), z, z, z, True, True)


def test_training_forward_fuses_clip_and_reparametrize():
    """In training mode the module clips and converts to real units in one launch; the result
    must equal clip_parameters followed by reparametrize(..., inverse=True) bit for bit."""
    from box_convolution import BoxConv2d, _native
    from box_convolution.box_convolution_function import reparametrize
    torch.manual_seed(3)
    for dtype in (torch.float32, torch.float64):
        m = BoxConv2d(3, 4, 20, 30).to("cuda", dtype)
        with torch.no_grad():      # push some boxes out of bounds / make some too thin
            m.x_min.mul_(3.0); m.y_max.add_(0.5); m.x_max.copy_(m.x_min + 1e-4)
        stored = [p.detach().clone() for p in (m.x_min, m.x_max, m.y_min, m.y_max)]
        _native.clip_parameters(*stored, m.reparametrization_h, m.reparametrization_w, 20, 30, True)
        want_real = reparametrize(*stored, m.reparametrization_h, m.reparametrization_w, inverse=True)
        live = [p.detach() for p in (m.x_min, m.x_max, m.y_min, m.y_max)]
        got_real = _native.clip_reparametrize(*live, m.reparametrization_h, m.reparametrization_w, 20, 30, True)
        for a, b in zip(live, stored):
            assert torch.equal(a, b)
        for a, b in zip(got_real, want_real):
            assert torch.equal(a, b)
        # and through the module: same output as the two-step path
        x = torch.randn(2, 3, 20, 30, device="cuda", dtype=dtype)
        m.train()
        out = m(x)
        from box_convolution.box_convolution_function import BoxConvolutionFunction
        # (the forward clipped once more; compare with the parameters as they are now)
        now = [p.detach() for p in (m.x_min, m.x_max, m.y_min, m.y_max)]
        ref = BoxConvolutionFunction.apply(x, *now, m.reparametrization_h, m.reparametrization_w, True, True)
        assert torch.equal(out, ref)


@pytest.mark.parametrize("shape", [(2, 3, 4, 20, 30), (1, 2, 2, 96, 256), (2, 1, 3, 70, 1024)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_training_forward_in_one_native_call(shape, dtype):
    """clip + unit conversion + integral image + sampling as one native call (the clip shares a
    launch with the preparation of the integral image's workspace where the single-pass
    integral-image kernel runs) against the same steps called one by one: identical bits."""
    from box_convolution import BoxConv2d, _native
    from box_convolution.box_convolution_function import reparametrize
    B, C, F, h, w = shape
    random.seed(17)
    m = BoxConv2d(C, F, h, w).to("cuda", dtype)
    with torch.no_grad():
        m.x_min.mul_(2.5); m.y_max.add_(0.3); m.y_min.copy_(m.y_max - 1e-5)
    x = torch.randn(B, C, h, w, device="cuda", dtype=dtype)
    stored = [p.detach().clone() for p in (m.x_min, m.x_max, m.y_min, m.y_max)]
    _native.clip_parameters(*stored, m.reparametrization_h, m.reparametrization_w, h, w, True)
    real = reparametrize(*stored, m.reparametrization_h, m.reparametrization_w, inverse=True)
    integ = _native.integral_image(x)
    out = _native.box_convolution_forward(integ, *real, True, True)

    live = [p.detach() for p in (m.x_min, m.x_max, m.y_min, m.y_max)]
    got_integ, got_out, got_real = _native.training_forward(
        x, *live, m.reparametrization_h, m.reparametrization_w, h, w, True, True)
    for a, b in zip(live, stored):
        assert torch.equal(a, b)
    for a, b in zip(got_real, real):
        assert torch.equal(a, b)
    assert torch.equal(got_integ, integ) and torch.equal(got_out, out)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("needs", [(True, True, True, True, True), (False, True, True, True, True),
                                   (True, False, False, False, False), (True, True, False, False, True)])
def test_cpp_autograd_node_matches_the_python_function(hip, dtype, needs):
    """BoxConv2d.forward in training mode goes through the C++ autograd node where that extension
    was built; BoxConvolutionFunction with `clip_to` is the same step in Python. Same native
    calls, so output, clipped parameters and every requested gradient agree bit for bit, and
    gradients that were not requested stay None."""
    if hip.glue() is None:
        pytest.skip("the C++ glue was not built")
    B, C, F, h, w = 2, 3, 4, 40, 130
    random.seed(5)
    torch.manual_seed(5)
    modules = [BoxConv2d(C, F, h, w).to(DEV, dtype) for _ in range(2)]
    modules[1].load_state_dict(modules[0].state_dict())
    x0 = torch.randn(B, C, h, w, device=DEV, dtype=dtype)
    g = torch.randn(B, C * F, h, w, device=DEV, dtype=dtype)
    results = []
    for which, m in enumerate(modules):
        with torch.no_grad():
            m.x_min.mul_(2.0)          # some boxes out of bounds: the clip has work to do
        names = ("x_min", "x_max", "y_min", "y_max")
        for name, need in zip(names, needs[1:]):
            getattr(m, name).requires_grad_(need)
        x = x0.clone().requires_grad_(needs[0])
        m.train()
        if which == 0:
            out = m(x)                                                      # C++ node
            assert type(out.grad_fn).__name__ != "BoxConvolutionFunctionBackward"
        else:
            out = BoxConvolutionFunction.apply(
                x, m.x_min, m.x_max, m.y_min, m.y_max, m.reparametrization_h, m.reparametrization_w,
                m.normalize, m.exact, (m.max_input_h, m.max_input_w))      # Python function
        out.backward(g)
        results.append((out.detach(), x.grad, [getattr(m, n).grad for n in names],
                        [getattr(m, n).detach().clone() for n in names]))
    (out_a, gx_a, gp_a, p_a), (out_b, gx_b, gp_b, p_b) = results
    assert torch.equal(out_a, out_b)
    assert (gx_a is None) == (not needs[0]) and (gx_b is None) == (not needs[0])
    if needs[0]:
        assert torch.equal(gx_a, gx_b)
    for a, b, need in zip(gp_a, gp_b, needs[1:]):
        assert (a is None) == (not need) and (b is None) == (not need)
        if need:
            assert torch.equal(a, b)
    for a, b in zip(p_a, p_b):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("grad", [True, False])
def test_cpp_autograd_node_in_eval_mode(hip, dtype, grad):
    """In eval mode the module's forward goes through the same C++ node without the clip
    (reference box_convolution/box_convolution_module.py:203-214: clip_parameters only when
    training): parameters that are out of bounds stay as they are, and output and gradients are
    those of BoxConvolutionFunction without `clip_to`, bit for bit; under no_grad there is no
    graph."""
    if hip.glue() is None:
        pytest.skip("the C++ glue was not built")
    B, C, F, h, w = 2, 3, 4, 33, 70
    random.seed(6)
    torch.manual_seed(6)
    m = BoxConv2d(C, F, h, w).to(DEV, dtype)
    m.eval()
    with torch.no_grad():
        m.x_min.mul_(3.0)              # out of bounds on purpose; eval mode must not touch them
    names = ("x_min", "x_max", "y_min", "y_max")
    before = [getattr(m, n).detach().clone() for n in names]
    x = torch.randn(B, C, h, w, device=DEV, dtype=dtype, requires_grad=grad)
    g = torch.randn(B, C * F, h, w, device=DEV, dtype=dtype)
    if grad:
        out = m(x)
        assert type(out.grad_fn).__name__ != "BoxConvolutionFunctionBackward"
        out.backward(g)
        got = (out.detach(), x.grad, [getattr(m, n).grad.clone() for n in names])
        for n in names:
            getattr(m, n).grad = None
        x2 = x.detach().clone().requires_grad_(True)
        ref = BoxConvolutionFunction.apply(x2, m.x_min, m.x_max, m.y_min, m.y_max, m.reparametrization_h,
                                           m.reparametrization_w, m.normalize, m.exact, None)
        ref.backward(g)
        assert torch.equal(got[0], ref.detach()) and torch.equal(got[1], x2.grad)
        for a, n in zip(got[2], names):
            assert torch.equal(a, getattr(m, n).grad)
    else:
        with torch.no_grad():
            out = m(x)
            ref = BoxConvolutionFunction.apply(x, m.x_min, m.x_max, m.y_min, m.y_max, m.reparametrization_h,
                                               m.reparametrization_w, m.normalize, m.exact, None)
        assert out.grad_fn is None and not out.requires_grad
        assert torch.equal(out, ref)
    for a, n in zip(before, names):
        assert torch.equal(a, getattr(m, n).detach())


def test_cpp_autograd_node_reports_the_reference_errors(hip):
    if hip.glue() is None:
        pytest.skip("the C++ glue was not built")
    m = BoxConv2d(2, 3, 8, 8).to(DEV)
    m.train()
    with pytest.raises(RuntimeError, match="as many rows as there are input channels"):
        m(torch.zeros(1, 5, 8, 8, device=DEV))
    with pytest.raises(AssertionError):
        BoxConv2d(2, 3, 8, 8, stride_h=2)


@pytest.mark.parametrize("w,rows,in_flight", [(256, 16, 2), (1024, 64, 8), (4096, 8, 4)])
def test_copy_probe_copies(hip, w, rows, in_flight):
    """The benchmark's yardstick kernel (a plain copy with the streaming pass's access pattern)
    moves exactly the bytes it is priced on: rows 1..h of every plane, nothing else."""
    planes, h = 5, 128
    src = torch.randn(planes, h, w, device="cuda")
    dst = torch.full((planes, h + 1, w), -7.0, device="cuda")
    hip.probe_copy_bands(src, dst, rows, in_flight)
    torch.cuda.synchronize()
    assert torch.equal(dst[:, 1:], src)
    assert bool((dst[:, 0] == -7.0).all())
    with pytest.raises(RuntimeError):
        hip.probe_copy_bands(src, dst, 48, 2)


def test_modules_on_concurrent_streams_give_the_serial_bits():
    """Three layers stepping at the same time on streams of their own (one of them at a shape that
    takes the single-pass integral image, whose workgroups wait for each other): every call keeps
    its scratch per stream and the results are those of the calls run one after the other, bit
    for bit."""
    random.seed(12)
    torch.manual_seed(12)
    shapes = [(2, 8, 4, 256, 512), (4, 16, 4, 64, 128), (1, 4, 8, 128, 1024)]
    mods, xs, gs, refs = [], [], [], []
    for (B, C, F, h, w) in shapes:
        m = BoxConv2d(C, F, h, w).to(DEV)
        m.train()
        x = torch.randn(B, C, h, w, device=DEV, requires_grad=True)
        g = torch.randn(B, C * F, h, w, device=DEV)
        out = m(x)
        out.backward(g)
        refs.append((out.detach().clone(), x.grad.clone(), [p.grad.clone() for p in m.parameters()]))
        x.grad = None
        for p in m.parameters():
            p.grad = None
        mods.append(m), xs.append(x), gs.append(g)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in shapes]
    for _ in range(5):
        outs = []
        for s, m, x, g in zip(streams, mods, xs, gs):
            s.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(s):
                out = m(x)
                out.backward(g)
                outs.append(out)
        for s in streams:
            torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        for m, x, out, ref in zip(mods, xs, outs, refs):
            assert torch.equal(out.detach(), ref[0]) and torch.equal(x.grad, ref[1])
            for p, want in zip(m.parameters(), ref[2]):
                assert torch.equal(p.grad, want)
                p.grad = None
            x.grad = None


def test_batches_too_large_for_one_native_call_go_through_in_slices(monkeypatch):
    """The library indexes with 32 bits and refuses batch * planes * filters * (h+1) * (w+1) >=
    2^31; the module then feeds the batch through in slices. Here with the limit lowered so that a
    small batch is cut into three uneven slices: output, grad_input and the parameter gradients
    are those of the single call."""
    random.seed(8)
    torch.manual_seed(8)
    B, C, F, h, w = 7, 2, 3, 20, 33
    m = BoxConv2d(C, F, h, w).to(DEV)
    m.train()
    x = torch.randn(B, C, h, w, device=DEV, requires_grad=True)
    g = torch.randn(B, C * F, h, w, device=DEV)
    m(x).backward(g)
    whole = (x.grad.clone(), [p.grad.clone() for p in m.parameters()])
    out_whole = m(x).detach()
    x.grad = None
    for p in m.parameters():
        p.grad = None
    per_item = C * F * (h + 1) * (w + 1)
    monkeypatch.setattr(BoxConv2d, "_MAX_ELEMENTS", 3 * per_item + 5)      # slices of 3, 3 and 1
    assert m._batch_limit(x) == 3
    out = m(x)
    out.backward(g)
    assert torch.equal(out.detach(), out_whole)
    assert torch.equal(x.grad, whole[0])
    for p, want in zip(m.parameters(), whole[1]):
        assert torch.allclose(p.grad, want, rtol=1e-5, atol=1e-6 * float(want.abs().max()))


def test_output_of_more_than_2_31_elements(hip):
    """The real thing: 130 x 4 planes x 8 filters of 512 x 1024 (8.7 GB of output, 2^31 elements
    are reached at batch 128). A single native call is refused; the module's forward and
    backward work, and agree with the batch items run one at a time."""
    free, _ = torch.cuda.mem_get_info()
    if free < 60 * 2 ** 30:
        pytest.skip("needs 60 GB of free device memory")
    random.seed(9)
    torch.manual_seed(9)
    B, C, F, h, w = 130, 4, 8, 512, 1024
    m = BoxConv2d(C, F, h, w).to(DEV)
    m.train()
    x = torch.randn(B, C, h, w, device=DEV, requires_grad=True)
    with pytest.raises(RuntimeError, match="2\\^31"):
        hip.integral_image(torch.empty(B * C * F, h, w, device=DEV))
    assert m._batch_limit(x) == 127
    g = torch.randn(B, C * F, h, w, device=DEV)
    out = m(x)
    assert out.shape == (B, C * F, h, w)
    out.backward(g)
    gin = x.grad
    gpar = [p.grad.clone() for p in m.parameters()]
    for p in m.parameters():
        p.grad = None
    acc = [torch.zeros(C, F, device=DEV, dtype=torch.float64) for _ in range(4)]
    worst_out = worst_gin = 0.0
    for b in range(B):
        xb = x.detach()[b:b + 1].clone().requires_grad_(True)
        ob = m(xb)
        ob.backward(g[b:b + 1])
        for a, p in zip(acc, m.parameters()):
            a += p.grad.double()
            p.grad = None
        if b in (0, 1, 63, 126, 127, 129):
            worst_out = max(worst_out, float((ob.detach() - out.detach()[b:b + 1]).abs().max() / ob.detach().abs().max()))
            worst_gin = max(worst_gin, float((xb.grad - gin[b:b + 1]).abs().max() / xb.grad.abs().max()))
    assert worst_out <= 2e-6 and worst_gin <= 2e-6, (worst_out, worst_gin)
    for got, want in zip(gpar, acc):
        assert float((got.double() - want).abs().max()) <= 1e-4 * float(want.abs().max())
    del out, gin, g, x
    torch.cuda.empty_cache()
    hip.release_workspaces()


def test_grad_input_pattern_probe_reads_the_rows_it_is_priced_on(hip):
    """The benchmark's second yardstick (the grad-input pass's loads and stores without its
    arithmetic): with every plane of the workspace holding its own constant the blend of the two
    runs cancels (mode 0) and the single run returns the sum of the constants (mode 1); with rows
    that hold their row index, mode 1 returns the clamped row positions."""
    planes, C, F, h = 8, 2, 3, 104
    x_lo = torch.tensor([[-5, -40, 2], [-1, -90, -7]], dtype=torch.int32, device="cuda")
    x_hi = torch.tensor([[6, 3, 30], [1, 80, -2]], dtype=torch.int32, device="cuda")
    consts = torch.arange(1, planes * F + 1, device="cuda", dtype=torch.float32).view(planes, F, 1, 1)
    m = consts.expand(planes, F, h + 1, 1024).contiguous()
    out = torch.full((planes, h, 1024), -1.0, device="cuda")
    hip.probe_grad_input_pattern(m, out, x_lo, x_hi, 0)
    assert bool((out == 0).all())
    hip.probe_grad_input_pattern(m, out, x_lo, x_hi, 1)
    assert torch.equal(out, consts.sum(1).expand(planes, h, 1024))
    rows = torch.arange(h + 1, device="cuda", dtype=torch.float32).view(1, 1, h + 1, 1)
    m = rows.expand(planes, F, h + 1, 1024).contiguous()
    hip.probe_grad_input_pattern(m, out, x_lo, x_hi, 1)
    i = torch.arange(h, device="cuda").view(1, h, 1)
    want = torch.zeros(planes, h, 1, device="cuda")
    for p in range(planes):
        for f in range(F):
            b0 = (i[0] + int(x_hi[p % C, f])).clamp(0, h).float()
            b1 = (i[0] + 1 + int(x_hi[p % C, f])).clamp(0, h).float()
            want[p] += b0 + 0.25 * (b1 - b0)
    assert torch.allclose(out, want.expand(planes, h, 1024), rtol=0, atol=1e-4)
    hip.probe_grad_input_pattern(m, out, x_lo, x_hi, 2)          # (runs; its values are not meaningful)
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError):
        hip.probe_grad_input_pattern(m, out, x_lo, x_hi, 3)
