"""Host-side layer (BoxConv2d, BoxConvolutionFunction, reparametrize) without a GPU: constructor
surface, seeded initialisation, training/eval clipping hooks, error behaviour."""
import random

import numpy as np
import pytest
import torch

from box_convolution import BoxConv2d, _native
from box_convolution.box_convolution_function import BoxConvolutionFunction, reparametrize


def test_constructor_surface_matches_reference():
    m = BoxConv2d(3, 5, 28, 40, reparametrization_factor=4)
    assert (m.in_planes, m.num_filters, m.max_input_h, m.max_input_w) == (3, 5, 28, 40)
    assert (m.reparametrization_h, m.reparametrization_w) == (28 * 4, 40 * 4)
    assert m.normalize is True and m.exact is True and (m.stride_h, m.stride_w) == (1, 1)
    assert sorted(n for n, _ in m.named_parameters()) == ["x_max", "x_min", "y_max", "y_min"]
    assert all(p.shape == (3, 5) and p.dtype == torch.float32 for p in m.parameters())
    assert sorted(m.state_dict()) == ["x_max", "x_min", "y_max", "y_min"]
    with pytest.raises(AssertionError):
        BoxConv2d(1, 1, 8, 8, stride_h=2)
    assert BoxConv2d(1, 1, 8, 8, 8, 1, 1, False).normalize is False


def reference_style_init(in_planes, num_filters, max_h, max_w, factor):
    """The initialisation loop written the way the reference does it (element-wise assignment
    into float32 tensors, then an in-place scale), for comparison with the vectorised module."""
    xs = [torch.empty(in_planes, num_filters) for _ in range(4)]
    min_h, min_w = 2, 2
    for c in range(in_planes):
        for f in range(num_filters):
            center_h = random.uniform(-max_h * 2 / 4.8 + 1 + min_h / 2, max_h * 2 / 4.8 - 1 - min_h / 2)
            center_w = random.uniform(-max_w * 2 / 4.8 + 1 + min_w / 2, max_w * 2 / 4.8 - 1 - min_w / 2)
            height = 2 * random.uniform(min_h / 2, min((max_h * 2 / 4.8 - 1) - center_h, center_h - (-max_h * 2 / 4.8 + 1)))
            width = 2 * random.uniform(min_w / 2, min((max_w * 2 / 4.8 - 1) - center_w, center_w - (-max_w * 2 / 4.8 + 1)))
            xs[0][c, f] = (center_h - height / 2) * 1.5
            xs[1][c, f] = (center_h + height / 2) * 1.5
            xs[2][c, f] = (center_w - width / 2) * 1.5
            xs[3][c, f] = (center_w + width / 2) * 1.5
    xs[0] *= 1 / (max_h * factor)
    xs[1] *= 1 / (max_h * factor)
    xs[2] *= 1 / (max_w * factor)
    xs[3] *= 1 / (max_w * factor)
    return xs


@pytest.mark.parametrize("shape", [(1, 40, 28, 28, 8), (4, 3, 64, 128, 2.5)])
def test_reset_parameters_draw_order_and_rounding(shape):
    C, F, H, W, factor = shape
    random.seed(1001)
    m = BoxConv2d(C, F, H, W, factor)
    after = random.getstate()
    random.seed(1001)
    want = reference_style_init(C, F, H, W, factor)
    assert random.getstate() == after          # same number of draws from the global generator
    for p, t in zip((m.x_min, m.x_max, m.y_min, m.y_max), want):
        assert torch.equal(p.detach(), t)
    # invariants of the initialisation: boxes at least 3 px thick, inside 1.5*(max*2/4.8 - 1)
    x_min, x_max, y_min, y_max = m.get_actual_parameters()
    assert torch.all(x_max - x_min >= 3 - 1e-3) and torch.all(y_max - y_min >= 3 - 1e-3)
    assert torch.all(x_max.abs() <= 1.5 * (H * 2 / 4.8 - 1) + 1e-3)
    assert torch.all(y_min.abs() <= 1.5 * (W * 2 / 4.8 - 1) + 1e-3)


def test_reparametrize_round_trip_and_modes():
    p = [torch.randn(2, 3) for _ in range(4)]
    real = reparametrize(*p, 224, 320, inverse=True)
    assert torch.equal(real[0], p[0] * 224) and torch.equal(real[3], p[3] * 320)
    stored = reparametrize(*real, 224, 320)
    for a, b in zip(stored, p):
        assert torch.allclose(a, b, rtol=1e-6)
    q = [t.clone() for t in p]
    assert reparametrize(*q, 224, 320, inplace=True, inverse=True) is None
    assert torch.equal(q[1], p[1] * 224)
    w = torch.nn.Parameter(torch.ones(1, 1))
    assert not reparametrize(w, w, w, w, 2, 2)[0].requires_grad


def test_train_and_forward_clip_hooks(monkeypatch):
    calls = []
    monkeypatch.setattr(_native, "clip_parameters", lambda *a: calls.append(a))
    m = BoxConv2d(1, 2, 8, 8)
    assert m.train() is m and m.training is True and calls == []
    assert m.eval() is m and m.training is False and len(calls) == 1
    args = calls[0]
    assert args[0] is m.x_min and args[3] is m.y_max
    assert args[4:] == (m.reparametrization_h, m.reparametrization_w, 8, 8, True)
    m.exact = False
    m.train(False)
    assert calls[-1][-1] is False
    # forward in training mode clips first, then runs the function
    seen = []
    monkeypatch.setattr(BoxConvolutionFunction, "apply", staticmethod(lambda *a: seen.append(a) or "out"))
    m.train()
    n = len(calls)
    assert m(torch.zeros(1, 1, 8, 8)) == "out" and len(calls) == n + 1
    # (parameters on the host: separate clip, no pre-scaled parameters handed over)
    assert seen[0][5:] == (m.reparametrization_h, m.reparametrization_w, True, False, None)
    m.training = False
    m(torch.zeros(1, 1, 8, 8))
    assert len(calls) == n + 1                 # no clip in eval mode


def test_tensors_can_replace_parameters():
    """The reference's test swaps plain tensors in for the Parameters (test.py:162-165)."""
    m = BoxConv2d(1, 1, 8, 8)
    t = torch.full((1, 1), 0.01)
    del m.x_min
    m.x_min = t
    assert m.get_actual_parameters()[0].item() == pytest.approx(0.01 * 64)


def test_host_tensors_are_refused():
    x = torch.zeros(1, 1, 4, 4)
    with pytest.raises(RuntimeError, match="no CPU path"):
        _native.integral_image(x)
    with pytest.raises(RuntimeError, match=">=2 dimensions"):
        _native.integral_image(torch.zeros(3))
    z = torch.zeros(1, 1)
    with pytest.raises(RuntimeError, match="no CPU path"):
        _native.box_convolution_forward(torch.zeros(1, 1, 5, 5), z, z, z, z, True, True)
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="no CPU path"):
            BoxConv2d(1, 1, 8, 8).eval()
        with pytest.raises(RuntimeError):
            BoxConv2d(1, 1, 8, 8)(x)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "LIB_PATH", str(tmp_path / "libboxconv_hip.so"))
    with pytest.raises(RuntimeError, match="is missing; build it"):
        _native.load()


def test_native_module_stand_in():
    import box_convolution_cpp_cuda as cpp
    for name in ("integral_image", "box_convolution_forward", "box_convolution_backward", "clip_parameters"):
        assert callable(getattr(cpp, name))


def test_baseline_workloads_are_reproducible():
    from baseline_workloads import algorithmic_bytes, make_workload
    a, b = make_workload(1), make_workload(1)
    assert torch.equal(a.x, b.x) and torch.equal(a.x_min, b.x_min) and a.x.shape == (32, 1, 28, 28)
    sub = make_workload(2, in_planes=3)
    full = make_workload(2)
    assert torch.equal(sub.x, full.x[:, :3]) and torch.equal(sub.y_max, full.y_max[:3])
    assert torch.equal(sub.grad_output, full.grad_output.view(4, 32, 4, 128, 256)[:, :3].reshape(4, 12, 128, 256))
    assert algorithmic_bytes(2, 16, 8, 512, 1024)["alg"] == 2486765952
    assert algorithmic_bytes(2, 16, 8, 512, 1024)["io"] == 1207959552


def test_draw_boxes_canvas_and_rectangles():
    """draw_boxes: canvas, centre lines, colour and geometry rules of the reference
    (box_convolution_module.py:99-181); the rasteriser is numpy instead of OpenCV."""
    m = BoxConv2d(2, 3, 20, 40)
    with torch.no_grad():
        for p, v in zip((m.x_min, m.x_max, m.y_min, m.y_max), (-5.0, 4.0, -10.0, 9.0)):
            p.fill_(v)
        m.x_min /= m.reparametrization_h; m.x_max /= m.reparametrization_h
        m.y_min /= m.reparametrization_w; m.y_max /= m.reparametrization_w
    img = m.draw_boxes(resolution=(200, 400))
    assert img.shape == (200, 400, 3) and img.dtype == np.uint8
    assert tuple(img[100, 0]) == (70, 70, 70) and tuple(img[0, 200]) == (70, 70, 70)
    # box rows -5 .. 4+1 of 20 -> 100 + (-5, 5) / 20 * 100 = 75, 125; columns 200 + (-10, 10) / 40 * 200
    color = (0, 255, 0)                              # several channels: colour of the last channel drawn
    for r, c in ((75, 150), (75, 250), (125, 150), (125, 250), (75, 200), (100, 150)):
        assert tuple(img[r, c]) == color, (r, c)
    assert tuple(img[90, 180]) == (0, 0, 0)          # inside the outline: untouched
    # one channel: colour per filter, weights darken, a box with min > max is filled
    with torch.no_grad():
        m.x_max[0, 2] = m.x_min[0, 2] - 4.0 / m.reparametrization_h
    w = torch.tensor([[1.0, 0.5, 1.0]])
    one = m.draw_boxes(channels=[0], resolution=(200, 400), weights=w)
    assert tuple(one[68, 220]) == (0, 0, 255)        # filter 2 (blue), filled between rows 60 and 75
    assert tuple(one[125, 200]) == (0, 127, 0)       # filter 1 (green) at half weight, bottom edge
    assert m.draw_boxes().shape == (600, 600, 3)
