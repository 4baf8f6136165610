"""The native calls under HIP graph capture: nothing in the library allocates, synchronises or
clears memory with a memset node, so integral image + forward + backward can be captured once and
replayed. Every replay is checked against the eager result for fresh inputs, with the program's
own eager work and synchronisations between the replays."""
import numpy as np
import pytest
import torch

from helpers import make_boxes

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [(2, 3, 4, 70, 130), (1, 2, 2, 96, 1024)])
def test_captured_step_replays_identically(hip, shape):
    B, C, F, h, w = shape
    rng = np.random.default_rng(B * 1000 + w)
    boxes = [torch.from_numpy(b).cuda() for b in make_boxes(rng, C, F, h, w, "hanging")]

    def step(x, g):
        integ = hip.integral_image(x)
        out = hip.box_convolution_forward(integ, *boxes, True, True)
        grads = hip.box_convolution_backward(integ, *boxes, g, out, 9.0, 7.0, True, True,
                                             True, True, True, True, True)
        return [out] + list(grads)

    static_x = torch.randn(B, C, h, w, device="cuda")
    static_g = torch.randn(B, C * F, h, w, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                       # warm-up outside the capture
        step(static_x, static_g)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = step(static_x, static_g)

    for _ in range(4):
        x = torch.randn_like(static_x)
        g = torch.randn_like(static_g)
        want = step(x, g)                               # eager work between the replays
        torch.cuda.synchronize()
        static_x.copy_(x)
        static_g.copy_(g)
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip(static_out, want):
            assert torch.equal(got, ref)


def test_captured_training_step_replays_identically(hip):
    """The same for the one-call training forward (clip and the marking of the single-pass
    integral image's hand-over words in one launch, no memset) followed by the backward."""
    B, C, F, h, w = 2, 3, 4, 96, 256                    # 3 bands: the single-pass kernel runs
    rng = np.random.default_rng(7)
    real = [torch.from_numpy(b).cuda() for b in make_boxes(rng, C, F, h, w, "inside")]
    reparam_h, reparam_w = 2.5 * h, 2.5 * w
    stored = [p / s for p, s in zip(real, (reparam_h, reparam_h, reparam_w, reparam_w))]

    def step(x, g):
        params = [p.clone() for p in stored]
        integ, out, real_now = hip.training_forward(x, *params, reparam_h, reparam_w, h, w, True, True)
        grads = hip.box_convolution_backward(integ, *real_now, g, None, reparam_h, reparam_w, True,
                                             True, True, True, True, True, True)
        return [out, integ] + list(grads) + list(real_now) + params

    static_x = torch.randn(B, C, h, w, device="cuda")
    static_g = torch.randn(B, C * F, h, w, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(static_x, static_g)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = step(static_x, static_g)

    for _ in range(4):
        x = torch.randn_like(static_x)
        g = torch.randn_like(static_g)
        want = step(x, g)
        torch.cuda.synchronize()
        static_x.copy_(x)
        static_g.copy_(g)
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip(static_out, want):
            assert torch.equal(got, ref)


def test_module_under_make_graphed_callables():
    """torch.cuda.make_graphed_callables captures the module's forward and backward (autograd
    included) into HIP graphs; replays must give the bits of the eager step. Nothing in the path
    allocates outside torch's capture-safe allocator, synchronises or records a memset node."""
    import warnings
    from box_convolution import BoxConv2d
    import random
    dev = torch.device("cuda:0")

    def make():
        random.seed(5)
        return BoxConv2d(3, 4, 40, 96).to(dev).train()

    gen = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn(2, 3, 40, 96, device=dev, generator=gen).requires_grad_(True)
    g = torch.randn(2, 12, 40, 96, device=dev, generator=gen)
    eager = make()
    out = eager(x)
    out.backward(g)
    want = [out.detach().clone(), x.grad.clone()] + [p.grad.clone() for p in eager.parameters()]

    module = make()
    sample = torch.randn_like(x).requires_grad_(True)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        graphed = torch.cuda.make_graphed_callables(module, (sample,))
        for _ in range(3):
            x.grad = None
            for p in module.parameters():
                p.grad = None
            out = graphed(x)
            out.backward(g)
            torch.cuda.synchronize()
            got = [out.detach(), x.grad] + [p.grad for p in module.parameters()]
            for a, b in zip(want, got):
                assert torch.equal(a, b)
