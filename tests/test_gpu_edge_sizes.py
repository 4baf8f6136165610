"""Edge cases of size on the GPU: empty batches, and a single plane of more than 2 GiB (64-bit
offsets inside a plane, which only the gather kernels and the tiled integral image handle).

The large case is far beyond what the CPU oracle finishes in seconds, so it is checked through
closed forms that do not depend on the size: the integral image against a float64 cumulative sum
(torch's, on the device), a box of exactly one pixel ([0,0]x[0,0], area 1) reproduces its input in
the forward pass and passes grad_output through in the backward pass, and d/dbound sums are
compared with the same sums formed by torch from shifted copies of the tensors.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_empty_batch(hip):
    from box_convolution import BoxConv2d
    module = BoxConv2d(3, 2, 8, 9).cuda()
    x = torch.zeros(0, 3, 8, 9, device="cuda", requires_grad=True)
    out = module(x)
    assert out.shape == (0, 6, 8, 9)
    out.sum().backward()
    assert x.grad.shape == x.shape
    for p in module.parameters():
        assert p.grad is not None and torch.count_nonzero(p.grad).item() == 0
    integ = hip.integral_image(torch.zeros(0, 5, 7, device="cuda"))
    assert integ.shape == (0, 6, 8)


def test_single_plane_above_two_gib(hip):
    h = w = 23200                                   # 538 M elements, 2.15 GB per float32 tensor
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(5)
    x = torch.rand(1, 1, h, w, device=dev, generator=gen) - 0.5
    integ = hip.integral_image(x)
    assert integ.shape == (1, 1, h + 1, w + 1)
    # float64 cumulative sums of the last 2048 rows need the column totals of everything above:
    # take them from a float64 sum over the rows above (an independent reduction)
    top = x[0, 0, :h - 2048].sum(dim=0, dtype=torch.float64)
    tail = x[0, 0, h - 2048:].double().cumsum(dim=0) + top
    want = tail.cumsum(dim=1)
    got = integ[0, 0, h - 2048 + 1:, 1:].double()
    scale = want.abs().max().item()
    assert (got - want).abs().max().item() <= 1e-6 * scale
    assert torch.count_nonzero(integ[0, 0, 0]).item() == 0 and torch.count_nonzero(integ[0, 0, :, 0]).item() == 0
    del top, tail, want, got

    # a one-pixel box: forward is the identity up to the float32 rounding of the integral image
    # (entries up to `scale`, so a difference of four of them is good to a few ulps of that)
    z = torch.zeros(1, 1, device=dev)
    out = hip.box_convolution_forward(integ, z, z, z, z, True, True)
    ulp = scale * 2.0 ** -23
    assert (out - x).abs().max().item() <= 8 * ulp
    # backward: grad_input is grad_output (one filter); the parameter gradients of a one-pixel box
    # are sums of grad_output times the neighbouring pixel minus ... : compare grad_x_max, whose
    # derivative is the row below (fractional border row i+1): sum g[i,j] * x[i+1,j]
    g = torch.rand(1, 1, h, w, device=dev, generator=gen) - 0.5
    grads = hip.box_convolution_backward(integ, z, z, z, z, g, None, 1.0, 1.0, False, True,
                                         True, True, True, True, True)
    torch.cuda.synchronize()
    assert (grads[0] - g).abs().max().item() <= 8 * ulp
    want_xmax = (g[0, 0, :-1].double() * x[0, 0, 1:].double()).sum().item()
    want_xmin = -(g[0, 0, 1:].double() * x[0, 0, :-1].double()).sum().item()
    want_ymax = (g[0, 0, :, :-1].double() * x[0, 0, :, 1:].double()).sum().item()
    want_ymin = -(g[0, 0, :, 1:].double() * x[0, 0, :, :-1].double()).sum().item()
    noise = ulp * (h * w) ** 0.5 * 4               # random walk of per-pixel rounding errors
    for got_t, want_v, name in zip(grads[1:], (want_xmin, want_xmax, want_ymin, want_ymax),
                                   ("x_min", "x_max", "y_min", "y_max")):
        assert abs(got_t.item() - want_v) <= 1e-3 * abs(want_v) + noise, (name, got_t.item(), want_v)
