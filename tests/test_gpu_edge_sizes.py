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


def _shifted(t, elems=1):
    """A contiguous copy of t whose first element sits `elems` elements past an aligned address."""
    flat = torch.empty(t.numel() + elems, device=t.device, dtype=t.dtype)
    out = flat[elems:].view_as(t)
    out.copy_(t)
    assert out.data_ptr() % 16 != 0 and out.is_contiguous()
    return out


@pytest.mark.parametrize("shape", [(2, 2, 3, 40, 256), (1, 2, 2, 33, 1024), (1, 1, 2, 70, 384), (2, 1, 4, 24, 64)])
def test_tensors_that_are_not_16_byte_aligned(hip, shape):
    """Inputs whose data pointers are only 4-byte aligned (views into a larger buffer): the vector
    loads must not be used on them. Same bits as with aligned tensors for the integral image and
    the forward pass; the backward is compared to a tight tolerance (its column workspace is
    private and aligned either way, only the loads of grad_output and of the integral differ; a
    grad_output that is not 16-byte aligned also takes the variant of the grad_output pass with
    wave-strided instead of consecutive columns per lane, whose float sums are associated
    differently)."""
    B, C, F, h, w = shape
    gen = torch.Generator(device="cuda").manual_seed(11)
    x = torch.randn(B, C, h, w, device="cuda", generator=gen)
    g = torch.randn(B, C * F, h, w, device="cuda", generator=gen)
    lo = -torch.rand(C, F, device="cuda", generator=gen) * 9 - 0.3
    hi = torch.rand(C, F, device="cuda", generator=gen) * 9 + 0.3
    boxes = (lo, hi, lo * 1.5, hi * 0.7)

    integ = hip.integral_image(x)
    integ_s = hip.integral_image(_shifted(x))
    assert torch.equal(integ, integ_s)
    out = hip.box_convolution_forward(integ, *boxes, True, True)
    out_s = hip.box_convolution_forward(_shifted(integ), *boxes, True, True)
    assert torch.equal(out, out_s)
    ref = hip.box_convolution_backward(integ, *boxes, g, None, 2.0, 3.0, True, True, True, True, True, True, True)
    got = hip.box_convolution_backward(_shifted(integ), *boxes, _shifted(g), None, 2.0, 3.0, True, True,
                                       True, True, True, True, True)
    torch.cuda.synchronize()
    for a, b in zip(ref, got):
        assert torch.allclose(a, b, rtol=1e-5, atol=4e-6 * float(a.abs().max()))
