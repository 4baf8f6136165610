"""Forward with half-precision output and the fused tail (scale, shift, residual, ReLU).

The reference has no such function; what it computes is the reference's forward followed by
element-wise steps (how its BottleneckBoxConv ends in eval mode,
examples/Cityscapes/models/ENet.py:290-304). Expected values therefore come from the CPU oracle:
oracle integral image -> oracle forward -> scale / shift / residual / ReLU in float32 on the host
-> rounded to the output type on the host. Tolerances against the oracle: the forward's 1e-4 of the
largest entry, plus one unit in the last place of the half type for half-precision output. On top
of that the entry point is held much tighter to the library's own plain forward (a few float32
roundings; half precision: the float32 result rounded once), which pins the tail arithmetic itself.
"""
import numpy as np
import pytest
import torch

from box_convolution import BoxConv2d
from helpers import make_boxes

pytestmark = pytest.mark.gpu
DEV = "cuda"

# B, C, F, h, w: partial rows, full rows at 256 and 512 threads, three columns per lane, gather
SHAPES = [(2, 3, 4, 37, 53), (1, 2, 2, 64, 256), (1, 1, 2, 40, 1024), (1, 2, 1, 18, 1536),
          (1, 1, 1, 8, 2100), (3, 1, 5, 9, 64)]
HALF_ULP = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}


class OracleForward:
    """The reference's forward on the host for one test case (float32, numpy)."""

    def __init__(self, oracle, x, boxes):
        self.oracle = oracle
        self.boxes = boxes
        self.integ = oracle.integral_image(x)

    def __call__(self, normalize, exact):
        return self.oracle.box_forward(self.integ, *self.boxes, normalize, exact)


def setup_case(hip, shape, seed, kind="inside", oracle=None):
    B, C, F, h, w = shape
    rng = np.random.default_rng(seed)
    boxes_np = make_boxes(rng, C, F, h, w, kind)
    boxes = [torch.from_numpy(b).to(DEV) for b in boxes_np]
    g = torch.Generator(device="cpu").manual_seed(seed)
    x_host = torch.randn(B, C, h, w, generator=g)
    x = x_host.to(DEV)
    integ = hip.integral_image(x)
    scale = (torch.rand(C * F, generator=g) * 2 - 0.7).to(DEV)
    shift = torch.randn(C * F, generator=g).to(DEV)
    residual = torch.randn(B, C * F, h, w, generator=g).to(DEV)
    if oracle is None:
        return integ, boxes, scale, shift, residual
    return integ, boxes, scale, shift, residual, OracleForward(oracle, x_host.numpy(), boxes_np)


def compose_host(plain, scale, shift, residual, relu):
    """The tail in float32 on the host: numpy in, numpy out."""
    y = plain.astype(np.float32)
    if scale is not None:
        y = y * scale.cpu().numpy()[None, :, None, None]
    if shift is not None:
        y = y + shift.cpu().numpy()[None, :, None, None]
    if residual is not None:
        y = y + residual.float().cpu().numpy()
    return np.maximum(y, 0) if relu else y


def to_half_on_host(a, dtype):
    """float32 numpy -> torch tensor of a half type, rounded to nearest even on the host."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dtype)


def compose(plain, scale, shift, residual, relu):
    y = plain
    if scale is not None:
        y = y * scale[None, :, None, None]
    if shift is not None:
        y = y + shift[None, :, None, None]
    if residual is not None:
        y = y + residual
    return torch.relu(y) if relu else y


@pytest.mark.parametrize("exact", [True, False])
@pytest.mark.parametrize("shape", SHAPES)
def test_fused_tail_float32(hip, oracle, shape, exact):
    integ, boxes, scale, shift, residual, ref = setup_case(hip, shape, 11, oracle=oracle)
    plain = hip.box_convolution_forward(integ, *boxes, True, exact)
    plain_c = ref(True, exact)
    # nothing to fuse: the very same numbers as the plain entry point, and the oracle's to 1e-4
    assert torch.equal(hip.box_convolution_forward_fused(integ, *boxes, True, exact), plain)
    assert np.abs(plain.cpu().numpy() - plain_c).max() <= 1e-4 * np.abs(plain_c).max()
    for use_scale, use_shift, use_res, relu in [(1, 1, 1, 1), (1, 0, 0, 0), (0, 1, 0, 0), (0, 0, 1, 0),
                                                (0, 0, 0, 1), (1, 1, 0, 1), (0, 0, 1, 1)]:
        args = (scale if use_scale else None, shift if use_shift else None,
                residual if use_res else None, bool(relu))
        got = hip.box_convolution_forward_fused(integ, *boxes, True, exact, torch.float32, *args)
        want = compose(plain, *args)
        # sizes of the terms that get rounded
        mag = (plain.abs() * (scale.abs().max() if use_scale else 1)).max().item() + 4.0
        assert (got - want).abs().max().item() <= 4e-7 * mag, (use_scale, use_shift, use_res, relu)
        # against the oracle's forward with the tail applied on the host
        want_c = compose_host(plain_c, *args)
        assert np.abs(got.cpu().numpy() - want_c).max() <= 1e-4 * mag, (use_scale, use_shift, use_res, relu)
        if relu:
            assert got.min().item() >= 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_half_precision_output(hip, oracle, shape, dtype):
    integ, boxes, scale, shift, residual, ref = setup_case(hip, shape, 23, kind="hanging", oracle=oracle)
    for normalize in (True, False):
        plain = hip.box_convolution_forward(integ, *boxes, normalize, True)
        got = hip.box_convolution_forward_fused(integ, *boxes, normalize, True, dtype)
        assert got.dtype == dtype and got.shape == plain.shape
        # against the oracle's forward rounded to the half type on the host: the forward's 1e-4
        # of the largest entry plus one unit in the last place of the half type
        plain_c = ref(normalize, True)
        want_c = to_half_on_host(plain_c, dtype).float().numpy()
        ok = np.isfinite(want_c)
        assert np.array_equal(np.isfinite(got.float().cpu().numpy()), ok)
        err = np.abs(got.float().cpu().numpy()[ok] - plain_c[ok])
        assert np.all(err <= HALF_ULP[dtype] * np.abs(plain_c[ok]) + 1e-4 * np.abs(plain_c[ok]).max())
        # (float16 overflows to inf where the unnormalized sums exceed 65504, as .to() does)
        want = plain.to(dtype)
        # The kernel may round the product sum * (1/area) to the half type in one step
        # (mixed-precision multiply); where the float32 product is a tie between two half
        # values that differs from rounding twice, and is then the closer one.
        assert (got != want).float().mean().item() < 1e-3
        finite = want.float().isfinite()
        assert torch.equal(got.float().isfinite(), finite)
        assert torch.all(((got.float() - plain).abs() <= (want.float() - plain).abs() * (1 + 1e-6))[finite])
    plain = hip.box_convolution_forward(integ, *boxes, True, True)
    res16 = residual.to(dtype)
    got = hip.box_convolution_forward_fused(integ, *boxes, True, True, dtype, scale, shift, res16, True)
    want = compose(plain, scale, shift, res16.float(), True)
    err = (got.float() - want).abs()
    bound = HALF_ULP[dtype] * want.abs().clamp_min(2.0 ** -14) + 1e-6
    assert torch.all(err <= bound)
    # and nearly all entries are the correctly rounded value of the float32 composition
    assert (got != want.to(dtype)).float().mean().item() < 0.02
    # the same against the oracle: forward on the host, tail on the host, rounded on the host
    want_c = compose_host(ref(True, True), scale, shift, res16, True)
    mag = (np.abs(ref(True, True)).max() * scale.abs().max().item()) + 4.0
    err_c = np.abs(got.float().cpu().numpy() - want_c)
    assert np.all(err_c <= HALF_ULP[dtype] * np.abs(want_c) + 1e-4 * mag)
    assert (got.cpu() != to_half_on_host(want_c, dtype)).float().mean().item() < 0.05


# planes, h, w: single pass (full rows), two passes (partial rows, vector and element loads),
# one band, 64 bands, wider than the direct path reads
HALF_INTEGRAL_SHAPES = [(3, 96, 256), (2, 130, 1024), (2, 70, 2048), (3, 200, 36), (1, 300, 1023),
                        (2, 100, 1000), (5, 9, 17), (40, 33, 257), (1, 2048, 64), (1, 12, 2500)]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("planes,h,w", HALF_INTEGRAL_SHAPES)
def test_integral_image_of_half_precision_input(hip, switches, planes, h, w, dtype):
    """float32 integral image straight from float16 / bfloat16: the same bits as converting the
    input to float32 first (which is pinned against the oracle in test_gpu_parity.py)."""
    x = (torch.randn(planes, h, w, device=DEV) * 3 + 0.5).to(dtype)
    want = hip.integral_image(x.float())
    got = hip.integral_image(x)
    assert got.dtype == torch.float32 and torch.equal(got, want)
    # an odd start address (no 8-byte alignment): element-wise loads
    flat = torch.empty(x.numel() + 1, device=DEV, dtype=dtype)
    shifted = flat[1:].view_as(x).copy_(x)
    assert shifted.data_ptr() % 8 != 0 and torch.equal(hip.integral_image(shifted), want)
    switches("BOXCONV_INTEGRAL_LOOKBACK", "2")     # single pass wherever it applies
    assert torch.equal(hip.integral_image(x), hip.integral_image(x.float()))


def test_argument_checks(hip):
    integ, boxes, scale, shift, residual = setup_case(hip, (1, 2, 2, 8, 8), 3)
    with pytest.raises(RuntimeError, match="float32 integral image"):
        hip.box_convolution_forward_fused(integ.double(), *boxes, True, True)
    with pytest.raises(RuntimeError, match="float32, float16 or bfloat16"):
        hip.box_convolution_forward_fused(integ, *boxes, True, True, torch.float64)
    with pytest.raises(RuntimeError, match="must hold 4 values"):
        hip.box_convolution_forward_fused(integ, *boxes, True, True, torch.float32, scale[:3])
    with pytest.raises(RuntimeError, match="shape of the output"):
        hip.box_convolution_forward_fused(integ, *boxes, True, True, torch.float32, None, None,
                                          residual[:, :3])


def make_module(C, F, h, w, seed):
    import random
    random.seed(seed)
    return BoxConv2d(C, F, h, w).to(DEV)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def oracle_module_forward(oracle, m, x_host):
    """The reference's BoxConv2d.forward on the host for module `m` (its stored parameters)."""
    stored = [p.detach().cpu().numpy() for p in (m.x_min, m.x_max, m.y_min, m.y_max)]
    out, _ = oracle.module_forward(np.ascontiguousarray(x_host, dtype=np.float32), *stored,
                                   m.reparametrization_h, m.reparametrization_w, m.normalize, m.exact)
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_module_takes_half_precision_input(oracle, dtype):
    m = make_module(3, 4, 40, 72, 5).eval()
    x = torch.randn(2, 3, 40, 72, device=DEV).to(dtype)
    with torch.no_grad():
        got = m(x)
        want = m(x.float())
    assert got.dtype == dtype and (got != want.to(dtype)).float().mean().item() < 1e-3
    assert torch.allclose(got.float(), want, rtol=HALF_ULP[dtype], atol=1e-7)
    # the oracle on the same (half-precision) input values, rounded to the half type on the host
    want_c = oracle_module_forward(oracle, m, x.float().cpu().numpy())
    err = np.abs(got.float().cpu().numpy() - want_c)
    assert np.all(err <= HALF_ULP[dtype] * np.abs(want_c) + 1e-4 * np.abs(want_c).max())
    # with autograd: float32 in between, gradients come back in the input's type
    m.train()
    xg = x.clone().requires_grad_(True)
    out = m(xg)
    assert out.dtype == dtype and out.requires_grad
    go = torch.randn_like(out)
    out.backward(go)
    x32 = x.float().requires_grad_(True)
    ref_grads = torch.autograd.grad(m(x32), [x32, m.x_min, m.y_max], go.float())
    assert xg.grad.dtype == dtype
    assert torch.allclose(xg.grad.float(), ref_grads[0], rtol=2 * HALF_ULP[dtype], atol=1e-3)
    assert torch.allclose(m.x_min.grad, ref_grads[1], rtol=1e-4, atol=1e-4 * ref_grads[1].abs().max().item())
    assert torch.allclose(m.y_max.grad, ref_grads[2], rtol=1e-4, atol=1e-4 * ref_grads[2].abs().max().item())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_bottleneck_tail_in_one_launch(oracle, dtype):
    """BoxConv2d -> BatchNorm2d -> Dropout2d -> + x -> ReLU in eval mode, as the reference's
    BottleneckBoxConv ends (ENet.py:290-304), against the same chain of torch modules."""
    C, F, h, w = 4, 4, 32, 64
    m = make_module(C, F, h, w, 9).eval()
    bn = torch.nn.BatchNorm2d(C * F).to(DEV)
    with torch.no_grad():
        bn.running_mean.normal_()
        bn.running_var.uniform_(0.5, 2.0)
        bn.weight.normal_()
        bn.bias.normal_()
    bn.eval()
    drop = torch.nn.Dropout2d(0.25).eval()
    x = torch.randn(2, C, h, w, device=DEV)
    skip = torch.randn(2, C * F, h, w, device=DEV).to(dtype)
    with torch.no_grad():
        want = torch.relu(skip.float() + drop(bn(m(x))))
        scale, shift = BoxConv2d.fold_batch_norm(bn)
        got = m.forward_fused(x.to(dtype), scale, shift, skip, relu=True)
        want_in = torch.relu(skip.float() + drop(bn(m(x.to(dtype).float()))))
    assert got.dtype == dtype
    if dtype == torch.float32:
        assert torch.allclose(got, want, rtol=1e-5, atol=1e-5)
    else:
        assert torch.all((got.float() - want_in).abs() <= HALF_ULP[dtype] * want_in.abs() + 1e-5)
    # the oracle's box convolution, then BatchNorm (eval) + residual + ReLU written out on the host
    conv_c = oracle_module_forward(oracle, m, x.to(dtype).float().cpu().numpy())
    g, b = bn.weight.detach().cpu().numpy(), bn.bias.detach().cpu().numpy()
    mu, var = bn.running_mean.cpu().numpy(), bn.running_var.cpu().numpy()
    y = (conv_c - mu[None, :, None, None]) / np.sqrt(var + bn.eps)[None, :, None, None]
    want_c = np.maximum(y * g[None, :, None, None] + b[None, :, None, None] + skip.float().cpu().numpy(), 0)
    err = np.abs(got.float().cpu().numpy() - want_c)
    ulp = HALF_ULP[dtype] if dtype != torch.float32 else 0.0
    assert np.all(err <= ulp * np.abs(want_c) + 1e-4 * (np.abs(want_c).max() + 4.0))


def test_forward_fused_modes_and_double_input():
    """forward_fused follows the module's normalize / exact switches and takes float64 input
    (integrated in float32, as the entry point works on a float32 integral image)."""
    m = make_module(2, 3, 24, 40, 21).eval()
    x = torch.randn(2, 2, 24, 40, device=DEV)
    for normalize, exact in ((True, True), (False, True), (True, False), (False, False)):
        m.normalize, m.exact = normalize, exact
        with torch.no_grad():
            want = m(x)
        assert torch.equal(m.forward_fused(x), want)
        got = m.forward_fused(x.double(), output_dtype=torch.float32)
        assert torch.allclose(got, want, rtol=1e-5, atol=1e-5)
    assert not m.forward_fused(x).requires_grad
