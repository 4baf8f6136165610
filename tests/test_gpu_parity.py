"""HIP kernels vs the CPU oracle on identical seeded inputs, through the C ABI (ctypes).

Tolerances: forward and grad_input max|gpu-cpu|/max|cpu| <= 1e-4, box-parameter gradients <= 1e-3
for float32 (the targets the build is held to); 1e-9 for float64.
"""
import os

import numpy as np
import pytest
import torch

from helpers import make_boxes, param_grad_floor, rel_err

pytestmark = pytest.mark.gpu

TOL = {np.float32: (1e-4, 1e-3), np.float64: (1e-9, 1e-9)}


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


# planes, h, w: chosen to hit one band / several bands, one wave / four waves, vector / scalar
# loads, several column tiles.
INTEGRAL_SHAPES = [
    (1, 2, 2), (3, 5, 7), (2, 10, 10), (6, 28, 28), (1, 33, 257), (2, 64, 128), (1, 200, 36),
    (1, 300, 1023), (2, 130, 1024), (1, 70, 2048), (1, 40, 2500), (1, 36, 4100), (1, 9, 9000),
    (2, 100, 4096), (1, 170, 3000),                     # sixteen waves per row, several bands
    (5, 1, 1), (2, 1, 300), (2, 300, 1),
    # single-pass kernel: many bands, partial last band, 64 bands, one band too many for it
    (3, 512, 1000), (1, 2048, 64), (1, 2100, 40), (40, 100, 520), (9, 97, 1536),
]


# (the single-pass kernel is float32 only)
@pytest.mark.parametrize("dtype,single_pass", [(np.float32, "where_faster"), (np.float64, "where_faster"),
                                               (np.float32, "wherever_possible")])
@pytest.mark.parametrize("planes,h,w", INTEGRAL_SHAPES)
def test_integral_image(hip, oracle, switches, planes, h, w, dtype, single_pass):
    if single_pass == "wherever_possible":
        # by default that kernel serves only the shapes it is faster on; reach the others too
        switches("BOXCONV_INTEGRAL_LOOKBACK", "2")
    rng = np.random.default_rng(planes * 1000003 + h * 1009 + w)
    x = (rng.random((planes, h, w)) * 2 - 0.5).astype(dtype)
    got = host(hip.integral_image(dev(x)))
    want = oracle.integral_image(x)
    assert got.shape == want.shape
    # closed form: float64 cumulative sums (the reference's own test oracle, test.py:12-35)
    exact = np.zeros((planes, h + 1, w + 1))
    exact[:, 1:, 1:] = x.astype(np.float64).cumsum(1).cumsum(2)
    assert np.all(got[:, 0, :] == 0) and np.all(got[:, :, 0] == 0)
    tol = 1e-6 if dtype == np.float32 else 1e-13
    assert rel_err(got, exact) <= tol
    assert rel_err(got, want) <= 10 * tol
    if dtype == np.float32:
        # sums are carried in double and rounded once: (almost) every entry is the correctly
        # rounded exact sum, and none is off by more than one unit in the last place
        ideal = exact.astype(np.float32)
        assert np.mean(got != ideal) < 1e-4
        assert np.all(np.abs(got - ideal) <= np.spacing(np.abs(ideal)))


@pytest.mark.parametrize("planes,h,w", [(1, 33, 257), (3, 200, 36), (2, 130, 1024), (2, 512, 1000),
                                        (1, 2048, 64), (17, 96, 2048)])
def test_integral_image_single_pass_waits_are_bounded(hip, switches, planes, h, w):
    """The single-pass kernel waits a bounded number of polls for the bands above; a band whose
    flag is still down is summed from the input instead. With a limit of zero polls every band
    goes that way, and the result is the same bit for bit. So is the three-launch path's."""
    x = torch.from_numpy(np.random.default_rng(h * w).random((planes, h, w), dtype=np.float32) - 0.3).cuda()
    switches("BOXCONV_INTEGRAL_LOOKBACK", "2")       # single pass for every shape it covers
    usual = hip.integral_image(x)
    for limit in ("0", "1", "2"):     # never wait / give up at once: a mix of both ways per launch
        switches("BOXCONV_INTEGRAL_SPIN", limit)
        assert torch.equal(hip.integral_image(x), usual)
    switches("BOXCONV_INTEGRAL_SPIN", None)
    switches("BOXCONV_INTEGRAL_LOOKBACK", "0")       # same bands, three launches
    three = hip.integral_image(x)
    switches("BOXCONV_INTEGRAL_LOOKBACK", None)
    # (the default may cut the planes into different bands: same sums, associated differently)
    assert torch.allclose(three, usual, rtol=2e-7, atol=0) and torch.allclose(hip.integral_image(x), usual, rtol=2e-7, atol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("planes,h,w", [(5, 1, 1), (3, 5, 7), (6, 28, 28), (2, 64, 128), (40, 64, 128), (3, 8, 256),
                                        (2, 9, 255), (4, 57, 100), (3, 128, 256), (2, 129, 33), (7, 135, 240),
                                        (2, 192, 256), (3, 191, 254), (2, 170, 3), (1, 100, 253)])
def test_integral_image_plane_per_workgroup(hip, switches, planes, h, w, dtype):
    """Planes of at most 192 rows and 256 columns are scanned by one workgroup each (a wave per
    band of 8 to 24 rows, the bands' column sums handed over through LDS);
    BOXCONV_INTEGRAL_PLANE=0 sends them through the launches that larger planes take (other bands:
    the same sums, associated differently). Both against float64 cumulative sums."""
    x = torch.from_numpy(np.random.default_rng(planes + 7 * h + 1000 * w).random((planes, h, w), dtype=np.float32)
                         * 4 - 1).cuda().to(dtype)
    exact = torch.zeros(planes, h + 1, w + 1, dtype=torch.float64, device="cuda")
    exact[:, 1:, 1:] = x.double().cumsum(1).cumsum(2)
    got = hip.integral_image(x)
    assert got.dtype == torch.float32 and got.shape == exact.shape
    ideal = exact.float()
    assert torch.all((got - ideal).abs() <= torch.from_numpy(np.spacing(np.abs(ideal.cpu().numpy()))).cuda())
    assert (got != ideal).float().mean().item() < 1e-4
    switches("BOXCONV_INTEGRAL_PLANE", "0")
    two_launches = hip.integral_image(x)
    switches("BOXCONV_INTEGRAL_PLANE", None)
    assert torch.allclose(got, two_launches, rtol=2e-7, atol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("planes,h,w", [(3, 28, 28), (5, 64, 128), (2, 100, 64), (4, 33, 256), (3, 64, 1024), (2, 40, 2048)])
def test_integral_image_of_a_misaligned_tensor(hip, planes, h, w, dtype):
    """A contiguous tensor whose first element is not 16-byte aligned (a view into a larger
    buffer) takes the kernels' element-wise loads instead of the 16-byte ones, and small planes
    other bands; the sums are the same."""
    for shift in (1, 3):
        flat = torch.randn(planes * h * w + shift, device="cuda").to(dtype)
        x = flat[shift:].view(planes, h, w)
        assert x.is_contiguous() and x.data_ptr() % 16 != 0
        assert torch.allclose(hip.integral_image(x), hip.integral_image(x.clone()), rtol=2e-7, atol=0)


INT_TYPES = [(np.uint8, torch.uint8), (np.int8, torch.int8), (np.int16, torch.int16),
             (np.int32, torch.int32), (np.int64, torch.int64)]


@pytest.mark.parametrize("np_dtype,torch_dtype", INT_TYPES)
@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 5, 7), (2, 33, 257), (1, 70, 2500), (2, 2, 130, 1024), (1, 300, 3)])
def test_integral_image_of_integer_tensors(hip, oracle, shape, np_dtype, torch_dtype):
    """Integer tensors (src/integral_image.cpp:14): bit-exact against the oracle and against
    numpy's wrapping cumulative sums, with values over the type's full range."""
    rng = np.random.default_rng(sum(shape) + np.dtype(np_dtype).itemsize)
    info = np.iinfo(np_dtype)
    x = rng.integers(info.min, info.max, size=shape, dtype=np_dtype, endpoint=True)
    got = hip.integral_image(torch.from_numpy(x).cuda())
    assert got.dtype == torch_dtype and tuple(got.shape) == shape[:-2] + (shape[-2] + 1, shape[-1] + 1)
    got = got.cpu().numpy()
    want = np.zeros(got.shape, dtype=np_dtype)
    want[..., 1:, 1:] = x.cumsum(-2, dtype=np_dtype).cumsum(-1, dtype=np_dtype)
    assert np.array_equal(got, oracle.integral_image(x))
    assert np.array_equal(got, want)


def test_integral_image_leading_dims(hip, oracle):
    x = np.random.default_rng(5).random((2, 3, 2, 17, 19)).astype(np.float32)
    got = host(hip.integral_image(dev(x)))
    assert got.shape == (2, 3, 2, 18, 20)
    assert rel_err(got, oracle.integral_image(x)) <= 1e-6
    x2 = np.random.default_rng(6).random((17, 19)).astype(np.float32)
    assert rel_err(host(hip.integral_image(dev(x2))), oracle.integral_image(x2)) <= 1e-6


def run_both(hip, oracle, x, boxes, reparam_h, reparam_w, normalize, exact, grad_out,
             needs=(True,) * 5):
    """Forward + backward of the native functions on both sides, parameters in real units."""
    integ_cpu = oracle.integral_image(x)
    out_cpu = oracle.box_forward(integ_cpu, *boxes, normalize, exact)
    back_cpu = oracle.box_backward(integ_cpu, *boxes, grad_out, out_cpu, reparam_h, reparam_w,
                                   normalize, exact, needs)
    integ = hip.integral_image(dev(x))
    b = [dev(p) for p in boxes]
    out = hip.box_convolution_forward(integ, *b, normalize, exact)
    back = hip.box_convolution_backward(integ, *b, dev(grad_out), out, reparam_h, reparam_w,
                                        normalize, exact, *needs)
    torch.cuda.synchronize()
    scales = dict(i_max=float(np.abs(integ_cpu).max()),
                  gi_max=float(np.abs(oracle.integral_image(grad_out)).max()),
                  pg_scale=float(np.abs(integ_cpu).max() * np.abs(grad_out).max()
                                 * max(abs(reparam_h), abs(reparam_w))
                                 * np.sqrt(grad_out.shape[-1] * grad_out.shape[-2])) if grad_out.size else 0.0)
    return (out_cpu, back_cpu), (host(out), [None if g is None else host(g) for g in back]), scales


# comparisons made by assert_parity in this process, and how many of them passed only thanks to
# the additive noise term or the sibling-tensor scale (see its docstring)
NOISE_STATS = {"comparisons": 0, "needed_noise_term": 0, "of_those_reference_all_zero": 0,
               "worst_ratio": 0.0, "worst_case": ""}


def assert_parity(cpu, gpu, dtype, what="", i_max=0.0, gi_max=0.0, pg_scale=0.0):
    """max|gpu-cpu| <= tol * scale + rounding noise, per tensor.

    forward / grad_input: scale = max|cpu|, noise = 8 eps * (largest integral-image entry): every
    output is a difference of integral-image entries, each known to half a unit in its last place;
    it only matters for tensors that are (nearly) zero, e.g. a box that misses the image.
    i_max / gi_max: largest |entry| of the integral image of the input / of grad_output.

    Parameter gradients: scale = max(max|cpu|, 1e-2 * largest of the four tensors), noise =
    eps * pg_scale with pg_scale = i_max * max|grad_output| * reparametrization * sqrt(h*w). They
    are sums over all pixels of grad_output times differences of integral-image entries, scaled
    by the reparametrization factor, so the float32 reference itself carries a random-walk error
    of that order (checked against the float64 oracle: e.g. input mean 3, 65x1535, whole-pixel
    boxes: the float32 CPU result is off by 0.55 %, the GPU result by 0.09 %); for boxes that miss
    the image the true gradients are exactly zero and the reference returns pure noise."""
    tol_f, tol_p = TOL[dtype]
    eps = float(np.finfo(dtype).eps)
    (out_c, back_c), (out_g, back_g) = cpu, gpu

    def close(got, want, tol, atol, name, scale_floor=0.0, magnitude=0.0):
        want = np.asarray(want, dtype=np.float64)
        diff = np.abs(np.asarray(got, dtype=np.float64) - want).max() if want.size else 0.0
        own_scale = np.abs(want).max() if want.size else 0.0
        ok = diff <= tol * max(own_scale, scale_floor) + atol
        # bookkeeping: how often the plain bound (tol * max|cpu| of the tensor itself) would not
        # have been enough; printed at the end of the run
        NOISE_STATS["comparisons"] += 1
        if ok and diff > tol * own_scale:
            NOISE_STATS["needed_noise_term"] += 1
            # a reference tensor a million times smaller than what it is made of (the integral
            # image for forward / grad_input; for a parameter gradient the largest sibling, or the
            # size of the sums it is a difference of) counts as zero: it lies below the float32
            # resolution of those sums, its entries are the reference's own rounding noise
            negligible = own_scale <= 1e-6 * magnitude
            NOISE_STATS["of_those_reference_all_zero"] += int(negligible)
            # how far beyond the plain bound the others sit: diff / (tol * max|cpu|)
            if not negligible and diff / (tol * own_scale) > NOISE_STATS["worst_ratio"]:
                NOISE_STATS["worst_ratio"] = diff / (tol * own_scale)
                NOISE_STATS["worst_case"] = "%s %s %s, max|cpu| %.3g, diff %.3g" % (
                    what, name, np.dtype(dtype).name, own_scale, diff)
        return ok

    assert close(out_g, out_c, tol_f, 8 * eps * i_max, "forward", magnitude=i_max), what + " forward"
    if back_c[0] is not None:
        assert close(back_g[0], back_c[0], tol_f, 8 * eps * gi_max, "grad_input", magnitude=gi_max), what + " grad_input"
    floor = param_grad_floor(back_c[1:])
    for k, name in enumerate(("x_min", "x_max", "y_min", "y_max")):
        if back_c[1 + k] is not None:
            assert close(back_g[1 + k], back_c[1 + k], tol_p, eps * pg_scale, "grad_" + name, floor, max(100 * floor, pg_scale)), what + " grad_" + name


SMALL_CASES = [
    # B, C, F, h, w
    (1, 1, 1, 2, 2), (1, 1, 1, 5, 9), (2, 3, 2, 7, 6), (1, 2, 3, 10, 10), (2, 1, 5, 28, 28),
    (1, 2, 2, 17, 65), (1, 1, 3, 40, 130), (1, 2, 2, 33, 300), (1, 1, 2, 20, 600),
    (1, 1, 2, 12, 1100), (1, 1, 1, 9, 2100), (1, 1, 2, 1, 1), (1, 1, 2, 1, 70), (1, 1, 2, 70, 1),
    (1, 1, 2, 12, 700), (1, 2, 1, 10, 768), (1, 1, 2, 11, 1300), (1, 1, 1, 9, 1536),   # three columns per lane
    (1, 1, 2, 40, 2048), (1, 2, 2, 21, 1800), (1, 1, 1, 10, 2047),      # 512 threads, four columns per lane
    # the same shape with an even number of row pairs per band (a band then ends in the second LDS
    # buffer; float64 in rounded mode once returned wrong parameter gradients exactly there)
    (1, 1, 2, 4, 1538), (2, 1, 3, 32, 1537), (1, 1, 4, 8, 1800), (1, 1, 2, 16, 2047), (1, 1, 2, 12, 1300),
    # narrow images with four filters or more: the waves of a grad-input workgroup share the
    # filters (one turn with idle waves, two turns with the second partial, full-width rows)
    (1, 2, 4, 9, 20), (1, 2, 11, 19, 33), (2, 1, 16, 12, 64),
    (1, 2, 2, 12, 128), (1, 1, 3, 35, 100),          # two waves per row, full and partial
    # the same sharing of filters for rows of two and four waves
    (1, 2, 5, 20, 100), (1, 1, 6, 12, 128), (1, 1, 4, 20, 200), (1, 2, 7, 9, 256),
    # one and two waves with three or four columns per lane (rows of 129 to 512 columns), rows that
    # fill the workgroup's column slots exactly and rows that do not
    (1, 2, 2, 14, 192), (1, 1, 2, 13, 150), (2, 1, 2, 10, 384), (1, 1, 3, 9, 512), (1, 1, 2, 11, 500),
    (1, 2, 1, 16, 257),
    # rows of 2049 to 4096 columns: 1024 threads, three or four columns per lane (float32; float64
    # rows this wide and anything wider take the gather kernels)
    (1, 1, 1, 8, 3072), (1, 2, 1, 7, 4096), (1, 1, 2, 6, 3500), (1, 1, 1, 5, 2049), (1, 1, 1, 5, 4100),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("kind", ["inside", "hanging", "integer"])
@pytest.mark.parametrize("B,C,F,h,w", SMALL_CASES)
def test_forward_backward_small(hip, oracle, B, C, F, h, w, kind, dtype):
    seed = (B * 7 + C * 11 + F * 13 + h * 17 + w * 19) * 3 + len(kind)
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((B, C, h, w)).astype(dtype)
    g = rng.standard_normal((B, C * F, h, w)).astype(dtype)
    boxes = make_boxes(rng, C, F, max(h, 4), max(w, 4), kind, dtype)
    for normalize in (True, False):
        for exact in (True, False):
            if not exact:
                # rounded mode needs boxes at least one whole pixel thick to have a finite area
                bx = list(boxes)
                bx[1] = (np.maximum(bx[1], np.ceil(bx[0]) + 1)).astype(dtype)
                bx[3] = (np.maximum(bx[3], np.ceil(bx[2]) + 1)).astype(dtype)
                use = tuple(bx)
            else:
                use = boxes
            cpu, gpu, sc = run_both(hip, oracle, x, use, 3.5 * h, 2.25 * w, normalize, exact, g)
            assert_parity(cpu, gpu, dtype, "%s normalize=%s exact=%s" % (kind, normalize, exact), **sc)


@pytest.mark.parametrize("kind", ["inside", "hanging", "inverted"])
@pytest.mark.parametrize("h,w", [(150, 90), (257, 256), (97, 520), (140, 400), (131, 170), (100, 2600), (3000, 40)])
def test_backward_across_row_bands(hip, oracle, h, w, kind):
    """Images tall enough that the backward pass cuts grad_output into several row bands, with
    boxes whose top and bottom rows fall into different bands; 'inverted' boxes have min > max
    along the rows (their bottom rows lie above their top rows)."""
    rng = np.random.default_rng(h * 1000 + w + len(kind))
    B, C, F = 1, 2, 3
    x = rng.standard_normal((B, C, h, w)).astype(np.float32)
    g = (rng.standard_normal((B, C * F, h, w)) + 0.5).astype(np.float32)
    boxes = list(make_boxes(rng, C, F, h, w, "hanging" if kind == "inverted" else kind,
                            away_from_integers=0.05))
    if kind == "inverted":
        lo = rng.uniform(-0.6 * h, 0.6 * h, (C, F))
        boxes[0] = lo.astype(np.float32)                                  # x_min
        boxes[1] = (lo - rng.uniform(3.3, 0.5 * h, (C, F))).astype(np.float32)   # x_max < x_min
    cpu, gpu, sc = run_both(hip, oracle, x, tuple(boxes), 3.5 * h, 2.25 * w, False, True, g)
    assert_parity(cpu, gpu, np.float32, "%s %dx%d" % (kind, h, w), **sc)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("exact", [True, False])
@pytest.mark.parametrize("h,w", [(12, 40), (70, 300), (40, 1024), (16, 512), (9, 700), (33, 1500), (36, 1800),
                                 (40, 2048), (18, 3000)])
def test_backward_lower_bound_one_ulp_above_an_integer(hip, oracle, h, w, exact, dtype):
    """A lower bound so close above an integer that `bound - 1` rounds to the integer below: the
    split the reference uses for the parameter gradients (src/box_convolution.cpp:80-96) and the
    mirrored split it uses for the input gradient (:51-67) then cut the box at different whole
    pixels. The grad_output pass computes separate column weights for the two in that case; in
    rounded mode a shared set would put a whole column of grad_input off. The widths reach every
    workgroup shape of that pass; the heights give bands with odd and with even numbers of row
    pairs."""
    rng = np.random.default_rng(h * 31 + w + int(exact))
    B, C, F = 1, 2, 2
    x = rng.standard_normal((B, C, h, w)).astype(dtype)
    g = rng.standard_normal((B, C * F, h, w)).astype(dtype)
    one = dtype(1.0)

    def above(v):
        return np.nextafter(dtype(v), dtype(0.0))

    just_above = above(-1.0)                                         # float32: -0.99999994
    assert dtype(just_above - one) == dtype(-2.0)
    x_min = np.array([[just_above, -3.3], [above(-3.0), -0.4]], dtype)
    x_max = np.array([[4.6, 2.2], [5.0, 3.5]], dtype)
    y_min = np.array([[just_above, just_above], [-7.25, above(-2.0)]], dtype)
    y_max = np.array([[6.4, 9.0], [3.75, 11.5]], dtype)
    for normalize in (False, True):
        # Rounded mode with normalisation: the reference's second summand multiplies grad_output with
        # the saved forward output (forward split), while the sums of the grad_output pass follow the
        # split of the parameter-gradient pass; at these bounds the two differ by a whole row or
        # column, and the GPU takes that one sum again with the forward split (finalize_box).
        cpu, gpu, sc = run_both(hip, oracle, x, (x_min, x_max, y_min, y_max), 3.5 * h, 2.25 * w,
                                normalize, exact, g)
        assert_parity(cpu, gpu, dtype, "normalize=%s exact=%s" % (normalize, exact), **sc)


@pytest.mark.parametrize("w", [48, 100, 200])
@pytest.mark.parametrize("kind", ["inside", "hanging"])
def test_backward_across_row_bands_narrow_image(hip, oracle, kind, w):
    """As above for images one, two and four waves wide with many filters, where the waves of a
    grad-input workgroup take the filters in turns."""
    rng = np.random.default_rng(77 + len(kind) + w)
    B, C, F, h = 2, 2, 9, 150
    x = rng.standard_normal((B, C, h, w)).astype(np.float32)
    g = (rng.standard_normal((B, C * F, h, w)) + 0.5).astype(np.float32)
    boxes = make_boxes(rng, C, F, h, w, kind, away_from_integers=0.05)
    for normalize in (False, True):
        cpu, gpu, sc = run_both(hip, oracle, x, tuple(boxes), 3.5 * h, 2.25 * w, normalize, True, g)
        assert_parity(cpu, gpu, np.float32, "%s normalize=%s" % (kind, normalize), **sc)


@pytest.mark.parametrize("B,C,F,h,w", [(2, 1, 9, 40, 48), (1, 2, 13, 70, 100), (1, 1, 6, 33, 256)])
def test_grad_input_filter_sharing_matches_one_set_per_workgroup(hip, switches, B, C, F, h, w):
    """Small problems on narrow images: the grad-input workgroups whose thread sets take the
    filters in turns give the same result, up to the order of the float32 additions over the
    filters, as workgroups that walk through all filters themselves."""
    rng = np.random.default_rng(B + C + F + h + w)
    x = dev(rng.standard_normal((B, C, h, w)).astype(np.float32))
    g = dev(rng.standard_normal((B, C * F, h, w)).astype(np.float32))
    boxes = [dev(b) for b in make_boxes(rng, C, F, h, w, "hanging")]
    integ = hip.integral_image(x)

    def grad_input():
        return hip.box_convolution_backward(integ, *boxes, g, None, 5.0, 3.0, True, True,
                                            True, False, False, False, False)[0].clone()
    preset = os.environ.get("BOXCONV_GI_SPLIT_FILTERS")     # (a run of the suite with the switch set)
    shared = grad_input()
    switches("BOXCONV_GI_SPLIT_FILTERS", "0")
    single = grad_input()
    if os.environ.get("BOXCONV_FORCE_GATHER") != "1" and preset is None:
        assert not torch.equal(shared, single) or F < 3   # really two different code paths
    scale = single.abs().max().item()
    assert (shared - single).abs().max().item() <= 4e-6 * scale


@pytest.mark.parametrize("exact", [True, False])
@pytest.mark.parametrize("h,w", [(67, 256), (130, 512), (70, 1024), (66, 2048),
                                 # rows that leave lanes of that workgroup idle (whole waves, half a wave, one lane)
                                 (36, 240), (30, 640), (40, 960), (64, 1000), (18, 1280), (22, 1800), (34, 1920),
                                 (20, 2044), (50, 160), (33, 44), (36, 100), (40, 96), (34, 92), (30, 272), (31, 132)])
def test_grad_output_pass_variants_agree(hip, oracle, switches, h, w, exact):
    """Rows of a multiple of four columns that fill at least three eighths of a workgroup at four
    columns per lane run the grad_output pass with consecutive columns per lane (the lanes past
    the row's end idle along); BOXCONV_STREAM_CONSEC=0 sends them to the kernel with wave-strided
    columns, as every other width. Both against the oracle, and against each other to the last
    few bits (the sums differ only in which columns share a lane)."""
    rng = np.random.default_rng(h + w + int(exact))
    B, C, F = 1, 2, 3
    x = rng.standard_normal((B, C, h, w)).astype(np.float32)
    g = (rng.standard_normal((B, C * F, h, w)) + 0.25).astype(np.float32)
    boxes = list(make_boxes(rng, C, F, h, w, "hanging", away_from_integers=0.05))
    if not exact:
        boxes[1] = np.maximum(boxes[1], np.ceil(boxes[0]) + 1).astype(np.float32)
        boxes[3] = np.maximum(boxes[3], np.ceil(boxes[2]) + 1).astype(np.float32)
    results = []
    for variant in (None, "0"):
        switches("BOXCONV_STREAM_CONSEC", variant)
        cpu, gpu, sc = run_both(hip, oracle, x, tuple(boxes), 3.5 * h, 2.25 * w, True, exact, g)
        assert_parity(cpu, gpu, np.float32, "consecutive=%s %dx%d exact=%s" % (variant, h, w, exact), **sc)
        results.append(gpu)
    (_, back_a), (_, back_b) = results
    assert np.abs(back_a[0] - back_b[0]).max() <= 2e-6 * np.abs(back_b[0]).max()
    for a, b in zip(back_a[1:], back_b[1:]):
        # (float32 sums of a few hundred thousand products in two different orders)
        assert np.abs(a - b).max() <= 1e-4 * max(np.abs(b).max(), 1e-30) + 1e-5 * max(np.abs(t).max() for t in back_b[1:])


@pytest.mark.parametrize("exact", [True, False])
@pytest.mark.parametrize("h,w", [(67, 256), (30, 640), (70, 1024), (22, 1800), (20, 2044), (36, 100), (33, 44), (25, 2048)])
def test_parameter_gradients_alone(hip, oracle, h, w, exact):
    """When the input needs no gradient (a network's first layer) the grad_output pass forms the
    parameter sums only: on rows that take the kernel with consecutive columns per lane, that
    kernel without its column workspace. The sums are formed the same way with or without it, so
    the four gradients equal those of the full backward bit for bit; and they meet the oracle."""
    rng = np.random.default_rng(11 * h + w + int(exact))
    B, C, F = 2, 2, 3
    x = rng.standard_normal((B, C, h, w)).astype(np.float32)
    g = (rng.standard_normal((B, C * F, h, w)) + 0.25).astype(np.float32)
    boxes = list(make_boxes(rng, C, F, h, w, "hanging", away_from_integers=0.05))
    if not exact:
        boxes[1] = np.maximum(boxes[1], np.ceil(boxes[0]) + 1).astype(np.float32)
        boxes[3] = np.maximum(boxes[3], np.ceil(boxes[2]) + 1).astype(np.float32)
    needs = (False, True, True, True, True)
    cpu, gpu, sc = run_both(hip, oracle, x, tuple(boxes), 3.5 * h, 2.25 * w, True, exact, g, needs)
    assert gpu[1][0] is None
    assert_parity(cpu, gpu, np.float32, "parameters only %dx%d exact=%s" % (h, w, exact), **sc)
    _, full, _ = run_both(hip, oracle, x, tuple(boxes), 3.5 * h, 2.25 * w, True, exact, g)
    for a, b in zip(gpu[1][1:], full[1][1:]):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("exact", [True, False])
@pytest.mark.parametrize("h,w", [(37, 130), (40, 256), (34, 300), (70, 512), (21, 700), (36, 1024), (18, 1025),
                                 (12, 1100), (16, 1536), (10, 1538), (14, 2047), (12, 2048)])
def test_float64_grad_output_pass_shapes_agree(hip, oracle, switches, h, w, exact):
    """float64 rows of up to 1024 columns run the grad_output pass with at most two columns per
    lane, and on four or eight waves as two launches (parameter sums, column workspace); rows of
    1025 to 2048 columns as two launches as well, the parameter sums by two workgroups per band
    with two columns per lane. BOXCONV_STREAM_F64_NARROW=0 gives all of them float32's three or
    four columns per lane and the one launch. Both against the oracle and against each other."""
    rng = np.random.default_rng(3 * h + w + int(exact))
    B, C, F = 2, 2, 3
    x = rng.standard_normal((B, C, h, w))
    g = rng.standard_normal((B, C * F, h, w)) + 0.25
    boxes = list(make_boxes(rng, C, F, h, w, "hanging", away_from_integers=0.05))
    if not exact:
        boxes[1] = np.maximum(boxes[1], np.ceil(boxes[0]) + 1)
        boxes[3] = np.maximum(boxes[3], np.ceil(boxes[2]) + 1)
    boxes = tuple(np.asarray(b, dtype=np.float64) for b in boxes)
    results = []
    for variant in (None, "0"):
        switches("BOXCONV_STREAM_F64_NARROW", variant)
        cpu, gpu, sc = run_both(hip, oracle, x, boxes, 3.5 * h, 2.25 * w, True, exact, g)
        assert_parity(cpu, gpu, np.float64, "narrow=%s %dx%d exact=%s" % (variant, h, w, exact), **sc)
        results.append(gpu)
    (_, back_a), (_, back_b) = results
    for a, b in zip(back_a, back_b):
        assert np.abs(a - b).max() <= 1e-11 * max(np.abs(b).max(), 1e-30) + 1e-12 * max(np.abs(t).max() for t in back_b[1:])


@pytest.mark.parametrize("h,w,F", [(64, 20, 3), (64, 40, 5), (96, 200, 3), (128, 256, 2), (256, 512, 3),
                                   (64, 1024, 3), (128, 2500, 2)])
def test_workspace_layouts_agree(hip, oracle, switches, h, w, F):
    """Planes that are cut into whole bands of a power-of-two number of rows keep the rows of the
    column workspace interleaved over the bands (row k of every band side by side);
    BOXCONV_M_INTERLEAVE=0 keeps them in their natural order. Only the place of a row changes,
    so the two give the same bits, and both meet the oracle."""
    rng = np.random.default_rng(h * 7 + w)
    B, C = 2, 2
    x = rng.standard_normal((B, C, h, w)).astype(np.float32)
    g = (rng.standard_normal((B, C * F, h, w)) + 0.25).astype(np.float32)
    boxes = tuple(make_boxes(rng, C, F, h, w, "hanging", away_from_integers=0.05))
    results = []
    for layout in ("1", "0"):
        switches("BOXCONV_M_INTERLEAVE", layout)
        cpu, gpu, sc = run_both(hip, oracle, x, boxes, 2.5 * h, 1.5 * w, True, True, g)
        assert_parity(cpu, gpu, np.float32, "interleave=%s %dx%d" % (layout, h, w), **sc)
        results.append(gpu)
    (_, back_a), (_, back_b) = results
    for a, b in zip(back_a, back_b):
        assert np.array_equal(a, b)


def test_parameter_gradients_are_reproducible(hip):
    """The streaming backward adds the per-workgroup partial sums in a fixed order (no atomics),
    so repeated calls agree bit for bit."""
    rng = np.random.default_rng(5)
    B, C, F, h, w = 3, 2, 3, 130, 200
    x = dev(rng.standard_normal((B, C, h, w)).astype(np.float32))
    g = dev(rng.standard_normal((B, C * F, h, w)).astype(np.float32))
    boxes = [dev(b) for b in make_boxes(rng, C, F, h, w, "hanging")]
    integ = hip.integral_image(x)
    out = hip.box_convolution_forward(integ, *boxes, True, True)
    runs = [hip.box_convolution_backward(integ, *boxes, g, out, 11.0, 7.0, True, True,
                                         True, True, True, True, True) for _ in range(3)]
    torch.cuda.synchronize()
    for other in runs[1:]:
        for a, b in zip(runs[0], other):
            assert torch.equal(a, b)


def test_unit_box_is_identity(hip):
    x = torch.randn(2, 3, 13, 31, device="cuda")
    z = torch.zeros(3, 2, device="cuda")
    out = hip.box_convolution_forward(hip.integral_image(x), z, z, z, z, True, True)
    want = x.repeat_interleave(2, dim=1)
    assert torch.allclose(out, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("needs", [(True, False, False, False, False), (False, True, True, True, True),
                                   (False, False, True, False, False), (True, True, False, False, True)])
def test_selective_gradients(hip, oracle, needs):
    rng = np.random.default_rng(77)
    B, C, F, h, w = 2, 2, 3, 19, 23
    x = rng.standard_normal((B, C, h, w)).astype(np.float32)
    g = rng.standard_normal((B, C * F, h, w)).astype(np.float32)
    boxes = make_boxes(rng, C, F, h, w, "hanging")
    cpu, gpu, sc = run_both(hip, oracle, x, boxes, 40.0, 50.0, True, True, g, needs)
    for k in range(5):
        assert (gpu[1][k] is None) == (not needs[k])
    assert_parity(cpu, gpu, np.float32, **sc)


def test_gather_kernels_match_row_streaming(hip, oracle, switches):
    """The per-pixel gather kernels (used for very wide images) against the oracle."""
    rng = np.random.default_rng(123)
    B, C, F, h, w = 2, 2, 3, 31, 77
    x = rng.standard_normal((B, C, h, w)).astype(np.float32)
    g = rng.standard_normal((B, C * F, h, w)).astype(np.float32)
    boxes = make_boxes(rng, C, F, h, w, "hanging")
    switches("BOXCONV_FORCE_GATHER", "1")
    for normalize in (True, False):
        for exact in (True, False):
            if not exact:
                boxes = make_boxes(rng, C, F, h, w, "inside")
            cpu, gpu, sc = run_both(hip, oracle, x, boxes, 40.0, 50.0, normalize, exact, g)
            assert_parity(cpu, gpu, np.float32, "gather normalize=%s exact=%s" % (normalize, exact), **sc)


def test_clip_parameters_matches_oracle(hip, oracle):
    rng = np.random.default_rng(9)
    for dtype in (np.float32, np.float64):
        for exact in (True, False):
            n = 257
            rh, rw, mh, mw = 8.0 * 28, 3.3 * 40, 28.0, 40.0
            p = [(rng.uniform(-1.5, 1.5, n) * s).astype(dtype) for s in (mh / rh, mh / rh, mw / rw, mw / rw)]
            p[1][:40] = p[0][:40] + rng.uniform(-0.5, 0.5, 40).astype(dtype) / rh   # thin / inverted boxes
            want = [a.copy() for a in p]
            oracle.clip_parameters(*want, rh, rw, mh, mw, exact)
            t = [dev(a) for a in p]
            hip.clip_parameters(*t, rh, rw, mh, mw, exact)
            for a, b in zip(t, want):
                assert np.array_equal(host(a), b)
