"""Pins for the CPU oracle (oracle/boxconv_oracle.cpp). Runs without a GPU.

Three independent anchors:
 (1) tests/golden/reference_vectors.npz -- outputs of the reference's own CPU kernels compiled
     unmodified (tests/golden/make_golden.py): covers every entry point, exact and rounded mode,
     whole-number bounds, float32 and float64.
 (2) oracle/_ref live, where it was built: randomized bit-for-bit comparison.
 (3) what the mathematics fixes, none of it written with the oracle's formulas: float64 cumulative
     sums; a brute-force overlap-area box filter (the reference test's definition,
     box_convolution/test.py:60-86); its transpose for grad_input; central finite differences of it
     for the parameter gradients; identity / plain box filter / constant image special cases; the
     closed form of the clip projection.
Pinned by (1)+(2)+(3): integral_image, box_forward, box_grad_input_planes, box_backward
(grad_input and the four parameter gradients incl. the normalisation term and reparametrization
scale), clip_parameters, the three splits. Nothing in the oracle is left unpinned.
"""
import os

import numpy as np
import pytest

from helpers import make_boxes, rel_err

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.npz")
CASES = ["inside_f32", "hanging_f32", "integer_f32", "unit_f32", "hanging_f64", "integer_f64", "tall_f32"]


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN)


# ---- (1) golden vectors ---------------------------------------------------------------------
@pytest.mark.parametrize("case", CASES)
def test_oracle_matches_golden_vectors(oracle, golden, case):
    x = golden[case + "/x"]
    g = golden[case + "/grad_output"]
    reparam_h, reparam_w = golden[case + "/reparam"]
    integ = oracle.integral_image(x)
    assert np.array_equal(integ, golden[case + "/integral"])
    ptol = 2e-5 if x.dtype == np.float32 else 1e-12
    for exact in (1, 0):
        bx = [golden["%s/exact%d/%s" % (case, exact, n)] for n in ("x_min", "x_max", "y_min", "y_max")]
        for normalize in (1, 0):
            tag = "%s/exact%d/norm%d" % (case, exact, normalize)
            out = oracle.box_forward(integ, *bx, normalize, exact)
            assert np.array_equal(out, golden[tag + "/output"]), tag
            back = oracle.box_backward(integ, *bx, g, out, reparam_h, reparam_w, normalize, exact)
            assert np.array_equal(back[0], golden[tag + "/grad_input"]), tag
            names = ("grad_x_min", "grad_x_max", "grad_y_min", "grad_y_max")
            scale = max(np.abs(golden[tag + "/" + n]).max() for n in names)
            for k, n in enumerate(names):
                # the reference sums float32 products with ATen's blocked float32 sum; the oracle
                # accumulates the same products in double
                assert np.abs(back[1 + k] - golden[tag + "/" + n]).max() <= ptol * scale, (tag, n)


@pytest.mark.parametrize("tag", ["clip_f32", "clip_f64"])
def test_oracle_clip_matches_golden_vectors(oracle, golden, tag):
    rh, rw, mh, mw = golden[tag + "/meta"]
    for exact in (1, 0):
        p = [golden["%s/in%d" % (tag, k)].copy() for k in range(4)]
        oracle.clip_parameters(*p, rh, rw, mh, mw, exact)
        for k in range(4):
            assert np.array_equal(p[k], golden["%s/exact%d/out%d" % (tag, exact, k)])


# ---- (2) compiled reference, live -------------------------------------------------------------
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_oracle_matches_compiled_reference(oracle, reference, dtype):
    rng = np.random.default_rng(11)
    for trial in range(12):
        B, C, F = (int(v) for v in rng.integers(1, 3, 3))
        h, w = (int(v) for v in rng.integers(2, 12, 2))
        x = rng.random((B, C, h, w)).astype(dtype)
        kind = ("inside", "hanging", "integer")[trial % 3]
        boxes = make_boxes(rng, C, F, max(h, 4), max(w, 4), kind, dtype)
        integ = oracle.integral_image(x)
        assert np.array_equal(integ, reference.integral_image(x))
        for variant in range(3):
            for c in range(C):
                args = [float(b[c, 0]) for b in boxes]
                io, fo = oracle.split(variant, *args, dtype=dtype)
                ir, fr = reference.split(variant, *args, dtype=dtype)
                assert np.array_equal(io, ir) and np.array_equal(fo, fr)
        for normalize in (0, 1):
            for exact in (0, 1):
                bx = list(boxes)
                if not exact:
                    bx[1] = np.maximum(bx[1], np.ceil(bx[0]) + 1).astype(dtype)
                    bx[3] = np.maximum(bx[3], np.ceil(bx[2]) + 1).astype(dtype)
                fo = oracle.box_forward(integ, *bx, normalize, exact)
                assert np.array_equal(fo, reference.box_forward(integ, *bx, normalize, exact))
                g = rng.standard_normal(fo.shape).astype(dtype)
                gint = oracle.integral_image(g.reshape(B, C, F, h, w))
                assert np.array_equal(oracle.grad_input_planes(gint, *bx, normalize, exact),
                                      reference.grad_input_planes(gint, *bx, normalize, exact))
                for which in range(4):
                    assert np.array_equal(oracle.grad_param_planes(integ, *bx, which, exact),
                                          reference.grad_param_planes(integ, *bx, which, exact))
                bo = oracle.box_backward(integ, *bx, g, fo, 3.7 * h, 2.2 * w, normalize, exact)
                br = reference.box_backward(integ, *bx, g, fo, 3.7 * h, 2.2 * w, normalize, exact)
                assert np.array_equal(bo[0], br[0])
                scale = max(np.abs(b).max() for b in br[1:]) + 1e-300
                for k in range(1, 5):
                    assert np.abs(bo[k] - br[k]).max() <= (2e-5 if dtype == np.float32 else 1e-12) * scale


# ---- (3) mathematics ------------------------------------------------------------------------
def overlap(a0, a1, b0, b1):
    return max(0.0, min(a1, b1) - max(a0, b0))


def brute_force_forward(x, xmin, xmax, ymin, ymax, normalize):
    """out[b, c*F+f, i, j] = sum_{i',j'} x[b,c,i',j'] * |rows [i',i'+1) ^ [i+xmin, i+xmax+1)| *
    |cols [j',j'+1) ^ [j+ymin, j+ymax+1)|, zero outside the image; / full box area if normalize."""
    B, C, h, w = x.shape
    F = xmin.shape[1]
    out = np.zeros((B, C * F, h, w))
    for c in range(C):
        for f in range(F):
            x0, x1, y0, y1 = (float(p[c, f]) for p in (xmin, xmax, ymin, ymax))
            rw_ = np.array([[overlap(ii, ii + 1, i + x0, i + x1 + 1) for ii in range(h)] for i in range(h)])
            cw_ = np.array([[overlap(jj, jj + 1, j + y0, j + y1 + 1) for jj in range(w)] for j in range(w)])
            res = np.einsum("ip,bpq,jq->bij", rw_, x[:, c].astype(np.float64), cw_)
            if normalize:
                res = res / ((x1 - x0 + 1) * (y1 - y0 + 1))
            out[:, c * F + f] = res
    return out


def oracle_forward64(oracle, x, boxes, normalize, exact=1):
    x = x.astype(np.float64)
    bx = [b.astype(np.float64) for b in boxes]
    integ = oracle.integral_image(x)
    return integ, bx, oracle.box_forward(integ, *bx, normalize, exact)


def test_integral_image_is_double_cumsum(oracle):
    rng = np.random.default_rng(0)
    for _ in range(20):
        shape = tuple(int(v) for v in rng.integers(1, 4, 2)) + tuple(int(v) for v in rng.integers(2, 11, 2))
        x = rng.random(shape).astype(np.float32)
        got = oracle.integral_image(x)
        want = np.zeros(shape[:-2] + (shape[-2] + 1, shape[-1] + 1))
        want[..., 1:, 1:] = x.astype(np.float64).cumsum(-2).cumsum(-1)
        assert np.all(got[..., 0, :] == 0) and np.all(got[..., :, 0] == 0)
        assert np.allclose(got, want, rtol=1e-5, atol=1e-8)     # tolerances of reference test.py:53
    xd = rng.random((2, 3, 7, 9))
    want = np.zeros((2, 3, 8, 10))
    want[..., 1:, 1:] = xd.cumsum(-2).cumsum(-1)
    assert np.allclose(oracle.integral_image(xd), want, rtol=1e-14, atol=1e-14)


@pytest.mark.parametrize("kind", ["inside", "hanging", "integer"])
@pytest.mark.parametrize("normalize", [0, 1])
def test_forward_is_overlap_area_filter(oracle, kind, normalize):
    rng = np.random.default_rng(3 + normalize)
    for _ in range(8):
        B, C, F = 1, 2, 2
        h, w = (int(v) for v in rng.integers(2, 8, 2))
        x = rng.standard_normal((B, C, h, w))
        boxes = make_boxes(rng, C, F, max(h, 4), max(w, 4), kind, np.float64)
        _, bx, got = oracle_forward64(oracle, x, boxes, normalize)
        want = brute_force_forward(x, *bx, normalize)
        assert np.abs(got - want).max() <= 1e-11 * max(1.0, np.abs(want).max())


def test_rounded_mode_is_exact_mode_on_rounded_bounds(oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((1, 2, 7, 9))
    boxes = make_boxes(rng, 2, 3, 7, 9, "inside", np.float64)
    integ = oracle.integral_image(x)
    rounded = [np.ceil(boxes[0]), np.floor(boxes[1]), np.ceil(boxes[2]), np.floor(boxes[3])]
    for normalize in (0, 1):
        a = oracle.box_forward(integ, *boxes, normalize, 0)
        b = brute_force_forward(x, *rounded, normalize)
        assert np.abs(a - b).max() <= 1e-11


def test_special_cases(oracle):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((2, 2, 6, 8)).astype(np.float32)
    integ = oracle.integral_image(x)
    z = np.zeros((2, 1), dtype=np.float32)
    # the zero box is the identity
    assert np.allclose(oracle.box_forward(integ, z, z, z, z, 1, 1), x, atol=1e-5)
    # whole-number box = plain sliding-window sum with zero padding
    xmin, xmax, ymin, ymax = (np.full((2, 1), v, dtype=np.float32) for v in (-1, 2, -2, 1))
    got = oracle.box_forward(integ, xmin, xmax, ymin, ymax, 0, 1)
    pad = np.zeros((2, 2, 6 + 8, 8 + 8))
    pad[:, :, 4:10, 4:12] = x
    want = np.zeros_like(x, dtype=np.float64)
    for i in range(6):
        for j in range(8):
            want[:, :, i, j] = pad[:, :, 4 + i - 1:4 + i + 3, 4 + j - 2:4 + j + 2].sum((-1, -2))
    assert np.allclose(got, want, atol=1e-4)
    # constant image: average = (box area inside the image) / (box area)
    ones = np.ones((1, 1, 5, 5))
    io = oracle.integral_image(ones)
    b = [np.array([[v]]) for v in (-1.5, 0.25, -0.75, 3.5)]
    got = oracle.box_forward(io, *b, 1, 1)
    for i in range(5):
        for j in range(5):
            inside = overlap(0, 5, i - 1.5, i + 1.25) * overlap(0, 5, j - 0.75, j + 4.5)
            assert abs(got[0, 0, i, j] - inside / (2.75 * 5.25)) < 1e-12


@pytest.mark.parametrize("normalize", [0, 1])
def test_grad_input_is_the_adjoint(oracle, normalize):
    rng = np.random.default_rng(8)
    B, C, F, h, w = 2, 2, 3, 6, 7
    x = rng.standard_normal((B, C, h, w))
    g = rng.standard_normal((B, C * F, h, w))
    boxes = make_boxes(rng, C, F, h, w, "hanging", np.float64)
    integ, bx, out = oracle_forward64(oracle, x, boxes, normalize)
    gin = oracle.box_backward(integ, *bx, g, out, 1.0, 1.0, normalize, 1, (1, 0, 0, 0, 0))[0]
    assert abs((out * g).sum() - (x * gin).sum()) <= 1e-10 * np.abs(out * g).sum()
    # and element-wise: grad_input[b,c,p,q] = d <out,g> / d x[b,c,p,q] by linearity
    for (b, c, p, q) in [(0, 0, 0, 0), (1, 1, 5, 6), (0, 1, 3, 2)]:
        e = np.zeros_like(x)
        e[b, c, p, q] = 1.0
        want = (brute_force_forward(e, *bx, normalize) * g).sum()
        assert abs(gin[b, c, p, q] - want) <= 1e-11 * max(1.0, abs(want))


@pytest.mark.parametrize("normalize", [0, 1])
def test_parameter_gradients_match_finite_differences(oracle, normalize):
    """The reference's own check (gradcheck in float64, test.py:280-301) restated with central
    differences of the brute-force filter; bounds kept away from whole numbers where the filter is
    not differentiable."""
    rng = np.random.default_rng(9 + normalize)
    for trial in range(5):
        B, C, F, h, w = 2, 2, 2, 5, 6
        x = rng.standard_normal((B, C, h, w))
        g = rng.standard_normal((B, C * F, h, w))
        boxes = list(make_boxes(rng, C, F, h, w, "hanging" if trial % 2 else "inside", np.float64,
                                away_from_integers=0.02))
        reparam_h, reparam_w = 3.0, 7.0
        integ, bx, out = oracle_forward64(oracle, x, boxes, normalize)
        grads = oracle.box_backward(integ, *bx, g, out, reparam_h, reparam_w, normalize, 1)[1:]
        eps = 1e-5
        for k in range(4):
            scale = reparam_h if k < 2 else reparam_w
            for c in range(C):
                for f in range(F):
                    hi = [b.copy() for b in bx]
                    lo = [b.copy() for b in bx]
                    hi[k][c, f] += eps
                    lo[k][c, f] -= eps
                    fd = ((brute_force_forward(x, *hi, normalize) - brute_force_forward(x, *lo, normalize)) * g).sum() / (2 * eps)
                    # gradient w.r.t. the STORED parameter = real-unit gradient * reparametrization
                    assert abs(grads[k][c, f] - fd * scale) <= 1e-6 * max(1.0, abs(fd * scale)), (trial, k, c, f)


def clip_closed_form(pmin, pmax, reparam, min_size, max_size, dtype):
    inv = 1.0 / reparam
    lo = min(max(float(pmin), -(max_size + 1) * inv), (max_size - 1) * inv)
    hi = min(max(float(pmax), -(max_size + 1) * inv), (max_size - 1) * inv)
    gap = (min_size - 0.9999) * inv
    if lo + gap > hi:
        mean = float(dtype(0.5 * (lo + hi)))
        lo, hi = mean - 0.5 * gap, mean + 0.5 * gap
    return dtype(lo), dtype(hi)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("exact", [1, 0])
def test_clip_projection_regimes(oracle, dtype, exact):
    rh, rw, mh, mw = 16.0, 40.0, 8.0, 10.0
    min_size = float(np.float32(1.001 if exact else 2.001))
    # (min, max) in real pixels: untouched / clamped high / clamped low / too thin / inverted
    pairs = [(-2.0, 3.0), (5.0, 30.0), (-30.0, -20.0), (1.0, 1.0005), (2.0, -1.0), (7.0, 7.0)]
    xmin = np.array([a / rh for a, _ in pairs], dtype=dtype)
    xmax = np.array([b / rh for _, b in pairs], dtype=dtype)
    ymin = np.array([a / rw for a, _ in pairs], dtype=dtype)
    ymax = np.array([b / rw for _, b in pairs], dtype=dtype)
    want_x = [clip_closed_form(a, b, rh, min_size, mh, dtype) for a, b in zip(xmin, xmax)]
    want_y = [clip_closed_form(a, b, rw, min_size, mw, dtype) for a, b in zip(ymin, ymax)]
    oracle.clip_parameters(xmin, xmax, ymin, ymax, rh, rw, mh, mw, exact)
    assert [(a, b) for a, b in zip(xmin, xmax)] == want_x
    assert [(a, b) for a, b in zip(ymin, ymax)] == want_y
    # invariants: inside the allowed range (re-centring a thin box may overshoot it by half the
    # minimum thickness) and at least min_size - 0.9999 thick (up to rounding)
    half = 0.5 * (min_size - 0.9999)
    assert np.all(xmax * rh <= mh - 1 + half + 1e-4) and np.all(xmin * rh >= -(mh + 1) - half - 1e-4)
    assert np.all((xmax - xmin) * rh >= min_size - 0.9999 - 1e-4)
    # an untouched pair stays bit-identical
    assert xmin[0] == dtype(-2.0 / rh) and xmax[0] == dtype(3.0 / rh)


def test_split_identities(oracle):
    rng = np.random.default_rng(10)
    for _ in range(200):
        x0, y0 = rng.uniform(-20, 20, 2)
        x1, y1 = x0 + rng.uniform(0, 10), y0 + rng.uniform(0, 10)
        ints, fr = oracle.split(0, x0, x1, y0, y1, dtype=np.float64)
        assert np.all((fr >= 0) & (fr < 1))
        assert np.isclose(ints[0] - fr[0], x0) and np.isclose(ints[1] - 1 + fr[1], x1)
        assert np.isclose(ints[2] - fr[2], y0) and np.isclose(ints[3] - 1 + fr[3], y1)
        # mirrored box (grad input): split of (-x1, -x0)
        gi, gf = oracle.split(1, x0, x1, y0, y1, dtype=np.float64)
        mi, mf = oracle.split(0, -x1, -x0, -y1, -y0, dtype=np.float64)
        assert np.array_equal(gi, mi) and np.allclose(gf, mf, atol=1e-12)
        # parameter-gradient split is the forward split shifted to 1-based pixels
        pi, pf = oracle.split(2, x0, x1, y0, y1, dtype=np.float64)
        assert np.array_equal(pi, ints - 1)
        assert np.allclose(pf, fr, atol=1e-12)


INT_DTYPES = [np.uint8, np.int8, np.int16, np.int32, np.int64]


@pytest.mark.parametrize("dtype", INT_DTYPES)
def test_integer_integral_image_is_wrapping_cumsum(oracle, dtype):
    """Integer tensors (the reference dispatches on every ATen type, src/integral_image.cpp:14):
    the exact sums modulo 2^bits, i.e. numpy's cumulative sums in the same type, full-range
    values included. Where the compiled reference exists it gives the same bits."""
    rng = np.random.default_rng(np.dtype(dtype).itemsize)
    info = np.iinfo(dtype)
    for shape in [(3, 37, 41), (1, 1, 1), (2, 5, 300), (2, 2, 130, 7)]:
        x = rng.integers(info.min, info.max, size=shape, dtype=dtype, endpoint=True)
        want = np.zeros(shape[:-2] + (shape[-2] + 1, shape[-1] + 1), dtype=dtype)
        want[..., 1:, 1:] = x.cumsum(-2, dtype=dtype).cumsum(-1, dtype=dtype)
        got = oracle.integral_image(x)
        assert got.dtype == x.dtype and np.array_equal(got, want)
        from oracle import cpu_checker
        ref = cpu_checker.reference()
        if ref is not None:
            assert np.array_equal(ref.integral_image(x), want)


# ---- what the rounding of the reference's integral image does to large-box gradients -----------
def test_large_box_parameter_gradients_carry_the_integral_images_rounding(oracle):
    """The recipe of the large-box workload (1024 x 2048 planes of uniform[0,1) + 10, boxes over
    more than 80 % of the image): integral-image entries reach 2.2e7, where a float32 ulp is 2.
    The reference rounds its integral image once per row (src/integral_image.cpp:28-31: the row
    sum in double plus the float32 entry above, stored as float32), so an entry is off by up to a
    few dozen ulps; the parameter gradients are differences of nearly equal sums of such entries.

    Same float32 sampling code, same boxes, same grad_output, only the integral image exchanged
    for the correctly rounded one (float64 sums rounded once): the y gradients move by more than
    the 1e-3 they are compared at, towards the float64 result. This is why an implementation that
    stores correctly rounded sums is compared with the reference on equal integral images at this
    workload (tests/test_gpu_baseline_configs.py)."""
    rng = np.random.default_rng(5)
    C, F, h, w = 2, 2, 1024, 2048
    x = rng.random((1, C, h, w), dtype=np.float32) + np.float32(10.0)
    g = rng.standard_normal((1, C * F, h, w), dtype=np.float32)
    boxes = make_boxes(rng, C, F, h, w, "large", away_from_integers=0.01)
    own = oracle.integral_image(x)
    i64 = oracle.integral_image(x.astype(np.float64))
    rounded_once = i64.astype(np.float32)
    ulp = np.spacing(np.float32(own.max()))
    assert np.abs(own.astype(np.float64) - i64).max() > 8 * ulp          # the reference's drift
    assert np.abs(rounded_once.astype(np.float64) - i64).max() <= 0.5 * ulp

    def gradients(integ, dtype):
        b = [p.astype(dtype) for p in boxes]
        out = oracle.box_forward(integ, *b, True, True)
        return oracle.box_backward(integ, *b, g.astype(dtype), out, 8.0 * h, 8.0 * w, True, True)[1:]
    lit, once, dbl = gradients(own, np.float32), gradients(rounded_once, np.float32), gradients(i64, np.float64)
    moved = [rel_err(a, b) for a, b in zip(lit, once)]
    lit64 = [rel_err(a, b) for a, b in zip(lit, dbl)]
    once64 = [rel_err(a, b) for a, b in zip(once, dbl)]
    # the reference's own float32 result is more than the tolerance away from float64 ...
    assert max(lit64) > 1.5e-3
    # ... all of it from the integral image: with the correctly rounded one it is within 1e-4
    assert max(once64) <= 1e-4
    assert max(moved) > 1.5e-3
    # and the x gradients hardly move: they sum differences of ADJACENT ROWS of the integral image,
    # which are one rounding apart, while the y gradients sum differences of adjacent columns of
    # box sums over some 900 rows, whose accumulated drifts are independent of each other
    assert max(moved[:2]) <= 1e-4
