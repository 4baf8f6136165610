"""Writes tests/golden/reference_vectors.npz: small input/output vectors of the reference's own
CPU kernels.

The outputs come from oracle/_ref/libboxconv_ref.so, i.e. the reference's src/integral_image.cpp
and src/box_convolution.cpp compiled unmodified (see oracle/Makefile, oracle/ref_driver.cpp), so
this script only runs where /root/reference exists. The fixture is data only: seeded inputs and
the reference's outputs for them. It pins what no closed form fixes: one-sided gradient choices at
whole-number box bounds, rounded-mode (exact=False) parameter gradients, and the float32 rounding
pattern of the reference's integral image.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from helpers import make_boxes  # noqa: E402
from oracle import cpu_checker  # noqa: E402

CASES = [
    # name, B, C, F, h, w, box kind, dtype
    ("inside_f32", 2, 2, 3, 9, 11, "inside", np.float32),
    ("hanging_f32", 1, 3, 2, 8, 13, "hanging", np.float32),
    ("integer_f32", 2, 1, 4, 7, 7, "integer", np.float32),
    ("unit_f32", 1, 2, 1, 5, 6, "unit", np.float32),
    ("hanging_f64", 1, 2, 2, 6, 9, "hanging", np.float64),
    ("integer_f64", 1, 2, 3, 10, 5, "integer", np.float64),
    ("tall_f32", 1, 1, 2, 40, 3, "hanging", np.float32),
]


def main():
    ref = cpu_checker.reference()
    if ref is None:
        sys.exit("oracle/_ref/libboxconv_ref.so not built (make -C oracle ref); needs /root/reference")
    out = {}
    for n, (name, B, C, F, h, w, kind, dtype) in enumerate(CASES):
        rng = np.random.default_rng(4200 + n)
        x = rng.standard_normal((B, C, h, w)).astype(dtype)
        g = rng.standard_normal((B, C * F, h, w)).astype(dtype)
        boxes = make_boxes(rng, C, F, h, w, kind, dtype)
        reparam_h, reparam_w = 2.5 * h, 3.25 * w
        out[name + "/x"] = x
        out[name + "/grad_output"] = g
        out[name + "/reparam"] = np.array([reparam_h, reparam_w], dtype=np.float64)
        integ = ref.integral_image(x)
        out[name + "/integral"] = integ
        for exact in (True, False):
            bx = list(boxes)
            if not exact:   # rounded mode needs at least one whole pixel inside the box
                bx[1] = np.maximum(bx[1], np.ceil(bx[0]) + 1).astype(dtype)
                bx[3] = np.maximum(bx[3], np.ceil(bx[2]) + 1).astype(dtype)
            for k, pname in enumerate(("x_min", "x_max", "y_min", "y_max")):
                out["%s/exact%d/%s" % (name, exact, pname)] = bx[k]
            for normalize in (True, False):
                tag = "%s/exact%d/norm%d" % (name, exact, normalize)
                fwd = ref.box_forward(integ, *bx, normalize, exact)
                back = ref.box_backward(integ, *bx, g, fwd, reparam_h, reparam_w, normalize, exact)
                out[tag + "/output"] = fwd
                for k, gname in enumerate(("grad_input", "grad_x_min", "grad_x_max", "grad_y_min", "grad_y_max")):
                    out[tag + "/" + gname] = back[k]
    # parameter clipping: stored-unit parameters covering the three regimes (inside, clamped,
    # too thin / inverted)
    rng = np.random.default_rng(77)
    for dtype, tag in ((np.float32, "clip_f32"), (np.float64, "clip_f64")):
        n = 64
        rh, rw, mh, mw = 8.0 * 28, 3.3 * 40, 28.0, 40.0
        p = [(rng.uniform(-1.6, 1.6, n) * s).astype(dtype) for s in (mh / rh, mh / rh, mw / rw, mw / rw)]
        p[1][:24] = p[0][:24] + (rng.uniform(-0.5, 0.5, 24) / rh).astype(dtype)
        p[3][:24] = p[2][:24] + (rng.uniform(-0.5, 0.5, 24) / rw).astype(dtype)
        out[tag + "/meta"] = np.array([rh, rw, mh, mw])
        for k in range(4):
            out["%s/in%d" % (tag, k)] = p[k].copy()
        for exact in (True, False):
            q = [a.copy() for a in p]
            ref.clip_parameters(*q, rh, rw, mh, mw, exact)
            for k in range(4):
                out["%s/exact%d/out%d" % (tag, exact, k)] = q[k]
    path = os.path.join(HERE, "reference_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote %s (%d arrays, %d bytes)" % (path, len(out), os.path.getsize(path)))


if __name__ == "__main__":
    main()
