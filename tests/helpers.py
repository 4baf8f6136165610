"""Shared generators for the tests: seeded inputs and boxes (real pixel units)."""
import numpy as np


def make_boxes(rng, C, F, h, w, kind="inside", dtype=np.float32, away_from_integers=0.0):
    """Four [C,F] arrays (x_min, x_max, y_min, y_max), x_min <= x_max, y_min <= y_max.

    kind: 'inside'   bounds within +-h/2, +-w/2 (the BASELINE configs 2-4 recipe)
          'hanging'  boxes reaching up to 1.5 image sizes outside the image
          'integer'  whole-number bounds (the non-smooth points)
          'large'    spanning more than 80 % of the image (BASELINE config 5 recipe)
          'unit'     x_min = x_max = y_min = y_max = 0 (identity filter)
    """
    def draw(lo_fn):
        while True:
            v = lo_fn()
            if away_from_integers <= 0 or abs(v - round(v)) > away_from_integers:
                return v

    out = np.zeros((4, C, F), dtype=np.float64)
    for c in range(C):
        for f in range(F):
            if kind == "inside":
                x0 = draw(lambda: rng.uniform(-h / 2, h / 2 - 3)); x1 = draw(lambda: rng.uniform(x0 + 1.5, h / 2))
                y0 = draw(lambda: rng.uniform(-w / 2, w / 2 - 3)); y1 = draw(lambda: rng.uniform(y0 + 1.5, w / 2))
            elif kind == "hanging":
                x0 = draw(lambda: rng.uniform(-1.5 * h, 1.2 * h)); x1 = draw(lambda: x0 + rng.uniform(0.1, 1.5 * h))
                y0 = draw(lambda: rng.uniform(-1.5 * w, 1.2 * w)); y1 = draw(lambda: y0 + rng.uniform(0.1, 1.5 * w))
            elif kind == "integer":
                x0 = float(rng.integers(-h, h)); x1 = x0 + float(rng.integers(0, h + 1))
                y0 = float(rng.integers(-w, w)); y1 = y0 + float(rng.integers(0, w + 1))
            elif kind == "large":
                x0 = draw(lambda: rng.uniform(-0.49 * h, -0.41 * h)); x1 = draw(lambda: rng.uniform(0.41 * h, 0.49 * h))
                y0 = draw(lambda: rng.uniform(-0.49 * w, -0.41 * w)); y1 = draw(lambda: rng.uniform(0.41 * w, 0.49 * w))
            elif kind == "unit":
                x0 = x1 = y0 = y1 = 0.0
            else:
                raise ValueError(kind)
            out[:, c, f] = (x0, x1, y0, y1)
    return tuple(np.ascontiguousarray(out[k].astype(dtype)) for k in range(4))


def rel_err(a, b, floor=0.0):
    """max|a-b| / max(max|b|, floor): the per-tensor error the parity targets are stated in.

    `floor` keeps the measure meaningful for a tensor whose exact value is zero and whose
    reference value is pure rounding noise (e.g. the gradient of a bound that lies outside the
    image for every pixel): pass a small fraction of the magnitude of the sibling tensors."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    denom = max(np.abs(b).max() if b.size else 0.0, floor)
    diff = np.abs(a - b).max() if b.size else 0.0
    return float(diff / denom) if denom > 0 else float(diff)


def param_grad_floor(grads):
    """1e-2 of the largest entry over the four parameter-gradient tensors that are present: a
    gradient tensor smaller than that is compared on this scale (absolute error <= tol * 1e-2 of
    the largest gradient), because its float32 value is dominated by cancellation noise."""
    vals = [np.abs(np.asarray(g, dtype=np.float64)).max() for g in grads if g is not None and g.size]
    return 1e-2 * max(vals) if vals else 0.0
