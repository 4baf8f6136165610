"""Seeded random shapes against the CPU oracle: widths on both sides of every workgroup-shape
boundary (64, 128, 192, 256, 384, 512, 768, 1024, 1536, 2048, 3072, 4096), heights that give one
or several row bands, 1 to 12 filters, all box kinds and the four (normalize, exact) modes.
The cases are fixed by their seeds, so a failure names a reproducible shape.
Tolerances as everywhere: forward / grad_input 1e-4, parameter gradients 1e-3 (test_gpu_parity);
the float64 runs of the same cases: 1e-9."""
import numpy as np
import pytest

from helpers import make_boxes
from test_gpu_parity import assert_parity, run_both

pytestmark = pytest.mark.gpu

EDGES = [64, 128, 192, 256, 384, 512, 768, 1024, 1536, 2048, 3072, 4096]


def random_case(seed):
    rng = np.random.default_rng(90000 + seed)
    if seed % 3 == 0:                      # right at, just below or just above a boundary
        w = int(EDGES[rng.integers(len(EDGES))] + rng.integers(-2, 3))
    else:
        w = int(rng.integers(1, 4200 if seed % 7 == 0 else 1300))
    # keep the oracle's work bounded: about 60 k pixels per plane and filter at most
    h = int(rng.integers(1, max(2, min(260, 60000 // w + 2))))
    B, C, F = int(rng.integers(1, 3)), int(rng.integers(1, 3)), int(rng.integers(1, 13))
    while B * C * F * h * w > 400000 and F > 1:
        F -= 1
    kind = ("inside", "hanging", "integer", "large")[int(rng.integers(4))]
    normalize, exact = bool(rng.integers(2)), bool(rng.integers(2))
    return rng, (B, C, F, max(h, 1), max(w, 1)), kind, normalize, exact


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("seed", range(72))
def test_random_shape(hip, oracle, seed, dtype):
    rng, (B, C, F, h, w), kind, normalize, exact = random_case(seed)
    if kind in ("inside", "large") and (h < 6 or w < 6):
        kind = "hanging"
    x = (rng.standard_normal((B, C, h, w)) + (0.5 if seed % 5 == 0 else 0.0)).astype(dtype)
    g = rng.standard_normal((B, C * F, h, w)).astype(dtype)
    # whole-number bounds are where the reference's own splits are discontinuous: keep the other
    # kinds away from them so that a last-bit difference in a bound cannot flip a pixel
    boxes = tuple(b.astype(dtype) for b in
                  make_boxes(rng, C, F, h, w, kind, away_from_integers=0.0 if kind == "integer" else 0.01))
    cpu, gpu, sc = run_both(hip, oracle, x, boxes, float(h), float(w), normalize, exact, g)
    if np.isnan(cpu[0]).any():
        # a box that rounds to nothing, normalised (the module's clip excludes it): 0/0 on both sides
        assert np.isnan(gpu[0]).any()
        return
    assert_parity(cpu, gpu, dtype,
                  "seed %d: %s, %s boxes, normalize=%s exact=%s" % (seed, (B, C, F, h, w), kind, normalize, exact), **sc)
