"""The five synthetic BoxConv2d workloads the build is measured and parity-checked on.

Everything is generated on the host from fixed seeds (1000 + k for workload k), so the GPU run and
the CPU checker see identical bits. Parameters are returned in STORED (reparametrized) units, the
way ``BoxConv2d`` keeps them; ``real = stored * reparametrization``.

k = 1  MNIST-scale     BoxConv2d(1, 40, 28, 28),      x [32,1,28,28]      uniform[0,1), module-seeded boxes
k = 2  BoxENet block   BoxConv2d(32, 4, 128, 256),    x [4,32,128,256]    N(0,1), boxes inside +-h/2, +-w/2
k = 3  full-res layer  BoxConv2d(16, 8, 512, 1024),   x [2,16,512,1024]   N(0,1)          (headline)
k = 4  grad stress     BoxConv2d(64, 4, 64, 128),     x [8,64,64,128]     N(0,1)
k = 5  large boxes     BoxConv2d(128, 2, 1024, 2048), x [1,128,1024,2048] uniform[0,1)+10, boxes > 80 % of h, w
"""
import random
from collections import namedtuple

import numpy as np
import torch

Workload = namedtuple(
    "Workload",
    "k name B C F h w reparametrization_factor x grad_output x_min x_max y_min y_max "
    "reparametrization_h reparametrization_w")

SHAPES = {
    1: ("mnist_1x40_28x28_b32", 32, 1, 40, 28, 28),
    2: ("boxenet_32x4_128x256_b4", 4, 32, 4, 128, 256),
    3: ("fullres_16x8_512x1024_b2", 2, 16, 8, 512, 1024),
    4: ("gradstress_64x4_64x128_b8", 8, 64, 4, 64, 128),
    5: ("largebox_128x2_1024x2048_b1", 1, 128, 2, 1024, 2048),
}


def algorithmic_bytes(B, C, F, h, w, elem=4):
    """Minimal data flow of one forward+backward through the integral-image algorithm:
    4*(2*N_in + 3*N_int + 2*N_out + 2*N_gint) for float32, plus the compulsory-I/O figure."""
    n_in = B * C * h * w
    n_int = B * C * (h + 1) * (w + 1)
    n_out = F * n_in
    n_gint = F * n_int
    return {
        "alg": elem * (2 * n_in + 3 * n_int + 2 * n_out + 2 * n_gint),
        "io": elem * (2 * n_in + 2 * n_out),
        "n_in": n_in, "n_int": n_int, "n_out": n_out, "n_gint": n_gint,
    }


def _uniform_away_from_integers(rng, lo, hi, margin=0.01):
    while True:
        v = rng.uniform(lo, hi)
        if abs(v - round(v)) > margin:
            return v


def _seeded_boxes(rng, C, F, h, w, large):
    real = np.empty((4, C, F), dtype=np.float64)
    for c in range(C):
        for f in range(F):
            if large:
                x0 = _uniform_away_from_integers(rng, -0.49 * h, -0.41 * h)
                x1 = _uniform_away_from_integers(rng, 0.41 * h, 0.49 * h)
                y0 = _uniform_away_from_integers(rng, -0.49 * w, -0.41 * w)
                y1 = _uniform_away_from_integers(rng, 0.41 * w, 0.49 * w)
            else:
                x0 = _uniform_away_from_integers(rng, -h / 2, h / 2 - 3)
                x1 = _uniform_away_from_integers(rng, x0 + 1.5, h / 2)
                y0 = _uniform_away_from_integers(rng, -w / 2, w / 2 - 3)
                y1 = _uniform_away_from_integers(rng, y0 + 1.5, w / 2)
            real[:, c, f] = (x0, x1, y0, y1)
    return real


def make_workload(k, batch=None, in_planes=None, reparametrization_factor=8):
    """Host tensors of workload k. `batch` / `in_planes` shrink the workload to its first planes
    (same seeds, same boxes for the planes that remain) for a bounded CPU sample."""
    name, B, C, F, h, w = SHAPES[k]
    seed = 1000 + k
    gen = torch.Generator().manual_seed(seed)
    reparam_h = h * reparametrization_factor
    reparam_w = w * reparametrization_factor

    if k == 1:
        # the module's own initialisation under random.seed (BoxConv2d imports lazily so that
        # this file can be used without the HIP library present)
        from box_convolution import BoxConv2d
        state = random.getstate()
        random.seed(seed)
        module = BoxConv2d(C, F, h, w, reparametrization_factor)
        random.setstate(state)
        stored = [p.detach().clone() for p in (module.x_min, module.x_max, module.y_min, module.y_max)]
        x = torch.rand(B, C, h, w, generator=gen)
    else:
        rng = np.random.default_rng(seed)
        real = _seeded_boxes(rng, C, F, h, w, large=(k == 5))
        scales = (reparam_h, reparam_h, reparam_w, reparam_w)
        stored = [torch.from_numpy((real[i] / scales[i]).astype(np.float32)) for i in range(4)]
        if k == 5:
            x = torch.rand(B, C, h, w, generator=gen) + 10.0
        else:
            x = torch.randn(B, C, h, w, generator=gen)
    g = torch.randn(B, C * F, h, w, generator=gen)

    wl = Workload(k, name, B, C, F, h, w, reparametrization_factor, x, g, *stored,
                  reparam_h, reparam_w)
    if batch is not None or in_planes is not None:
        wl = restrict(wl, 0, C if in_planes is None else in_planes, batch)
    return wl


def restrict(wl, c0, c1, batch=None):
    """The input planes [c0, c1) (and the first `batch` batch items) of a workload: same data,
    same boxes for the planes that remain. Box convolution is independent per input plane and a
    parameter gradient only sums over the batch, so a checker run on the restricted workload
    reproduces exactly the matching slices of the full result."""
    b = wl.B if batch is None else batch
    F, h, w = wl.F, wl.h, wl.w
    x = wl.x[:b, c0:c1].contiguous()
    g = wl.grad_output.view(wl.B, wl.C, F, h, w)[:b, c0:c1].reshape(b, (c1 - c0) * F, h, w).contiguous()
    stored = [p[c0:c1].contiguous() for p in (wl.x_min, wl.x_max, wl.y_min, wl.y_max)]
    return wl._replace(B=b, C=c1 - c0, x=x, grad_output=g, x_min=stored[0], x_max=stored[1],
                       y_min=stored[2], y_max=stored[3])
