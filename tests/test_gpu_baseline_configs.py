"""The five BASELINE workloads at full size on the GPU, through BoxConv2d (training mode, all
five gradients), against the CPU oracle.

Workloads 1 to 4 are compared in full. Workload 5 is compared on its first 16 of 128 input planes
(box convolution is independent per input plane, and a parameter gradient only sums over the
batch, so the oracle restricted to planes [0, c) reproduces exactly those slices of the full
result), plus a size-independent property on the whole tensors: the adjoint identity
<boxconv(x), g> = <x, grad_input(g)>.

Every run prints its measured errors; with BOXCONV_PARITY_REPORT=<file> they are appended to that
file as well (this is how profiles/parity_errors.txt is made).

Tolerances: forward, grad_input 1e-4; parameter gradients 1e-3 (max|gpu-cpu| / max|cpu|).

Workload 5 (inputs near 10.5, integral-image entries up to 2.2e7 where a float32 ulp is 2) is at
the precision limit of the float32 reference itself: its parameter gradients are differences of
two nearly equal terms (for a constant image the gradient of a normalised box vanishes), and the
reference's float32 result deviates from the same algorithm run in float64 by about 2e-3
(measured: y_max 1.8e-3), the GPU result by about 3e-4. There the GPU is held to 1e-3 against
the float64 oracle and must be at least as close to it as the float32 oracle is; its distance to
the float32 oracle is held to 1e-3 or, where the float32 oracle itself is further than that from
float64, to the sum of the two distances to float64 (nothing but the reference's own rounding
error may separate them).
"""
import os

import numpy as np
import pytest
import torch

from baseline_workloads import make_workload
from helpers import param_grad_floor, rel_err

pytestmark = pytest.mark.gpu

# planes the oracle is run on (None = all)
ORACLE_PLANES = {1: None, 2: None, 3: None, 4: None, 5: 16}


def report(line):
    print(line)
    path = os.environ.get("BOXCONV_PARITY_REPORT")
    if path:
        with open(path, "a") as fh:
            fh.write(line + "\n")


def run_gpu(wl):
    from box_convolution import BoxConv2d
    dev = torch.device("cuda:0")
    module = BoxConv2d(wl.C, wl.F, wl.h, wl.w, wl.reparametrization_factor).to(dev)
    stored = (wl.x_min, wl.x_max, wl.y_min, wl.y_max)
    with torch.no_grad():
        for p, v in zip((module.x_min, module.x_max, module.y_min, module.y_max), stored):
            p.copy_(v)
    module.train()
    x = wl.x.to(dev).requires_grad_(True)
    g = wl.grad_output.to(dev)
    out = module(x)
    for p, v in zip((module.x_min, module.x_max, module.y_min, module.y_max), stored):
        assert torch.equal(p.detach().cpu(), v), "workload boxes must survive clipping unchanged"
    out.backward(g)
    torch.cuda.synchronize()
    # adjoint identity on the full tensors, accumulated in float64 on the device
    lhs = (out.detach().double() * g.double()).sum().item()
    rhs = (x.detach().double() * x.grad.double()).sum().item()
    scale = (out.detach().double().abs() * g.double().abs()).sum().item()
    return (out.detach(), x.grad, [p.grad for p in (module.x_min, module.x_max, module.y_min, module.y_max)],
            (lhs, rhs, scale))


@pytest.mark.parametrize("k", [1, 2, 3, 4, 5])
def test_baseline_workload(oracle, k):
    wl = make_workload(k)
    out, gin, gpar, (lhs, rhs, scale) = run_gpu(wl)
    assert abs(lhs - rhs) <= 2e-5 * scale, "adjoint identity <y,g> = <x,grad_input>: %r vs %r" % (lhs, rhs)

    c = ORACLE_PLANES[k] or wl.C
    sub = make_workload(k, in_planes=c)
    args = [t.numpy() for t in (sub.x, sub.x_min, sub.x_max, sub.y_min, sub.y_max)]
    out_c, saved = oracle.module_forward(*args, sub.reparametrization_h, sub.reparametrization_w, True, True)
    grads_c = oracle.module_backward(saved, sub.grad_output.numpy(), sub.reparametrization_h,
                                     sub.reparametrization_w, True, True)

    F = wl.F
    e_out = rel_err(out[:, :c * F].cpu().numpy(), out_c)
    e_gin = rel_err(gin[:, :c].cpu().numpy(), grads_c[0])
    floor = param_grad_floor(grads_c[1:])
    e_par = [rel_err(gp[:c].cpu().numpy(), gc, floor) for gp, gc in zip(gpar, grads_c[1:])]
    report("workload %d (%s), oracle on %d of %d input planes: adjoint identity |lhs-rhs|/sum|terms| %.2e; "
           "max|gpu-cpu|/max|cpu|: forward %.2e grad_input %.2e grad_x_min %.2e grad_x_max %.2e "
           "grad_y_min %.2e grad_y_max %.2e"
           % (k, wl.name, c, wl.C, abs(lhs - rhs) / scale, e_out, e_gin, *e_par))
    assert e_out <= 1e-4
    assert e_gin <= 1e-4
    if k != 5:
        assert max(e_par) <= 1e-3
        return

    # workload 5: the same algorithm in float64 on the same (float32-rounded) real-unit boxes
    real = [(a.astype(np.float32) * np.float32(r)).astype(np.float64) for a, r in
            zip(args[1:], (sub.reparametrization_h,) * 2 + (sub.reparametrization_w,) * 2)]
    integ64 = oracle.integral_image(args[0].astype(np.float64))
    out64 = oracle.box_forward(integ64, *real, True, True)
    grads64 = oracle.box_backward(integ64, *real, sub.grad_output.numpy().astype(np.float64), out64,
                                  sub.reparametrization_h, sub.reparametrization_w, True, True)
    floor64 = param_grad_floor(grads64[1:])
    e_gpu64 = [rel_err(gp[:c].cpu().numpy(), g64, floor64) for gp, g64 in zip(gpar, grads64[1:])]
    e_cpu64 = [rel_err(gc, g64, floor64) for gc, g64 in zip(grads_c[1:], grads64[1:])]
    report("workload 5 parameter gradients vs the float64 oracle (x_min x_max y_min y_max): gpu %s ; "
           "float32 cpu oracle %s" % (" ".join("%.2e" % e for e in e_gpu64), " ".join("%.2e" % e for e in e_cpu64)))
    assert max(e_gpu64) <= 1e-3
    assert max(e_gpu64) <= max(max(e_cpu64), 1e-4)
    for e, eg, ec in zip(e_par, e_gpu64, e_cpu64):
        assert e <= max(1e-3, 1.05 * (eg + ec))
