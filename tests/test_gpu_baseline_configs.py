"""The five BASELINE workloads at full size on the GPU, through BoxConv2d (training mode, all
five gradients), against the CPU oracle.

Workloads 1, 2 and 4 are compared in full. Workloads 3 and 5 are compared on their first input
planes (box convolution is independent per input plane, and a parameter gradient only sums over
the batch, so the oracle restricted to planes [0, c) reproduces exactly those slices of the full
result), plus a size-independent property on the whole tensors: the adjoint identity
<boxconv(x), g> = <x, grad_input(g)>.

Tolerances: forward, grad_input 1e-4; parameter gradients 1e-3 (max|gpu-cpu| / max|cpu|).

Workload 5 (inputs near 10.5, integral-image entries up to 2.2e7 where a float32 ulp is 2) is at
the precision limit of the float32 reference itself: its parameter gradients are differences of
two nearly equal terms (for a constant image the gradient of a normalised box vanishes), and the
reference's float32 result deviates from the same algorithm run in float64 by about 2e-3
(measured: y_max 1.8e-3), the GPU result by about 3e-4. There the GPU is held to 1e-3 against
the float64 oracle, must be at least as close to it as the float32 oracle is, and to 4e-3
against the float32 oracle.
"""
import numpy as np
import pytest
import torch

from baseline_workloads import make_workload
from helpers import param_grad_floor, rel_err

pytestmark = pytest.mark.gpu

# planes the oracle is run on (None = all)
ORACLE_PLANES = {1: None, 2: None, 3: 2, 4: None, 5: 1}


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
    print("workload %d: forward %.2e grad_input %.2e grad_params %s" % (k, e_out, e_gin, ["%.2e" % e for e in e_par]))
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
    print("workload 5 vs float64 oracle: gpu %s  float32 oracle %s"
          % (["%.2e" % e for e in e_gpu64], ["%.2e" % e for e in e_cpu64]))
    assert max(e_gpu64) <= 1e-3
    assert max(e_gpu64) <= max(max(e_cpu64), 1e-4)
    assert max(e_par) <= 4e-3
