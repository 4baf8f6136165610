"""The five BASELINE workloads at full size on the GPU, through BoxConv2d (training mode, all
five gradients), against the CPU oracle.

Workloads 1, 2 and 4 are compared in full. Workloads 3 and 5 are compared on their first input
planes (box convolution is independent per input plane, and a parameter gradient only sums over
the batch, so the oracle restricted to planes [0, c) reproduces exactly those slices of the full
result), plus a size-independent property on the whole tensors: the adjoint identity
<boxconv(x), g> = <x, grad_input(g)>.

Tolerances: forward, grad_input 1e-4; parameter gradients 1e-3 (max|gpu-cpu| / max|cpu|).
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
    assert max(e_par) <= 1e-3
