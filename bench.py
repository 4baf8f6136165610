#!/usr/bin/env python3
"""Benchmark of the box-convolution hot path on one MI355X.

One step = BoxConv2d forward + backward (training mode: parameter clip, stored->real scaling,
integral image, box sampling; backward to the input and to all four box parameters) on the
headline workload: BoxConv2d(16, 8, 512, 1024), input float32 [2,16,512,1024], synthetic N(0,1)
data with seeded boxes, normalize=True, exact=True. Inputs are resident in HBM before timing.

Prints ONE JSON line. `value` is the effective bandwidth on the ALGORITHMIC byte count of one
step, 4*(2*N_in + 3*N_int + 2*N_out + 2*N_gint) bytes (each tensor of the integral-image data
flow moved once), divided by the measured time per step. `roofline` prices the dominant kernel
alone: its algorithmic bytes per launch over its average duration, taken with HIP events placed
around that kernel's launches on its stream during the timed steps (one launch in five, reported
as `launches_timed`: an event pair costs GPU time that would otherwise show up in `value`).
After the --warmup steps the script keeps stepping, untimed, until the step time has settled
(`prewarm_steps`); it then times --steps steps seven times over and reports the median region as
`ms_per_step` / `value`, with `ms_per_step_min` and `ms_per_step_max` beside it. `cpu_baseline` is the
reference's CPU path timed on this host on a bounded sample of the same workload.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload 1..5] [--no-cpu]

Other modes (never the default): --graph replays a captured HIP graph of the step's native calls;
--forward-only [--rounded] times the inference forward (eval mode, no autograd) on the forward's
own algorithmic bytes; `config.mode` and `metric` say which one a line came from.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "box-convolutions_amd"))

HBM_PEAK_GBS = 8000.0   # MI355X HBM3E
EVENT_EVERY = 5     # launches of the dominant kernel per HIP-event pair in the timed region
REPEATS = 7         # timed regions of --steps steps each; the median one is reported
PREWARM_MAX_S = 1.5 # upper bound on the untimed clock-up phase after --warmup
RANKING_STEPS = 3   # untimed eager steps per kernel name while the per-kernel times are taken
# every kernel a training step launches ("clip" is the parameter projection, which shares its
# launch with the marking of the single-pass integral image's hand-over words)
TIMED_KERNELS = ("grad_output_stream", "band_scan", "band_colsum", "forward_rows", "grad_input_cols", "clip")
METRIC = "BoxConv2d fwd+bwd ms/iter + effective HBM GB/s (% peak) at 2x16ch 512x1024 fp32"


def kernel_algorithmic_bytes(ab, elem=4):
    """Algorithmic bytes moved by ONE launch of each kernel at a given workload: the share of the
    step's data flow that the kernel is responsible for (each is launched once per step)."""
    return {
        "clip": 0,                                               # kilobytes of box parameters and marker words
        # read grad_output and the input's integral, write the (band-local) integral of grad_output
        "grad_output_stream": elem * (ab["n_out"] + ab["n_int"] + ab["n_gint"]),
        "band_scan": elem * (ab["n_in"] + ab["n_int"]),          # read input, write its integral
        "band_colsum": elem * ab["n_in"],                        # pre-pass over the input
        "forward_rows": elem * (ab["n_int"] + ab["n_out"]),      # read integral, write output
        "grad_input_cols": elem * (ab["n_gint"] + ab["n_in"]),   # read integral of grad_output, write grad_input
    }


def load_measured_traffic(kernel, workload_name):
    """HBM bytes per launch of `kernel` measured with rocprofv3 --pmc (FETCH_SIZE scaled by the
    copy-kernel factor, plus WRITE_SIZE), read from the summary recorded under profiles/ for this
    workload; None if there is none."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic_%s.txt" % workload_name)
    try:
        with open(path) as fh:
            for line in fh:
                parts = line.split()
                if parts and not line.startswith("#") and parts[0].startswith(kernel):
                    return int(parts[3])
    except (OSError, ValueError, IndexError):
        pass
    return None


def cpu_baseline(k, ab_full):
    """The reference's CPU kernels (oracle/_ref, built from the reference's own sources) or, where
    that library does not exist, the C++ restatement, timed on this host: whole steps of the same
    workload, repeated until at least 10 s of CPU work have been measured (at most 30 s)."""
    from baseline_workloads import SHAPES, make_workload
    from oracle import cpu_checker
    chk = cpu_checker.reference() or cpu_checker.oracle()
    name, B, C, F, h, w = SHAPES[k]
    # a step of the largest workloads takes minutes on one core: restrict those to their first
    # input planes (planes are independent and the reference's loops are single-threaded)
    full_px = B * C * F * h * w
    c = C
    while c > 1 and B * c * F * h * w > 150e6:
        c //= 2
    wl = make_workload(k, in_planes=c)
    args = [t.numpy() for t in (wl.x, wl.x_min, wl.x_max, wl.y_min, wl.y_max)]
    g = wl.grad_output.numpy()
    reps, total = 0, 0.0
    while reps < 1 or (total < 10.0 and total + total / reps < 30.0):
        t0 = time.perf_counter()
        out, saved = chk.module_forward(*args, wl.reparametrization_h, wl.reparametrization_w, True, True)
        chk.module_backward(saved, g, wl.reparametrization_h, wl.reparametrization_w, True, True)
        total += time.perf_counter() - t0
        reps += 1
    frac = (wl.B * wl.C * wl.F * wl.h * wl.w) / full_px
    step_s = total / reps / frac
    return {
        "value": ab_full["alg"] / step_s / 1e9,
        "unit": "GB/s",
        "cores": 1,
        "kind": chk.kind,
        "sample": "%d step(s) of %s%s, %.1f s of single-threaded CPU work in total, %.2f s per full step"
                  % (reps, name, "" if c == C else " restricted to its first %d of %d input planes" % (c, C),
                     total, step_s),
        "ms_per_step": 1e3 * step_s,
        "host_cpus": os.cpu_count(),
    }


def make_step(wl, dev):
    """(module, x, g, eager_step) for one workload, tensors resident on `dev`."""
    import torch
    from box_convolution import BoxConv2d
    module = BoxConv2d(wl.C, wl.F, wl.h, wl.w, wl.reparametrization_factor).to(dev)
    with torch.no_grad():
        for p, v in zip((module.x_min, module.x_max, module.y_min, module.y_max),
                        (wl.x_min, wl.x_max, wl.y_min, wl.y_max)):
            p.copy_(v)
    module.train()
    x = wl.x.to(dev).requires_grad_(True)
    g = wl.grad_output.to(dev)
    params = list(module.parameters())

    def eager_step():
        x.grad = None
        for p in params:
            p.grad = None
        out = module(x)
        out.backward(g)
    return module, x, g, eager_step


def capture_native_step(wl, module, x, g):
    """A HIP graph of the native calls of one training step (clip + integral image + forward,
    backward through the C ABI); returns (replay, keep_alive)."""
    import torch
    from box_convolution import _native
    stored = [p.detach() for p in (module.x_min, module.x_max, module.y_min, module.y_max)]
    x_static = x.detach()

    def native_step():
        integ, out, real = _native.training_forward(
            x_static, *stored, wl.reparametrization_h, wl.reparametrization_w, wl.h, wl.w, True, True)
        return out, _native.box_convolution_backward(
            integ, *real, g, None, wl.reparametrization_h, wl.reparametrization_w, True, True,
            True, True, True, True, True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        native_step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        keep_alive = native_step()
    return graph.replay, (graph, keep_alive)


def time_steps(step, steps, repeats):
    """Median, min, max seconds per region of `steps` steps between two synchronisations."""
    import torch
    regions = []
    for _ in range(repeats):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        regions.append(time.perf_counter() - t0)
    return sorted(regions)[len(regions) // 2], min(regions), max(regions)


def small_workload_extra(k, dev, steps=200):
    """Eager and captured-graph step time of a small workload (its kernels take tens of
    microseconds, so the eager figure is what the host can enqueue)."""
    import torch
    from baseline_workloads import algorithmic_bytes, make_workload
    wl = make_workload(k)
    module, x, g, eager_step = make_step(wl, dev)
    ab = algorithmic_bytes(wl.B, wl.C, wl.F, wl.h, wl.w)
    for _ in range(20):
        eager_step()
    eager, _, _ = time_steps(eager_step, steps, 3)
    replay, keep = capture_native_step(wl, module, x, g)
    for _ in range(20):
        replay()
    graph, _, _ = time_steps(replay, steps, 3)
    del keep
    # the inference forward of the same layer: module.eval(), no autograd
    module.eval()
    x_eval = x.detach()

    def eval_forward():
        with torch.no_grad():
            module(x_eval)
    for _ in range(20):
        eval_forward()
    infer, _, _ = time_steps(eval_forward, steps, 3)
    module.train()
    return {
        "workload": wl.name,
        "eager_ms_per_step": round(1e3 * eager / steps, 4),
        "graph_ms_per_step": round(1e3 * graph / steps, 4),
        "eager_GBps": round(ab["alg"] / (eager / steps) / 1e9, 1),
        "graph_GBps": round(ab["alg"] / (graph / steps) / 1e9, 1),
        "eager_over_graph": round(eager / graph, 2),
        "eval_forward_ms": round(1e3 * infer / steps, 4),
    }


def event_pair_overhead_ms(n=50):
    """What a pair of HIP events with nothing between them measures on the current stream."""
    import torch
    torch.cuda.synchronize()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for a, b in pairs:
        a.record()
        b.record()
    torch.cuda.synchronize()
    vals = sorted(a.elapsed_time(b) for a, b in pairs)
    return vals[len(vals) // 2]


def machine_probes(dev):
    """Rates of plain kernels on this machine, the yardsticks for the kernels' own rates."""
    import torch
    from box_convolution import _native

    def timed(fn, reps=20):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        times = []
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            e1.synchronize()
            times.append(e0.elapsed_time(e1) * 1e-3)
        return sorted(times)[len(times) // 2]

    print("plain kernels on one MI355X (median of 20 launches, HIP events around each; TB/s on the bytes named)")
    n = 512 * (1 << 20) // 4
    a = torch.randn(n, device=dev)
    b = torch.empty_like(a)
    c = torch.randn(n, device=dev)
    for name, fn, nbytes in (("torch sum, 512 MiB read", lambda: a.sum(), 4 * n),
                             ("torch copy_, 512 MiB read + 512 MiB written", lambda: b.copy_(a), 8 * n),
                             ("torch add, 2 x 512 MiB read + 512 MiB written", lambda: torch.add(a, c, out=b), 12 * n),
                             ("torch fill_, 512 MiB written", lambda: b.fill_(1.0), 4 * n)):
        t = timed(fn)
        print("%-72s %7.1f us  %.2f TB/s" % (name, t * 1e6, nbytes / t / 1e12))
    del a, b, c
    # the size of the headline's integral image: input planes in, integral planes out
    small_in = torch.randn(32, 512, 1024, device=dev)
    small_out = torch.empty_like(small_in)
    t = timed(lambda: small_out.copy_(small_in))
    print("%-72s %7.1f us  %.2f TB/s" % ("torch copy_, 64 MiB read + 64 MiB written (the integral image's bytes)",
                                         t * 1e6, 8 * small_in.numel() / t / 1e12))
    del small_in, small_out
    planes, h, w = 256, 512, 1024        # grad_output of the headline workload: 2 x 16 x 8 planes
    src = torch.randn(planes, h, w, device=dev)
    dst = torch.zeros(planes, h + 1, w, device=dev)
    nbytes = 8 * planes * h * w
    for rows, in_flight in ((64, 2), (64, 8), (32, 2), (16, 2), (8, 2), (8, 8)):
        t = timed(lambda: _native.probe_copy_bands(src, dst, rows, in_flight))
        print("%-72s %7.1f us  %.2f TB/s" % (
            "band copy of 256 planes of 512 x 1024 floats, %2d rows per workgroup, %d in flight" % (rows, in_flight),
            t * 1e6, nbytes / t / 1e12))
    assert torch.equal(dst[:, 1:], src)
    print("(the backward's streaming pass moves these 1074 MB plus 67 MB of integral images per launch, in "
          "workgroups of 64 rows)")
    del src, dst
    # the grad-input pass's loads and stores without its arithmetic, with the headline workload's boxes
    from baseline_workloads import make_workload
    wl = make_workload(3)
    x_lo = torch.ceil(-wl.x_max * wl.reparametrization_h).to(torch.int32).to(dev)
    x_hi = (torch.floor(-wl.x_min * wl.reparametrization_h) + 1).to(torch.int32).to(dev)
    planes = wl.B * wl.C
    m = torch.randn(planes, wl.F, wl.h + 1, wl.w, device=dev)
    out = torch.empty(planes, wl.h, wl.w, device=dev)
    m_bytes, out_bytes = 4 * m.numel(), 4 * out.numel()
    for mode, what in ((0, "both runs of 9 rows per filter (the kernel's pattern)"),
                       (1, "one run per filter: every row of the workspace read once"),
                       (2, "one run from the workspace, the other from a few MB resident in the L2")):
        t = timed(lambda: _native.probe_grad_input_pattern(m, out, x_lo, x_hi, mode))
        print("%-72s %7.1f us  %.2f TB/s" % ("grad-input pattern, " + what, t * 1e6, (m_bytes + out_bytes) / t / 1e12))
    print("(TB/s on the 537 MB of the column workspace read once plus the 67 MB written)")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", type=int, default=3, choices=[1, 2, 3, 4, 5])
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the eager/graph step time of the BoxENet-block workload (`extra`)")
    ap.add_argument("--phases", action="store_true", help="also print per-kernel times to stderr")
    ap.add_argument("--graph", action="store_true",
                    help="time replays of a captured HIP graph of the step's native calls (training "
                         "forward + backward through the C ABI) instead of the eager module step: "
                         "the same kernels without Python, autograd and launch latency, which bound "
                         "the small workloads")
    ap.add_argument("--shape", default=None, metavar="B,C,F,H,W",
                    help="instead of a baseline workload: batch B, C input planes, F filters per plane, "
                         "H x W images, N(0,1) data and the module's own seeded initial boxes (used for "
                         "shapes outside the five workloads, e.g. rows wider than 2048 columns; implies "
                         "--no-cpu)")
    ap.add_argument("--forward-only", action="store_true",
                    help="time the inference forward instead of the training step: module.eval(), no "
                         "autograd, out = module(x) (integral image + box sampling); `value` is then "
                         "the forward's algorithmic bytes 4*(N_in + 2*N_int + N_out) per second")
    ap.add_argument("--rounded", action="store_true",
                    help="with --forward-only: module.exact = False, the reference's fast inference "
                         "mode (box bounds rounded to whole pixels)")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MIB",
                    help="after the timed steps, run torch.neg on a float tensor of this many MiB "
                         "(reads MIB, writes MIB): the plain streaming kernel of known size that "
                         "the FETCH_SIZE / WRITE_SIZE counters are calibrated against")
    ap.add_argument("--machine-probes", action="store_true",
                    help="instead of a workload: what this machine's memory system gives plain kernels "
                         "(torch's sum, copy, add, fill on 512 MiB, and the library's band-wise copy with "
                         "the access pattern of the backward's streaming pass at the headline shape); "
                         "prints a table, not the JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; --gpus %d is not supported (box convolution "
                 "shards over batch and input planes with no exchange but a %d-float all-reduce, "
                 "which is outside this benchmark)" % (args.gpus, 4))

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    from baseline_workloads import algorithmic_bytes, make_workload
    from box_convolution import BoxConv2d, _native
    _native.load()

    dev = torch.device("cuda:0")
    if args.machine_probes:
        machine_probes(dev)
        return
    if args.shape:
        import random
        from baseline_workloads import Workload
        B, C, F, h, w = (int(v) for v in args.shape.split(","))
        state = random.getstate()
        random.seed(1234)
        init = BoxConv2d(C, F, h, w, 8)
        random.setstate(state)
        gen = torch.Generator().manual_seed(1234)
        wl = Workload(0, "custom_%dx%d_%dx%d_b%d" % (C, F, h, w, B), B, C, F, h, w, 8,
                      torch.randn(B, C, h, w, generator=gen), torch.randn(B, C * F, h, w, generator=gen),
                      *(p.detach().clone() for p in (init.x_min, init.x_max, init.y_min, init.y_max)),
                      h * 8, w * 8)
        args.no_cpu = True
    else:
        wl = make_workload(args.workload)
    ab = algorithmic_bytes(wl.B, wl.C, wl.F, wl.h, wl.w)

    module, x, g, eager_step = make_step(wl, dev)
    params = list(module.parameters())

    if args.forward_only:
        if args.graph:
            sys.exit("bench.py: --forward-only and --graph are separate modes")
        module.eval()
        module.exact = not args.rounded
        x.requires_grad_(False)
        # the forward's own data flow: input -> integral image -> output
        ab = dict(ab, alg=4 * (ab["n_in"] + 2 * ab["n_int"] + ab["n_out"]), io=4 * (ab["n_in"] + ab["n_out"]))

        def eager_step():
            with torch.no_grad():
                module(x)

    step = eager_step

    before = [p.detach().clone() for p in params]
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    for p, b in zip(params, before):
        assert args.shape or torch.equal(p.detach(), b), "workload boxes must be invariant under clipping"

    # A box that has just been handed over clocks up over the first milliseconds of work, and
    # --warmup steps of half a millisecond end before it has: go on with untimed blocks of steps
    # until two blocks in a row take the same time to 2 % (at most PREWARM_MAX_S seconds).
    def timed_block(n):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            step()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    prewarm_steps, last, t_start = 0, None, time.perf_counter()
    block = max(10, args.steps // 2)
    while time.perf_counter() - t_start < PREWARM_MAX_S:
        cur = timed_block(block)
        prewarm_steps += block
        if last is not None and abs(cur - last) <= 0.02 * last:
            break
        last = cur

    # which kernel takes the most time per step (RANKING_STEPS untimed eager steps per kernel
    # name). An event pair with nothing between its events already measures a few microseconds;
    # that is taken off every bracketed launch, so that the figures are the kernels' own time.
    pair_ms = event_pair_overhead_ms()
    per_kernel = {}
    for name in TIMED_KERNELS:
        _native.profile_arm(name)
        for _ in range(RANKING_STEPS):
            eager_step()
        ms, launches = _native.profile_collect()
        ms = max(ms - pair_ms * launches, 0.0)
        per_kernel[name] = (ms / RANKING_STEPS, launches // RANKING_STEPS, ms / max(launches, 1))
    dominant = max(per_kernel, key=lambda n: per_kernel[n][0])

    if args.graph:
        # the native calls of one step, captured once: clip + integral image + forward, backward
        replay, keep_alive = capture_native_step(wl, module, x, g)
        step = replay
        for _ in range(max(args.warmup, 5)):
            step()
        torch.cuda.synchronize()
    if args.phases:
        print("per-kernel ms per step:", {k: round(v[0], 4) for k, v in per_kernel.items()},
              file=sys.stderr)

    # ---- timed region ---------------------------------------------------------------------------
    # EXACTLY --steps steps between two synchronisations, REPEATS times over; ms_per_step (and
    # value) are the median region, the fastest and slowest are reported beside it.
    # An event pair around a kernel costs about 2.5 us of GPU time each side on this machine,
    # 1 % of a step: the dominant kernel is bracketed at one launch in EVENT_EVERY, so that the
    # whole-step figure is perturbed by a fraction of that.
    if not args.graph:
        _native.profile_arm(dominant, every=EVENT_EVERY)
    regions = [timed_block(args.steps) for _ in range(REPEATS)]
    if args.graph:
        # launches inside a replayed graph cannot be bracketed: the eager measurement above stands in
        dom_ms, dom_launches = per_kernel[dominant][2] * 3, 3
    else:
        dom_ms, dom_launches = _native.profile_collect()
        dom_ms = max(dom_ms - pair_ms * dom_launches, 0.0)
    elapsed = sorted(regions)[len(regions) // 2]

    if args.copy_probe > 0:
        src = torch.ones(args.copy_probe * (1 << 20) // 4, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.neg(src, out=dst)
        torch.cuda.synchronize()

    ms_per_step = 1e3 * elapsed / args.steps
    value = ab["alg"] / (elapsed / args.steps) / 1e9

    # (rows wider than 2048 columns run the grad_output pass as two launches: its bytes are then
    # priced against the time of both)
    launches_per_step = max(per_kernel[dominant][1], 1)
    bytes_per_launch = kernel_algorithmic_bytes(ab)[dominant] / launches_per_step
    avg_launch_s = dom_ms / 1e3 / max(dom_launches, 1)
    achieved = bytes_per_launch / avg_launch_s / 1e9

    result = {
        "metric": METRIC if not args.forward_only else
                  "BoxConv2d inference forward ms/iter + effective HBM GB/s (% peak) at 2x16ch 512x1024 fp32",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "ms_per_step_min": round(1e3 * min(regions) / args.steps, 4),
        "ms_per_step_max": round(1e3 * max(regions) / args.steps, 4),
        "timed_regions": REPEATS,
        "prewarm_steps": prewarm_steps,
        # every untimed step before the timed regions: --warmup, the clock-up phase, and the
        # RANKING_STEPS steps per kernel name during which the per-kernel times were taken
        "warmup_total": args.warmup + prewarm_steps + RANKING_STEPS * len(TIMED_KERNELS),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "%s: BoxConv2d(%d,%d,%d,%d) fwd+bwd, input [%d,%d,%d,%d], normalize, exact, "
                        "grads to input and 4 box parameters" % (
                            wl.name, wl.C, wl.F, wl.h, wl.w, wl.B, wl.C, wl.h, wl.w),
            "mode": ("inference forward, eval mode, %s box bounds" % ("rounded" if args.rounded else "exact")
                     if args.forward_only else
                     "captured HIP graph of the step's native calls" if args.graph else "eager module step"),
            "algorithmic_bytes_per_step": ab["alg"],
            "io_bytes_per_step": ab["io"],
            "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
            "io_GBps": round(ab["io"] / (elapsed / args.steps) / 1e9, 2),
        },
        "roofline": {
            "bound": "hbm",
            "kernel": dominant,
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": load_measured_traffic(dominant, wl.name),
            "traffic_source": "recorded rocprofv3 --pmc summary profiles/hbm_traffic_%s.txt "
                              "(not measured in this run)" % wl.name,
            "algorithmic_bytes_per_launch": int(bytes_per_launch),
            "avg_launch_us": round(1e6 * avg_launch_s, 2),
            "launches_timed": dom_launches,
        },
        # own time of every kernel of the step (HIP events around each launch, the empty event
        # pair's own reading taken off); their sum is what the step would take with no gaps
        "kernel_ms_per_step": {k: round(v[0], 4) for k, v in per_kernel.items()},
        "kernel_sum_ms": round(sum(v[0] for v in per_kernel.values()), 4),
        "event_pair_overhead_us": round(1e3 * pair_ms, 2),
    }
    if not (args.no_extra or args.graph or args.forward_only or args.shape):
        # the realistic layer shape of the reference's model zoo (a BoxENet block)
        result["extra"] = {"boxenet_block": small_workload_extra(2, dev)}
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(args.workload, ab)
        result["cpu_baseline"]["speedup_vs_cpu"] = round(result["cpu_baseline"]["ms_per_step"] / ms_per_step, 1)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
