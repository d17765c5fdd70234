#!/usr/bin/env python3
"""Benchmark of the distance-neuron hot path on one MI355X.

A step is one training pass of the 5x5120 SortNet-MLP on a batch of 512 synthetic CIFAR-shaped
inputs (3072 features in [0,1], 10 classes): forward through the distance layers (l-inf on the
first layer, masked order-statistic neuron with q = 0.3 on the others) with mean shift, hinge
loss on the 1-Lipschitz margin, backward through every layer (grad_input and grad_weight),
AdamW update, and the interval-bound (certification) pass with eps = 8/255 through all layers.

Prints one JSON line.  `value` belongs to the mask named in config.workload (--mask); the same line carries,
under "secondary", short runs of the other formulations of the same step: the other mask granularity, the pure
l-inf net (q = 1), the reference's own index-list training form at its published keep probability (p = inf and
p = 8) with its certification pass, one l-p distance layer at p = 8 and p = 64, and the wide 64x64-image
configuration.  See --help for the knobs.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

FP32_VECTOR_PEAK_TFLOPS = 157.3     # MI355X published fp32 vector peak
NBATCH = 4                          # distinct synthetic batches cycled through the steps of the masked workload
VALU_LANE_RATE = 78.64e12           # 256 CUs x 4 SIMD x 16 lanes x 2 issue ports x 2.4 GHz lane-instructions/s
# HBM bytes of one 512x5120x5120 launch come from the committed counter summary (two rocprofv3 --pmc runs,
# FETCH_SIZE and WRITE_SIZE, scaled by a plain copy of known size): the lines "traffic_bytes_per_launch" (interval
# forward, every term) and "traffic_bytes_per_launch_masked_forward" (l-inf forward under the factored mask)
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "bench_headline_hbm_traffic.txt")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=8,
                    help="untimed steps; a layer's table hints settle within its first seven calls")
    ap.add_argument("--batch", type=int, default=512)
    ap.add_argument("--width", type=int, default=5120)
    ap.add_argument("--depth", type=int, default=6, help="distance layers incl. the class layer (reference: depth=6)")
    ap.add_argument("--in-features", type=int, default=3072)
    ap.add_argument("--classes", type=int, default=10)
    ap.add_argument("--q", type=float, default=0.3)
    ap.add_argument("--eps", type=float, default=8.0 / 255)
    ap.add_argument("--mask", choices=["term", "factored"], default="factored",
                    help="granularity of the Bernoulli keep mask of the masked neuron that `value` is measured with: "
                         "term = an independent draw per (b, m, n) term; factored = keep_x(b, n) & keep_w(m, n)")
    ap.add_argument("--workload", choices=["masked", "index-lists"], default="masked",
                    help="masked: the headline step (fused masked neuron).  index-lists: only the reference's own "
                         "training form (kept-channel lists per 32-sample sub-batch, SortMLPModel) and its certification "
                         "pass (sort neuron and interval sort neuron), without roofline / cpu_baseline")
    ap.add_argument("--p", type=float, default=float("inf"),
                    help="index-lists workload: norm of the distance layers during training (the reference anneals it from 8 to 1000, then inf)")
    ap.add_argument("--weight-std", type=float, default=None,
                    help="standard deviation of the initial weights of the masked workload (default fan_in ** -0.5; "
                         "the reference initialises with 1.0)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true", help="skip the short runs of the other formulations")
    ap.add_argument("--no-overlap", action="store_true",
                    help="queue forward, backward, optimizer and certification pass in turn on the one stream, instead of "
                         "the certification pass on a second stream beside forward and backward and the optimizer's "
                         "steps layer by layer on a third (per-kernel durations in a profiler trace are then those of "
                         "kernels that have the device to themselves)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run one plain device copy of a width x width fp32 matrix after the timed steps "
                         "(a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE counters with)")
    ap.add_argument("--cpu-batch", type=int, default=0, help="samples of the CPU baseline (0 = pick for 10-25 s)")
    return ap.parse_args()


def cpu_baseline(args, model_dims):
    """The CPU oracle timed on this host's cores on a bounded sample of the same step:
    `nb` samples through forward (+positions), scatter backward and interval bounds of every layer."""
    import numpy as np
    import oracle
    oracle.build()
    cores = os.cpu_count() or 1
    cores = min(cores, 16)
    oracle.set_num_threads(cores)
    rng = np.random.default_rng(0)
    ws = [(rng.standard_normal((o, i)) * i ** -0.5).astype(np.float32) for i, o in zip(model_dims[:-1], model_dims[1:])]

    def run(nb):
        x = rng.random((nb, model_dims[0], 1), dtype=np.float32)
        lo, up = np.maximum(x - np.float32(args.eps), 0), np.minimum(x + np.float32(args.eps), 1)
        t0 = time.perf_counter()
        h, saved = x, []
        for li, w in enumerate(ws):
            if li == 0 or args.q >= 1.0:
                y, pos = oracle.inf_dist_forward(h, w)
            else:
                y, pos = oracle.masked_inf_dist_forward(h, w, args.q, li, oracle.MASK_TERM if args.mask == "term" else oracle.MASK_FACTORED)
            saved.append((h.shape, pos))
            h = y - y.mean(axis=(0, 2), keepdims=True) if li < len(ws) - 1 else y
        g = np.ones_like(h)
        for li in reversed(range(len(ws))):
            g, _ = oracle.inf_dist_backward(g, saved[li][1], saved[li][0], ws[li].shape)
        for li, w in enumerate(ws):
            lo, up = oracle.bound_inf_dist_forward(lo, up, w, need_pos=False)
        return time.perf_counter() - t0

    nb = args.cpu_batch
    if nb <= 0:
        t = run(2)
        nb = int(max(2, min(args.batch, 25.0 / max(t / 2, 1e-6))))
    t = run(nb)
    return {"value": nb / t, "unit": "samples/s", "cores": cores, "kind": "port",
            "sample": "%d samples through the same step (oracle forward+positions, scatter backward, interval "
                      "bounds of all %d layers; no optimizer), %.1f s" % (nb, len(ws), t)}


def run_index_lists(args, q, p, steps, warmup, certify_runs=0):
    """Training step of SortMLPModel in the reference's index-list form and, when asked for, the certification pass
    of the same model in evaluation mode (sort neuron for the value, interval sort neuron for the bounds)."""
    import torch
    from sortnet_amd.ell_inf_models import SortMLPModel
    from sortnet_amd.layers import DropoutRegistry, NormDistBase, set_mask_seed
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    reg = DropoutRegistry()
    torch.manual_seed(0)
    side = int(round((args.in_features / 3) ** 0.5))
    assert 3 * side * side == args.in_features, "--in-features must be 3 x side x side for this workload"
    net = SortMLPModel(args.depth, args.width, (3, side, side), num_classes=args.classes, dropout=q,
                       registry=reg).to(dev)
    opt = torch.optim.AdamW(net.parameters(), lr=1e-4, fused=True)
    dist_layers = [m for m in net.modules() if isinstance(m, NormDistBase)]

    def set_p(v):
        for m in dist_layers:
            m.p = v

    g = torch.Generator().manual_seed(0)
    x = torch.rand(args.batch, 3, side, side, generator=g).to(dev)
    t = torch.randint(0, args.classes, (args.batch,), generator=g).to(dev)
    up, down = torch.ones_like(x), torch.zeros_like(x)
    set_mask_seed(1, reg)

    def train_step():
        net.train()
        set_p(p)
        loss = torch.nn.functional.cross_entropy(net(x), t)
        opt.zero_grad(set_to_none=True)
        loss.backward()
        opt.step()

    def certify():
        net.eval()
        set_p(float("inf"))
        with torch.no_grad():
            return net(x, targets=t, eps=args.eps, up=up, down=down)

    def timed(fn, n):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n

    for _ in range(warmup):
        train_step()
    step_s = timed(train_step, steps)
    out = {"ms_per_step": step_s * 1e3, "samples_per_s": args.batch / step_s, "steps": steps,
           "workload": "SortMLPModel depth %d width %d, B=%d, keep probability %.2f, p=%g: forward + cross entropy + "
                       "backward + AdamW through kept-channel index lists (the reference's training form)"
                       % (args.depth, args.width, args.batch, q, p)}
    if certify_runs:
        certify()
        cert_s = timed(certify, certify_runs)
        out["certification_ms"] = cert_s * 1e3
    del net, opt
    torch.cuda.empty_cache()
    return out


_EXTRA_STREAMS = {}


def extra_streams(dev):
    """The two streams (default priority) beside torch's current one that the overlapped step uses, made once per
    process: the runtime deals streams to a few hardware queues in the order they are made, and two streams that
    share a queue do not overlap, so every run of the step uses the same two."""
    import torch
    if dev not in _EXTRA_STREAMS:
        _EXTRA_STREAMS[dev] = (torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev))
    return _EXTRA_STREAMS[dev]


def run_masked(args, mask, q, steps, warmup, batch=None, in_features=None, width=None, classes=None, eps=None,
               time_ibp=False, calib_copy=False, weight_std=None, overlap=None, pipeline=None, stages=None):
    """K timed steps of the fused-mask formulation; returns timings, phase split and the per-launch events of the
    interval-bound forward of the width x width layers."""
    import torch
    from sortnet_amd import ext, _lib
    from sortnet_amd.model import DistanceMLP, margins, hinge_loss
    overlap = (not args.no_overlap) if overlap is None else overlap
    pipeline = overlap if pipeline is None else (pipeline and overlap)
    batch = batch or args.batch
    in_features = in_features or args.in_features
    width = width or args.width
    classes = classes or args.classes
    eps = args.eps if eps is None else eps
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    mode = ext.MASK_TERM if mask == "term" else ext.MASK_FACTORED
    model = DistanceMLP(in_features, width, args.depth, classes, q=q, device=dev, seed=0, mask_mode=mode,
                        weight_std=weight_std)
    # AdamW couples no two parameters, so one optimizer per layer (the class layer's with the bias) takes the same
    # steps as one over all of them; with `pipeline` they are queued layer by layer on a stream of their own
    if pipeline:
        # three steps: the first layer's, the second layer's, and the rest in one (measured: the next step's first
        # two layers are enough to hide the rest's update, and fewer optimizer calls cost the host less)
        stages = stages or [st for st in ([0], [1], list(range(2, model.num_layers))) if st and st[0] < model.num_layers]
        groups = [[model.weights[i] for i in st] + ([model.bias] if model.num_layers - 1 in st else []) for st in stages]
    else:
        groups = [model.parameters()]
    opts = [torch.optim.AdamW(g, lr=1e-4, fused=True) for g in groups]
    # NBATCH distinct synthetic batches, step i takes batch i % NBATCH: the candidate tables and their hints see new
    # inputs every step, as in training
    g = torch.Generator().manual_seed(0)
    batches = []
    for _ in range(NBATCH):
        bx = torch.rand(batch, in_features, generator=g).to(dev)
        bt = torch.randint(0, classes, (batch,), generator=g).to(dev)
        batches.append((bx, bt, (bx - eps).clamp(min=0), (bx + eps).clamp(max=1)))

    ev = lambda: torch.cuda.Event(enable_timing=True)
    phase_ms = {"forward": 0.0, "backward": 0.0, "optimizer": 0.0, "bounds": 0.0}
    ibp_events = []
    ibp_kernel = [None]          # the tile kernel the library dispatched for the width x width interval layers
    probe = []                   # operands of the last width x width interval layer of the last step
    dense_ms = []                # every-term interval kernel, per launch
    fwd_ms, fwd_kernel = [], [None]   # masked l-inf forward tile kernel, per launch
    # per layer: the share of its terms that the forward / the interval forward formed (1 = every term), read from
    # the candidate-table counters in the extra one-stream steps
    fwd_share = [[] for _ in range(model.num_layers)]
    ibp_share = [[] for _ in range(model.num_layers)]

    # The certification pass needs the weights and nothing of the training step, so it is queued on a second stream
    # (default priority) beside forward and backward, on the weights the forward uses and a snapshot of the running
    # means; the optimizer waits for it before it changes the weights.  Its small kernels (tables, fills, shifts) and
    # the partly filled last rounds of workgroups of either stream then fill each other's gaps.
    #
    # With `pipeline` the optimizer's steps, layer by layer on a third stream, wait for the backward and for the
    # certification pass and each leaves an event; the next step's forward and certification pass wait for layer i's
    # event right before they read layer i's weights.  The update of the later layers, a stream of reads and writes to HBM,
    # then runs beside the next step's first layers, which are bound by the vector units.
    main = torch.cuda.current_stream(dev)
    side, upd_stream = extra_streams(dev) if overlap else (None, None)
    updated = [None] * model.num_layers          # per layer: the event after its last queued update

    def wait_updated(stream):
        def hook(i):
            if updated[i] is not None:
                stream.wait_event(updated[i])
        return hook

    def certification(timed, means, lower, upper, before_layer=None):
        if timed and time_ibp:
            # the pass spelled out, to time every call of the interval forward of a width x width layer with events on
            # the stream it is queued on (torch's current stream)
            lo, up = lower.unsqueeze(-1).contiguous(), upper.unsqueeze(-1).contiguous()
            with torch.no_grad():
                for li, w in enumerate(model.weights):
                    ylo = torch.empty(lo.size(0), w.size(0), 1, device=dev)
                    yup = torch.empty_like(ylo)
                    e0, e1 = ev(), ev()
                    e0.record()
                    ext.bound_inf_dist_forward_nograd(lo, up, w, ylo, yup, 1)
                    e1.record()
                    ibp_share[li].append(_lib.last_forward_term_share())
                    if w.size(0) == width and w.size(1) == width:
                        ibp_events.append((e0, e1))
                        probe[:] = [lo, up, w]
                    shift = (means[li].view(1, -1, 1) if li < model.num_layers - 1 else -model.bias.view(1, -1, 1))
                    lo, up = ylo - shift, yup - shift
            return lo.squeeze(-1), up.squeeze(-1)
        return model.bounds(lower, upper, means=means, before_layer=before_layer)

    def step(i, timed, after_layer=None, concurrent=None):
        x, targets, lower, upper = batches[i % NBATCH]
        concurrent = overlap if concurrent is None else concurrent
        piped = pipeline and concurrent
        if pipeline and not piped:
            main.wait_stream(upd_stream)                 # a step on one stream after pipelined ones
            updated[:] = [None] * len(updated)
        marks = [ev() for _ in range(7)]
        marks[0].record()
        if concurrent:
            means = [m.clone() for m in model.running_mean]
            side.wait_stream(main)                       # the snapshot; without `pipeline` also the previous step's optimizer
            with torch.cuda.stream(side):
                marks[5].record()
                lo, up = certification(timed, means, lower, upper, wait_updated(side) if piped else None)
                marks[6].record()
        dist = model.forward(x, step_seed=i, after_layer=after_layer,
                             before_layer=wait_updated(main) if piped else None)
        logits, worst = margins(dist, targets, eps)
        loss = hinge_loss(worst)
        marks[1].record()
        # (with `pipeline` the forward has waited for every layer's update by now, so the optimizer is done with the
        # gradients that are freed here)
        for opt in opts:
            opt.zero_grad(set_to_none=True)
        loss.backward()
        marks[2].record()
        if piped:
            upd_stream.wait_stream(main)                 # the gradients
            upd_stream.wait_stream(side)                 # the certification pass has read the weights
            with torch.cuda.stream(upd_stream):
                for st, opt in zip(stages, opts):
                    opt.step()
                    e = torch.cuda.Event()
                    e.record()
                    for li in st:
                        updated[li] = e
                marks[3].record()
        if concurrent:
            main.wait_stream(side)                       # the certification pass has read the weights
            lo.record_stream(main)
            up.record_stream(main)
        if not piped:
            for opt in opts:
                opt.step()
            marks[3].record()
        if not concurrent:
            marks[5].record()
            lo, up = certification(timed, model.running_mean, lower, upper)
            marks[6].record()
        cert = margins(dist.detach(), targets, eps, lo, up)[1]
        marks[4].record()
        return marks, loss, cert

    for i in range(warmup):
        step(i, False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    all_marks, trace = [], []
    for i in range(steps):
        marks, loss, cert = step(warmup + i, False)
        all_marks.append(marks)
        trace.append((loss.detach(), cert))      # read after the timed region
    queued = time.perf_counter() - t0
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    loss_trace = [float(l) for l, _ in trace]
    margin_trace = [float(c.double().sum()) for _, c in trace]
    del trace

    if time_ibp:
        # A few more steps on one stream, not part of `value`, for the figures about single kernels and calls: the
        # interval forward of every width x width layer between two events (roofline's in_step), and - the kernel with
        # the largest share of the step - the masked l-inf forward with chunk tracking of those layers by the library's
        # events around the tile kernel's launch, read back after every such layer (which makes the host wait).
        def read_timer(i, w):
            fwd_share[i].append(_lib.last_forward_term_share())
            if i > 0 and tuple(w.shape) == (width, width):
                ms = _lib.last_forward_kernel_ms()
                if ms is not None:
                    fwd_ms.append(ms)
                    fwd_kernel[0] = _lib.last_forward_kernel()

        _lib.time_forward_kernels(True)
        try:
            for k in range(max(4, steps // 4)):
                step(warmup + steps + k, True, after_layer=read_timer, concurrent=False)
        finally:
            _lib.time_forward_kernels(False)
        torch.cuda.synchronize()

    if time_ibp and probe:
        # The interval forward picks, on the device, between a kernel that evaluates only the inputs a table marks
        # and the kernel that evaluates every term.  The roofline entry is about the latter (its flops are the
        # algorithmic ones): the same call on the operands of the step's last width x width layer with the table
        # switched off, every launch between two events on the stream it is queued on.
        lo, up, w = probe
        ylo = torch.empty(lo.size(0), w.size(0), 1, device=dev)
        yup = torch.empty_like(ylo)
        _lib.set_bound_candidate_density(0.0)
        _lib.time_forward_kernels(True)      # events around the tile kernel's own launch, on the stream it is queued on
        try:
            with torch.no_grad():
                for k in range(2 + max(8, steps)):
                    ext.bound_inf_dist_forward_nograd(lo, up, w, ylo, yup, 1)
                    ms = _lib.last_forward_kernel_ms()
                    if k >= 2 and ms is not None:
                        dense_ms.append(ms)
            ibp_kernel[0] = _lib.last_forward_kernel()
        finally:
            _lib.set_bound_candidate_density(-1.0)
            _lib.time_forward_kernels(False)
        torch.cuda.synchronize()

    if calib_copy:
        src = model.weights[1]
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    for marks in all_marks:
        phase_ms["forward"] += marks[0].elapsed_time(marks[1]) / steps
        phase_ms["backward"] += marks[1].elapsed_time(marks[2]) / steps
        phase_ms["optimizer"] += marks[2].elapsed_time(marks[3]) / steps   # with `pipeline`: on its own stream, beside the next step
        phase_ms["bounds"] += marks[5].elapsed_time(marks[6]) / steps      # on its own stream with `overlap`
    mean = lambda v: sum(v) / len(v) if v else 1.0
    layer_terms = [w.numel() * batch for w in model.weights]
    executed = {"forward_terms": sum(t * mean(sh) for t, sh in zip(layer_terms, fwd_share)),
                "interval_terms": sum(t * mean(sh) for t, sh in zip(layer_terms, ibp_share)),
                "forward_share_by_layer": [mean(sh) for sh in fwd_share],
                "interval_share_by_layer": [mean(sh) for sh in ibp_share]} if time_ibp else None
    res = {
        "executed": executed,
        "ms_per_step": elapsed * 1e3 / steps, "samples_per_s": batch / (elapsed / steps), "steps": steps,
        "host_ms_per_step": queued * 1e3 / steps,      # the host's time to queue a step
        "phase_ms": phase_ms, "terms_per_step": model.terms_per_sample() * batch,
        "ibp_launch_ms": [a.elapsed_time(b) for a, b in ibp_events], "ibp_kernel": ibp_kernel[0],
        "ibp_every_term_ms": dense_ms, "fwd_kernel_ms": fwd_ms, "fwd_kernel": fwd_kernel[0],
        "loss": float(loss.detach()), "certified_frac": float((cert.max(dim=1)[0] < 0).float().mean()),
        # per timed step: the training loss, and the sum of the certification pass's worst-case margins
        "loss_trace": loss_trace, "margin_trace": margin_trace,
    }
    del model, opts
    torch.cuda.empty_cache()
    return res


def committed_traffic(key):
    """The figure `key` of the committed counter summary, or None."""
    try:
        m = re.search(r"^%s:\s*([0-9.eE+]+)" % key, open(TRAFFIC_PROFILE).read(), re.M)
        return float(m.group(1)) if m else None
    except OSError:
        return None


def workload_text(args, mask, q):
    return ("SortNet-MLP training step: %d->%s->%d distance layers, B=%d, q=%.2f (%s), "
            "forward+hinge loss+backward+AdamW+interval bounds eps=%.4f, weights ~ N(0, %s)"
            % (args.in_features, "x".join([str(args.width)] * (args.depth - 1)), args.classes, args.batch, q,
               "no mask: pure l-inf net" if q >= 1.0 else
               ("independent Bernoulli draw per term" if mask == "term" else
                "factored mask keep_x(b,n)&keep_w(m,n), each output a max over a Bernoulli(q) subset"), args.eps,
               "1/fan_in" if args.weight_std is None else "%g^2" % args.weight_std))


def run_lp_layer(args, p, steps, warmup):
    """One l-p distance layer of the headline width: forward, backward (grad_input and grad_weight) and the batch
    mean shift of the output, inputs ~ N(0, 1) and weights ~ N(0, 1/N) (the p-annealing phase of training)."""
    import torch
    from sortnet_amd import ext
    dev = torch.device("cuda:0")
    B, N = args.batch, args.width
    g = torch.Generator().manual_seed(0)
    x = torch.randn(B, N, 1, generator=g).to(dev)
    w = (torch.randn(N, N, generator=g) * N ** -0.5).to(dev)
    gy = torch.randn(B, N, 1, generator=g).to(dev)
    y, ys = torch.empty(B, N, 1, device=dev), torch.empty(B, N, 1, device=dev)
    mean = torch.empty(N, device=dev)
    gx, gw = torch.empty_like(x), torch.empty_like(w)

    def step():
        ext.norm_dist_forward(x, w, y, 1, p)
        ext.mean_shift_forward(y, mean, None, 0.1, ys)
        ext.norm_dist_backward_input_weight(gy, x, w, y, gx, gw, 1, p)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    return {"ms_per_step": ms, "samples_per_s": B / (ms * 1e-3), "steps": steps,
            "workload": "one l-p distance layer %dx%dx%d at p=%g: forward + mean shift + backward (input and weight), "
                        "x~N(0,1), w~N(0,1/N)" % (B, N, N, p)}


def run_interval_layer(args, steps, warmup):
    """One interval layer of the headline width as certified training differentiates it: forward with positions and
    backward (both input gradients and grad_weight), on bounds that are alike from sample to sample (those of a hidden
    layer) and weights ~ N(0, 1/N)."""
    import torch
    from sortnet_amd import ext
    dev = torch.device("cuda:0")
    B, N = args.batch, args.width
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1, N, 1, generator=g) * 0.02 + torch.randn(B, N, 1, generator=g) * 0.004
    r = 0.02 + torch.rand(B, N, 1, generator=g) * 0.002
    xl, xu = (x - r).contiguous().to(dev), (x + r).contiguous().to(dev)
    w = (torch.randn(N, N, generator=g) * N ** -0.5).to(dev)
    gl, gu = torch.randn(B, N, 1, generator=g).to(dev), torch.randn(B, N, 1, generator=g).to(dev)
    yl, yu = torch.empty(B, N, 1, device=dev), torch.empty(B, N, 1, device=dev)
    pl = torch.empty(B, N, 1, device=dev, dtype=torch.int32)
    pu = torch.empty_like(pl)
    gxl, gxu, gw = torch.empty_like(xl), torch.empty_like(xu), torch.empty_like(w)

    def step():
        ext.bound_inf_dist_forward(xl, xu, w, yl, yu, pl, pu, 1)
        ext.bound_inf_dist_backward_input_weight(gl, gu, pl, pu, gxl, gxu, gw, 1)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    return {"ms_per_step": ms, "samples_per_s": B / (ms * 1e-3), "steps": steps,
            "workload": "one interval layer %dx%dx%d with positions: forward + backward (both inputs and weight), "
                        "bounds alike from sample to sample, w~N(0,1/N)" % (B, N, N)}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (no collective path exists); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import torch
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.workload == "index-lists":
        r = run_index_lists(args, args.q, args.p, args.steps, args.warmup, certify_runs=max(2, args.steps // 4))
        print(json.dumps({
            "metric": "train samples/s, SortMLPModel in the reference's index-list form", "value": r["samples_per_s"],
            "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": r["ms_per_step"],
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": r["workload"]}, "certification_ms": r["certification_ms"]}))
        return

    head = run_masked(args, args.mask, args.q, args.steps, args.warmup, time_ibp=True, calib_copy=args.calib_copy,
                      weight_std=args.weight_std)
    step_s = head["ms_per_step"] * 1e-3
    step_flops = head["terms_per_step"] * (2 + 6)         # forward 2 flops/term, interval bounds 6 flops/term
    ex = head["executed"]
    executed_flops = 2.0 * ex["forward_terms"] + 6.0 * ex["interval_terms"] if ex else None
    layer_terms = args.batch * args.width * args.width
    launches, dense, fwd = head["ibp_launch_ms"], head["ibp_every_term_ms"], head["fwd_kernel_ms"]
    step_ms = sum(launches) / max(len(launches), 1)
    ibp_ms = sum(dense) / max(len(dense), 1)
    fwd_ms = sum(fwd) / max(len(fwd), 1)
    at_size = (args.batch, args.width) == (512, 5120)
    factored = args.mask == "factored"
    interval = {
        "kernel": "sd::%s, policy BoundNograd (interval-bound forward, every term, %dx%dx%d)" % (head["ibp_kernel"], args.batch, args.width, args.width),
        "achieved": 6.0 * layer_terms / (ibp_ms * 1e-3) / 1e12 if dense else None, "unit": "TFLOP/s",
        "frac": 6.0 * layer_terms / (ibp_ms * 1e-3) / 1e12 / FP32_VECTOR_PEAK_TFLOPS if dense else None,
        "traffic": committed_traffic("traffic_bytes_per_launch") if at_size else None,
        "algorithmic_bytes": 4.0 * (args.width * args.width + 4 * args.batch * args.width),
        "avg_launch_ms": ibp_ms if dense else None, "launches_timed": len(dense),
        "valu_issue_frac": 4.0 * layer_terms / (ibp_ms * 1e-3) / VALU_LANE_RATE if dense else None,
        "in_step": {
            "avg_call_ms": step_ms if launches else None, "calls_timed": len(launches),
            "algorithmic_tflops": 6.0 * layer_terms / (step_ms * 1e-3) / 1e12 if launches else None,
            "note": "the same entry point as the steps call it on their width x width layers (timed in a few further "
                    "steps that queue everything on one stream): a table of the "
                    "inputs that can hold a maximum (per weight row and tile of 128 batch rows) is built first and a "
                    "count taken on the device picks the table kernel or the every-term kernel; terms that cannot "
                    "hold a maximum are never formed, so this rate is not bounded by the vector peak",
        },
        "note": "6 flops per term in 4 VALU instructions; a register-only stream of this mix reaches 72 T "
                "lane-instructions/s on this part (floor 56 fs/term = 69% of peak) and the part sustains ~2.0 of its "
                "2.4 GHz under this kernel; the step itself takes this entry point's results from candidate tables "
                "(in_step), so these launches are queued after the steps, on the operands of their last width x width "
                "layer with the table switched off",
    }
    if fwd and args.q < 1.0:
        achieved = 2.0 * layer_terms / (fwd_ms * 1e-3) / 1e12
        roofline = {
            "bound": "valu",
            "kernel": "sd::%s, policy %s (l-inf forward %s with the winning chunk tracked for the positions, every "
                      "term, %dx%dx%d)" % (head["fwd_kernel"],
                                           "LinfChunkPacked" if factored else "MaskedTermChunk",
                                           "under the %s mask" % args.mask,
                                           args.batch, args.width, args.width),
            "achieved": achieved, "peak": FP32_VECTOR_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": achieved / FP32_VECTOR_PEAK_TFLOPS,
            "traffic": committed_traffic("traffic_bytes_per_launch_masked_forward") if at_size and factored else None,
            "algorithmic_bytes": 4.0 * (args.width * args.width + 3 * args.batch * args.width),
            "avg_launch_ms": fwd_ms, "launches_timed": len(fwd),
            "valu_issue_frac": 1.5 * layer_terms / (fwd_ms * 1e-3) / VALU_LANE_RATE if factored else None,
            "note": ("the kernel with the largest share of the step (four launches, about 30 %); tropical (sub/max) "
                     "contraction on the fp32 vector ALUs, not MFMA: 2 flops per term in 1.5 VALU instructions (one "
                     "subtraction, half a three-operand maximum), so a register-only stream at the part's 72 T "
                     "lane-instructions/s would give 61 % of the peak; " if factored else
                     "the kernel with the largest share of the step; 2 flops per term, and the keep decision of every "
                     "term comes from a counter hash that costs more than the term; ") +
                    "timed by events around the kernel's own launch (sd_time_forward_kernels) in a few further steps "
                    "after the timed ones, every width x width layer; those steps queue everything on one stream, so "
                    "that the kernel has the device to itself as in a profiler trace of --no-overlap",
            "interval_every_term": interval,
        }
    else:   # q = 1: no masked layers (and most l-inf layers are served from candidate tables); the interval kernel is the one to report
        roofline = dict(interval, bound="valu", peak=FP32_VECTOR_PEAK_TFLOPS)
    out = {
        "metric": "train samples/s (fwd+bwd+IBP) 5x5120 SortNet-MLP, B=512; % FP32 VALU peak",
        "value": head["samples_per_s"], "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": workload_text(args, args.mask, args.q),
                   "batch": args.batch, "width": args.width, "distance_layers": args.depth, "mask": args.mask,
                   "streams": 1 if args.no_overlap else 3},
        # ALGORITHMIC rate: 2 flops per forward term and 6 per interval term for EVERY term of every layer, over the
        # step time and the fp32 vector peak.  Not a utilisation: the step forms only the terms its candidate tables
        # mark (`executed`), so this figure can exceed what the vector units deliver.
        "step_algorithmic_rate_vs_fp32_peak": step_flops / step_s / (FP32_VECTOR_PEAK_TFLOPS * 1e12),
        # the same from the terms the step actually formed (table marks read back from the device in a few further
        # one-stream steps): what the vector units really did per second of the step, against their peak
        "step_executed_rate_vs_fp32_peak": (executed_flops / step_s / (FP32_VECTOR_PEAK_TFLOPS * 1e12)
                                            if executed_flops else None),
        "executed": head["executed"],
        "phase_ms": head["phase_ms"],
        "phase_note": ("the certification pass (bounds) is queued on a second stream beside forward and backward, on "
                       "the weights the forward uses; the optimizer, layer by layer on a third stream, waits for both, "
                       "and the next step's forward and certification pass wait for a layer's update right before they "
                       "read that layer's weights: the phases overlap and do not add up to ms_per_step, and each is "
                       "longer than alone because they share the device"
                       if not args.no_overlap else "one stream: forward, backward, optimizer, certification pass in turn"),
        "roofline": roofline,
        "loss": head["loss"], "certified_frac": head["certified_frac"],
    }

    if not args.no_secondary:
        sec = {}
        short, warm = max(3, args.steps // 4), 8   # a layer's table hints settle within its first seven calls

        def masked_entry(mask, q, steps=short, warmup=warm, **kw):
            r = run_masked(args, mask, q, steps, warmup, **kw)
            return {"ms_per_step": r["ms_per_step"], "samples_per_s": r["samples_per_s"], "steps": steps,
                    "phase_ms": r["phase_ms"]}

        # the same step with every candidate table switched off: each kernel forms every term, whatever the data
        from sortnet_amd import _lib
        setters = (_lib.set_bound_candidate_density, _lib.set_linf_candidate_density, _lib.set_sort_candidate_density,
                   _lib.set_lp_candidate_density)
        try:
            for f in setters:
                f(0.0)
            sec["tables_off"] = dict(masked_entry(args.mask, args.q),
                                     workload=workload_text(args, args.mask, args.q) + "; candidate tables off: every "
                                     "kernel evaluates every term (the data-independent floor of `value`)")
        finally:
            for f in setters:
                f(-1.0)
        other = "term" if args.mask == "factored" else "factored"
        sec[other + "_mask"] = dict(masked_entry(other, args.q), workload=workload_text(args, other, args.q))
        sec["q1"] = dict(masked_entry(args.mask, 1.0), workload=workload_text(args, args.mask, 1.0))
        # the same step from the reference's own initialisation (weights of unit scale, core/models/norm_dist.py:30)
        # (enough steps for the layers to have settled on their kernels: a layer reports three calls before it switches)
        sec["unit_weights"] = dict(masked_entry(args.mask, args.q, steps=max(short, 12), warmup=8, weight_std=1.0),
                                   workload=workload_text(args, args.mask, args.q).replace("N(0, 1/fan_in)", "N(0, 1)")
                                   + " as the reference initialises them")
        # the reference's own training form at the keep probability of its published commands (0.7-0.85)
        r = run_index_lists(args, 0.75, float("inf"), short, warm, certify_runs=3)
        sec["index_lists_q0.75_inf"] = {k: r[k] for k in ("ms_per_step", "samples_per_s", "steps", "workload")}
        sec["certification"] = {"ms_per_pass": r["certification_ms"],
                                "workload": "evaluation-mode pass of the same model: sort neuron (K=10) for the value, "
                                            "interval sort neuron for the bounds, all layers, B=%d" % args.batch}
        # the p-annealing phase of the reference's training (main.py:297-303: p from 8 to 1000 on a logarithmic schedule)
        for pp in (8.0, 24.0, 256.0):
            r = run_index_lists(args, 0.75, pp, short, warm)
            sec["index_lists_q0.75_p%g" % pp] = {k: r[k] for k in ("ms_per_step", "samples_per_s", "steps", "workload")}
        for pp in (8.0, 64.0):
            sec["lp_layer_p%g" % pp] = run_lp_layer(args, pp, short, warm)
        sec["interval_layer_with_pos"] = run_interval_layer(args, short, warm)
        if (args.batch, args.width, args.in_features, args.classes) == (512, 5120, 3072, 10):
            r = run_masked(args, args.mask, args.q, short, warm, batch=256, in_features=12288, width=10240, classes=200,
                           eps=1.0 / 255)
            sec["wide"] = {"ms_per_step": r["ms_per_step"], "samples_per_s": r["samples_per_s"], "steps": short,
                           "phase_ms": r["phase_ms"],
                           "workload": "same step, 64x64 images: 12288->4x10240->200, B=256, q=%.2f (%s mask), eps=1/255"
                                       % (args.q, args.mask)}
        out["secondary"] = sec

    dims = [args.in_features] + [args.width] * (args.depth - 1) + [args.classes]
    out["cpu_baseline"] = None if args.no_cpu_baseline else cpu_baseline(args, dims)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
