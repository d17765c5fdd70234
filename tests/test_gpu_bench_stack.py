"""The composed stack that bench.py times (sortnet_amd.model.DistanceMLP, margins, hinge_loss) against the same
chain composed from oracle calls.

Per layer the oracle is fed the very tensor the GPU layer consumed, so l-inf / masked values and positions and the
interval bounds are compared bit for bit (the mean shift between layers is a floating-point sum and is held to
rel 1e-5 on its own); the loss is checked against a numpy restatement of the reference's margin and hinge
formulas (ell_inf_models.py:45-50, main.py:329-335) and every weight gradient against the oracle's backward
chain at rel 1e-5.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL = 1e-5


def _dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def _close(got, ref, rtol=RTOL):
    got = got.detach().cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got)
    ref = np.asarray(ref)
    np.testing.assert_allclose(got, ref, rtol=rtol, atol=rtol * max(float(np.abs(ref).max()), 1e-30))


def _margins_np(dist, targets, eps, lower=None, upper=None):
    """ell_inf_models.py:45-50 in float32 numpy: logits = -dist, worst-case margin of every wrong class
    against the target, the target column zeroed, divided by 2 eps."""
    eps = np.float32(eps)
    lower = dist - eps if lower is None else lower
    upper = dist + eps if upper is None else upper
    lo, up = -upper, -lower
    rows = np.arange(dist.shape[0])
    margin = up - lo[rows, targets][:, None]
    margin[rows, targets] = 0
    return -dist, margin / (np.float32(2) * eps)


def _hinge_np(worst, mix=0.25):
    """main.py:329-335."""
    res = np.maximum(worst, 0)
    return (1 - mix) * res.max(axis=1).mean() + mix * res.mean()


def _hinge_grad_wrt_dist(dist, targets, eps, mix=0.25):
    """d loss / d dist by float64 autograd over an independent statement of the same formulas."""
    d = torch.tensor(dist, dtype=torch.float64, requires_grad=True)
    t = torch.tensor(targets, dtype=torch.long)
    lo, up = -(d + eps), -(d - eps)
    margin = up - lo.gather(1, t.view(-1, 1))
    keep = torch.ones_like(margin).scatter(1, t.view(-1, 1), 0)
    res = (margin * keep / (2 * eps)).clamp(min=0)
    loss = (1 - mix) * res.max(dim=1)[0].mean() + mix * res.mean()
    loss.backward()
    return d.grad.numpy().astype(np.float32), float(loss)


def _build(dev, dims, q, mode, B, seed=3):
    from sortnet_amd.model import DistanceMLP
    model = DistanceMLP(dims[0], dims[1], len(dims) - 1, dims[-1], q=q, device=dev, seed=seed, mask_mode=mode)
    assert [tuple(w.shape) for w in model.weights] == [(o, i) for i, o in zip(dims[:-1], dims[1:])]
    g = torch.Generator().manual_seed(seed + 1)
    x = torch.rand(B, dims[0], generator=g)
    t = torch.randint(0, dims[-1], (B,), generator=g)
    with torch.no_grad():   # a non-trivial bias and running means, so their signs matter
        model.bias.copy_(torch.randn(dims[-1], generator=g) * 0.05)
        for rm in model.running_mean:
            rm.copy_(torch.rand(rm.numel(), generator=g) * 0.1)
    return model, x, t


@pytest.mark.parametrize("variant", ["term", "factored", "q1"])
def test_training_step_matches_oracle_chain(oracle, variant):
    from sortnet_amd import ext
    from sortnet_amd.model import margins, hinge_loss
    dev = _dev()
    dims = [96, 160, 160, 160, 10]
    B, eps, step_seed = 70, 8.0 / 255, 5
    q = 1.0 if variant == "q1" else 0.3
    mode = ext.MASK_FACTORED if variant == "factored" else ext.MASK_TERM
    omode = oracle.MASK_FACTORED if variant == "factored" else oracle.MASK_TERM
    model, x, t = _build(dev, dims, q, mode, B)
    rm_before = [rm.clone() for rm in model.running_mean]
    trace = []
    dist = model.forward(x.to(dev), step_seed=step_seed, trace=trace)
    logits, worst = margins(dist, t.to(dev), eps)
    loss = hinge_loss(worst)
    loss.backward()

    # forward, layer by layer on the GPU's own layer inputs
    saved = []
    for i, (h_in, y, mean) in enumerate(trace):
        w = model.weights[i].detach().cpu().numpy()
        hin = h_in.cpu().numpy()
        if i == 0 or q == 1.0:
            ry, rpos = oracle.inf_dist_forward(hin, w)
        else:
            ry, rpos = oracle.masked_inf_dist_forward(hin, w, q, step_seed * 64 + i, omode)
        assert np.array_equal(y.cpu().numpy(), ry), (variant, i)
        saved.append((hin.shape, rpos))
        if i < len(trace) - 1:
            rout, rmean = oracle.mean_shift(ry)
            _close(mean, rmean)
            _close(trace[i + 1][0], rout)
            _close(model.running_mean[i], 0.9 * rm_before[i].cpu().numpy() + 0.1 * rmean)
    d_np = dist.detach().cpu().numpy()
    _close(d_np, trace[-1][1].cpu().numpy()[:, :, 0] + model.bias.detach().cpu().numpy()[None, :], rtol=1e-6)

    # loss
    rlogits, rworst = _margins_np(d_np, t.numpy(), eps)
    _close(logits, rlogits, rtol=1e-6)
    _close(worst, rworst, rtol=1e-6)
    assert abs(float(loss) - _hinge_np(rworst)) <= 1e-5 * abs(float(loss))
    gdist, loss64 = _hinge_grad_wrt_dist(d_np, t.numpy(), eps)
    assert abs(float(loss) - loss64) <= 1e-5 * abs(loss64)

    # backward chain: bias, then scatter backward through the positions, centring between the layers
    _close(model.bias.grad, gdist.sum(axis=0))
    g = gdist[:, :, None]
    for i in reversed(range(len(trace))):
        if i < len(trace) - 1:
            g = g - g.mean(axis=(0, 2), keepdims=True)
        gx, gw = oracle.inf_dist_backward(g, saved[i][1], saved[i][0], tuple(model.weights[i].shape))
        _close(model.weights[i].grad, gw)
        g = gx


def test_certification_pass_matches_oracle_chain(oracle):
    from sortnet_amd import ext
    from sortnet_amd.model import margins
    dev = _dev()
    dims = [96, 160, 160, 160, 10]
    B, eps = 70, 8.0 / 255
    model, x, t = _build(dev, dims, 0.3, ext.MASK_TERM, B)
    lower, upper = (x - eps).clamp(min=0), (x + eps).clamp(max=1)
    lo, up = model.bounds(lower.to(dev), upper.to(dev))
    rl, ru = lower.numpy()[:, :, None], upper.numpy()[:, :, None]
    for i, w in enumerate(model.weights):
        rl, ru = oracle.bound_inf_dist_forward(rl, ru, w.detach().cpu().numpy(), need_pos=False)
        shift = (model.running_mean[i].cpu().numpy() if i < len(model.weights) - 1
                 else -model.bias.detach().cpu().numpy())[None, :, None]
        rl, ru = rl - shift, ru - shift
    assert np.array_equal(lo.cpu().numpy(), rl[:, :, 0])
    assert np.array_equal(up.cpu().numpy(), ru[:, :, 0])
    # the bounds bracket the evaluation forward of the pure l-inf net
    val = model.predict(x.to(dev))
    assert bool((lo <= val).all()) and bool((val <= up).all())
    # certified margins from the propagated bounds against the numpy restatement
    cert = margins(val, t.to(dev), eps, lo, up)[1]
    _close(cert, _margins_np(val.cpu().numpy(), t.numpy(), eps, rl[:, :, 0], ru[:, :, 0])[1], rtol=1e-6)


def test_benchmark_size_stack(oracle):
    """The headline configuration itself (512 x 3072 -> 4 x 5120 -> 10): the first-layer and class-layer launches
    against the oracle on the first rows, and the certification pass bracketing the evaluation forward."""
    from sortnet_amd import ext
    dev = _dev()
    dims = [3072, 5120, 5120, 5120, 5120, 5120, 10]
    B, eps, rows = 512, 8.0 / 255, 6
    model, x, t = _build(dev, dims, 0.3, ext.MASK_FACTORED, B, seed=0)
    xd = x.to(dev)
    trace = []
    with torch.no_grad():
        model.forward(xd, step_seed=2, trace=trace)
    assert len(trace) == 6
    for i in (0, 5):      # 512 x 3072 x 5120 (plain l-inf) and 512 x 5120 x 10 (masked, factored)
        h_in, y, _ = trace[i]
        w = model.weights[i].detach().cpu().numpy()
        hin = h_in[:rows].cpu().numpy()
        if i == 0:
            ry = oracle.inf_dist_forward(hin, w, need_pos=False)
        else:
            ry = oracle.masked_inf_dist_forward(hin, w, 0.3, 2 * 64 + i, oracle.MASK_FACTORED, need_pos=False)
        assert np.array_equal(y[:rows].cpu().numpy(), ry), i
    lower, upper = (xd - eps).clamp(min=0), (xd + eps).clamp(max=1)
    lo, up = model.bounds(lower, upper)
    val = model.predict(xd)
    assert bool((lo <= val).all()) and bool((val <= up).all())
    assert bool((up - lo).max() <= 2 * eps * 1.0001 + 4e-10 * len(dims))   # 1-Lipschitz: the interval never widens
    # the class layer of the certification pass against the oracle on the first rows
    h_lo, h_up = lower.unsqueeze(-1).contiguous(), upper.unsqueeze(-1).contiguous()
    from sortnet_amd import functional as F
    with torch.no_grad():
        for i, w in enumerate(model.weights[:-1]):
            h_lo, h_up = F.bound_inf_dist(h_lo, h_up, w)
            h_lo, h_up = h_lo - model.running_mean[i].view(1, -1, 1), h_up - model.running_mean[i].view(1, -1, 1)
        y_lo, y_up = F.bound_inf_dist(h_lo, h_up, model.weights[-1])
    rl, ru = oracle.bound_inf_dist_forward(h_lo[:rows].cpu().numpy(), h_up[:rows].cpu().numpy(),
                                           model.weights[-1].detach().cpu().numpy(), need_pos=False)
    assert np.array_equal(y_lo[:rows].cpu().numpy(), rl) and np.array_equal(y_up[:rows].cpu().numpy(), ru)


def test_overlapped_steps_match_one_stream_step(monkeypatch):
    """bench.py's default step queues the certification pass on a second stream beside forward and backward and the
    optimizer layer by layer on a third, each reader of a layer's weights waiting for that layer's update; with
    --no-overlap everything follows in turn on one stream.  All train the same weights: the loss of every step agrees.
    An overlapped certification pass of step i + 1 reads the weights and running means that the one-stream pass of
    step i reads (those left by step i's optimizer and forward), so its margins agree with that pass's."""
    import os
    import sys
    _dev()
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench
    monkeypatch.setattr(sys, "argv", ["bench.py"])
    # one batch instead of the benchmark's four in turn: the certification passes compared below must see the same inputs
    monkeypatch.setattr(bench, "NBATCH", 1)
    args = bench.parse()
    args.batch, args.in_features, args.width, args.depth, args.classes = 256, 784, 1024, 4, 10
    steps, warmup = 6, 2
    one = bench.run_masked(args, "factored", 0.3, steps, warmup, overlap=False)
    # a step moves the margins by well more than the tolerance: the comparison below tells neighbouring steps apart
    m = np.asarray(one["margin_trace"])
    assert np.abs(np.diff(m)).min() > 5e-4 * np.abs(m).max()
    for pipeline in (True, False):
        two = bench.run_masked(args, "factored", 0.3, steps, warmup, overlap=True, pipeline=pipeline)
        np.testing.assert_allclose(two["loss_trace"], one["loss_trace"], rtol=1e-4, err_msg=str(pipeline))
        np.testing.assert_allclose(two["margin_trace"][1:], one["margin_trace"][:-1], rtol=1e-4, err_msg=str(pipeline))
