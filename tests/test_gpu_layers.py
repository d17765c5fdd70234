"""GPU tests of the layer callers (sortnet_amd.layers) and of the device-side mask sampler:
a small stack is run in the three modes of the reference's NormDistBase.forward and compared with
the same computation composed from oracle calls."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def _close(got, ref, rtol=1e-5):
    got = got.detach().cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got)
    ref = np.asarray(ref)
    np.testing.assert_allclose(got, ref, rtol=rtol, atol=rtol * max(float(np.abs(ref).max()), 1e-30))


@pytest.mark.parametrize("S,G,C,q", [(3, 1, 100, 0.3), (2, 2, 64, 0.75), (16, 1, 5120, 0.3), (1, 1, 7, 1.0),
                                     (2, 1, 8192, 0.5), (2, 1, 8193, 0.1), (1, 2, 20000, 0.9)])
def test_sampler_matches_oracle(oracle, S, G, C, q):
    from sortnet_amd import ext
    dev = _dev()
    for seed in (0, 12345):
        count = ext.mask_count(seed, C, q)
        assert count == oracle.mask_count(seed, C, q)
        assert abs(count - q * C) <= 6 * np.sqrt(C * q * (1 - q)) + 1
        idx = ext.sample_index_lists(seed, S, G, C, count, dev).cpu().numpy()
        ref = oracle.sample_index_lists(seed, S, G, C, count)
        assert np.array_equal(idx, ref)
        assert idx.shape == (S, G, count) and (np.diff(idx, axis=-1) > 0).all() and idx.min() >= 0 and idx.max() < C
    if S > 1 and 0 < count < C:
        assert not np.array_equal(idx[0], idx[1])    # sub-batches get different subsets


@pytest.mark.parametrize("C,count", [(5120, 1), (5120, 5120), (5120, 5119), (8192, 4096), (257, 128), (1, 1), (300, 299)])
def test_sampler_counts_at_the_ends(oracle, C, count):
    """Counts the probability does not produce (one channel, all but one, all), many seeds: the selection of the
    count-th smallest word has to name the right bin at every level of its histograms."""
    from sortnet_amd import ext
    dev = _dev()
    for seed in range(20, 28):
        idx = ext.sample_index_lists(seed, 3, 1, C, count, dev).cpu().numpy()
        assert np.array_equal(idx, oracle.sample_index_lists(seed, 3, 1, C, count)), seed


def test_plain_stack_value_and_bounds(oracle):
    from sortnet_amd.layers import NormDist, BoundSequential, DropoutRegistry
    dev = _dev()
    reg = DropoutRegistry()
    torch.manual_seed(0)
    net = BoundSequential(NormDist(48, 64, bias=False, std=0.2, registry=reg),
                          NormDist(64, 10, bias=True, mean_shift=False, std=0.2, registry=reg)).to(dev)
    x = torch.rand(40, 48, device=dev)
    eps = 0.02
    net.train()
    y, _, _ = net((x, None, None))
    w0, w1 = net[0].weight.detach().cpu().numpy(), net[1].weight.detach().cpu().numpy()
    xn = x.cpu().numpy()[:, :, None]
    h0, pos0 = oracle.inf_dist_forward(xn, w0)
    h, mean = oracle.mean_shift(h0)
    ref, pos1 = oracle.inf_dist_forward(h, w1)
    np.testing.assert_allclose(y.detach().cpu().numpy(), ref[:, :, 0], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(net[0].mean_shift.running_mean.cpu().numpy(), 0.1 * mean, rtol=1e-5, atol=1e-7)
    gy = torch.randn(40, 10, generator=torch.Generator().manual_seed(5))
    (y * gy.to(dev)).sum().backward()
    # the oracle's backward chain: bias, scatter through the positions, centring, scatter again
    g1 = gy.numpy()[:, :, None]
    _close(net[1].bias.grad, g1.sum(axis=(0, 2)))
    gh, gw1 = oracle.inf_dist_backward(g1, pos1, h.shape, w1.shape)
    _close(net[1].weight.grad, gw1)
    gh = gh - gh.mean(axis=(0, 2), keepdims=True)
    _, gw0 = oracle.inf_dist_backward(gh, pos0, xn.shape, w0.shape)
    _close(net[0].weight.grad, gw0)
    net.eval()
    with torch.no_grad():
        v, lo, up = net((x, x - eps, x + eps))
    rm = net[0].mean_shift.running_mean.cpu().numpy()
    xl, xu = (x - eps).cpu().numpy()[:, :, None], (x + eps).cpu().numpy()[:, :, None]
    l1, u1 = oracle.bound_inf_dist_forward(xl, xu, w0, need_pos=False)
    l2, u2 = oracle.bound_inf_dist_forward(l1 - rm[None, :, None], u1 - rm[None, :, None], w1, need_pos=False)
    np.testing.assert_allclose(lo.cpu().numpy(), l2[:, :, 0], rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(up.cpu().numpy(), u2[:, :, 0], rtol=1e-6, atol=1e-6)
    assert bool((lo <= v + 1e-6).all()) and bool((v <= up + 1e-6).all())


def test_index_list_training_and_sort_eval(oracle):
    from sortnet_amd.layers import NormDist, BoundSequential, DropoutRegistry, set_mask_seed
    dev = _dev()
    reg = DropoutRegistry()
    torch.manual_seed(1)
    q = 0.6
    net = BoundSequential(NormDist(40, 96, bias=False, std=0.2, registry=reg),
                          NormDist(96, 64, bias=False, std=0.2, dropout=q, registry=reg),
                          NormDist(64, 10, bias=True, mean_shift=False, std=0.2, dropout=q, registry=reg)).to(dev)
    x = torch.rand(70, 40, device=dev)
    set_mask_seed(7, reg)
    net.train()
    y, _, _ = net((x, None, None))
    gy = torch.randn(70, 10, generator=torch.Generator().manual_seed(6))
    (y * gy.to(dev)).sum().backward()
    # recompute with the oracle: layer 0 drops outputs (= inputs of layer 1), layer 1 drops outputs too
    S = 3
    seeds = [(7 * 1000003 + d) & 0xFFFFFFFF for d in (1, 2)]
    c1 = oracle.mask_count(seeds[0], 96, q)
    i1 = oracle.sample_index_lists(seeds[0], S, 1, 96, c1)
    c2 = oracle.mask_count(seeds[1], 64, q)
    i2 = oracle.sample_index_lists(seeds[1], S, 1, 64, c2)
    w = [m.weight.detach().cpu().numpy() for m in net]
    rows = np.arange(70) // 32

    def index_mean_shift(h, idx, channels):
        tot, cnt = np.zeros(channels), np.full(channels, 1e-10)
        for b in range(h.shape[0]):
            tot[idx[rows[b], 0]] += h[b, :, 0]
            cnt[idx[rows[b], 0]] += 1
        mean = (tot / cnt).astype(np.float32)
        return h - mean[idx[rows, 0]][:, :, None]

    xn = x.cpu().numpy()[:, :, None]
    h0, p0 = oracle.inf_dist_forward(xn, w[0], 1, True, None, i1)
    h0 = index_mean_shift(h0, i1, 96)
    h1, p1 = oracle.inf_dist_forward(h0, w[1], 1, True, i1, i2)
    h1 = index_mean_shift(h1, i2, 64)
    h2, p2 = oracle.inf_dist_forward(h1, w[2], 1, True, i2, None)
    np.testing.assert_allclose(y.detach().cpu().numpy(), h2[:, :, 0], rtol=2e-5, atol=2e-6)
    # backward chain through the same lists: scatter, then the centring of the gradient over the samples that
    # kept each channel (the backward of the index-list mean shift), layer by layer
    g = gy.numpy()[:, :, None]
    _close(net[2].bias.grad, g.sum(axis=(0, 2)))
    g, gw2 = oracle.inf_dist_backward(g, p2, h1.shape, w[2].shape, 1, True, i2, None)
    _close(net[2].weight.grad, gw2)
    g, gw1 = oracle.inf_dist_backward(index_mean_shift(g, i2, 64), p1, h0.shape, w[1].shape, 1, True, i1, i2)
    _close(net[1].weight.grad, gw1)
    _, gw0 = oracle.inf_dist_backward(index_mean_shift(g, i1, 96), p0, xn.shape, w[0].shape, 1, True, None, i1)
    _close(net[0].weight.grad, gw0)
    # evaluation mode: sort neuron for the value, its interval version for the bounds
    net.eval()
    eps = 0.01
    with torch.no_grad():
        v, lo, up = net((x, x - eps, x + eps))
    rm = [m.mean_shift.running_mean.cpu().numpy() if m.mean_shift is not None else None for m in net]
    xv = x.cpu().numpy()[:, :, None]
    a = oracle.inf_dist_forward(xv, w[0], need_pos=False) - rm[0][None, :, None]
    a = oracle.sort_neuron_forward(a, w[1], q, 10, need_pos=False) - rm[1][None, :, None]
    a = oracle.sort_neuron_forward(a, w[2], q, 10, need_pos=False)
    np.testing.assert_allclose(v.cpu().numpy(), a[:, :, 0], rtol=1e-5, atol=1e-6)
    assert bool((lo <= v + 1e-5).all()) and bool((v <= up + 1e-5).all())


def test_conv_layer_shapes_and_value(oracle):
    from sortnet_amd.layers import NormDistConv, DropoutRegistry
    dev = _dev()
    torch.manual_seed(2)
    layer = NormDistConv(3, 8, 3, stride=2, bias=False, mean_shift=False, std=0.3, registry=DropoutRegistry()).to(dev)
    x = torch.rand(4, 3, 9, 9, device=dev)
    with torch.no_grad():
        y, lo, up = layer(x, x - 0.01, x + 0.01)
    assert y.shape == (4, 8, 4, 4) and lo.shape == y.shape
    cols = torch.nn.functional.unfold(x, 3, stride=2).cpu().numpy()          # (4, 27, 16)
    ref = oracle.inf_dist_forward(cols, layer.weight.detach().cpu().numpy(), need_pos=False)
    assert np.array_equal(y.cpu().numpy().reshape(4, 8, 16), ref)
    assert bool((lo <= y).all()) and bool((y <= up).all())


@pytest.mark.parametrize("kind", ["mlp", "hybrid", "hybrid_conv", "hybrid_avg"])
def test_model_zoo_modes(kind):
    """The three uses of a model of every family: training step through the index-list path, plain evaluation, and
    certification with an input box.  Certified margins must dominate the margins at sampled points of the
    box, and the 1-Lipschitz margins (no box) must dominate the certified ones' nominal margins as well."""
    from sortnet_amd.ell_inf_models import SortMLPModel, SortHybridModel, SortHybridModel2, SortHybridModelAvg
    from sortnet_amd.layers import DropoutRegistry, set_mask_seed
    dev = _dev()
    reg = DropoutRegistry()
    torch.manual_seed(3)
    dims = (3, 8, 8)
    if kind == "mlp":
        net = SortMLPModel(4, 64, dims, num_classes=10, dropout=0.7, std=0.3, registry=reg)
    elif kind == "hybrid":
        net = SortHybridModel(5, 64, dims, hidden=32, num_classes=10, dropout=0.7, std=0.3, registry=reg)
    elif kind == "hybrid_conv":
        net = SortHybridModel2(5, 64, dims, hidden=32, num_classes=10, dropout=0.7, std=0.3, registry=reg)
    else:
        net = SortHybridModelAvg(5, 64, dims, hidden=32, num_classes=10, dropout=0.7, std=0.3, registry=reg)
        assert net.fc_linear[0].in_features == 64
    net = net.to(dev)
    B, eps = 70, 2.0 / 255
    x = torch.rand(B, *dims, device=dev)
    targets = torch.randint(0, 10, (B,), device=dev)
    set_mask_seed(11, reg)
    net.train()
    logits = net(x)
    assert logits.shape == (B, 10)
    torch.nn.functional.cross_entropy(logits, targets).backward()
    grads = [p.grad for p in net.parameters() if p.requires_grad]
    assert all(g is not None and torch.isfinite(g).all() for g in grads)
    # training-mode margins from the 1-Lipschitz ball around the distance features
    logits2, margin = net(x, targets=targets, eps=eps)
    assert margin.shape == (B, 10) and torch.isfinite(margin).all()
    net.eval()
    with torch.no_grad():
        plain = net(x)
        up, down = torch.ones_like(x), torch.zeros_like(x)
        cl, certified = net(x, targets=targets, eps=eps, up=up, down=down)
        torch.testing.assert_close(cl, plain, rtol=1e-5, atol=1e-6)
        scale = 2 * eps if kind == "mlp" else 1.0                 # the MLP reports margins in units of 2 eps
        g = torch.Generator().manual_seed(5)
        for _ in range(5):
            noise = (torch.rand(x.shape, generator=g) * 2 - 1).to(dev) * eps
            xp = torch.minimum(torch.maximum(x + noise, down), up)
            out = net(xp)
            m = out - out.gather(1, targets.view(-1, 1))
            s = net.scalar if not isinstance(net.scalar, (int, float)) else torch.tensor(float(net.scalar), device=dev)
            assert bool((m <= certified * scale * s + 1e-4).all())
        assert bool((certified.gather(1, targets.view(-1, 1)).abs() < 1e-6).all())


@pytest.mark.parametrize("B,G,Cg,cnt,HW", [(70, 1, 96, 29, 1), (64, 2, 40, 17, 4), (5, 1, 12, 12, 1), (512, 1, 5120, 1530, 1)])
def test_index_mean_shift_matches_float64_and_torch_ops(B, G, Cg, cnt, HW):
    """Fused index-list mean shift: forward against a float64 restatement of
    core/models/bound_basic_module.py:125-153, and forward + backward against the same computation written
    with differentiable torch ops (the layer's path when it has a bias)."""
    from sortnet_amd import functional as F
    from sortnet_amd.layers import MeanShiftDropout
    dev = _dev()
    g = torch.Generator().manual_seed(B + cnt)
    S = (B + 31) // 32
    index = torch.stack([torch.stack([torch.randperm(Cg, generator=g)[:cnt].sort().values for _ in range(G)])
                         for _ in range(S)]).to(torch.int32)
    x = torch.randn(B, G * cnt, HW, generator=g)
    running0 = torch.randn(G * Cg, generator=g)
    # float64 restatement
    xn, idx = x.double().numpy(), index.numpy()
    tot, seen = np.zeros((G, Cg)), np.full((G, Cg), 1e-10)
    for b in range(B):
        for gi in range(G):
            tot[gi, idx[b // 32, gi]] += xn[b, gi * cnt:(gi + 1) * cnt].sum(-1)
            seen[gi, idx[b // 32, gi]] += 1
    mean = tot / (seen * HW)
    ref = xn.copy()
    for b in range(B):
        for gi in range(G):
            ref[b, gi * cnt:(gi + 1) * cnt] -= mean[gi, idx[b // 32, gi]][:, None]
    xd = x.to(dev).requires_grad_(True)
    running = running0.to(dev).clone()
    y, m = F.mean_shift_index(xd, index.to(dev), G * Cg, running, 0.1)
    np.testing.assert_allclose(m.cpu().numpy(), mean.reshape(-1), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(y.detach().cpu().numpy(), ref, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(running.cpu().numpy(), 0.9 * running0.numpy() + 0.1 * mean.reshape(-1), rtol=1e-5, atol=1e-6)
    # the torch-op formulation, forward and backward
    layer = MeanShiftDropout(G * Cg, affine=True).to(dev).train()
    x2 = x.to(dev).requires_grad_(True)
    y2 = layer(x2, None, None, index=index.to(dev))[0]
    torch.testing.assert_close(y.detach(), y2.detach(), rtol=1e-5, atol=1e-5)
    gy = torch.randn(y.shape, generator=g).to(dev)
    y.backward(gy)
    y2.backward(gy)
    torch.testing.assert_close(xd.grad, x2.grad, rtol=1e-5, atol=1e-5)
    # deterministic: a second call gives the same bits
    y3, _ = F.mean_shift_index(x.to(dev), index.to(dev), G * Cg, None, 0.1)
    assert torch.equal(y3, y.detach())


def test_running_mean_refresh_protocol():
    """The reference refreshes the running means after training (main.py:184-202): training mode, no_grad, p = inf,
    momentum 1 / (batch index + 1), so that the running mean ends as the average of the batch means of the
    evaluation-form (sort neuron) outputs."""
    from sortnet_amd import functional as F
    from sortnet_amd.layers import NormDist, BoundSequential, DropoutRegistry
    dev = _dev()
    reg = DropoutRegistry()
    torch.manual_seed(4)
    net = BoundSequential(NormDist(40, 64, bias=False, std=0.3, registry=reg),
                          NormDist(64, 48, bias=False, std=0.3, dropout=0.7, registry=reg),
                          NormDist(48, 10, bias=True, mean_shift=False, std=0.3, dropout=0.7, registry=reg)).to(dev)
    net.train()
    batches = [torch.rand(50, 40, device=dev) for _ in range(3)]
    layers = list(net)
    expect0 = []
    with torch.no_grad():
        for i, xb in enumerate(batches):
            for m in net.modules():
                if hasattr(m, "momentum"):
                    m.momentum = 1 / (i + 1)
            net((xb, None, None))
            h0 = F.sort_neuron(xb.unsqueeze(-1), layers[0].weight, 1, q=None)
            expect0.append(h0.mean(dim=(0, 2)))
    torch.testing.assert_close(layers[0].mean_shift.running_mean, torch.stack(expect0).mean(0), rtol=1e-5, atol=1e-6)
    assert torch.isfinite(layers[1].mean_shift.running_mean).all() and layers[1].mean_shift.running_mean.abs().sum() > 0


def test_evaluation_mode_stack_is_differentiable(oracle):
    """The attack (attack.py:26-29) differentiates an evaluation-mode stack with respect to its input, weights
    frozen; with trainable weights the same graph must reach them.  Checked against the same layers written with
    the running means subtracted by plain torch broadcasting."""
    from sortnet_amd.layers import NormDist, BoundSequential, DropoutRegistry
    import sortnet_amd.functional as F
    dev = _dev()
    reg = DropoutRegistry()
    torch.manual_seed(3)
    net = BoundSequential(NormDist(48, 64, bias=False, std=0.2, registry=reg),
                          NormDist(64, 32, bias=False, std=0.2, registry=reg),
                          NormDist(32, 10, bias=True, mean_shift=False, std=0.2, registry=reg)).to(dev)
    with torch.no_grad():
        for m in net:
            if m.mean_shift is not None:
                m.mean_shift.running_mean.copy_(torch.rand_like(m.mean_shift.running_mean) * 0.2)
        net[2].bias.copy_(torch.randn(10, device=dev) * 0.1)
    net.eval()
    gy = torch.randn(24, 10, device=dev)

    def manual(x):
        h = x.unsqueeze(-1)
        for m in net:
            h = F.norm_dist(h, m.weight, float("inf"))
            if m.mean_shift is not None:
                h = h - m.mean_shift.running_mean.view(1, -1, 1)
            if m.bias is not None:
                h = h + m.bias.view(1, -1, 1)
        return h.squeeze(-1)

    for frozen in (True, False):
        for prm in net.parameters():
            prm.requires_grad_(not frozen)
            prm.grad = None
        x1 = torch.rand(24, 48, device=dev, generator=None).requires_grad_()
        x2 = x1.detach().clone().requires_grad_()
        y1, _, _ = net((x1, None, None))
        assert y1.grad_fn is not None
        (y1 * gy).sum().backward()
        got = [x1.grad.clone()] + [prm.grad.clone() for prm in net.parameters() if not frozen]
        for prm in net.parameters():
            prm.grad = None
        y2 = manual(x2)
        (y2 * gy).sum().backward()
        ref = [x2.grad] + [prm.grad for prm in net.parameters() if not frozen]
        assert torch.equal(y1.detach(), y2.detach())
        assert float(x1.grad.abs().sum()) > 0
        for a, b in zip(got, ref):
            _close(a, b.cpu().numpy())


def test_training_mode_bounds_share_the_batch_mean(oracle):
    """Training mode with bounds passed along (core/models/bound_basic_module.py:154): value, lower and upper
    all lose the batch mean of the value; the running mean is updated once."""
    from sortnet_amd.layers import NormDist, DropoutRegistry
    dev = _dev()
    torch.manual_seed(4)
    layer = NormDist(40, 56, bias=False, std=0.2, registry=DropoutRegistry()).to(dev)
    layer.train()
    x = torch.rand(33, 40, device=dev)
    eps = 0.03
    v, lo, up = layer(x, x - eps, x + eps)
    w = layer.weight.detach().cpu().numpy()
    xn = x.cpu().numpy()[:, :, None]
    y = oracle.inf_dist_forward(xn, w, need_pos=False)
    yl, yu = oracle.bound_inf_dist_forward(xn - np.float32(eps), xn + np.float32(eps), w, need_pos=False)
    mean = y.mean(axis=(0, 2), dtype=np.float64).astype(np.float32)
    np.testing.assert_allclose(v.detach().cpu().numpy(), (y - mean[None, :, None])[:, :, 0], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(lo.detach().cpu().numpy(), (yl - mean[None, :, None])[:, :, 0], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(up.detach().cpu().numpy(), (yu - mean[None, :, None])[:, :, 0], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(layer.mean_shift.running_mean.cpu().numpy(), 0.1 * mean, rtol=1e-5, atol=1e-7)
    assert bool((lo <= v + 1e-6).all()) and bool((v <= up + 1e-6).all())
    # the shift of the bounds is part of the graph: the weight gradient of a weighted sum of the lower bounds is the
    # interval layer's backward plus the l-inf backward of what flows through the batch mean
    r = torch.randn(33, 56, generator=torch.Generator().manual_seed(9))
    (lo * r.to(dev)).sum().backward()
    rn = r.numpy()[:, :, None]
    _, _, pl, pu = oracle.bound_inf_dist_forward(xn - np.float32(eps), xn + np.float32(eps), w)
    _, _, gw_bound = oracle.bound_inf_dist_backward(rn, np.zeros_like(rn), pl, pu, xn.shape, w.shape)
    _, pos = oracle.inf_dist_forward(xn, w)
    g_mean = np.broadcast_to(-rn.sum(axis=0, keepdims=True) / np.float32(33), rn.shape).copy()
    _, gw_mean = oracle.inf_dist_backward(g_mean, pos, xn.shape, w.shape)
    _close(layer.weight.grad, gw_bound + gw_mean)
