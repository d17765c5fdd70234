"""The 64x64-image configuration as composed (B=256, 12288 -> 4 x 10240 -> 200, keep probability 0.3, eps = 1/255):
the 256 x 10240 x 200 class layer (200 output channels: not a multiple of the 64- or 128-wide tiles, so it takes other
kernels than the hidden layers) against the oracle on its first rows, and the whole stack the benchmark times
(`secondary.wide`) through properties that do not depend on the size: the certified interval brackets the evaluation
forward, its width obeys the 1-Lipschitz bound, degenerate intervals collapse onto the forward bit for bit, and the
training step's loss and gradients are finite with every weight row of every layer receiving its share.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ROWS = 8


def _dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def test_class_layer_256x10240x200(oracle):
    from sortnet_amd import ext
    dev = _dev()
    B, N, M = 256, 10240, 200
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(B, N, generator=g) * 0.05).unsqueeze(-1).contiguous()     # centred activations of a hidden layer
    w = (torch.randn(M, N, generator=g) * N ** -0.5).contiguous()
    gy = torch.randn(B, M, 1, generator=g)
    xd, wd, gd = x.to(dev), w.to(dev), gy.to(dev)
    xs, wn = x[:ROWS].numpy(), w.numpy()
    y, yn = torch.empty(B, M, 1, device=dev), torch.empty(B, M, 1, device=dev)
    pos = torch.empty(B, M, 1, device=dev, dtype=torch.int32)
    ext.inf_dist_forward(xd, wd, y, pos, 1)
    ext.inf_dist_forward_nograd(xd, wd, yn, 1)
    ry, rpos = oracle.inf_dist_forward(xs, wn)
    assert np.array_equal(y[:ROWS].cpu().numpy(), ry) and np.array_equal(pos[:ROWS].cpu().numpy(), rpos)
    assert torch.equal(y, yn)
    for mode in (ext.MASK_FACTORED, ext.MASK_TERM):
        ym = torch.empty_like(y)
        pm = torch.empty_like(pos)
        ext.masked_inf_dist_forward(xd, wd, ym, pm, 1, 0.3, 9, mode)
        rm, rpm = oracle.masked_inf_dist_forward(xs, wn, 0.3, 9, mode)
        assert np.array_equal(ym[:ROWS].cpu().numpy(), rm) and np.array_equal(pm[:ROWS].cpu().numpy(), rpm)
    eps = np.float32(1.0 / 255)
    yl, yu = torch.empty_like(y), torch.empty_like(y)
    pl, pu = torch.empty_like(pos), torch.empty_like(pos)
    ext.bound_inf_dist_forward(xd - float(eps), xd + float(eps), wd, yl, yu, pl, pu, 1)
    rl, ru, rpl, rpu = oracle.bound_inf_dist_forward((xd[:ROWS] - float(eps)).cpu().numpy(), (xd[:ROWS] + float(eps)).cpu().numpy(), wn)
    assert np.array_equal(yl[:ROWS].cpu().numpy(), rl) and np.array_equal(yu[:ROWS].cpu().numpy(), ru)
    assert np.array_equal(pl[:ROWS].cpu().numpy(), rpl) and np.array_equal(pu[:ROWS].cpu().numpy(), rpu)
    nl, nu = torch.empty_like(y), torch.empty_like(y)
    ext.bound_inf_dist_forward_nograd(xd - float(eps), xd + float(eps), wd, nl, nu, 1)
    assert torch.equal(nl, yl) and torch.equal(nu, yu)
    # scatter backward of the whole batch against index_put_ on the device (grad_weight sums over all 256 rows)
    gx, gw = torch.empty_like(xd), torch.empty_like(wd)
    ext.inf_dist_backward_input_weight(gd, pos, gx, gw, 1)
    idx = (pos & 0x7FFFFFFF).long().view(B, M)
    s = torch.where(pos.view(B, M) < 0, -gd.view(B, M), gd.view(B, M))
    tgx = torch.zeros(B, N, device=dev).scatter_add_(1, idx, s)
    rows = torch.arange(M, device=dev).view(1, M).expand(B, M)
    tgw = torch.zeros(M, N, device=dev).index_put_((rows.reshape(-1), idx.reshape(-1)), -s.reshape(-1), accumulate=True)
    torch.testing.assert_close(gx.view(B, N), tgx, rtol=1e-5, atol=1e-5 * float(tgx.abs().max()))
    torch.testing.assert_close(gw, tgw, rtol=1e-5, atol=1e-5 * float(tgw.abs().max()))


def test_wide_stack_composed_properties():
    from sortnet_amd import ext
    from sortnet_amd.model import DistanceMLP, margins, hinge_loss
    dev = _dev()
    B, eps = 256, 1.0 / 255
    model = DistanceMLP(12288, 10240, 6, 200, q=0.3, device=dev, seed=0, mask_mode=ext.MASK_FACTORED)
    g = torch.Generator().manual_seed(0)
    x = torch.rand(B, 12288, generator=g).to(dev)
    targets = torch.randint(0, 200, (B,), generator=g).to(dev)
    # one training step's forward and backward (this also sets the running means the other passes shift by)
    dist = model.forward(x, step_seed=1)
    logits, worst = margins(dist, targets, eps)
    loss = hinge_loss(worst)
    loss.backward()
    assert bool(torch.isfinite(loss))
    for w in model.weights:
        assert bool(torch.isfinite(w.grad).all())
    assert bool(torch.isfinite(model.bias.grad).all())
    # the class layer's gradient: every output of every sample deposits on exactly one input, so each of the 200 rows
    # carries the (signed) sum of its column of the loss gradient
    assert int((model.weights[-1].grad != 0).any(dim=1).sum()) == 200
    # certified interval brackets the evaluation forward of the same weights, for the inputs and for points of the box
    lower, upper = (x - eps).clamp(min=0), (x + eps).clamp(max=1)
    lo, up = model.bounds(lower, upper)
    for pt in (x, lower, upper, lower + (upper - lower) * torch.rand(B, 12288, generator=g).to(dev)):
        val = model.predict(pt)
        assert bool((lo <= val).all()) and bool((val <= up).all())
    # every layer is 1-Lipschitz in the l-inf norm and the shifts cancel in the width: at most 2 eps (+ the 1e-10 floors
    # and one rounding per layer)
    assert float((up - lo).max()) <= 2 * eps * (1 + 1e-5) + 1e-6
    # a degenerate interval collapses onto the forward, bit for bit
    dl, du = model.bounds(x, x)
    assert torch.equal(dl, du) and torch.equal(dl, model.predict(x))
