"""Interval-bound dense head (sortnet_amd.heads) against float64 interval arithmetic: these layers are plain torch
matrix products, so every check runs on the CPU; the linear and margin layers (core/models/bound_basic_module.py:27-47,
79-103) run the same checks on device tensors under the gpu marker."""
import pytest
import torch

from sortnet_amd.heads import BoundConv2d, BoundFinalLinear, BoundLinear, BoundReLU, BoundTanh


DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


def _on(device):
    if device != "cpu" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device(device)


def _box(batch, features, seed, radius=0.1):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(batch, features, generator=g)
    r = torch.rand(batch, features, generator=g) * radius
    return x, x - r, x + r


@pytest.mark.parametrize("device", DEVICES)
def test_bound_linear_matches_interval_arithmetic_and_contains_samples(device):
    dev = _on(device)
    torch.manual_seed(0)
    layer = BoundLinear(24, 10, bias=True, w_scale=0.7)
    with torch.no_grad():
        layer.bias.normal_()
    layer = layer.to(dev)
    x, lo, up = (t.to(dev) for t in _box(6, 24, 1))
    y, ylo, yup = layer(x, lo, up)
    w = layer.weight.double() * layer.w_scale
    b = layer.bias.double() * layer.b_scale
    pos, neg = w.clamp(min=0), w.clamp(max=0)
    ref_lo = lo.double() @ pos.t() + up.double() @ neg.t() + b
    ref_up = up.double() @ pos.t() + lo.double() @ neg.t() + b
    torch.testing.assert_close(ylo.double(), ref_lo, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(yup.double(), ref_up, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(y.double(), x.double() @ w.t() + b, rtol=1e-5, atol=1e-5)
    g = torch.Generator().manual_seed(2)
    for _ in range(20):
        p = lo + (up - lo) * torch.rand(lo.shape, generator=g).to(dev)
        out = layer(p)[0]
        assert bool((out >= ylo - 1e-5).all()) and bool((out <= yup + 1e-5).all())
    assert layer(x)[1] is None and layer(None, lo, up)[0] is None


def test_monotone_activations_map_bounds():
    x, lo, up = _box(4, 7, 3)
    for act, fn in ((BoundTanh(), torch.tanh), (BoundReLU(), torch.relu)):
        y, ylo, yup = act(x, lo, up)
        assert torch.equal(y, fn(x)) and torch.equal(ylo, fn(lo)) and torch.equal(yup, fn(up))
        assert bool((ylo <= y).all()) and bool((y <= yup).all())


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("classes", [10, 40])
def test_final_linear_margins(classes, device):
    dev = _on(device)
    torch.manual_seed(1)
    layer = BoundFinalLinear(16, classes, bias=True)
    with torch.no_grad():
        layer.bias.normal_()
    layer = layer.to(dev)
    batch = 70
    x, lo, up = (t.to(dev) for t in _box(batch, 16, 4))
    targets = torch.randint(0, classes, (batch,), generator=torch.Generator().manual_seed(5)).to(dev)
    logits, res = layer(x, lo, up, targets=targets)
    w = layer.weight.double() * layer.w_scale
    b = layer.bias.double() * layer.b_scale
    dw = w.unsqueeze(0) - w[targets].unsqueeze(1)                    # (batch, classes, features)
    db = b.unsqueeze(0) - b[targets].unsqueeze(1)
    c, r = (lo.double() + up.double()) / 2, (up.double() - lo.double()) / 2
    ref = torch.einsum("bjf,bf->bj", dw, c) + db + torch.einsum("bjf,bf->bj", dw.abs(), r)
    torch.testing.assert_close(res.double(), ref, rtol=1e-5, atol=1e-5)
    assert bool((res.gather(1, targets.unsqueeze(1)).abs() < 1e-5).all())
    # the bound dominates the margin at any point of the box
    g = torch.Generator().manual_seed(6)
    for _ in range(10):
        p = lo + (up - lo) * torch.rand(lo.shape, generator=g).to(dev)
        out = layer(p)
        margin = out - out.gather(1, targets.unsqueeze(1))
        assert bool((margin <= res + 1e-4).all())
    torch.testing.assert_close(logits, layer(x))
    # the radius term formed for a few samples at a time (7 chunks here) agrees with the one-piece form
    layer.max_diff_elements = 11 * classes * 16
    torch.testing.assert_close(layer(x, lo, up, targets=targets)[1], res, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_final_linear_is_differentiable(device):
    dev = _on(device)
    torch.manual_seed(8)
    layer = BoundFinalLinear(8, 5).to(dev)
    x, lo, up = (t.to(dev) for t in _box(9, 8, 7))
    targets = (torch.arange(9) % 5).to(dev)
    _, res = layer(x, lo, up, targets=targets)
    res.sum().backward()
    # d(sum of margin bounds)/dW from the float64 closed form: row j gathers centre + sign * radius of every sample
    # whose target is not j, and loses the same for the samples whose target it is
    w = (layer.weight.detach().double() * layer.w_scale).cpu().requires_grad_()
    t = targets.cpu()
    c, r = ((lo + up) / 2).double().cpu(), ((up - lo) / 2).double().cpu()
    dw = w.unsqueeze(0) - w[t].unsqueeze(1)
    ref = (torch.einsum("bjf,bf->bj", dw, c) + torch.einsum("bjf,bf->bj", dw.abs(), r)).sum()
    ref.backward()
    torch.testing.assert_close(layer.weight.grad.double().cpu(), w.grad * layer.w_scale, rtol=1e-4, atol=1e-5)


def test_bound_conv2d_matches_interval_arithmetic_and_contains_samples():
    torch.manual_seed(2)
    layer = BoundConv2d(3, 5, 3, stride=2, padding=1, bias=True, w_scale=0.5)
    with torch.no_grad():
        layer.bias.normal_()
    assert abs(layer.w_scale - 1.0 / (3 * 3 * 3) ** 0.5) < 1e-12
    g = torch.Generator().manual_seed(6)
    x = torch.randn(4, 3, 9, 9, generator=g)
    r = torch.rand(4, 3, 9, 9, generator=g) * 0.2
    lo, up = x - r, x + r
    y, ylo, yup = layer(x, lo, up)
    w = layer.weight.double() * layer.w_scale
    b = layer.bias.double() * layer.b_scale
    conv = lambda inp, k, bias=None: torch.nn.functional.conv2d(inp.double(), k, bias, stride=2, padding=1)
    pos, neg = w.clamp(min=0), w.clamp(max=0)
    torch.testing.assert_close(y.double(), conv(x, w, b), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(ylo.double(), conv(lo, pos, b) + conv(up, neg), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(yup.double(), conv(up, pos, b) + conv(lo, neg), rtol=1e-5, atol=1e-5)
    for _ in range(10):
        p = lo + (up - lo) * torch.rand(lo.shape, generator=g)
        out = layer(p)[0]
        assert bool((out >= ylo - 1e-5).all()) and bool((out <= yup + 1e-5).all())
    assert layer(x)[1] is None and layer(None, lo, up)[0] is None
