"""The five training losses (sortnet_amd.losses) against float64 numpy restatements of the reference's formulas
(main.py:329-379), values and gradients, and the decay of the clean cross-entropy weight."""
import math

import numpy as np
import pytest
import torch

from sortnet_amd import losses


def _data(seed, B=37, C=10):
    g = torch.Generator().manual_seed(seed)
    outputs = torch.randn(B, C, generator=g, dtype=torch.float64)
    targets = torch.randint(0, C, (B,), generator=g)
    worst = torch.randn(B, C, generator=g, dtype=torch.float64) * 1.5
    worst.scatter_(1, targets.view(-1, 1), 0.0)       # the models zero the target column
    return outputs, worst, targets


def _ce_np(z, t):
    """-log softmax(z)[target], per sample."""
    z = z - z.max(axis=1, keepdims=True)
    return np.log(np.exp(z).sum(axis=1)) - z[np.arange(len(t)), t]


def _ref(name, o, w, t, lam, **kw):
    rows = np.arange(len(t))
    clean = _ce_np(o, t).mean()
    if name == "hinge":
        res = np.maximum(w, 0)
        mix = kw.get("mix", 0.25)
        return (1 - mix) * res.max(axis=1).mean() + mix * res.mean()
    if name == "crossentropy":
        return _ce_np(w, t).mean() + lam * clean
    if name == "mixture":
        res = np.clip(w, 0, kw.get("clip", 1))
        return res.max(axis=1).mean() + lam * clean
    correct = (o.argmax(axis=1) == t).astype(np.float64)
    if name == "ce_hinge":
        m = w - w[rows, t][:, None] + 1
        m[rows, t] = 0
        return (correct * m.max(axis=1)).mean() + lam * clean
    if name == "ce_mixture":
        return (correct * _ce_np(w, t)).mean() + lam * clean
    raise KeyError(name)


@pytest.mark.parametrize("name,kw", [("hinge", {}), ("hinge", {"mix": 0.6}), ("crossentropy", {}), ("mixture", {}),
                                     ("mixture", {"clip": 0.4}), ("ce_hinge", {}), ("ce_mixture", {})])
def test_loss_values_and_gradients(name, kw):
    o, w, t = _data(3)
    loss = losses.LOSSES[name](**kw) if name == "hinge" else losses.LOSSES[name](lam0=0.7, lam_end=0.07, **kw)
    loss.update(0.35)
    lam = 0.0 if name == "hinge" else 0.7 * (0.1 ** 0.35)
    o1, w1 = o.clone().requires_grad_(), w.clone().requires_grad_()
    val = loss(o1, w1, t)
    ref = _ref(name, o.numpy(), w.numpy(), t.numpy(), lam, **kw)
    assert abs(float(val) - ref) <= 1e-12 * max(1.0, abs(ref))
    val.backward()
    # central differences of the restated formula on a few coordinates of each argument
    rng = np.random.default_rng(0)
    for arr, grad in ((o, o1.grad), (w, w1.grad)):
        if grad is None:
            grad = torch.zeros_like(arr)
        for _ in range(12):
            i, j = int(rng.integers(arr.size(0))), int(rng.integers(arr.size(1)))
            if arr is w and j == int(t[i]):
                continue          # the zeroed target column sits exactly on the kink of clamp(min=0)
            h = 1e-6
            hi, lo = arr.numpy().copy(), arr.numpy().copy()
            hi[i, j] += h
            lo[i, j] -= h
            a = (hi, w.numpy()) if arr is o else (o.numpy(), hi)
            b = (lo, w.numpy()) if arr is o else (o.numpy(), lo)
            fd = (_ref(name, a[0], a[1], t.numpy(), lam, **kw) - _ref(name, b[0], b[1], t.numpy(), lam, **kw)) / (2 * h)
            assert abs(float(grad[i, j]) - fd) <= 1e-6 + 1e-5 * abs(fd), (name, i, j)


def test_lambda_decay_and_names():
    assert losses.lam_schedule(1.0, 0.01, 0.0) == 1.0
    assert math.isclose(losses.lam_schedule(1.0, 0.01, 1.0), 0.01, rel_tol=1e-12)
    assert math.isclose(losses.lam_schedule(0.05, 0.0005, 0.5), 0.005, rel_tol=1e-12)
    assert losses.lam_schedule(0.0, 0.01, 0.3) == 0.0
    assert set(losses.LOSSES) == {"hinge", "crossentropy", "mixture", "ce_hinge", "ce_mixture"}
    m = losses.mixture(lam0=0.05, lam_end=0.0005)
    assert m.lam == 0.05 and m.extra == {"clip": 1}
    m.update(1.0)
    assert math.isclose(m.lam, 0.0005, rel_tol=1e-12)


def test_float32_matches_float64():
    o, w, t = _data(5, B=64)
    for name, cls in losses.LOSSES.items():
        loss = cls()
        a = float(loss(o, w, t))
        b = float(loss(o.float(), w.float(), t))
        assert abs(a - b) <= 1e-5 * max(1.0, abs(a)), name
