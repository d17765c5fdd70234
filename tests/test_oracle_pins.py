"""Pins the CPU oracle against independent statements of the same mathematics.

The reference ships no tests or golden vectors for this path, so each oracle function is
checked against library routines (torch.cdist, torch.topk, torch autograd in fp64), brute
force on small shapes, closed forms and invariants chosen so that a wrong sign, index or
dropped term fails.
"""
import itertools

import numpy as np
import pytest
import torch

SIGN = np.uint32(0x80000000)


def _rand(shape, seed, kind="randn", scale=1.0):
    g = torch.Generator().manual_seed(seed)
    t = torch.rand(shape, generator=g) if kind == "rand" else torch.randn(shape, generator=g)
    return (t * scale).numpy().astype(np.float32)


def _brute_diff(x, w, groups):
    """(B, G, COg, CIg, HW) tensor of x - w."""
    B, CI, HW = x.shape
    xt = torch.from_numpy(x).view(B, groups, 1, CI // groups, HW)
    wt = torch.from_numpy(w).view(groups, -1, w.shape[1], 1)
    return xt - wt


def _split_pos(pos):
    p = pos.view(np.uint32)
    return (p & ~SIGN).astype(np.int64), (p & SIGN) != 0


# ------------------------------------------------------------------ l-inf forward
@pytest.mark.parametrize("B,CI,CO,G,HW", [(5, 37, 11, 1, 1), (4, 24, 12, 3, 1), (3, 20, 8, 2, 5), (33, 64, 7, 1, 1)])
def test_inf_forward_matches_bruteforce_and_cdist(oracle, B, CI, CO, G, HW):
    x = _rand((B, CI, HW), 1, "rand")
    w = _rand((CO, CI // G), 2)
    y, pos = oracle.inf_dist_forward(x, w, G)
    d = _brute_diff(x, w, G)                      # B,G,COg,CIg,HW
    ref = d.abs().amax(dim=3).reshape(B, CO, HW).numpy()
    assert np.array_equal(y, np.maximum(ref, np.float32(1e-10)))
    arg = d.abs().argmax(dim=3).reshape(B, CO, HW).numpy()   # first maximal index
    idx, neg = _split_pos(pos)
    assert np.array_equal(idx, arg)
    sign_ref = torch.gather(d, 3, d.abs().argmax(dim=3, keepdim=True)).reshape(B, CO, HW).numpy() < 0
    assert np.array_equal(neg, sign_ref)
    assert np.array_equal(oracle.inf_dist_forward(x, w, G, need_pos=False), y)
    if G == 1 and HW == 1:
        cd = torch.cdist(torch.from_numpy(x[:, :, 0]), torch.from_numpy(w), p=float("inf")).numpy()
        assert np.array_equal(y[:, :, 0], cd)


def test_inf_forward_ties_pick_lowest_index_and_eps_floor(oracle):
    x = np.zeros((2, 6, 1), np.float32)
    w = np.zeros((3, 6), np.float32)
    # row 0: |d| = 2 at n=1 (d=-2), n=3 (d=+2), n=4 (d=-2): lowest index 1 wins, sign bit set
    w[0, [1, 4]] = 2.0
    w[0, 3] = -2.0
    # row 1: every term <= 1e-10 -> value 1e-10, pos 0 without sign
    w[1, 2] = 1e-10
    # row 2: +3 at n=5 only
    w[2, 5] = -3.0
    y, pos = oracle.inf_dist_forward(x, w)
    p = pos.view(np.uint32)[0, :, 0]
    assert y[0, 0, 0] == 2.0 and p[0] == (1 | int(SIGN))
    assert y[0, 1, 0] == np.float32(1e-10) and p[1] == 0
    assert y[0, 2, 0] == 3.0 and p[2] == 5


def test_inf_forward_index_lists_equal_explicit_gather(oracle):
    B, CI, CO = 70, 40, 30      # 3 sub-batches of 32 (last one ragged)
    S, ci_n, co_n = 3, 13, 9
    rng = np.random.default_rng(3)
    w = _rand((CO, CI), 4)
    ci = np.stack([np.sort(rng.choice(CI, ci_n, replace=False)) for _ in range(S)]).astype(np.int32).reshape(S, 1, ci_n)
    co = np.stack([np.sort(rng.choice(CO, co_n, replace=False)) for _ in range(S)]).astype(np.int32).reshape(S, 1, co_n)
    x = _rand((B, ci_n, 1), 5, "rand")
    y, pos = oracle.inf_dist_forward(x, w, 1, True, ci, co)
    assert y.shape == (B, co_n, 1)
    for s in range(S):
        sub = w[co[s, 0]][:, ci[s, 0]]
        ys, ps = oracle.inf_dist_forward(x[32 * s:32 * s + 32], sub)
        assert np.array_equal(y[32 * s:32 * s + 32], ys)
        assert np.array_equal(pos[32 * s:32 * s + 32], ps)


# ------------------------------------------------------------------ scatter backward (autograd)
def _autograd_inf(x, w, gy, G):
    B, CI, HW = x.shape
    xt = torch.from_numpy(x).double().requires_grad_()
    wt = torch.from_numpy(w).double().requires_grad_()
    d = xt.view(B, G, 1, CI // G, HW) - wt.view(G, -1, w.shape[1], 1)
    y = d.abs().amax(dim=3).reshape(B, -1, HW)
    y.backward(torch.from_numpy(gy).double())
    return xt.grad.numpy(), wt.grad.numpy()


@pytest.mark.parametrize("B,CI,CO,G,HW", [(6, 19, 9, 1, 1), (4, 12, 8, 2, 3)])
def test_inf_backward_matches_autograd(oracle, B, CI, CO, G, HW):
    x = _rand((B, CI, HW), 11, "rand")
    w = _rand((CO, CI // G), 12)
    gy = _rand((B, CO, HW), 13)
    _, pos = oracle.inf_dist_forward(x, w, G)
    gx, gw = oracle.inf_dist_backward(gy, pos, x.shape, w.shape, G)
    rx, rw = _autograd_inf(x, w, gy, G)
    np.testing.assert_allclose(gx, rx, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(gw, rw, rtol=1e-6, atol=1e-6)
    assert np.array_equal(oracle.inf_dist_backward(gy, pos, x.shape, w.shape, G, need_weight=False), gx)


def test_inf_backward_index_lists_scatter_to_full_weight(oracle):
    B, CI, CO, S, ci_n, co_n = 40, 20, 16, 2, 7, 5
    rng = np.random.default_rng(7)
    w = _rand((CO, CI), 14)
    ci = np.stack([np.sort(rng.choice(CI, ci_n, replace=False)) for _ in range(S)]).astype(np.int32).reshape(S, 1, ci_n)
    co = np.stack([np.sort(rng.choice(CO, co_n, replace=False)) for _ in range(S)]).astype(np.int32).reshape(S, 1, co_n)
    x = _rand((B, ci_n, 1), 15, "rand")
    gy = _rand((B, co_n, 1), 16)
    _, pos = oracle.inf_dist_forward(x, w, 1, True, ci, co)
    gx, gw = oracle.inf_dist_backward(gy, pos, x.shape, w.shape, 1, True, ci, co)
    # autograd on the explicitly gathered weights
    xt = torch.from_numpy(x[:, :, 0]).double().requires_grad_()
    wt = torch.from_numpy(w).double().requires_grad_()
    ys = []
    for s in range(S):
        sub = wt[torch.from_numpy(co[s, 0]).long()][:, torch.from_numpy(ci[s, 0]).long()]
        ys.append((xt[32 * s:32 * s + 32, None, :] - sub[None]).abs().amax(-1))
    torch.cat(ys).backward(torch.from_numpy(gy[:, :, 0]).double())
    np.testing.assert_allclose(gx[:, :, 0], xt.grad.numpy(), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(gw, wt.grad.numpy(), rtol=1e-6, atol=1e-6)


# ------------------------------------------------------------------ IBP through the l-inf layer
def _ibp_closed_form(xl, xu, w, G):
    """The reference's torch fallback formula (after the xL>xU repair), evaluated in fp32."""
    bad = xl > xu
    mid = (xl + xu) * np.float32(0.5)
    xl = np.where(bad, mid, xl)
    xu = np.where(bad, mid, xu)
    B, CI, HW = xl.shape
    wv = torch.from_numpy(w).view(G, -1, w.shape[1], 1)
    t1 = wv - torch.from_numpy(xl).view(B, G, 1, CI // G, HW)
    t2 = torch.from_numpy(xu).view(B, G, 1, CI // G, HW) - wv
    z1 = torch.maximum(t1, t2).clamp(min=1e-10)
    z2 = torch.minimum(t1, t2).clamp(max=-1e-10)
    return (-z2).amax(3).reshape(B, -1, HW).numpy(), z1.amax(3).reshape(B, -1, HW).numpy(), t1, t2


@pytest.mark.parametrize("B,CI,CO,G,HW", [(5, 23, 10, 1, 1), (3, 16, 6, 2, 4)])
def test_bound_forward_closed_form_and_invariants(oracle, B, CI, CO, G, HW):
    x = _rand((B, CI, HW), 21, "rand")
    eps = np.float32(2 / 255)
    xl, xu = x - eps, x + eps
    xl[0, 0, 0], xu[0, 0, 0] = xu[0, 0, 0], xl[0, 0, 0]     # one inverted interval -> midpoint repair
    w = _rand((CO, CI // G), 22, scale=0.3)
    yl, yu, pl, pu = oracle.bound_inf_dist_forward(xl, xu, w, G)
    rl, ru, t1, t2 = _ibp_closed_form(xl, xu, w, G)
    assert np.array_equal(yl, rl) and np.array_equal(yu, ru)
    yl2, yu2 = oracle.bound_inf_dist_forward(xl, xu, w, G, need_pos=False)
    assert np.array_equal(yl, yl2) and np.array_equal(yu, yu2)
    # the point value lies inside the bounds; a degenerate box gives yL == yU == y
    y = oracle.inf_dist_forward(x, w, G, need_pos=False)
    xl_ok = np.minimum(xl, xu)
    assert np.all(yl <= y + 1e-6) and np.all(y <= yu + 1e-6) and np.all(xl_ok <= xu + 1)
    dl, du = oracle.bound_inf_dist_forward(x, x, w, G, need_pos=False)
    assert np.array_equal(du, y)
    # 1-Lipschitz: the width of the output box never exceeds the widest input interval
    assert np.all(yu - yl <= 2 * eps + 1e-6)
    # argmin / argmax indices and the branch bit
    lo = torch.minimum(t1, t2)
    hi = torch.maximum(t1, t2)
    il, sl = _split_pos(pl)
    iu, su = _split_pos(pu)
    has_l = (lo.amin(3) < -1e-10).reshape(B, CO, HW).numpy()
    assert np.array_equal(il[has_l], lo.argmin(3).reshape(B, CO, HW).numpy()[has_l])
    assert np.all(pl.view(np.uint32)[~has_l] == 0xFFFFFFFF)
    assert np.array_equal(iu, hi.argmax(3).reshape(B, CO, HW).numpy())
    br = (t1 > t2)
    assert np.array_equal(su, torch.gather(br, 3, hi.argmax(3, keepdim=True)).reshape(B, CO, HW).numpy())
    assert np.array_equal(sl[has_l], torch.gather(br, 3, lo.argmin(3, keepdim=True)).reshape(B, CO, HW).numpy()[has_l])


@pytest.mark.parametrize("B,CI,CO,G,HW", [(5, 17, 8, 1, 1), (3, 12, 6, 2, 2)])
def test_bound_backward_matches_autograd(oracle, B, CI, CO, G, HW):
    x = _rand((B, CI, HW), 31, "rand")
    eps = np.float32(0.05)
    xl, xu = x - eps, x + eps
    w = _rand((CO, CI // G), 32, scale=0.3)
    gl, gu = _rand((B, CO, HW), 33), _rand((B, CO, HW), 34)
    _, _, pl, pu = oracle.bound_inf_dist_forward(xl, xu, w, G)
    gxl, gxu, gw = oracle.bound_inf_dist_backward(gl, gu, pl, pu, x.shape, w.shape, G)
    tl = torch.from_numpy(xl).double().requires_grad_()
    tu = torch.from_numpy(xu).double().requires_grad_()
    tw = torch.from_numpy(w).double().requires_grad_()
    wv = tw.view(G, -1, w.shape[1], 1)
    t1 = wv - tl.view(B, G, 1, CI // G, HW)
    t2 = tu.view(B, G, 1, CI // G, HW) - wv
    yl = -(torch.minimum(t1, t2).amin(3)).reshape(B, CO, HW)
    yu = torch.maximum(t1, t2).amax(3).reshape(B, CO, HW)
    (yl * torch.from_numpy(gl).double() + yu * torch.from_numpy(gu).double()).sum().backward()
    np.testing.assert_allclose(gxl, tl.grad.numpy(), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(gxu, tu.grad.numpy(), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(gw, tw.grad.numpy(), rtol=1e-6, atol=1e-6)


def test_bound_backward_skips_sentinel(oracle):
    # an interval that contains w everywhere: min(t1,t2) >= 0 -> posL stays 0xffffffff -> no lower gradient
    xl = np.full((1, 4, 1), -1.0, np.float32)
    xu = np.full((1, 4, 1), 1.0, np.float32)
    w = np.zeros((2, 4), np.float32)
    yl, yu, pl, pu = oracle.bound_inf_dist_forward(xl, xu, w)
    assert np.all(pl.view(np.uint32) == 0xFFFFFFFF) and np.all(yl == np.float32(1e-10))
    gxl, gxu, gw = oracle.bound_inf_dist_backward(np.ones((1, 2, 1), np.float32), np.ones((1, 2, 1), np.float32),
                                                  pl, pu, xl.shape, w.shape)
    assert gxl.sum() == 0 and gxu.sum() == 2.0 and gw.sum() == -2.0


# ------------------------------------------------------------------ sort neuron
def _sort_ref(x, w, q, K, G):
    d = _brute_diff(x, w, G).double()
    B, HW = x.shape[0], x.shape[2]
    top = torch.topk(d.abs(), k=K, dim=3)[0]           # B,G,COg,K,HW
    c = ((1 - q) ** torch.arange(K, dtype=torch.float64) * q).view(1, 1, 1, K, 1)
    return ((top * c).sum(3) / (1 - (1 - q) ** K)).reshape(B, -1, HW).numpy()


@pytest.mark.parametrize("B,CI,CO,G,HW,K,q", [(4, 40, 9, 1, 1, 10, 0.3), (3, 24, 6, 2, 3, 5, 0.75), (2, 8, 4, 1, 1, 8, 0.5)])
def test_sort_forward_matches_topk(oracle, B, CI, CO, G, HW, K, q):
    x = _rand((B, CI, HW), 41, "rand")
    w = _rand((CO, CI // G), 42)
    y, pos = oracle.sort_neuron_forward(x, w, q, K, G)
    ref = _sort_ref(x, w, q, K, G)
    np.testing.assert_allclose(y, ref, rtol=2e-6, atol=1e-9)
    assert np.array_equal(oracle.sort_neuron_forward(x, w, q, K, G, need_pos=False), y)
    d = _brute_diff(x, w, G)
    order = torch.argsort(d.abs(), dim=3, descending=True, stable=True)[:, :, :, :K]   # distinct values w.p. 1
    idx, neg = _split_pos(pos)                       # K,B,CO,HW
    ref_idx = order.permute(3, 0, 1, 2, 4).reshape(K, B, CO, HW).numpy()
    assert np.array_equal(idx, ref_idx)
    sg = torch.gather(d, 3, order).permute(3, 0, 1, 2, 4).reshape(K, B, CO, HW).numpy() < 0
    assert np.array_equal(neg, sg)


def test_sort_forward_limits_and_tie_order(oracle):
    x = _rand((3, 12, 1), 43, "rand")
    w = _rand((5, 12), 44)
    linf = oracle.inf_dist_forward(x, w, need_pos=False)
    # q = 1: only the largest term has weight
    np.testing.assert_allclose(oracle.sort_neuron_forward(x, w, 1.0, 4, need_pos=False), linf, rtol=1e-6)
    # K = 1: (EPS + t0 q) / q
    np.testing.assert_allclose(oracle.sort_neuron_forward(x, w, 0.4, 1, need_pos=False), linf, rtol=1e-6)
    # equal values: the later index ranks higher; zero terms never enter (slots keep index 0)
    x = np.zeros((1, 5, 1), np.float32)
    w = np.array([[0.0, 1.0, -1.0, 1.0, 0.0]], np.float32)
    y, pos = oracle.sort_neuron_forward(x, w, 0.5, 4)
    p = pos.view(np.uint32)[:, 0, 0, 0]
    assert list(p) == [3 | int(SIGN), 2, 1 | int(SIGN), 0]


def test_sort_neuron_is_expected_max_over_bernoulli_subsets(oracle):
    # exhaustive expectation over all 2^n keep-masks (max of the empty set = 0)
    n, q = 7, 0.35
    x = _rand((1, n, 1), 45, "rand")
    w = _rand((2, n), 46)
    a = np.abs(x[0, :, 0][None] - w).astype(np.float64)     # 2,n
    exp = np.zeros(2)
    for mask in itertools.product([0, 1], repeat=n):
        m = np.array(mask, bool)
        pr = np.prod(np.where(m, q, 1 - q))
        if m.any():
            exp += pr * a[:, m].max(1)
    y = oracle.sort_neuron_forward(x, w, q, n, need_pos=False)[0, :, 0]
    np.testing.assert_allclose(y * (1 - (1 - q) ** n), exp, rtol=1e-5)


@pytest.mark.parametrize("G,HW", [(1, 1), (2, 2)])
def test_sort_backward_matches_autograd(oracle, G, HW):
    B, CI, CO, K, q = 4, 16, 6, 5, 0.4
    x = _rand((B, CI, HW), 47, "rand")
    w = _rand((CO, CI // G), 48)
    gy = _rand((B, CO, HW), 49)
    _, pos = oracle.sort_neuron_forward(x, w, q, K, G)
    gx, gw = oracle.sort_neuron_backward(gy, pos, x.shape, w.shape, q, K, G)
    xt = torch.from_numpy(x).double().requires_grad_()
    wt = torch.from_numpy(w).double().requires_grad_()
    d = xt.view(B, G, 1, CI // G, HW) - wt.view(G, -1, w.shape[1], 1)
    top = torch.topk(d.abs(), k=K, dim=3)[0]
    c = ((1 - q) ** torch.arange(K, dtype=torch.float64) * q).view(1, 1, 1, K, 1)
    y = ((top * c).sum(3) / (1 - (1 - q) ** K)).reshape(B, CO, HW)
    y.backward(torch.from_numpy(gy).double())
    np.testing.assert_allclose(gx, xt.grad.numpy(), rtol=2e-6, atol=1e-6)
    np.testing.assert_allclose(gw, wt.grad.numpy(), rtol=2e-6, atol=1e-6)


@pytest.mark.parametrize("G,HW,K,q", [(1, 1, 10, 0.3), (2, 3, 4, 0.6)])
def test_bound_sort_forward_bruteforce_and_bracket(oracle, G, HW, K, q):
    B, CI, CO = 4, 24, 6
    x = _rand((B, CI, HW), 51, "rand")
    eps = np.float32(0.03)
    xl, xu = x - eps, x + eps
    w = _rand((CO, CI // G), 52, scale=0.5)
    yl, yu = oracle.bound_sort_neuron_forward(xl, xu, w, q, K, G)
    wv = torch.from_numpy(w).view(G, -1, w.shape[1], 1).double()
    t1 = wv - torch.from_numpy(xl).view(B, G, 1, CI // G, HW).double()
    t2 = torch.from_numpy(xu).view(B, G, 1, CI // G, HW).double() - wv
    up = torch.topk(torch.maximum(t1, t2).clamp(min=0), k=K, dim=3)[0]
    lo = torch.topk((-torch.minimum(t1, t2)).clamp(min=0), k=K, dim=3)[0]
    c = ((1 - q) ** torch.arange(K, dtype=torch.float64) * q).view(1, 1, 1, K, 1)
    nrm = 1 - (1 - q) ** K
    np.testing.assert_allclose(yu, ((up * c).sum(3) / nrm).reshape(B, CO, HW).numpy(), rtol=2e-6, atol=1e-9)
    np.testing.assert_allclose(yl, ((lo * c).sum(3) / nrm).reshape(B, CO, HW).numpy(), rtol=2e-6, atol=1e-9)
    y = oracle.sort_neuron_forward(x, w, q, K, G, need_pos=False)
    assert np.all(yl <= y * (1 + 1e-5) + 1e-7) and np.all(y <= yu * (1 + 1e-5) + 1e-7)
    # degenerate box: upper bound equals the point value
    _, du = oracle.bound_sort_neuron_forward(x, x, w, q, K, G)
    np.testing.assert_allclose(du, y, rtol=1e-6)


# ------------------------------------------------------------------ l-p
@pytest.mark.parametrize("p", [1.0, 2.0, 3.0, 8.0, 9.5, 11.3, 64.0])
def test_norm_dist_forward_matches_cdist(oracle, p):
    x = _rand((6, 50, 1), 61)
    w = _rand((7, 50), 62, scale=0.2)
    y = oracle.norm_dist_forward(x, w, p)
    ref = torch.cdist(torch.from_numpy(x[:, :, 0]).double(), torch.from_numpy(w).double(), p=p).numpy()
    np.testing.assert_allclose(y[:, :, 0], ref, rtol=2e-6)


def test_norm_dist_forward_large_p_tends_to_linf_and_groups(oracle):
    x = _rand((4, 24, 2), 63)
    w = _rand((6, 12), 64)
    y = oracle.norm_dist_forward(x, w, 1000.0, groups=2)
    linf = oracle.inf_dist_forward(x, w, 2, need_pos=False)
    np.testing.assert_allclose(y, linf, rtol=3e-3)
    d = _brute_diff(x, w, 2).double()
    ref = d.abs().pow(3.0).sum(3).pow(1 / 3.0).reshape(4, 6, 2).numpy()
    np.testing.assert_allclose(oracle.norm_dist_forward(x, w, 3.0, groups=2), ref, rtol=2e-6)


@pytest.mark.parametrize("p,G,HW", [(8.0, 1, 1), (2.0, 2, 2), (11.5, 1, 1), (64.0, 1, 1)])
def test_norm_dist_backward_matches_autograd(oracle, p, G, HW):
    B, CI, CO = 5, 12, 6
    x = _rand((B, CI, HW), 65)
    w = _rand((CO, CI // G), 66, scale=0.3)
    gy = _rand((B, CO, HW), 67)
    y = oracle.norm_dist_forward(x, w, p, G)
    gx, gw = oracle.norm_dist_backward(gy, x, w, y, p, G)
    xt = torch.from_numpy(x).double().requires_grad_()
    wt = torch.from_numpy(w).double().requires_grad_()
    d = xt.view(B, G, 1, CI // G, HW) - wt.view(G, -1, w.shape[1], 1)
    nrm = d.detach().abs().amax(3, keepdim=True)
    yy = ((d / nrm).abs().pow(p).sum(3, keepdim=True).pow(1 / p) * nrm).reshape(B, CO, HW)
    yy.backward(torch.from_numpy(gy).double())
    scale = np.abs(xt.grad.numpy()).max()
    np.testing.assert_allclose(gx, xt.grad.numpy(), rtol=1e-5, atol=1e-5 * scale)
    np.testing.assert_allclose(gw, wt.grad.numpy(), rtol=1e-5, atol=1e-5 * np.abs(wt.grad.numpy()).max())
    assert np.array_equal(oracle.norm_dist_backward(gy, x, w, y, p, G, need_weight=False), gx)


def test_norm_dist_backward_euler_identity(oracle):
    # single neuron: sum_n grad_x[b,n] (x[b,n]-w[n]) = g[b] y[b]   and   grad_w = -sum_b grad_x
    p = 8.0
    x = _rand((9, 30, 1), 68)
    w = _rand((1, 30), 69)
    gy = _rand((9, 1, 1), 70)
    y = oracle.norm_dist_forward(x, w, p)
    gx, gw = oracle.norm_dist_backward(gy, x, w, y, p)
    lhs = (gx[:, :, 0].astype(np.float64) * (x[:, :, 0] - w).astype(np.float64)).sum(1)
    np.testing.assert_allclose(lhs, (gy * y)[:, 0, 0], rtol=1e-5)
    np.testing.assert_allclose(gw[0], -gx[:, :, 0].astype(np.float64).sum(0), rtol=1e-5, atol=1e-6)


def test_norm_dist_index_lists(oracle):
    B, CI, CO, S, ci_n, co_n, p = 40, 20, 16, 2, 7, 5, 8.0
    rng = np.random.default_rng(9)
    w = _rand((CO, CI), 71)
    ci = np.stack([np.sort(rng.choice(CI, ci_n, replace=False)) for _ in range(S)]).astype(np.int32).reshape(S, 1, ci_n)
    co = np.stack([np.sort(rng.choice(CO, co_n, replace=False)) for _ in range(S)]).astype(np.int32).reshape(S, 1, co_n)
    x = _rand((B, ci_n, 1), 72)
    gy = _rand((B, co_n, 1), 73)
    y = oracle.norm_dist_forward(x, w, p, 1, ci, co)
    gx, gw = oracle.norm_dist_backward(gy, x, w, y, p, 1, True, ci, co)
    xt = torch.from_numpy(x[:, :, 0]).double().requires_grad_()
    wt = torch.from_numpy(w).double().requires_grad_()
    ys = []
    for s in range(S):
        sub = wt[torch.from_numpy(co[s, 0]).long()][:, torch.from_numpy(ci[s, 0]).long()]
        ys.append(torch.cdist(xt[32 * s:32 * s + 32], sub, p=p))
    yy = torch.cat(ys)
    np.testing.assert_allclose(y[:, :, 0], yy.detach().numpy(), rtol=2e-6)
    yy.backward(torch.from_numpy(gy[:, :, 0]).double())
    # the saved y is fp32, so (|d|/y)^(p-1) carries ~(p-1)*6e-8 relative error per term
    np.testing.assert_allclose(gx[:, :, 0], xt.grad.numpy(), rtol=1e-5, atol=1e-5 * np.abs(xt.grad.numpy()).max())
    np.testing.assert_allclose(gw, wt.grad.numpy(), rtol=1e-5, atol=1e-5 * np.abs(wt.grad.numpy()).max())


# ------------------------------------------------------------------ counter RNG and the masked neuron
def _mix(h):
    h = np.asarray(h, np.uint64) & 0xFFFFFFFF
    h ^= h >> 16
    h = (h * 0x21F0AAAD) & 0xFFFFFFFF
    h ^= h >> 15
    h = (h * 0x735A2D97) & 0xFFFFFFFF
    h ^= h >> 15
    return h


def _word(seed, stream, row, col):
    key = _mix(((seed ^ ((stream * 0x9E3779B9) & 0xFFFFFFFF)) + np.asarray(row, np.uint64)) & 0xFFFFFFFF)
    return _mix((key + (np.asarray(col, np.uint64) + 1) * 0x85EBCA6B) & 0xFFFFFFFF)


def test_rng_known_answers_and_uniformity(oracle):
    for args in [(0, 0, 0, 0), (1, 2, 3, 4), (0xDEADBEEF, 1, 123456, 789), (7, 2, 0xFFFFFFF0, 5119)]:
        assert oracle.rng_word(*args) == int(_word(*args))
    # hand-evaluated: mix(0) = 0, so word(0,0,0,0) = mix(0x85ebca6b)
    assert oracle.rng_word(0, 0, 0, 0) == int(_mix(0x85EBCA6B))
    words = _word(5, 0, np.arange(4096)[:, None], np.arange(64)[None])
    bytes_ = (words[..., None] >> (8 * np.arange(4, dtype=np.uint64))) & 0xFF
    assert abs(bytes_.mean() - 127.5) < 0.5
    assert abs((bytes_ < oracle.mask_threshold8(0.3)).mean() - 77 / 256) < 2e-3
    assert oracle.mask_threshold8(0.3) == 77 and oracle.mask_threshold16(0.3) == round(np.sqrt(0.3) * 65536)


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("B,CI,CO,G,HW", [(6, 50, 9, 1, 1), (3, 24, 8, 2, 2)])
def test_masked_forward_matches_numpy_mask(oracle, mode, B, CI, CO, G, HW):
    q, seed = 0.3, 1234
    x = _rand((B, CI, HW), 81, "rand")
    w = _rand((CO, CI // G), 82)
    y, pos = oracle.masked_inf_dist_forward(x, w, q, seed, mode, G)
    CIg, COg = CI // G, CO // G
    b, c, hw, n = np.meshgrid(np.arange(B), np.arange(CO), np.arange(HW), np.arange(CIg), indexing="ij")
    if mode == 0:
        out_lin = (b * CO + c) * HW + hw
        keep = ((_word(seed, 0, out_lin, n >> 2) >> (8 * (n & 3)).astype(np.uint64)) & 0xFF) < oracle.mask_threshold8(q)
    else:
        t16 = oracle.mask_threshold16(q)
        g = c // COg
        keep = ((_word(seed, 1, (b * G + g) * HW + hw, n) >> np.uint64(16)) < t16) & ((_word(seed, 2, c, n) >> np.uint64(16)) < t16)
    assert abs(keep.mean() - q) < 0.1   # few independent draws in the factored mode at this size
    d = _brute_diff(x, w, G).permute(0, 1, 2, 4, 3).reshape(B, CO, HW, CIg).numpy()
    a = np.where(keep, np.abs(d), -1.0)
    ref = np.maximum(a.max(-1), np.float32(1e-10)).astype(np.float32)
    assert np.array_equal(y, ref)
    idx, neg = _split_pos(pos)
    won = a.max(-1) > 1e-10
    assert np.array_equal(idx[won], a.argmax(-1)[won]) and np.all(pos[~won] == 0)
    sg = np.take_along_axis(d, a.argmax(-1)[..., None], -1)[..., 0] < 0
    assert np.array_equal(neg[won], sg[won])
    # q = 1 keeps everything
    y1 = oracle.masked_inf_dist_forward(x, w, 1.0, seed, mode, G, need_pos=False)
    assert np.array_equal(y1, oracle.inf_dist_forward(x, w, G, need_pos=False))


def test_mean_shift(oracle):
    x = _rand((7, 5, 3), 91)
    out, mean = oracle.mean_shift(x)
    np.testing.assert_allclose(mean, x.mean((0, 2)), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(out, x - x.mean((0, 2))[None, :, None], rtol=1e-6, atol=1e-7)
