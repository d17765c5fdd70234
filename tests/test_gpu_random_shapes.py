"""GPU parity on randomly drawn shapes (seeded): ragged sizes, groups, spatial positions, one- and two-sided
kept-channel index lists, data on a coarse grid (exact ties), inverted intervals.  Same bars as the other
parity tests: bit-exact l-inf / masked / interval values and positions and sort-neuron positions, rel 1e-5 for
l-p values, sort-neuron sums and every gradient accumulation."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def close(a, b, what):
    b = np.asarray(b)
    a = a.cpu().numpy()
    np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-5 * max(float(np.abs(b).max()), 1e-30), err_msg=what)


@pytest.mark.parametrize("seed", [1, 2])
def test_index_list_paths_on_random_shapes(oracle, seed):
    from sortnet_amd import ext, functional as F
    dev = _dev()
    rng = np.random.default_rng(seed)
    for trial in range(25):
        G = int(rng.choice([1, 1, 2, 3]))
        HW = int(rng.choice([1, 1, 2, 3]))
        B = int(rng.integers(1, 100)); CIg = int(rng.integers(1, 400)); COg = int(rng.integers(1, 150))
        cn = int(rng.integers(1, CIg + 1)); cm = int(rng.integers(1, COg + 1))
        S = (B + 31) // 32
        use_ci, use_co = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        ci = np.stack([[np.sort(rng.choice(CIg, cn, replace=False)) for _ in range(G)] for _ in range(S)]).astype(np.int32) if use_ci else None
        co = np.stack([[np.sort(rng.choice(COg, cm, replace=False)) for _ in range(G)] for _ in range(S)]).astype(np.int32) if use_co else None
        nin, nout = (cn if use_ci else CIg), (cm if use_co else COg)
        x = torch.from_numpy(rng.random((B, nin * G, HW), dtype=np.float32))
        w = torch.from_numpy((rng.standard_normal((COg * G, CIg)) * 0.3).astype(np.float32))
        if trial % 3 == 0:   # ties
            x, w = torch.round(x * 4) / 4, torch.round(w * 2) / 2
        gy = torch.from_numpy(rng.standard_normal((B, nout * G, HW)).astype(np.float32))
        ry, rpos = oracle.inf_dist_forward(x.numpy(), w.numpy(), G, True, ci, co)
        xd, wd, gd = x.to(dev), w.to(dev), gy.to(dev)
        cid = None if ci is None else torch.from_numpy(ci).to(dev); cod = None if co is None else torch.from_numpy(co).to(dev)
        y = torch.empty(B, nout * G, HW, device=dev); pos = torch.empty(B, nout * G, HW, device=dev, dtype=torch.int32)
        ext.inf_dist_forward(xd, wd, y, pos, G, cid, cod)
        assert np.array_equal(y.cpu().numpy(), ry), "linf value"
        assert np.array_equal(pos.cpu().numpy(), rpos), "linf pos"
        rgx, rgw = oracle.inf_dist_backward(gy.numpy(), rpos, x.shape, w.shape, G, True, ci, co)
        gx, gw = torch.empty_like(xd), torch.empty_like(wd)
        ext.inf_dist_backward_input_weight(gd, pos, gx, gw, G, cid, cod)
        close(gx, rgx, "gx"); close(gw, rgw, "gw")
        for p in (3.0, 12.5):
            ryp = oracle.norm_dist_forward(x.numpy(), w.numpy(), p, G, ci, co)
            ext.norm_dist_forward(xd, wd, y, G, p, cid, cod)
            np.testing.assert_allclose(y.cpu().numpy(), ryp, rtol=1e-5, err_msg="lp fwd p=%g" % p)
            rgx, rgw = oracle.norm_dist_backward(gy.numpy(), x.numpy(), w.numpy(), ryp, p, G, True, ci, co)
            ext.norm_dist_backward_input_weight(gd, xd, wd, torch.from_numpy(ryp).to(dev), gx, gw, G, p, cid, cod)
            close(gx, rgx, "lp gx"); close(gw, rgw, "lp gw")
            gx.fill_(float("nan"))
            ext.norm_dist_backward_input(gd, xd, wd, torch.from_numpy(ryp).to(dev), gx, G, p, cid, cod)
            close(gx, rgx, "lp gx (input only)")
        # index-list mean shift against float64
        if use_co:
            yv = torch.from_numpy(rng.standard_normal((B, cm * G, HW)).astype(np.float32))
            out, mean = F.mean_shift_index(yv.to(dev), cod, G * COg, None, 0.1)
            tot, seen = np.zeros((G, COg)), np.full((G, COg), 1e-10)
            yn = yv.double().numpy()
            for b in range(B):
                for gi in range(G):
                    tot[gi, co[b // 32, gi]] += yn[b, gi * cm:(gi + 1) * cm].sum(-1); seen[gi, co[b // 32, gi]] += 1
            np.testing.assert_allclose(mean.cpu().numpy(), (tot / (seen * HW)).reshape(-1), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("seed", [3, 4])
def test_dense_paths_on_random_shapes(oracle, seed):
    from sortnet_amd import ext
    dev = _dev()
    rng = np.random.default_rng(seed)
    for trial in range(20):
        G = int(rng.choice([1, 1, 2]))
        HW = int(rng.choice([1, 1, 1, 2, 5]))
        B = int(rng.integers(1, 90)); CIg = int(rng.choice([rng.integers(1, 300), 4 * rng.integers(1, 200)])); COg = int(rng.integers(1, 160))
        x = torch.from_numpy(rng.random((B, CIg * G, HW), dtype=np.float32))
        w = torch.from_numpy((rng.standard_normal((COg * G, CIg)) * 0.3).astype(np.float32))
        if trial % 3 == 0:
            x, w = torch.round(x * 4) / 4, torch.round(w * 2) / 2
        xd, wd = x.to(dev), w.to(dev)
        y = torch.empty(B, COg * G, HW, device=dev); pos = torch.empty(B, COg * G, HW, device=dev, dtype=torch.int32)
        ry, rpos = oracle.inf_dist_forward(x.numpy(), w.numpy(), G)
        ext.inf_dist_forward(xd, wd, y, pos, G)
        assert np.array_equal(y.cpu().numpy(), ry) and np.array_equal(pos.cpu().numpy(), rpos), "linf"
        ext.inf_dist_forward_nograd(xd, wd, y, G)
        assert np.array_equal(y.cpu().numpy(), ry), "linf nograd"
        for mode in (0, 1):
            q, seed = float(rng.choice([0.3, 0.7, 1.0])), int(rng.integers(0, 2**31))
            my, mpos = oracle.masked_inf_dist_forward(x.numpy(), w.numpy(), q, seed, mode, G)
            ext.masked_inf_dist_forward(xd, wd, y, pos, G, q, seed, mode)
            assert np.array_equal(y.cpu().numpy(), my) and np.array_equal(pos.cpu().numpy(), mpos), "masked mode %d" % mode
            ext.masked_inf_dist_forward(xd, wd, y, None, G, q, seed, mode)
            assert np.array_equal(y.cpu().numpy(), my), "masked nograd mode %d" % mode
        eps = np.float32(rng.choice([0.01, 0.2]))
        xl, xu = (x - eps).contiguous(), (x + eps).contiguous()
        if trial % 4 == 0:
            xl[0], xu[0] = xu[0].clone(), xl[0].clone()      # inverted interval: repaired to the midpoint
        rl, ru, rpl, rpu = oracle.bound_inf_dist_forward(xl.numpy(), xu.numpy(), w.numpy(), G)
        yl, yu = torch.empty_like(y), torch.empty_like(y); pl, pu = torch.empty_like(pos), torch.empty_like(pos)
        ext.bound_inf_dist_forward(xl.to(dev), xu.to(dev), wd, yl, yu, pl, pu, G)
        assert np.array_equal(yl.cpu().numpy(), rl) and np.array_equal(yu.cpu().numpy(), ru), "bound values"
        assert np.array_equal(pl.cpu().numpy(), rpl) and np.array_equal(pu.cpu().numpy(), rpu), "bound pos"
        ext.bound_inf_dist_forward_nograd(xl.to(dev), xu.to(dev), wd, yl, yu, G)
        assert np.array_equal(yl.cpu().numpy(), rl) and np.array_equal(yu.cpu().numpy(), ru), "bound nograd"
        K = int(rng.integers(2, min(CIg, 25) + 1)) if CIg >= 2 else 0
        if K:
            qs = float(rng.choice([0.3, 0.5, 0.9]))
            sy, spos = oracle.sort_neuron_forward(x.numpy(), w.numpy(), qs, K, G)
            posK = torch.empty(K, B, COg * G, HW, device=dev, dtype=torch.int32)
            ext.sort_neuron_forward(xd, wd, y, posK, G, qs, K)
            assert np.array_equal(posK.cpu().numpy(), spos), "sort pos"
            close(y, sy, "sort y")
            ext.sort_neuron_forward_nograd(xd, wd, y, G, qs, K)
            close(y, sy, "sort nograd")
            bl, bu = oracle.bound_sort_neuron_forward(xl.numpy(), xu.numpy(), w.numpy(), qs, K, G)
            ext.bound_sort_neuron_forward(xl.to(dev), xu.to(dev), wd, yl, yu, G, qs, K)
            close(yl, bl, "bound sort lo"); close(yu, bu, "bound sort up")
