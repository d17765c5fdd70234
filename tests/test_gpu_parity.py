"""GPU parity: every C-ABI entry point (reached through sortnet_amd.ext -> ctypes) against the
CPU oracle on identical seeded inputs.

Bit-exact sets (compared with array_equal): l-inf values and positions, masked-neuron values and
positions, interval bounds and their positions, sort-neuron positions.  Tolerance sets
(rel 1e-5, absolute floor 1e-5 of the largest reference magnitude): sort-neuron weighted sums,
l-p values, every gradient accumulation.
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


def _gen(shape, seed, kind="randn", scale=1.0):
    g = torch.Generator().manual_seed(seed)
    t = torch.rand(shape, generator=g) if kind == "rand" else torch.randn(shape, generator=g)
    return (t * scale).float().contiguous()


def _close(gpu, ref, rtol=RTOL):
    ref = np.asarray(ref)
    got = gpu.cpu().numpy()
    np.testing.assert_allclose(got, ref, rtol=rtol, atol=rtol * max(float(np.abs(ref).max()), 1e-30))


def _index_lists(B, CI, CO, ci_n, co_n, G, seed):
    rng = np.random.default_rng(seed)
    S = (B + 31) // 32
    ci = np.stack([[np.sort(rng.choice(CI // G, ci_n, replace=False)) for _ in range(G)] for _ in range(S)])
    co = np.stack([[np.sort(rng.choice(CO // G, co_n, replace=False)) for _ in range(G)] for _ in range(S)])
    return ci.astype(np.int32), co.astype(np.int32)


SHAPES = [
    # B, CI, CO, G, HW
    (5, 37, 11, 1, 1),        # ragged everything
    (70, 96, 200, 1, 1),      # several tiles, vector path
    (33, 64, 48, 2, 1),       # groups
    (6, 20, 24, 2, 3),        # groups and spatial positions
    (130, 260, 140, 1, 1),    # tails in every dimension, split-N candidate
]


@pytest.mark.parametrize("B,CI,CO,G,HW", SHAPES)
def test_inf_dist_forward_and_backward(oracle, B, CI, CO, G, HW):
    from sortnet_amd import ext
    dev = _dev()
    x, w, gy = _gen((B, CI, HW), 1, "rand"), _gen((CO, CI // G), 2, scale=0.3), _gen((B, CO, HW), 3)
    ry, rpos = oracle.inf_dist_forward(x.numpy(), w.numpy(), G)
    xd, wd, gd = x.to(dev), w.to(dev), gy.to(dev)
    y = torch.empty(B, CO, HW, device=dev)
    pos = torch.empty(B, CO, HW, device=dev, dtype=torch.int32)
    ext.inf_dist_forward(xd, wd, y, pos, G)
    assert np.array_equal(y.cpu().numpy(), ry)
    assert np.array_equal(pos.cpu().numpy(), rpos)
    y2 = torch.empty_like(y)
    ext.inf_dist_forward_nograd(xd, wd, y2, G)
    assert np.array_equal(y2.cpu().numpy(), ry)
    rgx, rgw = oracle.inf_dist_backward(gy.numpy(), rpos, x.shape, w.shape, G)
    gx, gw = torch.empty_like(xd), torch.empty_like(wd)
    ext.inf_dist_backward_input_weight(gd, pos, gx, gw, G)
    _close(gx, rgx)
    _close(gw, rgw)
    gx2 = torch.full_like(xd, 7.0)
    ext.inf_dist_backward_input(gd, pos, gx2, G)
    _close(gx2, rgx)


def test_backward_long_rows_use_global_atomics(oracle):
    """Reduction length above the LDS row-histogram limit: the atomic fallback kernels."""
    from sortnet_amd import ext
    dev = _dev()
    B, CI, CO = 3, 12300, 5
    x, w, gy = _gen((B, CI, 1), 61, "rand"), _gen((CO, CI), 62, scale=0.3), _gen((B, CO, 1), 63)
    ry, rpos = oracle.inf_dist_forward(x.numpy(), w.numpy())
    y = torch.empty(B, CO, 1, device=dev)
    pos = torch.empty(B, CO, 1, device=dev, dtype=torch.int32)
    ext.inf_dist_forward(x.to(dev), w.to(dev), y, pos, 1)
    assert np.array_equal(y.cpu().numpy(), ry) and np.array_equal(pos.cpu().numpy(), rpos)
    rgx, rgw = oracle.inf_dist_backward(gy.numpy(), rpos, x.shape, w.shape)
    gx, gw = torch.empty(B, CI, 1, device=dev), torch.empty(CO, CI, device=dev)
    ext.inf_dist_backward_input_weight(gy.to(dev), pos, gx, gw, 1)
    _close(gx, rgx)
    _close(gw, rgw)
    xl, xu = (x - 0.01).contiguous(), (x + 0.01).contiguous()
    rl, ru, rpl, rpu = oracle.bound_inf_dist_forward(xl.numpy(), xu.numpy(), w.numpy())
    rgl, rgu, rgw2 = oracle.bound_inf_dist_backward(gy.numpy(), gy.numpy(), rpl, rpu, x.shape, w.shape)
    gl, gu, gw2 = torch.empty(B, CI, 1, device=dev), torch.empty(B, CI, 1, device=dev), torch.empty(CO, CI, device=dev)
    ext.bound_inf_dist_backward_input_weight(gy.to(dev), gy.to(dev), torch.from_numpy(rpl).to(dev),
                                             torch.from_numpy(rpu).to(dev), gl, gu, gw2, 1)
    _close(gl, rgl)
    _close(gu, rgu)
    _close(gw2, rgw2)


def test_inf_dist_ties_and_floor(oracle):
    from sortnet_amd import ext
    dev = _dev()
    x = np.zeros((2, 70, 1), np.float32)
    w = np.zeros((3, 70), np.float32)
    w[0, [1, 40, 66]] = 2.0
    w[0, 35] = -2.0
    w[1, 2] = 1e-10
    w[2, 69] = -3.0
    ry, rpos = oracle.inf_dist_forward(x, w)
    y = torch.empty(2, 3, 1, device=dev)
    pos = torch.empty(2, 3, 1, device=dev, dtype=torch.int32)
    ext.inf_dist_forward(torch.from_numpy(x).to(dev), torch.from_numpy(w).to(dev), y, pos, 1)
    assert np.array_equal(y.cpu().numpy(), ry) and np.array_equal(pos.cpu().numpy(), rpos)
    assert pos.cpu().numpy().view(np.uint32)[0, 0, 0] == (1 | 0x80000000) and pos[0, 1, 0].item() == 0


@pytest.mark.parametrize("B,CI,CO,G,ci_n,co_n", [(70, 96, 64, 1, 29, 21), (40, 64, 48, 2, 12, 8), (64, 128, 160, 1, 128, 37),
                                                  (96, 1024, 300, 1, 701, 150)])
def test_inf_dist_index_lists(oracle, B, CI, CO, G, ci_n, co_n):
    from sortnet_amd import ext
    dev = _dev()
    ci, co = _index_lists(B, CI, CO, ci_n, co_n, G, 5)
    w = _gen((CO, CI // G), 6, scale=0.3)
    x, gy = _gen((B, ci_n * G, 1), 7, "rand"), _gen((B, co_n * G, 1), 8)
    ry, rpos = oracle.inf_dist_forward(x.numpy(), w.numpy(), G, True, ci, co)
    xd, wd, gd = x.to(dev), w.to(dev), gy.to(dev)
    cid, cod = torch.from_numpy(ci).to(dev), torch.from_numpy(co).to(dev)
    y = torch.empty(B, co_n * G, 1, device=dev)
    pos = torch.empty(B, co_n * G, 1, device=dev, dtype=torch.int32)
    ext.inf_dist_forward(xd, wd, y, pos, G, cid, cod)
    assert np.array_equal(y.cpu().numpy(), ry) and np.array_equal(pos.cpu().numpy(), rpos)
    rgx, rgw = oracle.inf_dist_backward(gy.numpy(), rpos, x.shape, w.shape, G, True, ci, co)
    gx, gw = torch.empty_like(xd), torch.empty_like(wd)
    ext.inf_dist_backward_input_weight(gd, pos, gx, gw, G, cid, cod)
    _close(gx, rgx)
    _close(gw, rgw)
    # only output channels dropped / only input channels dropped
    y3 = torch.empty(B, co_n * G, 1, device=dev)
    p3 = torch.empty_like(pos)
    xfull = _gen((B, CI, 1), 9, "rand")
    ext.inf_dist_forward(xfull.to(dev), wd, y3, p3, G, None, cod)
    r3, rp3 = oracle.inf_dist_forward(xfull.numpy(), w.numpy(), G, True, None, co)
    assert np.array_equal(y3.cpu().numpy(), r3) and np.array_equal(p3.cpu().numpy(), rp3)
    y4 = torch.empty(B, CO, 1, device=dev)
    p4 = torch.empty(B, CO, 1, device=dev, dtype=torch.int32)
    ext.inf_dist_forward(xd, wd, y4, p4, G, cid, None)
    r4, rp4 = oracle.inf_dist_forward(x.numpy(), w.numpy(), G, True, ci, None)
    assert np.array_equal(y4.cpu().numpy(), r4) and np.array_equal(p4.cpu().numpy(), rp4)
    # their backward passes: weight rows nobody kept come back as zeros, rows kept by some sub-batches only from those
    rgx3, rgw3 = oracle.inf_dist_backward(gy.numpy(), rp3, xfull.shape, w.shape, G, True, None, co)
    gx3, gw3 = torch.empty(B, CI, 1, device=dev), torch.full_like(wd, float("nan"))
    ext.inf_dist_backward_input_weight(gd, p3, gx3, gw3, G, None, cod)
    _close(gx3, rgx3)
    _close(gw3, rgw3)
    gy4 = _gen((B, CO, 1), 10)
    rgx4, rgw4 = oracle.inf_dist_backward(gy4.numpy(), rp4, x.shape, w.shape, G, True, ci, None)
    gx4, gw4 = torch.empty_like(xd), torch.full_like(wd, float("nan"))
    ext.inf_dist_backward_input_weight(gy4.to(dev), p4, gx4, gw4, G, cid, None)
    _close(gx4, rgx4)
    _close(gw4, rgw4)


def test_inf_dist_index_lists_with_spatial_positions(oracle):
    """Index lists on a layer with HW = 3 and two groups: forward bits and both gradients."""
    from sortnet_amd import ext
    dev = _dev()
    B, CI, CO, G, HW, ci_n, co_n = 40, 64, 48, 2, 3, 12, 8
    ci, co = _index_lists(B, CI, CO, ci_n, co_n, G, 25)
    w = _gen((CO, CI // G), 26, scale=0.3)
    x, gy = _gen((B, ci_n * G, HW), 27, "rand"), _gen((B, co_n * G, HW), 28)
    ry, rpos = oracle.inf_dist_forward(x.numpy(), w.numpy(), G, True, ci, co)
    xd, wd, gd = x.to(dev), w.to(dev), gy.to(dev)
    cid, cod = torch.from_numpy(ci).to(dev), torch.from_numpy(co).to(dev)
    y = torch.empty(B, co_n * G, HW, device=dev)
    pos = torch.empty(B, co_n * G, HW, device=dev, dtype=torch.int32)
    ext.inf_dist_forward(xd, wd, y, pos, G, cid, cod)
    assert np.array_equal(y.cpu().numpy(), ry) and np.array_equal(pos.cpu().numpy(), rpos)
    rgx, rgw = oracle.inf_dist_backward(gy.numpy(), rpos, x.shape, w.shape, G, True, ci, co)
    gx, gw = torch.empty_like(xd), torch.full_like(wd, float("nan"))
    ext.inf_dist_backward_input_weight(gd, pos, gx, gw, G, cid, cod)
    _close(gx, rgx)
    _close(gw, rgw)


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("B,CI,CO,G,HW", SHAPES)
def test_masked_inf_dist(oracle, mode, B, CI, CO, G, HW):
    from sortnet_amd import ext
    dev = _dev()
    x, w = _gen((B, CI, HW), 11, "rand"), _gen((CO, CI // G), 12, scale=0.3)
    q, seed = 0.3, 20240
    ry, rpos = oracle.masked_inf_dist_forward(x.numpy(), w.numpy(), q, seed, mode, G)
    y = torch.empty(B, CO, HW, device=dev)
    pos = torch.empty(B, CO, HW, device=dev, dtype=torch.int32)
    ext.masked_inf_dist_forward(x.to(dev), w.to(dev), y, pos, G, q, seed, mode)
    assert np.array_equal(y.cpu().numpy(), ry)
    assert np.array_equal(pos.cpu().numpy(), rpos)
    y2 = torch.empty_like(y)
    ext.masked_inf_dist_forward(x.to(dev), w.to(dev), y2, None, G, q, seed, mode)
    assert np.array_equal(y2.cpu().numpy(), ry)


@pytest.mark.parametrize("B,CI,CO,G,HW", SHAPES)
def test_bound_inf_dist_forward_and_backward(oracle, B, CI, CO, G, HW):
    from sortnet_amd import ext
    dev = _dev()
    x, w = _gen((B, CI, HW), 21, "rand"), _gen((CO, CI // G), 22, scale=0.3)
    eps = np.float32(2 / 255)
    xl, xu = (x - eps).contiguous(), (x + eps).contiguous()
    xl[0, 0, 0], xu[0, 0, 0] = xu[0, 0, 0].item(), xl[0, 0, 0].item()   # inverted interval -> midpoint repair
    gl, gu = _gen((B, CO, HW), 23), _gen((B, CO, HW), 24)
    rl, ru, rpl, rpu = oracle.bound_inf_dist_forward(xl.numpy(), xu.numpy(), w.numpy(), G)
    xld, xud, wd = xl.to(dev), xu.to(dev), w.to(dev)
    yl = torch.empty(B, CO, HW, device=dev)
    yu = torch.empty_like(yl)
    pl = torch.empty(B, CO, HW, device=dev, dtype=torch.int32)
    pu = torch.empty_like(pl)
    ext.bound_inf_dist_forward(xld, xud, wd, yl, yu, pl, pu, G)
    assert np.array_equal(yl.cpu().numpy(), rl) and np.array_equal(yu.cpu().numpy(), ru)
    assert np.array_equal(pl.cpu().numpy(), rpl) and np.array_equal(pu.cpu().numpy(), rpu)
    yl2, yu2 = torch.empty_like(yl), torch.empty_like(yl)
    ext.bound_inf_dist_forward_nograd(xld, xud, wd, yl2, yu2, G)
    assert np.array_equal(yl2.cpu().numpy(), rl) and np.array_equal(yu2.cpu().numpy(), ru)
    rgl, rgu, rgw = oracle.bound_inf_dist_backward(gl.numpy(), gu.numpy(), rpl, rpu, x.shape, w.shape, G)
    gxl, gxu, gw = torch.empty_like(xld), torch.empty_like(xld), torch.empty_like(wd)
    ext.bound_inf_dist_backward_input_weight(gl.to(dev), gu.to(dev), pl, pu, gxl, gxu, gw, G)
    _close(gxl, rgl)
    _close(gxu, rgu)
    _close(gw, rgw)
    gxl2, gxu2 = torch.empty_like(xld), torch.empty_like(xld)
    ext.bound_inf_dist_backward_input(gl.to(dev), gu.to(dev), pl, pu, gxl2, gxu2, G)
    _close(gxl2, rgl)
    _close(gxu2, rgu)


def test_bound_inf_dist_sentinel(oracle):
    from sortnet_amd import ext
    dev = _dev()
    xl = torch.full((3, 8, 1), -1.0)
    xu = torch.full((3, 8, 1), 1.0)
    w = torch.zeros(5, 8)
    rl, ru, rpl, rpu = oracle.bound_inf_dist_forward(xl.numpy(), xu.numpy(), w.numpy())
    yl, yu = torch.empty(3, 5, 1, device=dev), torch.empty(3, 5, 1, device=dev)
    pl = torch.empty(3, 5, 1, device=dev, dtype=torch.int32)
    pu = torch.empty_like(pl)
    ext.bound_inf_dist_forward(xl.to(dev), xu.to(dev), w.to(dev), yl, yu, pl, pu, 1)
    assert np.array_equal(pl.cpu().numpy(), rpl) and np.all(pl.cpu().numpy() == -1)
    assert np.array_equal(yl.cpu().numpy(), rl) and np.array_equal(yu.cpu().numpy(), ru)
    g = torch.ones(3, 5, 1, device=dev)
    gxl, gxu, gw = torch.empty(3, 8, 1, device=dev), torch.empty(3, 8, 1, device=dev), torch.empty(5, 8, device=dev)
    ext.bound_inf_dist_backward_input_weight(g, g, pl, pu, gxl, gxu, gw, 1)
    rgl, rgu, rgw = oracle.bound_inf_dist_backward(g.cpu().numpy(), g.cpu().numpy(), rpl, rpu, (3, 8, 1), (5, 8))
    _close(gxl, rgl)
    _close(gxu, rgu)
    _close(gw, rgw)


@pytest.mark.parametrize("K,q", [(10, 0.3), (2, 0.75), (25, 0.6), (7, 1.0)])
@pytest.mark.parametrize("B,CI,CO,G,HW", SHAPES[:4])
def test_sort_neuron(oracle, K, q, B, CI, CO, G, HW):
    from sortnet_amd import ext
    dev = _dev()
    if K > CI // G:
        pytest.skip("K larger than the reduction length is clamped by the Python wrapper")
    x, w, gy = _gen((B, CI, HW), 31, "rand"), _gen((CO, CI // G), 32, scale=0.3), _gen((B, CO, HW), 33)
    ry, rpos = oracle.sort_neuron_forward(x.numpy(), w.numpy(), q, K, G)
    xd, wd, gd = x.to(dev), w.to(dev), gy.to(dev)
    y = torch.empty(B, CO, HW, device=dev)
    pos = torch.empty(K, B, CO, HW, device=dev, dtype=torch.int32)
    ext.sort_neuron_forward(xd, wd, y, pos, G, q, K)
    assert np.array_equal(pos.cpu().numpy(), rpos)
    _close(y, ry)
    y2 = torch.empty_like(y)
    ext.sort_neuron_forward_nograd(xd, wd, y2, G, q, K)
    _close(y2, ry)
    rgx, rgw = oracle.sort_neuron_backward(gy.numpy(), rpos, x.shape, w.shape, q, K, G)
    gx, gw = torch.empty_like(xd), torch.empty_like(wd)
    ext.sort_neuron_backward_input_weight(gd, pos, gx, gw, G, q, K)
    _close(gx, rgx)
    _close(gw, rgw)
    gx2 = torch.empty_like(xd)
    ext.sort_neuron_backward_input(gd, pos, gx2, G, q, K)
    _close(gx2, rgx)
    # interval version
    eps = np.float32(0.02)
    xl, xu = (x - eps).contiguous(), (x + eps).contiguous()
    rl, ru = oracle.bound_sort_neuron_forward(xl.numpy(), xu.numpy(), w.numpy(), q, K, G)
    yl, yu = torch.empty_like(y), torch.empty_like(y)
    ext.bound_sort_neuron_forward(xl.to(dev), xu.to(dev), wd, yl, yu, G, q, K)
    _close(yl, rl)
    _close(yu, ru)


def test_sort_neuron_tie_order(oracle):
    from sortnet_amd import ext
    dev = _dev()
    x = np.zeros((1, 5, 1), np.float32)
    w = np.array([[0.0, 1.0, -1.0, 1.0, 0.0]], np.float32)
    ry, rpos = oracle.sort_neuron_forward(x, w, 0.5, 4)
    y = torch.empty(1, 1, 1, device=dev)
    pos = torch.empty(4, 1, 1, 1, device=dev, dtype=torch.int32)
    ext.sort_neuron_forward(torch.from_numpy(x).to(dev), torch.from_numpy(w).to(dev), y, pos, 1, 0.5, 4)
    assert np.array_equal(pos.cpu().numpy(), rpos)
    _close(y, ry)


@pytest.mark.parametrize("case", ["random", "grid", "flat", "sparse", "groups"])
@pytest.mark.parametrize("K", [10, 4, 12])
def test_sort_neuron_long_rows(oracle, case, K):
    """Rows long enough for the two-level path (chunk lists, then a candidate scan): continuous data, data
    on a coarse grid (exact ties inside and across chunks), chunk maxima that are all equal (the exhaustive
    scan of the second pass), rows with fewer than K non-zero terms, and groups."""
    from sortnet_amd import ext
    dev = _dev()
    G = 2 if case == "groups" else 1
    B, CI, CO = 37, 2048 * G, 24 * G
    x, w = _gen((B, CI, 1), 51, "rand"), _gen((CO, CI // G), 52, scale=0.3)
    if case == "grid":
        x, w = torch.round(x * 8) / 8, torch.round(w * 4) / 4
    elif case == "flat":
        x, w = torch.round(x * 2) / 2, torch.zeros_like(w)       # every chunk maximum is 1
    elif case == "sparse":
        keep = torch.zeros(CI)
        keep[[5, 700, 701, 1500]] = 1.0
        x, w = x * keep.view(1, -1, 1), w * 0
    x, w = x.contiguous(), w.contiguous()
    q = 0.3
    ry, rpos = oracle.sort_neuron_forward(x.numpy(), w.numpy(), q, K, G)
    xd, wd = x.to(dev), w.to(dev)
    y = torch.empty(B, CO, 1, device=dev)
    pos = torch.empty(K, B, CO, 1, device=dev, dtype=torch.int32)
    ext.sort_neuron_forward(xd, wd, y, pos, G, q, K)
    assert np.array_equal(pos.cpu().numpy(), rpos)
    _close(y, ry)
    y2 = torch.empty_like(y)
    ext.sort_neuron_forward_nograd(xd, wd, y2, G, q, K)
    _close(y2, ry)


def test_sort_neuron_widest_rows(oracle):
    """12288 inputs per row (the widest first layer): the candidate scan needs more than 64 KiB of LDS; the
    row length is not a multiple of the chunk size in the second case."""
    from sortnet_amd import ext
    dev = _dev()
    for CI in (12288, 12268):
        B, CO, K, q = 70, 9, 10, 0.3
        x, w = _gen((B, CI, 1), 61, "rand"), _gen((CO, CI), 62, scale=0.3)
        ry, rpos = oracle.sort_neuron_forward(x.numpy(), w.numpy(), q, K)
        xd, wd = x.to(dev), w.to(dev)
        y = torch.empty(B, CO, 1, device=dev)
        pos = torch.empty(K, B, CO, 1, device=dev, dtype=torch.int32)
        ext.sort_neuron_forward(xd, wd, y, pos, 1, q, K)
        assert np.array_equal(pos.cpu().numpy(), rpos)
        _close(y, ry)
        ext.sort_neuron_forward_nograd(xd, wd, y, 1, q, K)
        _close(y, ry)


# every integer-power chain (forward p = 1..8, backward p - 1 = 0..8), exponents below 1 on either side, general p
@pytest.mark.parametrize("p", [0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0, 9.0, 9.5, 11.3, 64.0, 300.0])
@pytest.mark.parametrize("B,CI,CO,G,HW", [SHAPES[1], SHAPES[3], SHAPES[4]])
def test_norm_dist(oracle, p, B, CI, CO, G, HW):
    from sortnet_amd import ext
    dev = _dev()
    x, w, gy = _gen((B, CI, HW), 41), _gen((CO, CI // G), 42, scale=0.3), _gen((B, CO, HW), 43)
    ry = oracle.norm_dist_forward(x.numpy(), w.numpy(), p, G)
    xd, wd, gd = x.to(dev), w.to(dev), gy.to(dev)
    y = torch.empty(B, CO, HW, device=dev)
    ext.norm_dist_forward(xd, wd, y, G, p)
    np.testing.assert_allclose(y.cpu().numpy(), ry, rtol=RTOL)
    # backward from the oracle's saved output, so both sides differentiate the same y
    yd = torch.from_numpy(ry).to(dev)
    rgx, rgw = oracle.norm_dist_backward(gy.numpy(), x.numpy(), w.numpy(), ry, p, G)
    gx, gw = torch.empty_like(xd), torch.empty_like(wd)
    ext.norm_dist_backward_input_weight(gd, xd, wd, yd, gx, gw, G, p)
    _close(gx, rgx)
    _close(gw, rgw)
    gx2 = torch.empty_like(xd)
    ext.norm_dist_backward_input(gd, xd, wd, yd, gx2, G, p)
    _close(gx2, rgx)
    # forward with a caller-supplied maximum (any positive scale gives the same norm)
    mx = torch.from_numpy(oracle.inf_dist_forward(x.numpy(), w.numpy(), G, need_pos=False)).to(dev)
    y3 = torch.empty_like(y)
    ext.norm_dist_forward_with_max(xd, wd, mx, y3, G, p)
    np.testing.assert_allclose(y3.cpu().numpy(), ry, rtol=RTOL)


@pytest.mark.parametrize("p", [8.0, 20.0, 24.0, 64.0, 256.0, 300.0])
@pytest.mark.parametrize("B,CI,CO,G,ci_n,co_n", [(70, 96, 64, 1, 29, 21), (40, 64, 48, 2, 12, 8), (96, 1024, 300, 1, 701, 150)])
def test_norm_dist_index_lists(oracle, p, B, CI, CO, G, ci_n, co_n):
    from sortnet_amd import ext
    dev = _dev()
    ci, co = _index_lists(B, CI, CO, ci_n, co_n, G, 15)
    w = _gen((CO, CI // G), 46, scale=0.3)
    x, gy = _gen((B, ci_n * G, 1), 47), _gen((B, co_n * G, 1), 48)
    ry = oracle.norm_dist_forward(x.numpy(), w.numpy(), p, G, ci, co)
    xd, wd, gd = x.to(dev), w.to(dev), gy.to(dev)
    cid, cod = torch.from_numpy(ci).to(dev), torch.from_numpy(co).to(dev)
    y = torch.empty(B, co_n * G, 1, device=dev)
    ext.norm_dist_forward(xd, wd, y, G, p, cid, cod)
    np.testing.assert_allclose(y.cpu().numpy(), ry, rtol=RTOL)
    rgx, rgw = oracle.norm_dist_backward(gy.numpy(), x.numpy(), w.numpy(), ry, p, G, True, ci, co)
    gx, gw = torch.empty_like(xd), torch.empty_like(wd)
    ext.norm_dist_backward_input_weight(gd, xd, wd, torch.from_numpy(ry).to(dev), gx, gw, G, p, cid, cod)
    _close(gx, rgx)
    _close(gw, rgw)
    # caller-supplied maximum with index lists (any scale at or above the true maximum gives the same norm)
    mx = torch.from_numpy(oracle.inf_dist_forward(x.numpy(), w.numpy(), G, False, ci, co) * np.float32(1.25)).to(dev)
    y2 = torch.empty_like(y)
    ext.norm_dist_forward_with_max(xd, wd, mx, y2, G, p, cid, cod)
    np.testing.assert_allclose(y2.cpu().numpy(), ry, rtol=RTOL)
    # only output channels dropped / only input channels dropped
    xfull = _gen((B, CI, 1), 49)
    y3 = torch.empty(B, co_n * G, 1, device=dev)
    ext.norm_dist_forward(xfull.to(dev), wd, y3, G, p, None, cod)
    np.testing.assert_allclose(y3.cpu().numpy(), oracle.norm_dist_forward(xfull.numpy(), w.numpy(), p, G, None, co), rtol=RTOL)
    y4 = torch.empty(B, CO, 1, device=dev)
    ext.norm_dist_forward(xd, wd, y4, G, p, cid, None)
    np.testing.assert_allclose(y4.cpu().numpy(), oracle.norm_dist_forward(x.numpy(), w.numpy(), p, G, ci, None), rtol=RTOL)


@pytest.mark.parametrize("p", [40.0, 100.0, 400.0, 1000.0])
@pytest.mark.parametrize("kind", ["grid", "continuous"])
def test_norm_dist_large_p(oracle, p, kind):
    """Large p, where the kernels evaluate r^p only for terms that can matter: rows with many terms at or near
    the maximum (coarse grid: hundreds of exact ties at the top and at fixed ratios below it) and continuous data,
    dense and with index lists, forward and backward against the double-precision oracle.  The values keep
    rel 1e-5.  The gradients are (d / y)^(p-1): the ratio is rounded to fp32 once before the power, so any fp32
    evaluation of all terms is off by about (p - 1) * 6e-8 relative (measured on these inputs: 2.8e-5 at p = 400,
    5e-4 at p = 1000, bit for bit the same as the kernels); their tolerance is max(1e-5, 1e-6 p)."""
    from sortnet_amd import ext
    dev = _dev()
    B, CI, CO = 70, 2048, 96
    x, w, gy = _gen((B, CI, 1), 71), _gen((CO, CI), 72, scale=0.3), _gen((B, CO, 1), 73)
    if kind == "grid":
        x, w = torch.round(x * 2) / 2, torch.round(w * 2) / 2
    ci, co = _index_lists(B, CI, CO, 1500, 70, 1, 74)
    for lists in (False, True):
        a, b = (ci, co) if lists else (None, None)
        xs = x[:, :1500].contiguous() if lists else x
        gs = gy[:, :70].contiguous() if lists else gy
        ry = oracle.norm_dist_forward(xs.numpy(), w.numpy(), p, 1, a, b)
        xd, wd, gd = xs.to(dev), w.to(dev), gs.to(dev)
        ad = None if a is None else torch.from_numpy(a).to(dev)
        bd = None if b is None else torch.from_numpy(b).to(dev)
        y = torch.empty(B, ry.shape[1], 1, device=dev)
        ext.norm_dist_forward(xd, wd, y, 1, p, ad, bd)
        np.testing.assert_allclose(y.cpu().numpy(), ry, rtol=RTOL)
        rgx, rgw = oracle.norm_dist_backward(gs.numpy(), xs.numpy(), w.numpy(), ry, p, 1, True, a, b)
        gx, gw = torch.empty_like(xd), torch.empty_like(wd)
        ext.norm_dist_backward_input_weight(gd, xd, wd, torch.from_numpy(ry).to(dev), gx, gw, 1, p, ad, bd)
        _close(gx, rgx, rtol=max(RTOL, 1e-6 * p))
        _close(gw, rgw, rtol=max(RTOL, 1e-6 * p))
        gx.fill_(float("nan"))
        ext.norm_dist_backward_input(gd, xd, wd, torch.from_numpy(ry).to(dev), gx, 1, p, ad, bd)
        _close(gx, rgx, rtol=max(RTOL, 1e-6 * p))


@pytest.mark.parametrize("p", [128.0, 400.0])
def test_norm_dist_large_p_adam_update(oracle, p):
    """The reference trains with AdamW at eps = 1e-10 (main.py:38,432): a gradient entry of 1e-9 still produces a
    full-size update.  The backward kernels leave out terms with (|d| / y)^(p-1) < 1e-16; the first Adam update
    g / (|g| + eps) from their gradients must agree with the one from the oracle's gradients (which sum every
    term in double precision), also where whole gradient entries consist of tiny terms only."""
    from sortnet_amd import ext
    dev = _dev()
    B, CI, CO = 64, 1024, 96
    x, w, gy = _gen((B, CI, 1), 81), _gen((CO, CI), 82, scale=0.3), _gen((B, CO, 1), 83)
    ry = oracle.norm_dist_forward(x.numpy(), w.numpy(), p)
    rgx, rgw = oracle.norm_dist_backward(gy.numpy(), x.numpy(), w.numpy(), ry, p)
    xd, wd, gd, yd = x.to(dev), w.to(dev), gy.to(dev), torch.from_numpy(ry).to(dev)
    gx, gw = torch.empty_like(xd), torch.empty_like(wd)
    ext.norm_dist_backward_input_weight(gd, xd, wd, yd, gx, gw, 1, p)
    gx2 = torch.empty_like(xd)
    ext.norm_dist_backward_input(gd, xd, wd, yd, gx2, 1, p)
    eps = 1e-10
    for got, ref in ((gw, rgw), (gx, rgx), (gx2, rgx)):
        got = got.cpu().numpy().astype(np.float64)
        ref = ref.astype(np.float64)
        upd_got, upd_ref = got / (np.abs(got) + eps), ref / (np.abs(ref) + eps)
        assert np.abs(ref).min() < 1e-8 < np.abs(ref).max()       # the data does hold entries in Adam's eps range
        assert np.abs(upd_got - upd_ref).max() < 2e-3, p


def test_config1_full_size(oracle):
    """Single l-inf layer at B=128, N=3072, M=1024: x ~ U[0,1], w ~ N(0, 1/N), grad ~ N(0,1), seed 0."""
    from sortnet_amd import ext
    dev = _dev()
    g = torch.Generator().manual_seed(0)
    x = torch.rand(128, 3072, generator=g).unsqueeze(-1).contiguous()
    w = (torch.randn(1024, 3072, generator=g) * 3072 ** -0.5).contiguous()
    gy = torch.randn(128, 1024, generator=g).unsqueeze(-1).contiguous()
    ry, rpos = oracle.inf_dist_forward(x.numpy(), w.numpy())
    xd, wd = x.to(dev), w.to(dev)
    y = torch.empty(128, 1024, 1, device=dev)
    pos = torch.empty(128, 1024, 1, device=dev, dtype=torch.int32)
    ext.inf_dist_forward(xd, wd, y, pos, 1)
    assert np.array_equal(y.cpu().numpy(), ry) and np.array_equal(pos.cpu().numpy(), rpos)
    y2 = torch.empty_like(y)
    ext.inf_dist_forward_nograd(xd, wd, y2, 1)
    assert np.array_equal(y2.cpu().numpy(), ry)
    rgx, rgw = oracle.inf_dist_backward(gy.numpy(), rpos, x.shape, w.shape)
    gx, gw = torch.empty_like(xd), torch.empty_like(wd)
    ext.inf_dist_backward_input_weight(gy.to(dev), pos, gx, gw, 1)
    _close(gx, rgx)
    _close(gw, rgw)


def test_full_size_properties():
    """B=512, N=M=5120 (too large for the scalar oracle in a test): properties that do not depend
    on size.  Every path must agree on the l-inf value; bounds bracket the point value and a
    degenerate box reproduces it bit for bit; arg-max positions reproduce the value when gathered."""
    from sortnet_amd import ext
    dev = _dev()
    B, N, M = 512, 5120, 5120
    g = torch.Generator().manual_seed(0)
    x = torch.rand(B, N, generator=g).unsqueeze(-1).contiguous().to(dev)
    w = (torch.randn(M, N, generator=g) * N ** -0.5).contiguous().to(dev)
    y = torch.empty(B, M, 1, device=dev)
    y2 = torch.empty_like(y)
    pos = torch.empty(B, M, 1, device=dev, dtype=torch.int32)
    ext.inf_dist_forward_nograd(x, w, y, 1)
    ext.inf_dist_forward(x, w, y2, pos, 1)
    assert torch.equal(y, y2)
    idx = (pos & 0x7FFFFFFF).long().squeeze(-1)
    xv = torch.gather(x.squeeze(-1), 1, idx)
    wv = w[torch.arange(M, device=dev)[None, :], idx]
    d = xv - wv
    assert torch.equal(d.abs(), y.squeeze(-1))
    assert torch.equal(d < 0, (pos.squeeze(-1) < 0))
    eps = 2.0 / 255
    xl, xu = (x - eps).contiguous(), (x + eps).contiguous()
    yl, yu = torch.empty_like(y), torch.empty_like(y)
    ext.bound_inf_dist_forward_nograd(xl, xu, w, yl, yu, 1)
    assert bool((yl <= y).all()) and bool((y <= yu).all()) and bool((yu - yl <= 2 * eps + 1e-6).all())
    dl, du = torch.empty_like(y), torch.empty_like(y)
    ext.bound_inf_dist_forward_nograd(x, x, w, dl, du, 1)
    assert torch.equal(du, y)
    # the masked neuron never exceeds the dense one, and equals it when everything is kept
    ym = torch.empty_like(y)
    ext.masked_inf_dist_forward(x, w, ym, None, 1, 0.3, 1, 0)
    assert bool((ym <= y).all())
    ext.masked_inf_dist_forward(x, w, ym, None, 1, 1.0, 1, 0)
    assert torch.equal(ym, y)


@pytest.mark.parametrize("B,C,HW", [(70, 200, 1), (33, 37, 1), (6, 24, 3), (512, 5120, 1)])
def test_mean_shift(oracle, B, C, HW):
    from sortnet_amd import ext
    import sortnet_amd.functional as F
    dev = _dev()
    x = _gen((B, C, HW), 71)
    rout, rmean = oracle.mean_shift(x.numpy())
    xd = x.to(dev)
    y, mean = torch.empty_like(xd), torch.empty(C, device=dev)
    running = torch.full((C,), 0.5, device=dev)
    ext.mean_shift_forward(xd, mean, running, 0.1, y)
    np.testing.assert_allclose(mean.cpu().numpy(), rmean, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(y.cpu().numpy(), rout, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(running.cpu().numpy(), 0.45 + 0.1 * rmean, rtol=1e-5, atol=1e-6)
    z = torch.empty_like(xd)
    ext.channel_shift(xd, mean, -1.0, z)
    assert torch.equal(z, y)
    # autograd: the gradient of the centring is the centring of the gradient
    xg = xd.clone().requires_grad_()
    g = _gen((B, C, HW), 72).to(dev)
    out, _ = F.mean_shift(xg)
    out.backward(g)
    ref = g - g.mean(dim=(0, 2), keepdim=True)
    np.testing.assert_allclose(xg.grad.cpu().numpy(), ref.cpu().numpy(), rtol=1e-5, atol=1e-6)


def test_argument_errors():
    from sortnet_amd import ext
    dev = _dev()
    x = torch.rand(4, 8, 1, device=dev)
    w = torch.rand(6, 8, device=dev)
    y = torch.empty(4, 6, 1, device=dev)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        ext.inf_dist_forward_nograd(x.cpu(), w, y, 1)
    with pytest.raises(RuntimeError, match="contiguous"):
        ext.inf_dist_forward_nograd(torch.rand(8, 4, 1, device=dev).transpose(0, 1), w, y, 1)
    with pytest.raises(RuntimeError, match="K="):
        ext.sort_neuron_forward_nograd(x, w, y, 1, 0.5, 40)
    with pytest.raises(RuntimeError, match="multiples of G"):
        ext.inf_dist_forward_nograd(x, w, y, 3)


def test_autograd_api(oracle):
    """The functional API on top: shapes, dtypes, gradient routing."""
    import sortnet_amd.functional as sa
    dev = _dev()
    x = _gen((40, 48, 1), 51, "rand").to(dev).requires_grad_()
    w = _gen((24, 48), 52, scale=0.3).to(dev).requires_grad_()
    y = sa.norm_dist(x, w, float("inf"))
    y.sum().backward()
    ry, rpos = oracle.inf_dist_forward(x.detach().cpu().numpy(), w.detach().cpu().numpy())
    rgx, rgw = oracle.inf_dist_backward(np.ones_like(ry), rpos, tuple(x.shape), tuple(w.shape))
    assert np.array_equal(y.detach().cpu().numpy(), ry)
    _close(x.grad, rgx)
    _close(w.grad, rgw)
    with torch.no_grad():
        assert torch.equal(sa.norm_dist(x, w, float("inf")), y)
        yl, yu = sa.bound_inf_dist(x - 0.01, x + 0.01, w)
        sl, su = sa.bound_sort_neuron(x - 0.01, x + 0.01, w, q=0.3)
        s = sa.sort_neuron(x, w, q=0.3)
    assert bool((yl <= y).all()) and bool((y <= yu).all())
    assert bool((sl <= s * (1 + 1e-5)).all()) and bool((s <= su * (1 + 1e-5)).all())
    x.grad = None
    w.grad = None
    y8 = sa.norm_dist(x, w, 8.0)
    y8.sum().backward()
    r8 = oracle.norm_dist_forward(x.detach().cpu().numpy(), w.detach().cpu().numpy(), 8.0)
    np.testing.assert_allclose(y8.detach().cpu().numpy(), r8, rtol=RTOL)
    assert x.grad.shape == x.shape and w.grad.shape == w.shape
    ym = sa.masked_inf_dist(x, w, 0.3, seed=5)
    ym.sum().backward()
    rm, _ = oracle.masked_inf_dist_forward(x.detach().cpu().numpy(), w.detach().cpu().numpy(), 0.3, 5, 0)
    assert np.array_equal(ym.detach().cpu().numpy(), rm)
    # the torch-op formulation of the same functions (core/norm_dist.py:181-185) on the same device tensors
    np.testing.assert_allclose(sa.norm_dist(x, w, 8.0, use_custom_cuda_func=False).detach().cpu().numpy(), r8, rtol=RTOL)
