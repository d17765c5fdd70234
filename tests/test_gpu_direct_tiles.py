"""Shapes that tile exactly (rows a multiple of 64, channels of 128, inputs of 32) and are large enough for 64-row
tiles take the LDS-direct forward kernels; the seeded random shapes of the other GPU tests never do.  Every op that has
such a path is compared with the oracle here: l-inf values and positions (ties, NaN inputs, the 1e-10 floor), the
factored-mask neuron, interval bounds with inverted intervals, l-p values -- dense, with groups, always with a split
reduction range.  sd_last_forward_kernel() confirms which kernel served the call; the small exact shapes check the
register-staged kernels on the same cases."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

# B, CI, CO, G
EXACT = [(256, 2048, 2048, 1), (256, 2048, 4096, 2), (128, 256, 256, 1), (64, 2048, 128, 1)]
DIRECT = {EXACT[0], EXACT[1]}       # large enough for 64-row tiles


def _served_by(shape, kind="fwd_kernel_direct<4,8>"):
    from sortnet_amd import _lib
    name = _lib.last_forward_kernel()
    if shape in DIRECT:
        assert name == kind, name
    else:
        assert "direct" not in name, name


def _dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def _data(B, CI, CO, G, seed, grid=None):
    g = torch.Generator().manual_seed(seed)
    x = torch.rand(B, CI, 1, generator=g)
    w = torch.randn(CO, CI // G, generator=g) * 0.3
    if grid:
        x, w = (x * grid).round() / grid, (w * grid).round() / grid
    return x.contiguous(), w.contiguous()


@pytest.mark.parametrize("B,CI,CO,G", EXACT)
@pytest.mark.parametrize("grid", [None, 4])
def test_linf_values_and_positions(oracle, B, CI, CO, G, grid):
    from sortnet_amd import ext
    dev = _dev()
    x, w = _data(B, CI, CO, G, 3, grid)
    if grid is None:
        x[1, 5, 0] = float("nan")          # NaN terms never win
        w[7, 9] = float("nan")
        x[2] = 0.25                         # a row whose distance to an equal weight row is below the 1e-10 floor
        w[3] = 0.25
    ry, rpos = oracle.inf_dist_forward(x.numpy(), w.numpy(), G)
    xd, wd = x.to(dev), w.to(dev)
    y = torch.empty(B, CO, 1, device=dev)
    pos = torch.empty(B, CO, 1, device=dev, dtype=torch.int32)
    ext.inf_dist_forward(xd, wd, y, pos, G)
    _served_by((B, CI, CO, G))
    assert np.array_equal(y.cpu().numpy(), ry)
    assert np.array_equal(pos.cpu().numpy(), rpos)
    y2 = torch.empty_like(y)
    ext.inf_dist_forward_nograd(xd, wd, y2, G)
    _served_by((B, CI, CO, G))
    assert np.array_equal(y2.cpu().numpy(), ry)
    if grid is None:
        assert ry[2, 3, 0] == np.float32(1e-10) and rpos[2, 3, 0] == 0


@pytest.mark.parametrize("B,CI,CO,G", EXACT[:3])
@pytest.mark.parametrize("q", [0.3, 0.9])
def test_factored_mask_neuron(oracle, B, CI, CO, G, q):
    from sortnet_amd import ext
    dev = _dev()
    x, w = _data(B, CI, CO, G, 5)
    ry, rpos = oracle.masked_inf_dist_forward(x.numpy(), w.numpy(), q, 11, oracle.MASK_FACTORED, G)
    xd, wd = x.to(dev), w.to(dev)
    y = torch.empty(B, CO, 1, device=dev)
    pos = torch.empty(B, CO, 1, device=dev, dtype=torch.int32)
    ext.masked_inf_dist_forward(xd, wd, y, pos, G, q, 11, ext.MASK_FACTORED)
    _served_by((B, CI, CO, G))
    assert np.array_equal(y.cpu().numpy(), ry)
    assert np.array_equal(pos.cpu().numpy(), rpos)
    y2 = torch.empty_like(y)
    ext.masked_inf_dist_forward(xd, wd, y2, None, G, q, 11, ext.MASK_FACTORED)
    _served_by((B, CI, CO, G))
    assert np.array_equal(y2.cpu().numpy(), ry)


@pytest.mark.parametrize("B,CI,CO,G", EXACT)
def test_interval_bounds_with_inverted_intervals(oracle, B, CI, CO, G):
    from sortnet_amd import ext
    dev = _dev()
    x, w = _data(B, CI, CO, G, 7)
    g = torch.Generator().manual_seed(8)
    r = torch.rand(B, CI, 1, generator=g) * 0.1
    xl, xu = x - r, x + r
    flip = torch.rand(B, CI, 1, generator=g) < 0.05      # inverted intervals are replaced by their midpoint
    xl, xu = torch.where(flip, xu, xl).contiguous(), torch.where(flip, xl, xu).contiguous()
    rl, ru = oracle.bound_inf_dist_forward(xl.numpy(), xu.numpy(), w.numpy(), G, need_pos=False)
    yl = torch.empty(B, CO, 1, device=dev)
    yu = torch.empty_like(yl)
    ext.bound_inf_dist_forward_nograd(xl.to(dev), xu.to(dev), w.to(dev), yl, yu, G)
    _served_by((B, CI, CO, G))
    assert np.array_equal(yl.cpu().numpy(), rl)
    assert np.array_equal(yu.cpu().numpy(), ru)
    # with positions: the chunk-tracking form (4 x 4 outputs, chunk numbers packed two outputs to a register), also on
    # coarse-grid data where many terms tie for a bound inside a chunk and across chunks
    for grid in (None, 8):
        if grid:
            xl, xu, wq = (xl * grid).round() / grid, (xu * grid).round() / grid, (w * grid).round() / grid
        else:
            wq = w
        rl, ru, rpl, rpu = oracle.bound_inf_dist_forward(xl.numpy(), xu.numpy(), wq.numpy(), G)
        zl, zu = torch.empty(B, CO, 1, device=dev), torch.empty(B, CO, 1, device=dev)
        pl = torch.empty(B, CO, 1, device=dev, dtype=torch.int32)
        pu = torch.empty_like(pl)
        ext.bound_inf_dist_forward(xl.to(dev), xu.to(dev), wq.to(dev), zl, zu, pl, pu, G)
        _served_by((B, CI, CO, G), "fwd_kernel_direct<4,4>")
        assert np.array_equal(zl.cpu().numpy(), rl) and np.array_equal(zu.cpu().numpy(), ru), grid
        assert np.array_equal(pl.cpu().numpy(), rpl) and np.array_equal(pu.cpu().numpy(), rpu), grid


@pytest.mark.parametrize("B,CI,CO,G", [EXACT[0], EXACT[2], EXACT[3]])
@pytest.mark.parametrize("p", [3.0, 8.0, 9.5, 24.0, 300.0])
def test_lp_values(oracle, B, CI, CO, G, p):
    from sortnet_amd import ext
    dev = _dev()
    g = torch.Generator().manual_seed(9)
    x = torch.randn(B, CI, 1, generator=g)
    w = torch.randn(CO, CI // G, generator=g) * 0.3
    ry = oracle.norm_dist_forward(x.numpy(), w.numpy(), p, G)
    xd, wd = x.to(dev), w.to(dev)
    y = torch.empty(B, CO, 1, device=dev)
    ext.norm_dist_forward(xd, wd, y, G, p)
    _served_by((B, CI, CO, G))
    np.testing.assert_allclose(y.cpu().numpy(), ry, rtol=1e-5)
    mx = torch.from_numpy(oracle.inf_dist_forward(x.numpy(), w.numpy(), G, need_pos=False)).to(dev)
    y2 = torch.empty_like(y)
    ext.norm_dist_forward_with_max(xd, wd, mx, y2, G, p)      # always the 32-row register-staged tile
    np.testing.assert_allclose(y2.cpu().numpy(), ry, rtol=1e-5)
