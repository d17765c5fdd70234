"""GPU parity of the dense l-p kernels that work from candidate tables (general p, single group, CI % 32 == 0).

A dense l-p call queues two kernels for the same result and a count taken on the device picks one; the tests
force either kernel (density 1 = always the table kernel, 0 = never) and the built-in limits, on data where the
table marks few inputs (small weights), where it marks most (weights as large as the inputs) and on ties, and
compare values (rel 1e-5) and gradients (rel max(1e-5, 1e-6 p) of the largest entry) with the double-precision
oracle (core/cuda/norm_dist_cuda.cu:36-160, 261-504 semantics)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL = 1e-5


def _dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def _gen(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).float().contiguous()


@pytest.fixture
def density():
    from sortnet_amd import _lib

    def set_(d):
        _lib.set_lp_candidate_density(d)
    yield set_
    _lib.set_lp_candidate_density(-1.0)


def _check(oracle, x, w, gy, p, tag):
    from sortnet_amd import ext
    dev = _dev()
    B, CO = x.shape[0], w.shape[0]
    ry = oracle.norm_dist_forward(x.numpy(), w.numpy(), p, 1)
    rgx, rgw = oracle.norm_dist_backward(gy.numpy(), x.numpy(), w.numpy(), ry, p, 1)
    xd, wd, gd, yd = x.to(dev), w.to(dev), gy.to(dev), torch.from_numpy(ry).to(dev)
    y = torch.full((B, CO, 1), float("nan"), device=dev)
    ext.norm_dist_forward(xd, wd, y, 1, p)
    np.testing.assert_allclose(y.cpu().numpy(), ry, rtol=RTOL, err_msg=tag)
    tol = max(RTOL, 1e-6 * p)
    gx, gw = torch.full_like(xd, float("nan")), torch.full_like(wd, float("nan"))
    ext.norm_dist_backward_input_weight(gd, xd, wd, yd, gx, gw, 1, p)
    for got, ref in ((gx, rgx), (gw, rgw)):
        np.testing.assert_allclose(got.cpu().numpy(), ref, rtol=tol, atol=tol * float(np.abs(ref).max()), err_msg=tag)
    gx2 = torch.full_like(xd, float("nan"))
    ext.norm_dist_backward_input(gd, xd, wd, yd, gx2, 1, p)
    np.testing.assert_allclose(gx2.cpu().numpy(), rgx, rtol=tol, atol=tol * float(np.abs(rgx).max()), err_msg=tag)


@pytest.mark.parametrize("dens", [1.0, 0.0, -1.0])
@pytest.mark.parametrize("B,CI,CO", [(70, 96, 64), (33, 2048, 300), (130, 1024, 513), (64, 160, 256), (1, 32, 1)])
def test_candidate_kernels_match_oracle(oracle, density, dens, B, CI, CO):
    """Ragged rows and channels (B not a multiple of 32 / 128, CO not a multiple of 256), one and several column
    tiles, both workgroup sizes of the forward (B <= 64 and above)."""
    density(dens)
    for wscale in (0.02, 1.5):
        for p in (24.0, 100.0, 400.0):
            x, w, gy = _gen((B, CI, 1), 1), _gen((CO, CI), 2, wscale), _gen((B, CO, 1), 3)
            _check(oracle, x, w, gy, p, "dens=%g wscale=%g p=%g" % (dens, wscale, p))


@pytest.mark.parametrize("dens", [1.0, -1.0])
def test_candidate_kernels_ties_and_zero_rows(oracle, density, dens):
    """Grid data (hundreds of exact ties at the maximum and at fixed ratios below it), a batch row that equals a
    weight row (distance at the 1e-10 floor, every ratio huge) and an all-zero input row."""
    density(dens)
    B, CI, CO = 40, 512, 70
    x, w, gy = _gen((B, CI, 1), 11), _gen((CO, CI), 12, 0.3), _gen((B, CO, 1), 13)
    x, w = torch.round(x * 2) / 2, torch.round(w * 2) / 2
    x[3, :, 0] = w[5]
    x[7] = 0.0
    for p in (50.0, 300.0):
        _check(oracle, x.contiguous(), w.contiguous(), gy, p, "dens=%g p=%g" % (dens, p))


@pytest.mark.parametrize("dens", [1.0, 0.0])
def test_candidate_kernels_undefined_entries_reach_their_outputs(oracle, density, dens):
    """An undefined input makes every output of its row undefined, an undefined weight every output of its channel
    (the reference sums all terms): the table must keep such entries as candidates whatever their size."""
    from sortnet_amd import ext
    dev = _dev()
    density(dens)
    B, CI, CO, p = 70, 256, 300, 64.0
    x, w = _gen((B, CI, 1), 21), _gen((CO, CI), 22, 0.05)
    x[5, 100, 0] = float("nan")
    w[17, 3] = float("nan")
    w[280, 200] = float("nan")
    with np.errstate(invalid="ignore"):
        ry = oracle.norm_dist_forward(x.numpy(), w.numpy(), p, 1)
    assert np.isnan(ry[5]).all() and np.isnan(ry[:, 17]).all() and np.isnan(ry).sum() == CO + 2 * B - 2
    y = torch.zeros(B, CO, 1, device=dev)
    ext.norm_dist_forward(x.to(dev), w.to(dev), y, 1, p)
    got = y.cpu().numpy()
    assert np.array_equal(np.isnan(got), np.isnan(ry))
    ok = ~np.isnan(ry)
    np.testing.assert_allclose(got[ok], ry[ok], rtol=RTOL)


@pytest.mark.parametrize("dens", [1.0, 0.0])
@pytest.mark.parametrize("p", [24.0, 256.0])
def test_candidate_kernels_infinite_entries_reach_their_outputs(oracle, density, dens, p):
    """An infinite input or weight makes the distance of every output it meets infinite and its scaled terms
    undefined in the reference (inf / inf); here such an output is never finite either (undefined, or infinite where
    the kernel skips the undefined term), and every other output is unchanged.  The scale of the affected rows is
    infinite, which must not unmark the row's inputs in the table."""
    from sortnet_amd import ext
    dev = _dev()
    density(dens)
    B, CI, CO = 70, 352, 300
    x, w = _gen((B, CI, 1), 31), _gen((CO, CI), 32, 0.3)
    x[5, 100, 0] = float("inf")
    x[40, 7, 0] = float("-inf")
    w[17, 3] = float("inf")
    w[280, 200] = float("-inf")
    w[281, 7] = float("nan")
    with np.errstate(invalid="ignore", over="ignore"):
        ry = oracle.norm_dist_forward(x.numpy(), w.numpy(), p, 1)
    bad = ~np.isfinite(ry)
    assert bad[5].all() and bad[40].all() and bad[:, 17].all() and bad[:, 280].all() and bad[:, 281].all()
    assert bad.sum() == 2 * CO + 3 * (B - 2)
    y = torch.zeros(B, CO, 1, device=dev)
    ext.norm_dist_forward(x.to(dev), w.to(dev), y, 1, p)
    got = y.cpu().numpy()
    assert np.array_equal(~np.isfinite(got), bad)
    np.testing.assert_allclose(got[~bad], ry[~bad], rtol=RTOL)


def test_candidate_density_argument(density):
    from sortnet_amd import _lib
    with pytest.raises(RuntimeError):
        _lib.set_lp_candidate_density(1.5)
    density(0.3)


def test_candidate_kernels_config3_size(oracle, density):
    """B = 512, N = M = 5120, x ~ N(0, 1), w ~ N(0, 1/N) at p = 64: the forced table kernels against the kernels
    that evaluate every term (the oracle takes minutes at this size; the latter are held to it at full size
    elsewhere), and the first rows against the oracle."""
    from sortnet_amd import ext
    dev = _dev()
    B, N, M, p = 512, 5120, 5120, 64.0
    g = torch.Generator().manual_seed(0)
    x = torch.randn(B, N, 1, generator=g)
    w = (torch.randn(M, N, generator=g) * N ** -0.5).contiguous()
    gy = torch.randn(B, M, 1, generator=g)
    xd, wd, gd = x.to(dev), w.to(dev), gy.to(dev)
    out = {}
    for dens in (0.0, 1.0):
        density(dens)
        y = torch.empty(B, M, 1, device=dev)
        ext.norm_dist_forward(xd, wd, y, 1, p)
        gx, gw = torch.empty_like(xd), torch.empty_like(wd)
        ext.norm_dist_backward_input_weight(gd, xd, wd, y, gx, gw, 1, p)
        out[dens] = (y.cpu().numpy(), gx.cpu().numpy(), gw.cpu().numpy())
    np.testing.assert_allclose(out[1.0][0], out[0.0][0], rtol=RTOL)
    for k in (1, 2):
        ref = out[0.0][k]
        np.testing.assert_allclose(out[1.0][k], ref, rtol=1e-4, atol=1e-4 * float(np.abs(ref).max()))
    rows = 4
    ry = oracle.norm_dist_forward(x[:rows].numpy(), w.numpy(), p, 1)
    np.testing.assert_allclose(out[1.0][0][:rows], ry, rtol=RTOL)
    rgx, _ = oracle.norm_dist_backward(gy[:rows].numpy(), x[:rows].numpy(), w.numpy(), ry, p, 1)
    # grad_input of a row depends on that row only
    yd = torch.from_numpy(ry).to(dev)
    gx4 = torch.empty(rows, N, 1, device=dev)
    density(1.0)
    ext.norm_dist_backward_input(gd[:rows].contiguous(), xd[:rows].contiguous(), wd, yd, gx4, 1, p)
    tol = 1e-6 * p
    np.testing.assert_allclose(gx4.cpu().numpy(), rgx, rtol=tol, atol=tol * float(np.abs(rgx).max()))


def test_candidate_kernels_long_slices(density):
    """Enough output tiles that the forward does not cut its input range (B = 2048, CO = 4096) and more than 64
    chunks of inputs (CI = 2112): the forward table kernel stages its mark words in two segments.  Against the
    every-term kernels (held to the oracle elsewhere)."""
    from sortnet_amd import ext
    dev = _dev()
    B, CI, CO, p = 2048, 2112, 4096, 64.0
    g = torch.Generator().manual_seed(7)
    x = torch.randn(B, CI, 1, generator=g).to(dev)
    w = (torch.randn(CO, CI, generator=g) * 0.02).to(dev)
    gy = torch.randn(B, CO, 1, generator=g).to(dev)
    y, grads = {}, {}
    for dens in (0.0, 1.0):
        density(dens)
        y[dens] = torch.empty(B, CO, 1, device=dev)
        ext.norm_dist_forward(x, w, y[dens], 1, p)
    np.testing.assert_allclose(y[1.0].cpu().numpy(), y[0.0].cpu().numpy(), rtol=RTOL)
    for dens in (0.0, 1.0):
        density(dens)
        gx, gw = torch.empty_like(x), torch.empty_like(w)
        ext.norm_dist_backward_input_weight(gy, x, w, y[0.0], gx, gw, 1, p)
        grads[dens] = (gx.cpu().numpy(), gw.cpu().numpy())
    for a, b in zip(grads[1.0], grads[0.0]):
        np.testing.assert_allclose(a, b, rtol=1e-4, atol=1e-4 * float(np.abs(b).max()))
