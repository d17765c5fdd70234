"""GPU parity of the interval-bound forward (values only) that works from candidate tables (dense single-group
layers, CI % 32 == 0).

`bound_inf_dist_forward_nograd` queues a kernel that evaluates only the inputs a table marks as able to hold a
maximum, and the kernel that evaluates every term; a count taken on the device picks one.  Both must give the
bits of the oracle (core/cuda/bound_inf_dist_cuda.cu:15-118 semantics, inverted intervals repaired to their
midpoint): the tests force either kernel (density 1 / 0) and the built-in limit, on batches whose rows are nearly
alike (the bounds of hidden layers: the table marks little), on unrelated rows (it marks nearly everything) and on
inverted intervals."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture
def density():
    from sortnet_amd import _lib

    def set_(d, form=0):
        _lib.set_bound_candidate_density(d)
        _lib.set_bound_candidate_form(form)
    yield set_
    _lib.set_bound_candidate_density(-1.0)
    _lib.set_bound_candidate_form(0)


def _intervals(B, CI, kind, seed):
    g = torch.Generator().manual_seed(seed)
    if kind == "rows_alike":
        x = torch.randn(1, CI, 1, generator=g) * 0.5 + torch.randn(B, CI, 1, generator=g) * 0.01
    elif kind == "images":
        x = torch.rand(B, CI, 1, generator=g)
    else:
        x = torch.randn(B, CI, 1, generator=g)
    r = torch.rand(B, CI, 1, generator=g) * 0.05
    xl, xu = (x - r).contiguous(), (x + r).contiguous()
    if kind == "inverted":
        m = torch.rand(B, CI, 1, generator=g) < 0.1
        xl, xu = torch.where(m, xu, xl).contiguous(), torch.where(m, xl, xu).contiguous()
    return xl, xu


@pytest.mark.parametrize("dens,form", [(1.0, 1), (1.0, 2), (0.0, 0), (-1.0, 0), (-1.0, 2)])
@pytest.mark.parametrize("B,CI,CO", [(70, 96, 64), (33, 2048, 300), (130, 1024, 513), (1, 32, 1), (257, 320, 129),
                                     (512, 512, 640), (700, 160, 72)])
def test_bound_candidate_kernel_matches_oracle(oracle, density, dens, form, B, CI, CO):
    """Ragged batch tiles (B not a multiple of 128) and weight tiles (CO not a multiple of 128), one and several of
    each, input ranges cut in slices or not; both table kernels (staged tiles, walk over transposed inputs)."""
    from sortnet_amd import ext
    dev = _dev()
    density(dens, form)
    for kind in ("rows_alike", "random", "inverted", "images"):
        for wscale in (0.02, 1.0):
            xl, xu = _intervals(B, CI, kind, B + CI)
            g = torch.Generator().manual_seed(2)
            w = (torch.randn(CO, CI, generator=g) * wscale).contiguous()
            rl, ru = oracle.bound_inf_dist_forward(xl.numpy(), xu.numpy(), w.numpy(), 1, need_pos=False)
            yl = torch.full((B, CO, 1), float("nan"), device=dev)
            yu = torch.full((B, CO, 1), float("nan"), device=dev)
            ext.bound_inf_dist_forward_nograd(xl.to(dev), xu.to(dev), w.to(dev), yl, yu, 1)
            tag = "dens=%g form=%d %s wscale=%g" % (dens, form, kind, wscale)
            assert np.array_equal(yl.cpu().numpy(), rl), tag
            assert np.array_equal(yu.cpu().numpy(), ru), tag


@pytest.mark.parametrize("dens", [1.0, 0.0, -1.0])
@pytest.mark.parametrize("B,CI,CO", [(70, 96, 64), (33, 2048, 300), (130, 1024, 513), (1, 32, 1), (257, 320, 129),
                                     (512, 512, 640), (700, 160, 72)])
def test_bound_candidate_kernel_with_positions_matches_oracle(oracle, density, dens, B, CI, CO):
    """The forward that also returns positions: values, positions and the "no gradient" position of a lower bound that
    stayed at its floor are the oracle's bits whether the table kernel (with its chunk tracking) or the every-term
    kernel leaves the (value, chunk) pairs; ties between inputs included (columns duplicated)."""
    from sortnet_amd import ext
    dev = _dev()
    density(dens)
    for kind in ("rows_alike", "random", "inverted", "images"):
        for wscale in (0.02, 1.0):
            xl, xu = _intervals(B, CI, kind, B + CI + 1)
            g = torch.Generator().manual_seed(3)
            w = (torch.randn(CO, CI, generator=g) * wscale).contiguous()
            if CI >= 64:   # equal terms at different inputs, in one chunk and in different chunks: the lowest input wins
                for src, dst in ((3, 17), (5, CI - 2)):
                    xl[:, dst], xu[:, dst], w[:, dst] = xl[:, src], xu[:, src], w[:, src]
            rl, ru, rpl, rpu = oracle.bound_inf_dist_forward(xl.numpy(), xu.numpy(), w.numpy(), 1, need_pos=True)
            yl = torch.full((B, CO, 1), float("nan"), device=dev)
            yu = torch.full((B, CO, 1), float("nan"), device=dev)
            pl = torch.full((B, CO, 1), -7, device=dev, dtype=torch.int32)
            pu = torch.full((B, CO, 1), -7, device=dev, dtype=torch.int32)
            ext.bound_inf_dist_forward(xl.to(dev), xu.to(dev), w.to(dev), yl, yu, pl, pu, 1)
            tag = "dens=%g %s wscale=%g" % (dens, kind, wscale)
            assert np.array_equal(yl.cpu().numpy(), rl), tag
            assert np.array_equal(yu.cpu().numpy(), ru), tag
            assert np.array_equal(pl.cpu().numpy(), rpl), tag
            assert np.array_equal(pu.cpu().numpy(), rpu), tag


@pytest.mark.parametrize("kind", ["images", "rows_alike"])
def test_bound_candidate_kernels_with_rows_longer_than_the_mark_lists(oracle, density, kind):
    """The kernel of the tables per batch row lists marked inputs as 16-bit numbers: a layer with more than 65536 inputs
    per row, forced into the tables, still gives the oracle's values and positions (from the tables per weight row or
    from every term)."""
    from sortnet_amd import ext
    dev = _dev()
    B, CI, CO = 8, 65568, 32
    density(1.0)
    xl, xu = _intervals(B, CI, kind, 11)
    g = torch.Generator().manual_seed(12)
    w = (torch.randn(CO, CI, generator=g) * 0.02).contiguous()
    rl, ru, rpl, rpu = oracle.bound_inf_dist_forward(xl.numpy(), xu.numpy(), w.numpy(), 1, need_pos=True)
    yl, yu = (torch.full((B, CO, 1), float("nan"), device=dev) for _ in range(2))
    pl, pu = (torch.full((B, CO, 1), -7, device=dev, dtype=torch.int32) for _ in range(2))
    ext.bound_inf_dist_forward(xl.to(dev), xu.to(dev), w.to(dev), yl, yu, pl, pu, 1)
    assert np.array_equal(yl.cpu().numpy(), rl) and np.array_equal(yu.cpu().numpy(), ru)
    assert np.array_equal(pl.cpu().numpy(), rpl) and np.array_equal(pu.cpu().numpy(), rpu)
    yl2, yu2 = (torch.full((B, CO, 1), float("nan"), device=dev) for _ in range(2))
    ext.bound_inf_dist_forward_nograd(xl.to(dev), xu.to(dev), w.to(dev), yl2, yu2, 1)
    assert np.array_equal(yl2.cpu().numpy(), rl) and np.array_equal(yu2.cpu().numpy(), ru)


def test_bound_candidate_kernel_with_positions_at_layer_size(density):
    """B = 512, N = M = 5120 with rows that are nearly alike: table kernel, every-term kernel and the built-in choice
    give the same values and positions."""
    from sortnet_amd import ext
    dev = _dev()
    B, N, M = 512, 5120, 5120
    g = torch.Generator().manual_seed(4)
    x = torch.randn(1, N, 1, generator=g) * 0.02 + torch.randn(B, N, 1, generator=g) * 0.004
    r = 0.02 + torch.rand(B, N, 1, generator=g) * 0.002
    xl, xu = (x - r).contiguous().to(dev), (x + r).contiguous().to(dev)
    w = (torch.randn(M, N, generator=g) * N ** -0.5).contiguous().to(dev)
    out = {}
    for dens in (0.0, 1.0, -1.0):
        density(dens)
        yl, yu = torch.empty(B, M, 1, device=dev), torch.empty(B, M, 1, device=dev)
        pl = torch.empty(B, M, 1, device=dev, dtype=torch.int32)
        pu = torch.empty(B, M, 1, device=dev, dtype=torch.int32)
        ext.bound_inf_dist_forward(xl, xu, w, yl, yu, pl, pu, 1)
        out[dens] = (yl, yu, pl, pu)
    for dens in (1.0, -1.0):
        for a, b in zip(out[dens], out[0.0]):
            assert torch.equal(a, b), dens


@pytest.mark.parametrize("dens,form", [(1.0, 1), (1.0, 2), (0.0, 0)])
@pytest.mark.parametrize("kind", ["rows_alike", "images"])
def test_bound_candidate_kernel_undefined_and_infinite_entries(oracle, density, dens, form, kind):
    """A term with an undefined operand is dropped by the reference's strict compares (an interval with one
    undefined end keeps the other end's term), so a row that holds NaN where its neighbours hold their maximum has
    a smaller result than they do: the tables must not conclude anything from such a column.  Infinite ends and
    weights likewise.  Both orientations of the table (rows alike / images) and the every-term kernel."""
    from sortnet_amd import ext
    dev = _dev()
    density(dens, form)
    B, CI, CO = 200, 256, 150
    xl, xu = _intervals(B, CI, kind, 5)
    g = torch.Generator().manual_seed(6)
    w = (torch.randn(CO, CI, generator=g) * (0.02 if kind == "images" else 0.5)).contiguous()
    # the column where most outputs have their maximum gets an undefined entry in a few rows
    rl, ru = oracle.bound_inf_dist_forward(xl.numpy(), xu.numpy(), w.numpy(), 1, need_pos=False)
    t = np.maximum(w.numpy()[None] - xl.numpy()[:, :, 0][:, None], xu.numpy()[:, :, 0][:, None] - w.numpy()[None])
    hot = np.bincount(t.argmax(2).ravel(), minlength=CI).argsort()[::-1][:6]
    nan, inf = float("nan"), float("inf")
    xl[3, hot[0], 0] = nan; xu[3, hot[0], 0] = nan
    xl[150, hot[1], 0] = nan
    xu[77, hot[2], 0] = nan
    xl[10, hot[3], 0] = -inf
    xu[11, hot[4], 0] = inf
    xl[12, hot[5], 0] = inf; xu[12, hot[5], 0] = inf
    w[5, hot[0]] = nan
    w[6, hot[1]] = inf
    w[7, hot[5]] = inf
    w[8, 17] = -inf
    with np.errstate(invalid="ignore"):
        rl, ru = oracle.bound_inf_dist_forward(xl.numpy(), xu.numpy(), w.numpy(), 1, need_pos=False)
    yl = torch.full((B, CO, 1), float("nan"), device=dev)
    yu = torch.full((B, CO, 1), float("nan"), device=dev)
    ext.bound_inf_dist_forward_nograd(xl.to(dev), xu.to(dev), w.to(dev), yl, yu, 1)
    assert np.array_equal(yl.cpu().numpy(), rl, equal_nan=True)
    assert np.array_equal(yu.cpu().numpy(), ru, equal_nan=True)


def test_bound_candidate_kernel_at_layer_size(density):
    """B = 512, N = M = 5120 with rows that are nearly alike (as the bounds of a hidden layer are): the table kernel
    and the every-term kernel give the same bits, and the built-in limit does too."""
    from sortnet_amd import ext
    dev = _dev()
    B, N, M = 512, 5120, 5120
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, N, 1, generator=g) * 0.02 + torch.randn(B, N, 1, generator=g) * 0.004
    r = 0.02 + torch.rand(B, N, 1, generator=g) * 0.002
    xl, xu = (x - r).contiguous().to(dev), (x + r).contiguous().to(dev)
    w = (torch.randn(M, N, generator=g) * N ** -0.5).contiguous().to(dev)
    out = {}
    for dens, form in ((0.0, 0), (1.0, 1), (-1.0, 0), (1.0, 2)):
        density(dens, form)
        yl, yu = torch.empty(B, M, 1, device=dev), torch.empty(B, M, 1, device=dev)
        ext.bound_inf_dist_forward_nograd(xl, xu, w, yl, yu, 1)
        out[(dens, form)] = (yl, yu)
    for key in ((1.0, 1), (-1.0, 0), (1.0, 2)):
        assert torch.equal(out[key][0], out[(0.0, 0)][0]) and torch.equal(out[key][1], out[(0.0, 0)][1]), key


def test_bound_results_do_not_depend_on_the_table_hint(oracle, density):
    """With the built-in limits (layers of at least 2^31 terms) a layer (same weights, same shape) whose tables did not
    pay a few times in a row is given none for a while: calls before, during and after that stretch give the bits of
    the every-term kernel on all rows and of the oracle on the first rows, on data of either kind."""
    from sortnet_amd import ext
    dev = _dev()
    B, CI, CO = 512, 2048, 2048
    g = torch.Generator().manual_seed(11)
    w = (torch.randn(CO, CI, generator=g) * 0.3).contiguous().to(dev)
    calls = []
    density(-1.0)
    for call in range(12):
        kind = "random" if call < 8 else "rows_alike"     # unrelated rows: every term; rows alike: the table
        xl, xu = _intervals(B, CI, kind, 100 + call)
        xl, xu = xl.to(dev), xu.to(dev)
        yl = torch.full((B, CO, 1), float("nan"), device=dev)
        yu = torch.full((B, CO, 1), float("nan"), device=dev)
        ext.bound_inf_dist_forward_nograd(xl, xu, w, yl, yu, 1)
        torch.cuda.synchronize()   # lets the next call see which kernel ran
        calls.append((xl, xu, yl, yu))
    density(0.0)
    for call, (xl, xu, yl, yu) in enumerate(calls):
        el, eu = torch.empty_like(yl), torch.empty_like(yu)
        ext.bound_inf_dist_forward_nograd(xl, xu, w, el, eu, 1)
        assert torch.equal(yl, el) and torch.equal(yu, eu), call
        rl, ru = oracle.bound_inf_dist_forward(xl[:8].cpu().numpy(), xu[:8].cpu().numpy(), w.cpu().numpy(), 1,
                                               need_pos=False)
        assert np.array_equal(yl[:8].cpu().numpy(), rl) and np.array_equal(yu[:8].cpu().numpy(), ru), call


def test_bound_candidate_density_argument(density):
    from sortnet_amd import _lib
    with pytest.raises(RuntimeError):
        _lib.set_bound_candidate_density(1.5)
    density(0.3)


def test_bound_candidate_kernel_long_slices(density):
    """Enough output tiles that the input range is not cut (B = 2048, CO = 4096) and more than 64 chunks of inputs
    (CI = 2112: 33 stages of 64 inputs in one slice).  Same bits as the every-term kernel."""
    from sortnet_amd import ext
    dev = _dev()
    B, CI, CO = 2048, 2112, 4096
    g = torch.Generator().manual_seed(7)
    x = torch.randn(1, CI, 1, generator=g) * 0.5 + torch.randn(B, CI, 1, generator=g) * 0.01
    r = torch.rand(B, CI, 1, generator=g) * 0.02
    xl, xu = (x - r).contiguous().to(dev), (x + r).contiguous().to(dev)
    w = (torch.randn(CO, CI, generator=g) * 0.3).to(dev)
    out = {}
    for dens in (0.0, 1.0):
        density(dens)
        yl, yu = torch.empty(B, CO, 1, device=dev), torch.empty(B, CO, 1, device=dev)
        ext.bound_inf_dist_forward_nograd(xl, xu, w, yl, yu, 1)
        out[dens] = (yl, yu)
    assert torch.equal(out[0.0][0], out[1.0][0]) and torch.equal(out[0.0][1], out[1.0][1])
