"""GPU parity of the l-inf forward (plain and under the factored mask) when it works from candidate tables (dense
single-group layers, CI % 32 == 0).

The entry points queue a kernel that evaluates only the inputs a table marks as able to hold the maximum of a weight
row, and the kernels that evaluate every term; a count taken on the device picks one.  Values AND positions must be
the oracle's bits either way (core/cuda/inf_dist_cuda.cu:110-212 semantics: the first of equal terms wins, the 1e-10
floor with position 0 when nothing exceeds it): the tests force either side (density 1 / 0) and the built-in limit,
on batches whose rows are alike against weights of unit scale (the table marks little), on unrelated rows, on grid
data with many exact ties, and under the mask with a shallow bound so that some outputs are recomputed from every
input.  Inputs in [0, 1] against small weights ("images", "image_ties") are the case of the other table orientation:
per batch row and tile of 128 weight rows, where the batch row decides which inputs can hold a maximum."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture
def knobs():
    from sortnet_amd import _lib

    def set_(density, depth=0):
        _lib.set_linf_candidate_density(density)
        _lib.set_linf_candidate_depth(depth)
    yield set_
    _lib.set_linf_candidate_density(-1.0)
    _lib.set_linf_candidate_depth(0)


def _data(B, CI, CO, kind, seed):
    g = torch.Generator().manual_seed(seed)
    if kind == "rows_alike":
        x = torch.randn(1, CI, 1, generator=g) * 0.3 + torch.randn(B, CI, 1, generator=g) * 0.05
        w = torch.randn(CO, CI, generator=g)
    elif kind == "images":
        x = torch.rand(B, CI, 1, generator=g)
        w = torch.randn(CO, CI, generator=g) * CI ** -0.5
    elif kind == "image_ties":      # the batch decides, and many terms are equal: 17 input levels, 9 weight levels
        x = torch.round(torch.rand(B, CI, 1, generator=g) * 16) / 16
        w = torch.round(torch.randn(CO, CI, generator=g) * 0.03 * 64) / 64
    elif kind == "ties":
        x = torch.round(torch.randn(B, CI, 1, generator=g) * 0.2 * 4) / 4
        w = torch.round(torch.randn(CO, CI, generator=g) * 4) / 4
    else:
        x = torch.randn(B, CI, 1, generator=g)
        w = torch.randn(CO, CI, generator=g)
    return x.contiguous(), w.contiguous()


def _served_from_tables(expect, tag):
    """With the limit forced to 1 on data where the batch decides, a table kernel must have served the call."""
    from sortnet_amd import _lib
    if expect:
        assert _lib.last_forward_term_share() < 1.0, tag


def _check_plain(oracle, x, w, tag, expect_tables=False):
    from sortnet_amd import ext
    dev = _dev()
    B, CO = x.shape[0], w.shape[0]
    ry, rpos = oracle.inf_dist_forward(x.numpy(), w.numpy(), 1)
    y = torch.full((B, CO, 1), float("nan"), device=dev)
    pos = torch.full((B, CO, 1), -7, device=dev, dtype=torch.int32)
    ext.inf_dist_forward(x.to(dev), w.to(dev), y, pos, 1)
    _served_from_tables(expect_tables, tag)
    assert np.array_equal(y.cpu().numpy(), ry), tag
    assert np.array_equal(pos.cpu().numpy(), rpos), tag
    y2 = torch.full((B, CO, 1), float("nan"), device=dev)
    ext.inf_dist_forward_nograd(x.to(dev), w.to(dev), y2, 1)
    _served_from_tables(expect_tables, tag)
    assert np.array_equal(y2.cpu().numpy(), ry), tag


def _check_masked(oracle, x, w, q, seed, tag, expect_tables=False):
    from sortnet_amd import ext
    dev = _dev()
    B, CO = x.shape[0], w.shape[0]
    ry, rpos = oracle.masked_inf_dist_forward(x.numpy(), w.numpy(), q, seed, ext.MASK_FACTORED, 1)
    y = torch.full((B, CO, 1), float("nan"), device=dev)
    pos = torch.full((B, CO, 1), -7, device=dev, dtype=torch.int32)
    ext.masked_inf_dist_forward(x.to(dev), w.to(dev), y, pos, 1, q, seed, ext.MASK_FACTORED)
    _served_from_tables(expect_tables, tag)
    assert np.array_equal(y.cpu().numpy(), ry), tag
    assert np.array_equal(pos.cpu().numpy(), rpos), tag
    y2 = torch.full((B, CO, 1), float("nan"), device=dev)
    ext.masked_inf_dist_forward(x.to(dev), w.to(dev), y2, None, 1, q, seed, ext.MASK_FACTORED)
    assert np.array_equal(y2.cpu().numpy(), ry), tag


SHAPES = [(70, 96, 64), (33, 2048, 300), (130, 1024, 513), (1, 32, 1), (257, 320, 129), (700, 160, 72), (512, 2112, 96)]


@pytest.mark.parametrize("dens", [1.0, 0.0, -1.0])
@pytest.mark.parametrize("B,CI,CO", SHAPES)
def test_linf_candidate_kernels_match_oracle(oracle, knobs, dens, B, CI, CO):
    """Ragged batch tiles and weight rows, rows of more than 64 chunks (several loads of table words per row)."""
    knobs(dens)
    for kind in ("rows_alike", "random", "images", "ties", "image_ties"):
        x, w = _data(B, CI, CO, kind, B + CI)
        # inputs in [0, 1] against small weights: the tables per batch row serve (rows of at least a few chunks)
        expect = dens == 1.0 and kind in ("images", "image_ties") and CI >= 160 and B > 1
        _check_plain(oracle, x, w, "dens=%g %s" % (dens, kind), expect)


@pytest.mark.parametrize("dens,depth", [(1.0, 0), (1.0, 8), (0.0, 0), (-1.0, 0)])
@pytest.mark.parametrize("B,CI,CO", SHAPES)
def test_masked_candidate_kernels_match_oracle(oracle, knobs, dens, depth, B, CI, CO):
    """Factored mask at q = 0.3, 0.75 and 1.  Depth 8 at q = 0.3: a row keeps none of the eight inputs the bound
    rests on about once in 600 outputs, so many wavefronts walk their weight row a second time over every input."""
    knobs(dens, depth)
    for kind in ("rows_alike", "random", "ties", "images", "image_ties"):
        for q, seed in ((0.3, 5), (0.75, 77), (1.0, 3)):
            x, w = _data(B, CI, CO, kind, B + CI + 1)
            expect = dens == 1.0 and kind in ("images", "image_ties") and CI >= 160 and B > 1
            _check_masked(oracle, x, w, q, seed, "dens=%g depth=%d %s q=%g" % (dens, depth, kind, q), expect)


@pytest.mark.parametrize("dens", [1.0, 0.0])
@pytest.mark.parametrize("kind", ["rows_alike", "images", "ties"])
def test_linf_candidate_kernels_with_undefined_and_infinite_operands(oracle, knobs, dens, kind):
    """NaN and +-inf sprinkled into inputs and weights: an undefined difference never becomes the maximum (strict
    comparisons, core/cuda/inf_dist_cuda.cu:176-190), an infinite one does, lowest input first.  Both table
    orientations (rows alike / images) and the every-term kernels against the oracle, plain and under the mask."""
    knobs(dens)
    B, CI, CO = 150, 1024, 200
    x, w = _data(B, CI, CO, kind, 41)
    g = torch.Generator().manual_seed(42)
    for t, frac in ((x, 0.002), (w, 0.0005)):
        m = torch.rand(t.shape, generator=g)
        t[m < frac] = float("nan")
        t[(m >= frac) & (m < 2 * frac)] = float("inf")
        t[(m >= 2 * frac) & (m < 3 * frac)] = float("-inf")
    _check_plain(oracle, x, w, "dens=%g %s" % (dens, kind))
    for q, seed in ((0.3, 5), (1.0, 3)):
        _check_masked(oracle, x, w, q, seed, "dens=%g %s q=%g" % (dens, kind, q))


def test_linf_candidate_kernels_at_layer_size(knobs):
    """B = 512, N = M = 5120, unit-scale weights against rows that are nearly alike: table kernels and every-term
    kernels give the same values and positions, plain and masked, and the built-in limit picks the table."""
    from sortnet_amd import ext
    dev = _dev()
    B, N, M = 512, 5120, 5120
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(1, N, 1, generator=g) * 0.3 + torch.randn(B, N, 1, generator=g) * 0.1).contiguous().to(dev)
    w = torch.randn(M, N, generator=g).contiguous().to(dev)
    out = {}
    for dens in (0.0, 1.0, -1.0):
        knobs(dens)
        y, ym = torch.empty(B, M, 1, device=dev), torch.empty(B, M, 1, device=dev)
        p = torch.empty(B, M, 1, device=dev, dtype=torch.int32)
        pm = torch.empty_like(p)
        ext.inf_dist_forward(x, w, y, p, 1)
        ext.masked_inf_dist_forward(x, w, ym, pm, 1, 0.3, 9, ext.MASK_FACTORED)
        out[dens] = (y, p, ym, pm)
    for dens in (1.0, -1.0):
        for a, b in zip(out[dens], out[0.0]):
            assert torch.equal(a, b), dens


def test_linf_row_tables_at_layer_size_with_built_in_limits(knobs):
    """B = 512, N = M = 5120: images against small weights.  With the built-in limits the tables per batch row serve the
    plain and the masked forward, and values and positions are the every-term kernels' bits."""
    from sortnet_amd import ext, _lib
    dev = _dev()
    B, N, M = 512, 5120, 5120
    g = torch.Generator().manual_seed(5)
    x = torch.rand(B, N, 1, generator=g).contiguous().to(dev)
    w = (torch.randn(M, N, generator=g) * N ** -0.5).contiguous().to(dev)
    out = {}
    for dens in (0.0, -1.0):
        knobs(dens)
        y, yn, ym = (torch.empty(B, M, 1, device=dev) for _ in range(3))
        p = torch.empty(B, M, 1, device=dev, dtype=torch.int32)
        pm = torch.empty_like(p)
        ext.inf_dist_forward(x, w, y, p, 1)
        share = _lib.last_forward_term_share()
        ext.inf_dist_forward_nograd(x, w, yn, 1)
        ext.masked_inf_dist_forward(x, w, ym, pm, 1, 0.3, 9, ext.MASK_FACTORED)
        share_masked = _lib.last_forward_term_share()
        out[dens] = (y, p, yn, ym, pm)
        if dens < 0:
            assert share < 0.15 and share_masked < 0.15, (share, share_masked)
        else:
            assert share == 1.0 and share_masked == 1.0, (share, share_masked)
    for a, b in zip(out[-1.0], out[0.0]):
        assert torch.equal(a, b)


def test_linf_candidate_arguments(knobs):
    from sortnet_amd import _lib
    with pytest.raises(RuntimeError):
        _lib.set_linf_candidate_density(1.5)
    with pytest.raises(RuntimeError):
        _lib.set_linf_candidate_depth(5)
    knobs(0.3, 12)
