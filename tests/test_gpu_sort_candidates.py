"""GPU parity of the sort neuron (values, values with positions) and its interval bounds when they work from candidate tables (dense
single-group layers, CI % 32 == 0).

Both entry points queue a kernel that evaluates only the inputs a table marks as able to be among the K largest
terms of a weight row, and the kernels that evaluate every term; a count taken on the device picks one.  Both must
give the results of the oracle (core/cuda/sort_neuron.cu:16-109, 216-314 semantics; the geometric sum is taken in the
reference's order over the same K values, so the comparison is exact): the tests force either side (density 1 / 0)
and the built-in limit, on batches whose rows are alike against weights of unit scale (the table marks little), on
unrelated rows (it marks nearly everything), on inverted intervals and on ties."""
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

    def set_(d):
        _lib.set_sort_candidate_density(d)
    yield set_
    _lib.set_sort_candidate_density(-1.0)


def _data(B, CI, CO, kind, seed):
    g = torch.Generator().manual_seed(seed)
    if kind == "rows_alike":
        x = torch.randn(1, CI, 1, generator=g) * 0.3 + torch.randn(B, CI, 1, generator=g) * 0.05
    elif kind in ("images", "pixels", "pixel_ties"):
        x = torch.rand(B, CI, 1, generator=g)
    else:
        x = torch.randn(B, CI, 1, generator=g)
    r = torch.rand(B, CI, 1, generator=g) * (0.01 if kind.startswith("pixels") else 0.05)
    if kind == "pixel_ties":
        x = torch.round(x * 16) / 16
        r = torch.full_like(x, 1.0 / 64)
    xl, xu = (x - r).contiguous(), (x + r).contiguous()
    if kind == "inverted":
        m = torch.rand(B, CI, 1, generator=g) < 0.1
        xl, xu = torch.where(m, xu, xl).contiguous(), torch.where(m, xl, xu).contiguous()
    w = torch.randn(CO, CI, generator=g).contiguous()
    if kind == "pixels":            # inputs in [0, 1] against small weights: the batch row decides where the largest terms sit
        w = (w * CI ** -0.5).contiguous()
    if kind == "pixel_ties":        # the same with 17 input levels and a few weight levels: many equal terms
        w = (torch.round(w * 0.03 * 64) / 64).contiguous()
    if kind == "ties":
        x, w = torch.round(x * 4) / 4, torch.round(w * 4) / 4
        xl, xu = x - 0.25, x + 0.25
    return x.contiguous(), xl.contiguous(), xu.contiguous(), w.contiguous()


RTOL = 1e-5


def _run(x, xl, xu, w, q, K):
    from sortnet_amd import ext
    dev = _dev()
    B, CO = x.shape[0], w.shape[0]
    y, yl, yu = (torch.full((B, CO, 1), float("nan"), device=dev) for _ in range(3))
    ext.sort_neuron_forward_nograd(x.to(dev), w.to(dev), y, 1, q, K)
    ext.bound_sort_neuron_forward(xl.to(dev), xu.to(dev), w.to(dev), yl, yu, 1, q, K)
    yp = torch.full((B, CO, 1), float("nan"), device=dev)
    pos = torch.full((K, B, CO, 1), -7, device=dev, dtype=torch.int32)
    ext.sort_neuron_forward(x.to(dev), w.to(dev), yp, pos, 1, q, K)
    return y.cpu().numpy(), yl.cpu().numpy(), yu.cpu().numpy(), yp.cpu().numpy(), pos.cpu().numpy()


def _check(oracle, density, dens, x, xl, xu, w, q, K, tag, expect_tables=False):
    """Against the oracle at the sort neuron's bar (rel 1e-5), and bit for bit against the every-term kernels."""
    ry, rpos = oracle.sort_neuron_forward(x.numpy(), w.numpy(), q, K)
    rl, ru = oracle.bound_sort_neuron_forward(xl.numpy(), xu.numpy(), w.numpy(), q, K)
    density(dens)
    got = _run(x, xl, xu, w, q, K)
    if expect_tables:   # (the last call of _run: values with positions)
        from sortnet_amd import _lib
        assert _lib.last_forward_term_share() < 1.0, tag
    for g, r in zip(got[:4], (ry, rl, ru, ry)):
        np.testing.assert_allclose(g, r, rtol=RTOL, err_msg=tag)
    assert np.array_equal(got[4], rpos), tag   # positions: exact, ties included
    if dens != 0.0:
        density(0.0)
        for g, e in zip(got, _run(x, xl, xu, w, q, K)):
            assert np.array_equal(g, e), tag


@pytest.mark.parametrize("dens", [1.0, 0.0, -1.0])
@pytest.mark.parametrize("B,CI,CO", [(70, 96, 64), (33, 2048, 300), (130, 1024, 513), (1, 32, 1), (257, 320, 129), (700, 160, 72),
                                     (512, 1088, 96)])
def test_sort_candidate_kernels_match_oracle(oracle, density, dens, B, CI, CO):
    """Ragged batch tiles (B not a multiple of 128) and weight rows (CO not a multiple of 32 / 64 / 128), rows of
    more than 32 chunks (several batches of marks per row), rows shorter than K."""
    for kind in ("rows_alike", "random", "inverted", "images", "ties", "pixels", "pixel_ties"):
        for q, K in ((0.3, 10), (0.75, 4)):
            x, xl, xu, w = _data(B, CI, CO, kind, B + CI)
            # (the bound of a batch row rests on the K largest of its per-chunk maxima: rows of at least K chunks)
            expect = dens == 1.0 and kind.startswith("pixel") and CI >= 32 * K and B > 1
            _check(oracle, density, dens, x, xl, xu, w, q, K, "dens=%g %s K=%d" % (dens, kind, K), expect)


@pytest.mark.parametrize("K", [2, 3, 7, 13, 16, 25])
def test_sort_candidate_kernels_every_k(oracle, density, K):
    x, xl, xu, w = _data(140, 512, 100, "rows_alike", K)
    _check(oracle, density, 1.0, x, xl, xu, w, 0.4, K, "K=%d" % K)


@pytest.mark.parametrize("K", [2, 3, 5, 6, 8, 9, 11, 13, 16, 20, 21, 25])
def test_sort_row_table_kernels_every_k(oracle, density, K):
    """The tables per batch row at every size of the top-K lists, for values, interval bounds and positions."""
    for kind in ("pixels", "pixel_ties"):
        x, xl, xu, w = _data(150, 1024, 200, kind, K)
        _check(oracle, density, 1.0, x, xl, xu, w, 0.4, K, "%s K=%d" % (kind, K), expect_tables=True)


def test_sort_candidate_kernels_at_layer_size(density):
    """B = 512, N = M = 5120, unit-scale weights against rows that are nearly alike: the table kernels and the
    every-term kernels give the same bits, and the built-in limit picks the table."""
    from sortnet_amd import ext
    dev = _dev()
    B, N, M, q, K = 512, 5120, 5120, 0.75, 10
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(1, N, 1, generator=g) * 0.3 + torch.randn(B, N, 1, generator=g) * 0.1).to(dev)
    r = 0.03 + torch.rand(B, N, 1, generator=g).to(dev) * 0.01
    xl, xu = (x - r).contiguous(), (x + r).contiguous()
    w = torch.randn(M, N, generator=g).contiguous().to(dev)
    out = {}
    for dens in (0.0, 1.0, -1.0):
        density(dens)
        y, yl, yu, yp = (torch.empty(B, M, 1, device=dev) for _ in range(4))
        pos = torch.empty(K, B, M, 1, device=dev, dtype=torch.int32)
        ext.sort_neuron_forward_nograd(x.contiguous(), w, y, 1, q, K)
        ext.bound_sort_neuron_forward(xl, xu, w, yl, yu, 1, q, K)
        ext.sort_neuron_forward(x.contiguous(), w, yp, pos, 1, q, K)
        out[dens] = (y, yl, yu, yp, pos)
    for dens in (1.0, -1.0):
        for a, b in zip(out[dens], out[0.0]):
            assert torch.equal(a, b), dens


@pytest.mark.parametrize("kind", ["rows_alike", "pixels", "ties"])
def test_sort_candidate_kernels_drop_undefined_terms(oracle, density, kind):
    """Undefined and infinite inputs and weights: a term with an undefined operand is left out of the K largest
    (include/sortdist.h), an infinite one counts.  The table kernels keep some of their lists as bit patterns, where an
    undefined value would order above every number: they must agree with the every-term kernels and the oracle, in
    both orientations of the tables (rows alike / pixels) and on ties."""
    B, CI, CO, q, K = 150, 1024, 200, 0.4, 10
    x, xl, xu, w = _data(B, CI, CO, kind, 11)
    g = torch.Generator().manual_seed(12)
    mx, mw = torch.rand(x.shape, generator=g), torch.rand(w.shape, generator=g)
    for t in (x, xl, xu):
        t[mx < 0.002] = float("nan")
        t[(mx >= 0.002) & (mx < 0.003)] = float("inf")
        t[(mx >= 0.003) & (mx < 0.004)] = float("-inf")
    w[mw < 0.0005] = float("nan")
    w[(mw >= 0.0005) & (mw < 0.001)] = float("inf")
    w[(mw >= 0.001) & (mw < 0.0015)] = float("-inf")
    ry, rpos = oracle.sort_neuron_forward(x.numpy(), w.numpy(), q, K)
    rl, ru = oracle.bound_sort_neuron_forward(xl.numpy(), xu.numpy(), w.numpy(), q, K)
    density(0.0)
    every = _run(x, xl, xu, w, q, K)
    for got, want in zip(every[:4], (ry, rl, ru, ry)):
        np.testing.assert_allclose(got, want, rtol=RTOL, err_msg=kind)   # (infinities and undefined sums compare equal)
    assert np.array_equal(every[4], rpos), kind
    density(1.0)
    for got, want in zip(_run(x, xl, xu, w, q, K), every):
        assert np.array_equal(got, want, equal_nan=got.dtype.kind == "f"), kind


def test_rows_longer_than_the_mark_lists_take_the_every_term_kernels(oracle, density):
    """The table kernels list marked inputs as 16-bit numbers: a dense layer with more than 65536 inputs per row
    (a multiple of 32, enough terms for the tables, density forced on) must fall back to the every-term kernels
    instead of being rejected."""
    x, xl, xu, w = _data(8, 65568, 32, "random", 5)
    _check(oracle, density, 1.0, x, xl, xu, w, 0.3, 10, "CI=65568")


def test_sort_candidate_density_argument(density):
    from sortnet_amd import _lib
    with pytest.raises(RuntimeError):
        _lib.set_sort_candidate_density(1.5)
    density(0.3)
