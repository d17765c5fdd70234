"""Seeded random cases of every entry point that can work from candidate tables: the table kernels (forced: staged
interval kernel and the walk over transposed inputs, sort neuron with and without positions, l-inf forward plain and
under the factored mask at several depths) against the kernels that evaluate every term, which the other GPU tests
hold to the oracle.  Values and positions must be the same bits.  Random batch sizes (ragged tiles, more than four
tiles), row lengths, channel counts, K, keep probabilities, inverted intervals and four kinds of data."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _data(rng, B, CI, CO, kind, g, dev):
    if kind == 0:      # rows alike against unit-scale weights: few marks
        x = torch.randn(1, CI, 1, generator=g) * 0.3 + torch.randn(B, CI, 1, generator=g) * float(rng.choice([0.01, 0.05, 0.2]))
        w = torch.randn(CO, CI, generator=g)
    elif kind == 1:    # images against small weights: the batch row decides
        x = torch.rand(B, CI, 1, generator=g)
        w = torch.randn(CO, CI, generator=g) * CI ** -0.5
    elif kind == 2:    # grid data: exact ties
        x = torch.round(torch.randn(B, CI, 1, generator=g) * 0.8) / 4
        w = torch.round(torch.randn(CO, CI, generator=g) * 4) / 4
    else:              # unrelated rows: nearly everything is marked
        x = torch.randn(B, CI, 1, generator=g)
        w = torch.randn(CO, CI, generator=g) * float(rng.choice([0.1, 1.0, 3.0]))
    return x.contiguous().to(dev), w.contiguous().to(dev)


@pytest.mark.parametrize("case", range(16))
def test_table_kernels_equal_every_term_kernels(case):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from sortnet_amd import ext, _lib
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(1000 + case)
    B = int(rng.integers(1, 700)); CI = 32 * int(rng.integers(1, 80)); CO = int(rng.integers(1, 700))
    kind = case % 4
    K = min(int(rng.integers(2, 26)), CI)
    q = float(rng.choice([0.2, 0.3, 0.5, 0.75, 1.0]))
    g = torch.Generator().manual_seed(case)
    x, w = _data(rng, B, CI, CO, kind, g, dev)
    r = torch.rand(B, CI, 1, generator=g).to(dev) * 0.05
    xl, xu = (x - r).contiguous(), (x + r).contiguous()
    if case % 3 == 0:   # some inverted intervals
        m = (torch.rand(B, CI, 1, generator=g) < 0.1).to(dev)
        xl, xu = torch.where(m, xu, xl).contiguous(), torch.where(m, xl, xu).contiguous()
    seed = int(rng.integers(0, 2 ** 31))
    depth = int(rng.choice([0, 8, 12, 24]))
    out = {}
    try:
        for dens, form in ((0.0, 0), (1.0, 1), (1.0, 2)):
            _lib.set_sort_candidate_density(dens)
            _lib.set_linf_candidate_density(dens)
            _lib.set_bound_candidate_density(dens)
            _lib.set_bound_candidate_form(form)
            _lib.set_linf_candidate_depth(depth)
            o = [torch.full((B, CO, 1), float("nan"), device=dev) for _ in range(9)]
            p1 = torch.full((B, CO, 1), -7, device=dev, dtype=torch.int32)
            p2 = torch.full_like(p1, -7)
            pk = torch.full((K, B, CO, 1), -7, device=dev, dtype=torch.int32)
            ext.sort_neuron_forward_nograd(x, w, o[0], 1, q, K)
            ext.sort_neuron_forward(x, w, o[1], pk, 1, q, K)
            ext.bound_sort_neuron_forward(xl, xu, w, o[2], o[3], 1, q, K)
            ext.inf_dist_forward(x, w, o[4], p1, 1)
            ext.inf_dist_forward_nograd(x, w, o[5], 1)
            ext.masked_inf_dist_forward(x, w, o[6], p2, 1, q, seed, ext.MASK_FACTORED)
            ext.bound_inf_dist_forward_nograd(xl, xu, w, o[7], o[8], 1)
            out[(dens, form)] = o + [p1, p2, pk]
    finally:
        _lib.set_sort_candidate_density(-1.0)
        _lib.set_linf_candidate_density(-1.0)
        _lib.set_bound_candidate_density(-1.0)
        _lib.set_bound_candidate_form(0)
        _lib.set_linf_candidate_depth(0)
    names = ("sort nograd", "sort", "bound sort L", "bound sort U", "l-inf", "l-inf nograd", "masked", "bound L", "bound U",
             "l-inf pos", "masked pos", "sort pos")
    for key in ((1.0, 1), (1.0, 2)):
        for name, a, b in zip(names, out[key], out[(0.0, 0)]):
            assert torch.equal(a, b), "%s, tables %s: B=%d CI=%d CO=%d kind=%d K=%d q=%g depth=%d" % (
                name, key, B, CI, CO, kind, K, q, depth)
