"""Known-answer vectors (tests/golden/vectors.json, written by tests/golden/make_fixtures.py from pure
Python / numpy statements of each op) against the CPU oracle (no GPU needed) and against the GPU library
(through the C ABI).  Bit-exact sets: l-inf, masked neuron, interval bounds, sort positions, RNG words,
thresholds, sampler lists.  Tolerance sets (rel 1e-5): sort-neuron sums, l-p values and gradients."""
import json
import os

import numpy as np
import pytest
import torch

RTOL = 1e-5
HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def vec():
    with open(os.path.join(HERE, "golden", "vectors.json")) as f:
        return json.load(f)


def _f(a):
    return np.asarray(a, dtype=np.float32)


def _pos(a):
    return (np.asarray(a, dtype=np.int64) & 0xFFFFFFFF).astype(np.uint32)


def _u(a):
    return np.ascontiguousarray(a).view(np.uint32)


def _close(got, ref):
    ref = np.asarray(ref, dtype=np.float64)
    np.testing.assert_allclose(np.asarray(got, dtype=np.float64), ref, rtol=RTOL, atol=RTOL * float(np.abs(ref).max()))


# ---------------------------------------------------------------------------- oracle (CPU)
def test_oracle_linf_and_masked(oracle, vec):
    x, w = _f(vec["linf"]["x"])[:, :, None], _f(vec["linf"]["w"])
    y, pos = oracle.inf_dist_forward(x, w)
    assert np.array_equal(y[:, :, 0], _f(vec["linf"]["y"])) and np.array_equal(_u(pos)[:, :, 0], _pos(vec["linf"]["pos"]))
    for name, mode in (("masked_term", oracle.MASK_TERM), ("masked_factored", oracle.MASK_FACTORED)):
        v = vec[name]
        y, pos = oracle.masked_inf_dist_forward(x, w, v["q"], v["seed"], mode)
        assert np.array_equal(y[:, :, 0], _f(v["y"])), name
        assert np.array_equal(_u(pos)[:, :, 0], _pos(v["pos"])), name


def test_oracle_bound(oracle, vec):
    v = vec["bound"]
    yl, yu, pl, pu = oracle.bound_inf_dist_forward(_f(v["xl"])[:, :, None], _f(v["xu"])[:, :, None], _f(v["w"]))
    assert np.array_equal(yl[:, :, 0], _f(v["yl"])) and np.array_equal(yu[:, :, 0], _f(v["yu"]))
    assert np.array_equal(_u(pl)[:, :, 0], _pos(v["pl"])) and np.array_equal(_u(pu)[:, :, 0], _pos(v["pu"]))
    assert (_pos(v["pl"]) == 0xFFFFFFFF).any(), "fixture must exercise the no-gradient sentinel"


def test_oracle_sort(oracle, vec):
    v = vec["sort"]
    y, pos = oracle.sort_neuron_forward(_f(v["x"])[:, :, None], _f(v["w"]), v["q"], v["K"])
    _close(y[:, :, 0], v["y"])
    assert np.array_equal(_u(pos)[:, :, :, 0], _pos(v["pos"]))


def test_oracle_lp(oracle, vec):
    v = vec["lp"]
    x, w, g = _f(v["x"])[:, :, None], _f(v["w"]), _f(v["g"])[:, :, None]
    for c in v["cases"]:
        y = oracle.norm_dist_forward(x, w, c["p"])
        _close(y[:, :, 0], c["y"])
        gx, gw = oracle.norm_dist_backward(g, x, w, y, c["p"])
        _close(gx[:, :, 0], c["gx"])
        _close(gw, c["gw"])


def test_oracle_rng_and_sampler(oracle, vec):
    for s, st, r, c, expect in vec["rng"]["words"]:
        assert oracle.rng_word(s, st, r, c) == expect
    for q, t in vec["rng"]["t8"]:
        assert oracle.mask_threshold8(q) == t
    for q, t in vec["rng"]["t16"]:
        assert oracle.mask_threshold16(q) == t
    for v in vec["sampler"]:
        assert oracle.mask_count(v["seed"], v["C"], v["q"]) == v["count"]
        lists = oracle.sample_index_lists(v["seed"], v["S"], v["G"], v["C"], v["count"])
        assert np.array_equal(lists, np.asarray(v["lists"], dtype=np.int32).reshape(v["S"], v["G"], v["count"]))


# ---------------------------------------------------------------------------- GPU library
def _dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def _t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


@pytest.mark.gpu
def test_gpu_linf_masked_bound(vec):
    from sortnet_amd import ext
    dev = _dev()
    x, w = _t(_f(vec["linf"]["x"])[:, :, None], dev), _t(_f(vec["linf"]["w"]), dev)
    B, M = x.size(0), w.size(0)
    y = torch.empty(B, M, 1, device=dev)
    pos = torch.empty(B, M, 1, device=dev, dtype=torch.int32)
    ext.inf_dist_forward(x, w, y, pos, 1)
    assert np.array_equal(y.cpu().numpy()[:, :, 0], _f(vec["linf"]["y"]))
    assert np.array_equal(_u(pos.cpu().numpy())[:, :, 0], _pos(vec["linf"]["pos"]))
    ext.inf_dist_forward_nograd(x, w, y, 1)
    assert np.array_equal(y.cpu().numpy()[:, :, 0], _f(vec["linf"]["y"]))
    for name, mode in (("masked_term", ext.MASK_TERM), ("masked_factored", ext.MASK_FACTORED)):
        v = vec[name]
        ext.masked_inf_dist_forward(x, w, y, pos, 1, v["q"], v["seed"], mode)
        assert np.array_equal(y.cpu().numpy()[:, :, 0], _f(v["y"])), name
        assert np.array_equal(_u(pos.cpu().numpy())[:, :, 0], _pos(v["pos"])), name
        ext.masked_inf_dist_forward(x, w, y, None, 1, v["q"], v["seed"], mode)
        assert np.array_equal(y.cpu().numpy()[:, :, 0], _f(v["y"])), name
    v = vec["bound"]
    xl, xu, w = _t(_f(v["xl"])[:, :, None], dev), _t(_f(v["xu"])[:, :, None], dev), _t(_f(v["w"]), dev)
    yl, yu = torch.empty(B, M, 1, device=dev), torch.empty(B, M, 1, device=dev)
    pl, pu = torch.empty_like(pos), torch.empty_like(pos)
    ext.bound_inf_dist_forward(xl, xu, w, yl, yu, pl, pu, 1)
    assert np.array_equal(yl.cpu().numpy()[:, :, 0], _f(v["yl"])) and np.array_equal(yu.cpu().numpy()[:, :, 0], _f(v["yu"]))
    assert np.array_equal(_u(pl.cpu().numpy())[:, :, 0], _pos(v["pl"]))
    assert np.array_equal(_u(pu.cpu().numpy())[:, :, 0], _pos(v["pu"]))
    ext.bound_inf_dist_forward_nograd(xl, xu, w, yl, yu, 1)
    assert np.array_equal(yl.cpu().numpy()[:, :, 0], _f(v["yl"])) and np.array_equal(yu.cpu().numpy()[:, :, 0], _f(v["yu"]))


@pytest.mark.gpu
def test_gpu_sort_lp_sampler(vec):
    from sortnet_amd import ext
    dev = _dev()
    v = vec["sort"]
    x, w = _t(_f(v["x"])[:, :, None], dev), _t(_f(v["w"]), dev)
    B, M, K = x.size(0), w.size(0), v["K"]
    y = torch.empty(B, M, 1, device=dev)
    pos = torch.empty(K, B, M, 1, device=dev, dtype=torch.int32)
    ext.sort_neuron_forward(x, w, y, pos, 1, v["q"], K)
    _close(y.cpu().numpy()[:, :, 0], v["y"])
    assert np.array_equal(_u(pos.cpu().numpy())[:, :, :, 0], _pos(v["pos"]))
    ext.sort_neuron_forward_nograd(x, w, y, 1, v["q"], K)
    _close(y.cpu().numpy()[:, :, 0], v["y"])
    v = vec["lp"]
    x, w, g = _t(_f(v["x"])[:, :, None], dev), _t(_f(v["w"]), dev), _t(_f(v["g"])[:, :, None], dev)
    gx, gw = torch.empty_like(x), torch.empty_like(w)
    for c in v["cases"]:
        ext.norm_dist_forward(x, w, y, 1, c["p"])
        _close(y.cpu().numpy()[:, :, 0], c["y"])
        ext.norm_dist_backward_input_weight(g, x, w, y, gx, gw, 1, c["p"])
        _close(gx.cpu().numpy()[:, :, 0], c["gx"])
        _close(gw.cpu().numpy(), c["gw"])
    for s, st, r, c, expect in vec["rng"]["words"]:
        assert ext.rng_word(s, st, r, c) == expect
    for v in vec["sampler"]:
        assert ext.mask_count(v["seed"], v["C"], v["q"]) == v["count"]
        lists = ext.sample_index_lists(v["seed"], v["S"], v["G"], v["C"], v["count"], dev)
        assert np.array_equal(lists.cpu().numpy(), np.asarray(v["lists"], dtype=np.int32).reshape(v["S"], v["G"], v["count"]))
