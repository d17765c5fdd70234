"""CPU-side checks of the drop-in boundary: the shared library loads without a GPU and exports
every symbol that include/sortdist.h declares; the host-side helpers that need no device agree
with the oracle."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "sortdist.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sd_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    from sortnet_amd import _lib
    lib = _lib.load()
    names = _declared()
    assert len(names) >= 23
    for n in names:
        assert hasattr(lib, n), n
    bound = set(_lib.SIGNATURES) | set(_lib._OTHER)
    assert set(names) == bound


def test_host_helpers_match_oracle(oracle):
    from sortnet_amd import _lib
    lib = _lib.load()
    for args in [(0, 0, 0, 0), (1, 2, 3, 4), (0xDEADBEEF, 1, 123456, 789)]:
        assert lib.sd_rng_word(*args) == oracle.rng_word(*args)
    for q in [0.0, 0.1, 0.3, 0.5, 0.75, 1.0]:
        assert lib.sd_mask_threshold8(q) == oracle.mask_threshold8(q)
        assert lib.sd_mask_threshold16(q) == oracle.mask_threshold16(q)
    assert lib.sd_version() >= 100


def test_functional_api_surface():
    import inspect
    import sortnet_amd.norm_dist as nd
    sig = {n: list(inspect.signature(getattr(nd, n)).parameters) for n in
           ["norm_dist", "norm_dist_dropout", "sort_neuron", "bound_sort_neuron", "bound_inf_dist"]}
    assert sig["norm_dist"] == ["input", "weight", "p", "groups", "use_custom_cuda_func", "tag"]
    assert sig["norm_dist_dropout"] == ["input", "weight", "w_index_ci", "w_index_co", "p", "groups",
                                        "use_custom_cuda_func", "tag"]
    assert sig["sort_neuron"] == ["input", "weight", "groups", "q", "truncate", "use_custom_cuda_func", "tag"]
    assert sig["bound_sort_neuron"] == ["x_lower", "x_upper", "weight", "groups", "q", "truncate", "tag"]
    assert sig["bound_inf_dist"] == ["x_lower", "x_upper", "weight", "groups", "use_custom_cuda_func", "tag"]
    for cls in ["NormDistF", "NormDistDropoutF", "SortNeuronF", "BoundInfDistF"]:
        assert hasattr(getattr(nd, cls), "apply")
