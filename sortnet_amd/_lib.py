"""ctypes binding of libsortdist.so (declarations: include/sortdist.h).

There is no fallback: if the library has not been built, importing anything that needs it
raises.  Build it with `make -C sortnet_amd/csrc` (or `__graft_entry__.build()`).
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsortdist.so")

_F = ctypes.c_void_p          # device pointer to float
_I = ctypes.c_void_p          # device pointer to int32
_S = ctypes.c_void_p          # hipStream_t
_i = ctypes.c_int
_f = ctypes.c_float
_u = ctypes.c_uint32

# name -> argument types, in the order of include/sortdist.h
SIGNATURES = {
    "sd_inf_dist_forward_nograd": [_F, _F, _i, _i, _i, _i, _i, _F, _S],
    "sd_inf_dist_forward": [_F, _F, _i, _i, _i, _i, _i, _F, _I, _I, _I, _i, _i, _S],
    "sd_inf_dist_forward_noalloc": [_F, _F, _i, _i, _i, _i, _i, _F, _I, _I, _I, _i, _i, _S],
    "sd_inf_dist_backward_input": [_F, _I, _i, _i, _i, _i, _i, _F, _S],
    "sd_inf_dist_backward_input_weight": [_F, _I, _i, _i, _i, _i, _i, _F, _F, _I, _I, _i, _i, _S],
    "sd_bound_inf_dist_forward_nograd": [_F, _F, _F, _i, _i, _i, _i, _i, _F, _F, _S],
    "sd_bound_inf_dist_forward": [_F, _F, _F, _i, _i, _i, _i, _i, _F, _F, _I, _I, _S],
    "sd_bound_inf_dist_backward_input": [_F, _F, _I, _I, _i, _i, _i, _i, _i, _F, _F, _S],
    "sd_bound_inf_dist_backward_input_weight": [_F, _F, _I, _I, _i, _i, _i, _i, _i, _F, _F, _F, _S],
    "sd_sort_neuron_forward_nograd": [_F, _F, _i, _i, _i, _i, _i, _F, _f, _i, _S],
    "sd_sort_neuron_forward": [_F, _F, _i, _i, _i, _i, _i, _F, _I, _f, _i, _S],
    "sd_sort_neuron_backward_input": [_F, _I, _i, _i, _i, _i, _i, _F, _f, _i, _S],
    "sd_sort_neuron_backward_input_weight": [_F, _I, _i, _i, _i, _i, _i, _F, _F, _f, _i, _S],
    "sd_bound_sort_neuron_forward": [_F, _F, _F, _i, _i, _i, _i, _i, _F, _F, _f, _i, _S],
    "sd_norm_dist_forward": [_F, _F, _i, _i, _i, _i, _i, _F, _f, _I, _I, _i, _i, _S],
    "sd_norm_dist_forward_with_max": [_F, _F, _F, _i, _i, _i, _i, _i, _F, _f, _I, _I, _i, _i, _S],
    "sd_norm_dist_backward_input": [_F, _F, _F, _F, _i, _i, _i, _i, _i, _F, _f, _I, _I, _i, _i, _S],
    "sd_norm_dist_backward_input_weight": [_F, _F, _F, _F, _i, _i, _i, _i, _i, _F, _F, _f, _I, _I, _i, _i, _S],
    "sd_masked_inf_dist_forward": [_F, _F, _i, _i, _i, _i, _i, _F, _I, _f, _u, _i, _S],
    "sd_mean_shift_forward": [_F, _i, _i, _i, _F, _F, _f, _F, _S],
    "sd_mean_shift_index_forward": [_F, _I, _i, _i, _i, _i, _i, _F, _F, _f, _F, _S],
    "sd_channel_shift": [_F, _F, _i, _i, _i, _f, _F, _S],
    "sd_sample_index_lists": [_u, _i, _i, _i, _i, _I, _S],
}
_OTHER = {
    "sd_version": ([], _i),
    "sd_last_error": ([], ctypes.c_char_p),
    "sd_last_forward_kernel": ([], ctypes.c_char_p),
    "sd_time_forward_kernels": ([_i], _i),
    "sd_last_forward_kernel_ms": ([], ctypes.c_float),
    "sd_last_forward_term_share": ([_S], ctypes.c_float),
    "sd_set_lp_candidate_density": ([_f], _i),
    "sd_set_bound_candidate_density": ([_f], _i),
    "sd_set_bound_candidate_form": ([_i], _i),
    "sd_set_sort_candidate_density": ([_f], _i),
    "sd_set_linf_candidate_density": ([_f], _i),
    "sd_set_linf_candidate_depth": ([_i], _i),
    "sd_rng_word": ([_u, _u, _u, _u], _u),
    "sd_mask_threshold8": ([_f], _u),
    "sd_mask_threshold16": ([_f], _u),
    "sd_mask_count": ([_u, _i, _f], _i),
}

_lib = None


def load():
    """Loads libsortdist.so once; raises RuntimeError if it is missing or incomplete."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "sortnet_amd: %s not found - build the HIP library first (make -C sortnet_amd/csrc); "
            "there is no fallback path" % LIB_PATH)
    # torch first: the library must bind the HIP runtime that torch ships and has initialised, not a second copy of it
    import torch  # noqa: F401
    lib = ctypes.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = _i
    for name, (args, res) in _OTHER.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = res
    _lib = lib
    return lib


def call(name, *args):
    """Calls an entry point and turns a non-zero status into RuntimeError."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.sd_last_error()
        raise RuntimeError("%s failed (status %d): %s" % (name, rc, msg.decode() if msg else "?"))


def set_lp_candidate_density(density):
    """Share of marked candidate-table entries up to which the dense l-p kernels work from the table (0: never)."""
    lib = load()
    rc = lib.sd_set_lp_candidate_density(float(density))
    if rc != 0:
        raise RuntimeError("sd_set_lp_candidate_density failed: %s" % lib.sd_last_error().decode())


def set_bound_candidate_density(density):
    """Share of marked candidate-table entries up to which the dense interval forward works from the table (0: never)."""
    lib = load()
    rc = lib.sd_set_bound_candidate_density(float(density))
    if rc != 0:
        raise RuntimeError("sd_set_bound_candidate_density failed: %s" % lib.sd_last_error().decode())


def set_bound_candidate_form(form):
    """Table kernel of the dense interval forward: 0 chosen per layer, 1 staged tiles, 2 walk over transposed inputs."""
    lib = load()
    rc = lib.sd_set_bound_candidate_form(int(form))
    if rc != 0:
        raise RuntimeError("sd_set_bound_candidate_form failed: %s" % lib.sd_last_error().decode())


def set_sort_candidate_density(density):
    """Share of marked candidate-table entries up to which the dense sort neuron (values only) and its interval
    bounds work from the table (0: never; negative: built-in limit, large layers only)."""
    lib = load()
    rc = lib.sd_set_sort_candidate_density(float(density))
    if rc != 0:
        raise RuntimeError("sd_set_sort_candidate_density failed: %s" % lib.sd_last_error().decode())


def set_linf_candidate_density(density):
    """Share of marked candidate-table entries up to which the dense l-inf forward (plain and under the factored
    mask) works from the table (0: never; negative: built-in limit, large layers only)."""
    lib = load()
    rc = lib.sd_set_linf_candidate_density(float(density))
    if rc != 0:
        raise RuntimeError("sd_set_linf_candidate_density failed: %s" % lib.sd_last_error().decode())


def set_linf_candidate_depth(depth):
    """Inputs per weight row the table's bound rests on under the factored mask (0: from the keep probability)."""
    lib = load()
    rc = lib.sd_set_linf_candidate_depth(int(depth))
    if rc != 0:
        raise RuntimeError("sd_set_linf_candidate_depth failed: %s" % lib.sd_last_error().decode())


def last_forward_kernel():
    """Name and register tile of the forward tile kernel that this thread's last forward call dispatched."""
    return load().sd_last_forward_kernel().decode()


def time_forward_kernels(on):
    """Switches the events around this thread's forward tile kernel launches on or off."""
    load().sd_time_forward_kernels(1 if on else 0)


def last_forward_kernel_ms():
    """Duration of the forward tile kernel this thread launched last with timing on (waits for it), or None."""
    ms = load().sd_last_forward_kernel_ms()
    return None if ms < 0 else ms


def last_forward_term_share(stream=None):
    """Share of its terms that this thread's last forward call formed (waits for `stream`, default torch's current
    one): the marked share when a candidate-table kernel served the call, 1.0 when every term was evaluated."""
    if stream is None:
        import torch
        stream = torch.cuda.current_stream().cuda_stream
    share = load().sd_last_forward_term_share(stream)
    if share < 0:
        raise RuntimeError("sd_last_forward_term_share failed")
    return share
