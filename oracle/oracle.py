"""numpy front-end of liboracle.so (built from sortdist_oracle.c by oracle/Makefile).

TEST INFRASTRUCTURE ONLY.  Every function takes and returns numpy arrays (fp32 / int32,
C-contiguous) shaped like the reference's tensors: x (B, CI, HW), weight (W_CO, W_CI/G),
outputs (B, CO, HW), sort-neuron pos (K, B, CO, HW).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

MASK_TERM = 0
MASK_FACTORED = 1

__all__ = [
    "build", "MASK_TERM", "MASK_FACTORED", "rng_word", "mask_threshold8", "mask_threshold16",
    "inf_dist_forward", "inf_dist_backward", "masked_inf_dist_forward",
    "bound_inf_dist_forward", "bound_inf_dist_backward",
    "sort_neuron_forward", "sort_neuron_backward", "bound_sort_neuron_forward",
    "norm_dist_forward", "norm_dist_backward", "mean_shift", "set_num_threads",
    "mask_count", "sample_index_lists",
]


def build(force=False):
    """Compile liboracle.so with gcc (a couple of seconds)."""
    src = os.path.join(_HERE, "sortdist_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.sdo_rng_word.restype = ctypes.c_uint32
        _lib.sdo_rng_word.argtypes = [ctypes.c_uint32] * 4
        _lib.sdo_mask_threshold8.restype = ctypes.c_uint32
        _lib.sdo_mask_threshold8.argtypes = [ctypes.c_float]
        _lib.sdo_mask_threshold16.restype = ctypes.c_uint32
        _lib.sdo_mask_threshold16.argtypes = [ctypes.c_float]
    return _lib


def set_num_threads(n):
    """Number of OpenMP threads the oracle uses (for the timed CPU baseline)."""
    gomp = ctypes.CDLL("libgomp.so.1")
    gomp.omp_set_num_threads(int(n))


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _i(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.int32)


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c_int(*v):
    return [ctypes.c_int(int(t)) for t in v]


def _dims(x, weight, groups, w_index_ci=None, w_index_co=None):
    B, CI, HW = x.shape
    CO = weight.shape[0] if w_index_co is None else w_index_co.shape[-1] * groups
    return B, CO, CI, HW, weight.shape[0], weight.shape[1] * groups


def rng_word(seed, stream, row, col):
    return int(_load().sdo_rng_word(seed & 0xFFFFFFFF, stream, row & 0xFFFFFFFF, col & 0xFFFFFFFF))


def mask_threshold8(q):
    return int(_load().sdo_mask_threshold8(ctypes.c_float(q)))


def mask_threshold16(q):
    return int(_load().sdo_mask_threshold16(ctypes.c_float(q)))


def inf_dist_forward(x, weight, groups=1, need_pos=True, w_index_ci=None, w_index_co=None):
    x, weight = _f(x), _f(weight)
    ci, co = _i(w_index_ci), _i(w_index_co)
    B, CO, CI, HW, W_CO, W_CI = _dims(x, weight, groups, ci, co)
    y = np.empty((B, CO, HW), np.float32)
    pos = np.empty((B, CO, HW), np.int32) if need_pos else None
    _load().sdo_inf_dist_forward(_p(x), _p(weight), *_c_int(B, CO, CI, groups, HW), _p(y), _p(pos),
                                 _p(ci), _p(co), *_c_int(W_CO, W_CI))
    return (y, pos) if need_pos else y


def masked_inf_dist_forward(x, weight, q, seed, mode=MASK_TERM, groups=1, need_pos=True):
    x, weight = _f(x), _f(weight)
    B, CO, CI, HW, _, _ = _dims(x, weight, groups)
    y = np.empty((B, CO, HW), np.float32)
    pos = np.empty((B, CO, HW), np.int32) if need_pos else None
    _load().sdo_masked_inf_dist_forward(_p(x), _p(weight), *_c_int(B, CO, CI, groups, HW), _p(y), _p(pos),
                                        ctypes.c_float(q), ctypes.c_uint32(seed & 0xFFFFFFFF), ctypes.c_int(mode))
    return (y, pos) if need_pos else y


def inf_dist_backward(grad_y, pos, x_shape, weight_shape, groups=1, need_weight=True,
                      w_index_ci=None, w_index_co=None):
    gy, pos = _f(grad_y), _i(pos)
    ci, co = _i(w_index_ci), _i(w_index_co)
    B, CI, HW = x_shape
    CO = gy.shape[1]
    gx = np.empty(x_shape, np.float32)
    gw = np.empty(weight_shape, np.float32) if need_weight else None
    _load().sdo_inf_dist_backward(_p(gy), _p(pos), *_c_int(B, CO, CI, groups, HW), _p(gx), _p(gw),
                                  _p(ci), _p(co), *_c_int(weight_shape[0], weight_shape[1] * groups))
    return (gx, gw) if need_weight else gx


def bound_inf_dist_forward(x_lower, x_upper, weight, groups=1, need_pos=True):
    xl, xu, weight = _f(x_lower), _f(x_upper), _f(weight)
    B, CO, CI, HW, _, _ = _dims(xl, weight, groups)
    yl = np.empty((B, CO, HW), np.float32)
    yu = np.empty_like(yl)
    pl = np.empty((B, CO, HW), np.int32) if need_pos else None
    pu = np.empty((B, CO, HW), np.int32) if need_pos else None
    _load().sdo_bound_inf_dist_forward(_p(xl), _p(xu), _p(weight), *_c_int(B, CO, CI, groups, HW),
                                       _p(yl), _p(yu), _p(pl), _p(pu))
    return (yl, yu, pl, pu) if need_pos else (yl, yu)


def bound_inf_dist_backward(grad_yl, grad_yu, pos_lower, pos_upper, x_shape, weight_shape, groups=1,
                            need_weight=True):
    gl, gu = _f(grad_yl), _f(grad_yu)
    pl, pu = _i(pos_lower), _i(pos_upper)
    B, CI, HW = x_shape
    CO = gl.shape[1]
    gxl = np.empty(x_shape, np.float32)
    gxu = np.empty(x_shape, np.float32)
    gw = np.empty(weight_shape, np.float32) if need_weight else None
    _load().sdo_bound_inf_dist_backward(_p(gl), _p(gu), _p(pl), _p(pu), *_c_int(B, CO, CI, groups, HW),
                                        _p(gxl), _p(gxu), _p(gw))
    return (gxl, gxu, gw) if need_weight else (gxl, gxu)


def sort_neuron_forward(x, weight, q, K, groups=1, need_pos=True):
    x, weight = _f(x), _f(weight)
    B, CO, CI, HW, _, _ = _dims(x, weight, groups)
    y = np.empty((B, CO, HW), np.float32)
    pos = np.empty((K, B, CO, HW), np.int32) if need_pos else None
    rc = _load().sdo_sort_neuron_forward(_p(x), _p(weight), *_c_int(B, CO, CI, groups, HW), _p(y), _p(pos),
                                         ctypes.c_float(q), ctypes.c_int(K))
    if rc:
        raise ValueError("K out of range")
    return (y, pos) if need_pos else y


def sort_neuron_backward(grad_y, pos, x_shape, weight_shape, q, K, groups=1, need_weight=True):
    gy, pos = _f(grad_y), _i(pos)
    B, CI, HW = x_shape
    CO = gy.shape[1]
    gx = np.empty(x_shape, np.float32)
    gw = np.empty(weight_shape, np.float32) if need_weight else None
    _load().sdo_sort_neuron_backward(_p(gy), _p(pos), *_c_int(B, CO, CI, groups, HW), _p(gx), _p(gw),
                                     ctypes.c_float(q), ctypes.c_int(K))
    return (gx, gw) if need_weight else gx


def bound_sort_neuron_forward(x_lower, x_upper, weight, q, K, groups=1):
    xl, xu, weight = _f(x_lower), _f(x_upper), _f(weight)
    B, CO, CI, HW, _, _ = _dims(xl, weight, groups)
    yl = np.empty((B, CO, HW), np.float32)
    yu = np.empty_like(yl)
    rc = _load().sdo_bound_sort_neuron_forward(_p(xl), _p(xu), _p(weight), *_c_int(B, CO, CI, groups, HW),
                                               _p(yl), _p(yu), ctypes.c_float(q), ctypes.c_int(K))
    if rc:
        raise ValueError("K out of range")
    return yl, yu


def norm_dist_forward(x, weight, p, groups=1, w_index_ci=None, w_index_co=None):
    x, weight = _f(x), _f(weight)
    ci, co = _i(w_index_ci), _i(w_index_co)
    B, CO, CI, HW, W_CO, W_CI = _dims(x, weight, groups, ci, co)
    y = np.empty((B, CO, HW), np.float32)
    _load().sdo_norm_dist_forward(_p(x), _p(weight), *_c_int(B, CO, CI, groups, HW), _p(y), ctypes.c_float(p),
                                  _p(ci), _p(co), *_c_int(W_CO, W_CI))
    return y


def norm_dist_backward(grad_y, x, weight, y, p, groups=1, need_weight=True, w_index_ci=None, w_index_co=None):
    gy, x, weight, y = _f(grad_y), _f(x), _f(weight), _f(y)
    ci, co = _i(w_index_ci), _i(w_index_co)
    B, CO, CI, HW, W_CO, W_CI = _dims(x, weight, groups, ci, co)
    gx = np.empty_like(x)
    gw = np.empty_like(weight) if need_weight else None
    _load().sdo_norm_dist_backward(_p(gy), _p(x), _p(weight), _p(y), *_c_int(B, CO, CI, groups, HW),
                                   _p(gx), _p(gw), ctypes.c_float(p), _p(ci), _p(co), *_c_int(W_CO, W_CI))
    return (gx, gw) if need_weight else gx


def mean_shift(x):
    x = _f(x)
    B, C, HW = x.shape
    mean = np.empty((C,), np.float32)
    out = np.empty_like(x)
    _load().sdo_mean_shift(_p(x), *_c_int(B, C, HW), _p(mean), _p(out))
    return out, mean


def mask_count(seed, channels, q):
    lib = _load()
    lib.sdo_mask_count.restype = ctypes.c_int
    return int(lib.sdo_mask_count(ctypes.c_uint32(seed & 0xFFFFFFFF), ctypes.c_int(channels), ctypes.c_float(q)))


def sample_index_lists(seed, sub_batches, groups, channels, count):
    out = np.empty((sub_batches, groups, count), np.int32)
    _load().sdo_sample_index_lists(ctypes.c_uint32(seed & 0xFFFFFFFF), *_c_int(sub_batches, groups, channels, count), _p(out))
    return out
