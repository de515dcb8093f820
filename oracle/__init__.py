"""ctypes binding of the CPU oracle (oracle/nnf_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by bench.py's
cpu_baseline leg as the checker / the timed baseline. Nothing under nnforge_amd/ imports it.
All functions take and return numpy float32 arrays in nnForge's [entry][feature_map][y][x] layout.
"""

import ctypes
import os
import subprocess

import numpy as np

ORACLE_DIR = os.path.dirname(os.path.abspath(__file__))
LIBRARY = os.path.join(ORACLE_DIR, "libnnf_oracle.so")

_lib = None
_FP = ctypes.POINTER(ctypes.c_float)
_UP = ctypes.POINTER(ctypes.c_uint)


def build():
    """Compiles oracle/nnf_oracle.c with the Makefile beside it."""
    proc = subprocess.run(["make", "-C", ORACLE_DIR, "-B", "libnnf_oracle.so"], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("oracle build failed:\n" + proc.stdout)
    return LIBRARY


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIBRARY):
            build()
        lib = ctypes.CDLL(LIBRARY)
        lib.nnf_oracle_max_threads.restype = ctypes.c_int
        lib.nnf_oracle_average_subsampling_plain_mult.restype = ctypes.c_float
        lib.nnf_oracle_average_subsampling_plain_mult.argtypes = [ctypes.c_uint, ctypes.c_uint, ctypes.c_int, ctypes.c_float]
        lib.nnf_oracle_average_subsampling_full_mult.restype = ctypes.c_float
        lib.nnf_oracle_average_subsampling_full_mult.argtypes = [ctypes.c_int, _UP, ctypes.c_uint, ctypes.c_uint, ctypes.c_int, ctypes.c_float]
        lib.nnf_oracle_batch_norm.argtypes = [_FP, _FP, _FP, _FP, _FP, _FP, ctypes.c_uint, ctypes.c_uint, ctypes.c_uint, ctypes.c_int]
        lib.nnf_oracle_rectified_linear.argtypes = [_FP, _FP, ctypes.c_float, ctypes.c_longlong, ctypes.c_int]
        lib.nnf_oracle_parametric_rectified_linear.argtypes = [_FP, _FP, _FP, ctypes.c_uint, ctypes.c_uint, ctypes.c_uint, ctypes.c_int]
        lib.nnf_oracle_exponential_linear.argtypes = [_FP, _FP, ctypes.c_longlong, ctypes.c_int]
        lib.nnf_oracle_sigmoid.argtypes = [_FP, _FP, ctypes.c_longlong, ctypes.c_int]
        lib.nnf_oracle_hyperbolic_tangent.argtypes = [_FP, _FP, ctypes.c_float, ctypes.c_float, ctypes.c_longlong, ctypes.c_int]
        lib.nnf_oracle_add.argtypes = [_FP, ctypes.POINTER(_FP), ctypes.c_int, ctypes.c_float, ctypes.c_longlong, ctypes.c_int]
        lib.nnf_oracle_softmax.argtypes = [_FP, _FP, ctypes.c_uint, ctypes.c_uint, ctypes.c_uint, ctypes.c_int]
        lib.nnf_oracle_average_subsampling.argtypes = [_FP, _FP, ctypes.c_uint, ctypes.c_uint, ctypes.c_uint, ctypes.c_int,
                                                       _UP, _UP, _UP, ctypes.c_uint, ctypes.c_uint, ctypes.c_float, ctypes.c_int]
        lib.nnf_oracle_absolute.argtypes = [_FP, _FP, ctypes.c_size_t, ctypes.c_int]
        lib.nnf_oracle_dropout.argtypes = [_FP, _FP, ctypes.c_size_t]
        lib.nnf_oracle_concat.argtypes = [_FP, ctypes.POINTER(_FP), _UP, ctypes.c_int, ctypes.c_uint]
        lib.nnf_oracle_maxout.argtypes = [_FP, _FP, ctypes.c_uint, ctypes.c_uint, ctypes.c_uint, ctypes.c_uint, ctypes.c_int]
        lib.nnf_oracle_max_subsampling.argtypes = [_FP, _FP, ctypes.c_uint, ctypes.c_uint, ctypes.c_uint, ctypes.c_int,
                                                   _UP, _UP, _UP, _UP, ctypes.c_uint, ctypes.c_uint, ctypes.c_int, ctypes.c_int,
                                                   ctypes.c_int]
        lib.nnf_oracle_max_subsampling_tiling.argtypes = [_FP, _FP, ctypes.c_uint, ctypes.c_uint, ctypes.c_int, _UP, _UP, _UP,
                                                          ctypes.c_int, ctypes.c_int]
        lib.nnf_oracle_feature_map_stat_init.argtypes = [ctypes.c_void_p, ctypes.c_uint]
        lib.nnf_oracle_feature_map_stat_write.argtypes = [ctypes.c_void_p, _FP, ctypes.c_uint, ctypes.c_uint, ctypes.c_uint, ctypes.c_int]
        lib.nnf_oracle_feature_map_stat_get.argtypes = [ctypes.c_void_p, ctypes.c_uint, _FP, _FP, _FP, _FP]
        lib.nnf_oracle_update_bn_weights.argtypes = [_FP, _FP, _FP, _FP, ctypes.c_uint]
        _lib = lib
    return _lib


def max_threads():
    return load().nnf_oracle_max_threads()


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _ptr(a):
    return a.ctypes.data_as(_FP)


def _out_for(x, out):
    if out is None:
        return np.empty_like(x)
    assert out.dtype == np.float32 and out.flags.c_contiguous and out.size == x.size
    return out


def _shape3(x):
    """(entry_count, feature_map_count, neuron_count_per_feature_map) of an [N][C][...] array."""
    n, c = x.shape[0], x.shape[1]
    plane = int(np.prod(x.shape[2:], dtype=np.int64)) if x.ndim > 2 else 1
    return n, c, plane


def batch_norm(x, gamma, beta, mean, inverse_sigma, out=None, threads=0):
    x = _f32(x)
    n, c, plane = _shape3(x)
    g, b, m, s = (_f32(v) for v in (gamma, beta, mean, inverse_sigma))
    assert g.size == b.size == m.size == s.size == c
    out = _out_for(x, out)
    load().nnf_oracle_batch_norm(_ptr(out), _ptr(x), _ptr(g), _ptr(b), _ptr(m), _ptr(s), n, c, plane, threads)
    return out


def rectified_linear(x, negative_slope=0.0, out=None, threads=0):
    x = _f32(x)
    out = _out_for(x, out)
    load().nnf_oracle_rectified_linear(_ptr(out), _ptr(x), negative_slope, x.size, threads)
    return out


def parametric_rectified_linear(x, slopes, out=None, threads=0):
    x = _f32(x)
    n, c, plane = _shape3(x)
    a = _f32(slopes)
    assert a.size == c
    out = _out_for(x, out)
    load().nnf_oracle_parametric_rectified_linear(_ptr(out), _ptr(x), _ptr(a), n, c, plane, threads)
    return out


def exponential_linear(x, out=None, threads=0):
    x = _f32(x)
    out = _out_for(x, out)
    load().nnf_oracle_exponential_linear(_ptr(out), _ptr(x), x.size, threads)
    return out


def sigmoid(x, out=None, threads=0):
    x = _f32(x)
    out = _out_for(x, out)
    load().nnf_oracle_sigmoid(_ptr(out), _ptr(x), x.size, threads)
    return out


def hyperbolic_tangent(x, scale=1.0, steepness=1.0, out=None, threads=0):
    x = _f32(x)
    out = _out_for(x, out)
    load().nnf_oracle_hyperbolic_tangent(_ptr(out), _ptr(x), scale, steepness, x.size, threads)
    return out


def add(inputs, alpha=1.0, out=None, threads=0):
    arrays = [_f32(a) for a in inputs]
    assert all(a.size == arrays[0].size for a in arrays)
    out = _out_for(arrays[0], out)
    ptrs = (_FP * len(arrays))(*[_ptr(a) for a in arrays])
    load().nnf_oracle_add(_ptr(out), ptrs, len(arrays), alpha, arrays[0].size, threads)
    return out


def softmax(x, out=None, threads=0):
    x = _f32(x)
    n, c, plane = _shape3(x)
    out = _out_for(x, out)
    load().nnf_oracle_softmax(_ptr(out), _ptr(x), n, c, plane, threads)
    return out


def average_subsampling(x, window_sizes, feature_map_window=1, entry_window=1, mult=None, alpha=None, threads=0):
    """x: [N][C][d_last]...[d_0] (numpy order, x last). window_sizes: per spatial dimension in
    nnForge order (x first). mult None: the plain tester's own multiplier (see the C file)."""
    x = _f32(x)
    dims = list(x.shape[2:])[::-1]  # nnForge order: x first
    if not dims:
        dims = [1]
    window_sizes = list(window_sizes)
    assert len(window_sizes) == len(dims)
    out_dims = [d // w for d, w in zip(dims, window_sizes)]
    n_out = x.shape[0] // entry_window
    c_out = x.shape[1] // feature_map_window
    if mult is None:
        mult = load().nnf_oracle_average_subsampling_plain_mult(feature_map_window, entry_window, int(alpha is not None),
                                                                 float(alpha or 0.0))
    out = np.empty([n_out, c_out] + out_dims[::-1], dtype=np.float32)
    arr = lambda v: (ctypes.c_uint * len(v))(*v)
    load().nnf_oracle_average_subsampling(_ptr(out), _ptr(x), n_out, x.shape[1], c_out, len(dims), arr(dims), arr(out_dims),
                                          arr(window_sizes), feature_map_window, entry_window, mult, threads)
    return out


def average_subsampling_full_mult(window_sizes, feature_map_window=1, entry_window=1, alpha=None):
    w = list(window_sizes)
    return load().nnf_oracle_average_subsampling_full_mult(len(w), (ctypes.c_uint * len(w))(*w), feature_map_window,
                                                           entry_window, int(alpha is not None), float(alpha or 0.0))


def absolute(x, out=None, threads=0):
    x = _f32(x)
    out = _out_for(x, out)
    load().nnf_oracle_absolute(_ptr(out), _ptr(x), x.size, threads)
    return out


def dropout(x, out=None):
    x = _f32(x)
    out = _out_for(x, out)
    load().nnf_oracle_dropout(_ptr(out), _ptr(x), x.size)
    return out


def concat(inputs):
    """inputs: arrays [N][C_i][spatial...] with equal N and spatial sizes; joined along feature maps."""
    arrays = [_f32(a) for a in inputs]
    n = arrays[0].shape[0]
    assert all(a.shape[0] == n and a.shape[2:] == arrays[0].shape[2:] for a in arrays)
    counts = [a.size // n if n else 0 for a in arrays]
    out = np.empty((n, sum(a.shape[1] for a in arrays)) + arrays[0].shape[2:], dtype=np.float32)
    ptrs = (_FP * len(arrays))(*[_ptr(a) for a in arrays])
    load().nnf_oracle_concat(_ptr(out), ptrs, (ctypes.c_uint * len(counts))(*counts), len(arrays), n)
    return out


def maxout(x, feature_map_subsampling_size, threads=0):
    x = _f32(x)
    n, c, plane = _shape3(x)
    assert c % feature_map_subsampling_size == 0
    c_out = c // feature_map_subsampling_size
    out = np.empty((n, c_out) + x.shape[2:], dtype=np.float32)
    load().nnf_oracle_maxout(_ptr(out), _ptr(x), n, c_out, plane, feature_map_subsampling_size, threads)
    return out


def max_subsampling_output_sizes(dims, window_sizes, strides=None, round_ups=None, tiling=False):
    """nnForge order (x first); nnforge/max_subsampling_layer.cpp:119-141."""
    strides = list(strides) if strides else list(window_sizes)
    round_ups = list(round_ups) if round_ups else [False] * len(dims)
    if tiling:
        return [(d - (w - 1)) // w for d, w in zip(dims, window_sizes)]
    return [(d + s - w + (w - 1 if r else 0)) // s for d, w, s, r in zip(dims, window_sizes, strides, round_ups)]


def max_subsampling(x, window_sizes, strides=None, round_ups=None, feature_map_window=1, entry_window=1, is_min=False,
                    tiling=False, threads=0):
    """x: [N][C][d_last]...[d_0]; window_sizes, strides, round_ups per spatial dimension, x first."""
    x = _f32(x)
    dims = list(x.shape[2:])[::-1]
    if not dims:
        dims = [1]
    window_sizes = list(window_sizes)
    assert len(window_sizes) == len(dims)
    strides = list(strides) if strides else list(window_sizes)
    out_dims = max_subsampling_output_sizes(dims, window_sizes, strides, round_ups, tiling)
    assert all(o > 0 for o in out_dims)
    arr = lambda v: (ctypes.c_uint * len(v))(*v)
    if tiling:
        assert feature_map_window == 1 and entry_window == 1 and not (round_ups and any(round_ups))
        tiles = int(np.prod(window_sizes))
        out = np.empty([x.shape[0] * tiles, x.shape[1]] + out_dims[::-1], dtype=np.float32)
        load().nnf_oracle_max_subsampling_tiling(_ptr(out), _ptr(x), x.shape[0], x.shape[1], len(dims), arr(dims), arr(out_dims),
                                                 arr(window_sizes), int(is_min), threads)
        return out
    n_out = x.shape[0] // entry_window
    c_out = x.shape[1] // feature_map_window
    out = np.empty([n_out, c_out] + out_dims[::-1], dtype=np.float32)
    truncate = int(bool(round_ups) and any(round_ups))
    load().nnf_oracle_max_subsampling(_ptr(out), _ptr(x), n_out, x.shape[1], c_out, len(dims), arr(dims), arr(out_dims),
                                      arr(window_sizes), arr(strides), feature_map_window, entry_window, int(is_min), truncate,
                                      threads)
    return out


class RunningStat(ctypes.Structure):
    """nnforge/stat_data_bunch_writer.h:45-63"""
    _fields_ = [("n", ctypes.c_double), ("mean", ctypes.c_double), ("m2", ctypes.c_double),
                ("min_val", ctypes.c_float), ("max_val", ctypes.c_float)]


STAT_DTYPE = np.dtype([("n", "<f8"), ("mean", "<f8"), ("m2", "<f8"), ("min_val", "<f4"), ("max_val", "<f4")])


class FeatureMapStat:
    """stat_data_bunch_writer for one layer: write() batches of entries, then get()."""

    def __init__(self, feature_map_count):
        self.state = np.zeros(feature_map_count, dtype=STAT_DTYPE)
        load().nnf_oracle_feature_map_stat_init(self.state.ctypes.data_as(ctypes.c_void_p), feature_map_count)

    def write(self, x, threads=0):
        x = _f32(x)
        n, c, plane = _shape3(x)
        assert c == self.state.size
        load().nnf_oracle_feature_map_stat_write(self.state.ctypes.data_as(ctypes.c_void_p), _ptr(x), n, c, plane, threads)
        return self

    def get(self):
        """{'min', 'max', 'average', 'std_dev'}: float32 arrays per feature map"""
        c = self.state.size
        res = {k: np.empty(c, dtype=np.float32) for k in ("min", "max", "average", "std_dev")}
        load().nnf_oracle_feature_map_stat_get(self.state.ctypes.data_as(ctypes.c_void_p), c, _ptr(res["min"]), _ptr(res["max"]),
                                               _ptr(res["average"]), _ptr(res["std_dev"]))
        return res


def update_bn_weights(mean, inverse_sigma, average, std_dev):
    """Returns the refreshed (mean, inverse_sigma)."""
    m, s = _f32(mean).copy(), _f32(inverse_sigma).copy()
    load().nnf_oracle_update_bn_weights(_ptr(m), _ptr(s), _ptr(_f32(average)), _ptr(_f32(std_dev)), m.size)
    return m, s
