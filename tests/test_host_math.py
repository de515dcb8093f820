"""The kernels' scalar formulas (nnforge_amd/csrc/nnf_math.h), compiled for the host, against libm
and against the oracle: pins the arithmetic of the device code without a GPU."""

import ctypes
import os
import subprocess

import numpy as np
import pytest

import nnf_testing as T
import oracle

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host_math")
_FP = ctypes.POINTER(ctypes.c_float)


@pytest.fixture(scope="module")
def host():
    proc = subprocess.run(["make", "-C", HERE], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout
    lib = ctypes.CDLL(os.path.join(HERE, "libnnf_math_host.so"))
    lib.nnf_host_expf_mismatches.restype = ctypes.c_ulonglong
    lib.nnf_host_expf_mismatches.argtypes = [ctypes.c_ulonglong, ctypes.c_ulonglong, ctypes.c_ulonglong, ctypes.POINTER(ctypes.c_uint32)]
    lib.nnf_host_apply.argtypes = [ctypes.c_int, _FP, _FP, ctypes.c_longlong] + [ctypes.c_float] * 4
    return lib


def test_expf_equals_libm_on_a_sweep_of_all_floats(host):
    """Every 13th fp32 bit pattern (330 million inputs, all exponents, both signs) plus every input
    in the windows where expf leaves the normal range: the double-precision scheme returns libm's
    bits. (All 2^32 inputs were compared once with the same routine: zero mismatches.)"""
    bad = ctypes.c_uint32(0)
    n = host.nnf_host_expf_mismatches(0, 13, (1 << 32) // 13, ctypes.byref(bad))
    assert n == 0, "first differing input bits: 0x%08x" % bad.value
    for centre in (88.72, -87.3, -103.97, 0.0, -0.0):
        first = int(np.array(centre, np.float32).view(np.uint32)) - (1 << 16)
        n = host.nnf_host_expf_mismatches(max(first, 0), 1, 1 << 17, ctypes.byref(bad))
        assert n == 0, "first differing input bits: 0x%08x" % bad.value


def apply(host, kind, x, p=(0.0, 0.0, 0.0, 0.0)):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty_like(x)
    host.nnf_host_apply(kind, out.ctypes.data_as(_FP), x.ctypes.data_as(_FP), x.size, *[float(v) for v in p])
    return out


def test_layer_formulas_equal_the_oracle_bit_for_bit(host):
    gen = T.rng(30, 0)
    x = np.concatenate([T.normal(gen, 200000, 16.0), np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 88.8, -104.0, 50, -50], np.float32)])
    g, b, m, s = 1.3, -0.2, 0.4, 0.9
    one = lambda v: np.array([v], np.float32)
    cases = [
        (1, (g, b, m, s), oracle.batch_norm(x.reshape(1, 1, -1), one(g), one(b), one(m), one(s)).reshape(-1)),
        (2, (0.0,), oracle.rectified_linear(x, 0.0)),
        (2, (0.3,), oracle.rectified_linear(x, 0.3)),
        (3, (0.25,), oracle.parametric_rectified_linear(x.reshape(1, 1, -1), one(0.25)).reshape(-1)),
        (4, (), oracle.exponential_linear(x)),
        (5, (), oracle.sigmoid(x)),
        (6, (1.7159, 0.6666), oracle.hyperbolic_tangent(x, 1.7159, 0.6666)),
        (6, (1.0, 1.0), oracle.hyperbolic_tangent(x, 1.0, 1.0)),
    ]
    for kind, params, want in cases:
        got = apply(host, kind, x, tuple(params) + (0.0,) * (4 - len(params)))
        assert T.bit_mismatches(got, want) == 0, "op kind %d" % kind
