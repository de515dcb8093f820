"""Writes tests/golden/expf_vectors.npy: 8192 fp32 inputs and glibc's expf of them, as bit patterns.

The reference's ELU, Sigmoid, TanH and Softmax testers call libm's expf (nnforge/plain/exponential_linear_layer_tester_plain.cpp:50,
sigmoid_layer_tester_plain.cpp:51, hyperbolic_tangent_layer_tester_plain.cpp:52, softmax_layer_tester_plain.cpp:69); the
reference holds no vectors of its own for them. These were produced by the C library of the image the kernels were
developed in (glibc 2.35, x86-64, through ctypes - no reference code runs here) and pin two things wherever the tests run
later: that the host's expf, which the oracle calls, is still that function, and that the device's expf equals it without
the host's libm being involved at test time.

Inputs: every exponent from 2^-30 to 2^7 with both signs and random mantissas, the range edges of expf (underflow to
subnormals and to zero near -87.3 ... -103.97, overflow at 88.72), zeros, infinities, a NaN.

    python tests/golden/make_expf_vectors.py
"""

import ctypes
import os

import numpy as np


def main():
    libm = ctypes.CDLL("libm.so.6")
    libm.expf.argtypes = [ctypes.c_float]
    libm.expf.restype = ctypes.c_float
    gen = np.random.Generator(np.random.MT19937(20240607))
    values = []
    for exponent in range(-30, 8):
        m = gen.random(96, dtype=np.float32) + np.float32(1.0)
        v = np.ldexp(m, exponent).astype(np.float32)
        values.append(v)
        values.append(-v)
    edges = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 88.72283, 88.72284, 88.7229, 89.0, 128.0, -87.33654, -87.33655, -87.4,
                      -100.0, -103.27892, -103.97207, -103.97208, -103.9721, -104.0, -150.0, 1e-45, -1e-45, 1.17549435e-38, 3.4e38, -3.4e38],
                     dtype=np.float32)
    values.append(edges)
    near = (np.float32(88.0) + gen.random(400, dtype=np.float32)).astype(np.float32)
    values.append(near)
    values.append((np.float32(-86.0) - np.float32(18.5) * gen.random(471, dtype=np.float32)).astype(np.float32))
    x = np.concatenate(values)[:8192]
    assert x.size == 8192, x.size
    y = np.array([libm.expf(float(v)) for v in x], dtype=np.float32)
    out = np.stack([x.view(np.uint32), y.view(np.uint32)])
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "expf_vectors.npy")
    np.save(path, out)
    print("wrote", path, out.shape, "glibc", os.confstr("CS_GNU_LIBC_VERSION"))


if __name__ == "__main__":
    main()
