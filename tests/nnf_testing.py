"""Shared helpers of the tests: seeded synthetic tensors of the benchmark configurations, ULP
distances, and a thin harness that runs the C ABI on torch-allocated device memory."""

import ctypes

import numpy as np

from nnforge_amd import capi

BASE_SEED = 0x6E6E4600

TANH_SCALE = 1.7159
TANH_STEEPNESS = 0.6666


def rng(config_id, tensor_id):
    return np.random.Generator(np.random.MT19937(BASE_SEED + 16 * config_id + tensor_id))


def normal(gen, shape, variance=1.0):
    return (gen.standard_normal(shape, dtype=np.float32) * np.float32(np.sqrt(variance))).astype(np.float32)


def uniform(gen, shape, lo, hi):
    return (gen.random(shape, dtype=np.float32) * np.float32(hi - lo) + np.float32(lo)).astype(np.float32)


def bn_params(gen, c, eps=1e-5):
    """gamma~U(0.5,1.5), beta~N(0,0.1), mean~N(0,0.1), variance~U(0.5,2.0); chunk 3 of nnForge's
    batch_norm_layer is the inverse standard deviation, computed here once in fp32."""
    gamma = uniform(gen, c, 0.5, 1.5)
    beta = normal(gen, c, 0.1)
    mean = normal(gen, c, 0.1)
    var = uniform(gen, c, 0.5, 2.0)
    inv_sigma = (np.float32(1.0) / np.sqrt(var + np.float32(eps), dtype=np.float32)).astype(np.float32)
    return gamma, beta, mean, inv_sigma


def ordered_bits(a):
    """Maps fp32 bit patterns to integers ordered like the floats (-0 and +0 coincide)."""
    b = np.ascontiguousarray(a, dtype=np.float32).view(np.int32).astype(np.int64)
    return np.where(b < 0, np.int64(-0x80000000) - b, b)


def ulp_distance(a, b):
    """Element-wise distance in units in the last place; 0 where both are NaN, huge where one is."""
    a = np.asarray(a, dtype=np.float32)
    b = np.asarray(b, dtype=np.float32)
    d = np.abs(ordered_bits(a) - ordered_bits(b))
    both_nan = np.isnan(a) & np.isnan(b)
    one_nan = np.isnan(a) ^ np.isnan(b)
    d = np.where(both_nan, 0, d)
    d = np.where(one_nan, np.int64(1) << 40, d)
    return d


def bit_mismatches(a, b):
    """Number of elements whose bit patterns differ (NaN == NaN; +0 and -0 are different)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    diff = a.view(np.uint32) != b.view(np.uint32)
    diff &= ~(np.isnan(a) & np.isnan(b))
    return int(diff.sum())


def assert_close_elementwise(got, want, ulps=2, rel=1e-6, what=""):
    """The element-wise bar: |got - want| <= max(ulps ULP, rel * |want|)."""
    got = np.asarray(got, dtype=np.float32)
    want = np.asarray(want, dtype=np.float32)
    assert got.shape == want.shape, (got.shape, want.shape)
    d_ulp = ulp_distance(got, want)
    with np.errstate(invalid="ignore", over="ignore"):
        abs_err = np.abs(got.astype(np.float64) - want.astype(np.float64))
        ok = (d_ulp <= ulps) | (abs_err <= rel * np.abs(want.astype(np.float64)))
    if not ok.all():
        idx = np.flatnonzero(~ok.ravel())[:5]
        raise AssertionError("%s: %d of %d elements outside max(%d ulp, %g rel); first: %s" % (
            what, int((~ok).sum()), ok.size, ulps, rel,
            [(int(i), float(got.ravel()[i]), float(want.ravel()[i])) for i in idx]))


class GpuHarness:
    """Runs the C ABI on device memory owned by torch tensors (torch is only the allocator)."""

    def __init__(self, lib):
        import torch

        self.torch = torch
        self.lib = lib
        self.device = torch.device("cuda:0")
        torch.cuda.set_device(0)

    @property
    def stream(self):
        return self.torch.cuda.current_stream().cuda_stream

    def to_device(self, array):
        t = self.torch.from_numpy(np.ascontiguousarray(array, dtype=np.float32)).to(self.device)
        assert t.data_ptr() % 16 == 0
        return t

    def empty_like(self, array):
        return self.torch.empty(int(np.asarray(array).size) if not hasattr(array, "numel") else array.numel(),
                                dtype=self.torch.float32, device=self.device)

    def to_host(self, tensor, shape=None):
        self.torch.cuda.synchronize()
        a = tensor.cpu().numpy()
        return a.reshape(shape) if shape is not None else a

    def chain(self, shape3, arms, tail, inputs, chunks=(), has_add=None, alpha=1.0, in_place=False, expect=0):
        """shape3 = (entry_count, feature_map_count, plane). inputs/chunks: numpy arrays.
        Returns the output as a numpy array (flat)."""
        n, c, plane = shape3
        desc = capi.make_desc(n, c, plane, arms, tail, has_add=has_add, add_alpha=alpha)
        d_in = [self.to_device(a) for a in inputs]
        d_chunks = [self.to_device(a) for a in chunks]
        d_out = d_in[0] if in_place else self.torch.full((n * c * plane,), float("nan"), dtype=self.torch.float32, device=self.device)
        ins = capi.pointer_array([t.data_ptr() for t in d_in])
        chk = capi.pointer_array([t.data_ptr() for t in d_chunks])
        rc = self.lib.nnf_hip_chain_forward(self.stream, ctypes.byref(desc), d_out.data_ptr(), ins, chk if d_chunks else None)
        assert rc == expect, capi.error_string(rc)
        return self.to_host(d_out)


def _chain_batch(self, groups, in_place=None):
    """groups: [(shape3, arms, tail, inputs, chunks, has_add, alpha)]; one nnf_hip_chain_forward_batch call.
    in_place[i]: group i writes over its first input. Returns the outputs as flat numpy arrays."""
    count = len(groups)
    descs = (capi.ChainDesc * count)()
    keep, outs, in_arrays, chunk_arrays = [], [], [], []
    for i, (shape3, arms, tail, inputs, chunks, has_add, alpha) in enumerate(groups):
        n, c, plane = shape3
        descs[i] = capi.make_desc(n, c, plane, arms, tail, has_add=has_add, add_alpha=alpha)
        # a tensor without elements still needs an address to hand over
        d_in = [self.to_device(a) if a.size else self.torch.empty(4, dtype=self.torch.float32, device=self.device) for a in inputs]
        d_chunks = [self.to_device(a) for a in chunks]
        if in_place is not None and in_place[i]:
            d_out = d_in[0]
        else:
            d_out = self.torch.full((max(4, n * c * plane),), float("nan"), dtype=self.torch.float32, device=self.device)
        keep.append((d_in, d_chunks, d_out))
        outs.append(d_out)
        in_arrays.append(capi.pointer_array([t.data_ptr() for t in d_in]))
        chunk_arrays.append(capi.pointer_array([t.data_ptr() for t in d_chunks]) if d_chunks else None)
    pp = ctypes.POINTER(ctypes.c_void_p)
    in_ptrs = (pp * count)(*[ctypes.cast(a, pp) for a in in_arrays])
    chunk_ptrs = (pp * count)(*[ctypes.cast(a, pp) if a is not None else pp() for a in chunk_arrays])
    rc = self.lib.nnf_hip_chain_forward_batch(self.stream, count, descs, capi.pointer_array([t.data_ptr() for t in outs]), in_ptrs, chunk_ptrs)
    assert rc == 0, capi.error_string(rc)
    self.torch.cuda.synchronize()
    return [t.cpu().numpy()[:g[0][0] * g[0][1] * g[0][2]] for t, g in zip(outs, groups)]


GpuHarness.chain_batch = _chain_batch


def golden_expf():
    """(x, expf(x)) of tests/golden/expf_vectors.npy: 8192 inputs and glibc 2.35's expf of them (see make_expf_vectors.py)."""
    import os

    data = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "expf_vectors.npy"))
    return data[0].view(np.float32).copy(), data[1].view(np.float32).copy()


def layers_from_golden_expf(x, e):
    """What ELU, Sigmoid(-x) and TanH(steepness 0.5, scale 1) must return for inputs x whose expf is e, by the reference's
    formulas in IEEE fp32 operations (numpy float32 arithmetic rounds once per operation):
    nnforge/plain/exponential_linear_layer_tester_plain.cpp:50, sigmoid_layer_tester_plain.cpp:51,
    hyperbolic_tangent_layer_tester_plain.cpp:49-55."""
    one = np.float32(1.0)
    with np.errstate(all="ignore"):
        elu = np.where(x >= 0, x, e - one).astype(np.float32)
        elu = np.where(np.isnan(x), (e - one), elu).astype(np.float32)  # NaN >= 0 is false: the expf branch
        sigmoid_of_minus_x = (one / (e + one)).astype(np.float32)
        tanh = (((e - one) / (e + one)) * one).astype(np.float32)
    return elu, sigmoid_of_minus_x, tanh

