"""GPU parity of the layers next to the hot path in the same chains: Absolute, Dropout (inference),
Concat, Maxout and MaxSubsampling, through the C ABI against the CPU oracle. All of it is selection
and copying, so the bar is bit equality - including which of +0.0 / -0.0 wins a tie, what NaN does
and the -1.0e37F start value of the pooling fold."""

import ctypes

import numpy as np
import pytest

import nnf_testing as T
import oracle
from nnforge_amd import capi

pytestmark = pytest.mark.gpu

F = np.float32


def u32(values):
    return (ctypes.c_uint32 * max(1, len(values)))(*values)


def spiced(gen, shape, scale=3.0):
    """Normal data with the values that make max/min order-dependent sprinkled in."""
    x = T.normal(gen, shape, scale)
    flat = x.reshape(-1)
    idx = gen.integers(0, flat.size, size=max(4, flat.size // 7))
    flat[idx] = gen.choice(np.array([0.0, -0.0, np.nan, np.inf, -np.inf, -3.0e38, 3.0e38, 1.0], F), size=idx.size)
    return x


def run_flat(gpu, fn, x, in_place=False):
    d_x = gpu.to_device(x)
    d_out = d_x if in_place else gpu.torch.full((x.size,), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    rc = fn(gpu.stream, d_out.data_ptr(), d_x.data_ptr(), x.size)
    assert rc == 0, capi.error_string(rc)
    return gpu.to_host(d_out, x.shape)


@pytest.mark.parametrize("size", [1, 5, 4096, 100003, 1 << 22])
def test_absolute_and_dropout(gpu, size):
    x = spiced(T.rng(60, size), (size,))
    got = run_flat(gpu, gpu.lib.nnf_hip_absolute_forward, x)
    assert T.bit_mismatches(got, oracle.absolute(x)) == 0
    assert T.bit_mismatches(run_flat(gpu, gpu.lib.nnf_hip_absolute_forward, x, in_place=True), oracle.absolute(x)) == 0
    assert T.bit_mismatches(run_flat(gpu, gpu.lib.nnf_hip_dropout_forward, x), oracle.dropout(x)) == 0
    assert T.bit_mismatches(run_flat(gpu, gpu.lib.nnf_hip_dropout_forward, x, in_place=True), x) == 0


def test_absolute_and_dropout_inside_a_fused_group(gpu):
    """BatchNorm -> Absolute -> Dropout -> ReLU as one launch equals the layers one by one."""
    gen = T.rng(61, 0)
    n, c, plane = 3, 10, 28 * 28
    x = T.normal(gen, (n, c, plane), 2.0)
    g, b, m, s = T.bn_params(gen, c)
    want = oracle.rectified_linear(oracle.dropout(oracle.absolute(oracle.batch_norm(x, g, b, m, s))), 0.0)
    arms = [[(capi.OP_BATCH_NORM, 0), (capi.OP_ABSOLUTE,), (capi.OP_DROPOUT,), (capi.OP_RELU, 0, 0.0)]]
    got = gpu.chain((n, c, plane), arms, [], [x], [g, b, m, s])
    assert T.bit_mismatches(got.reshape(x.shape), want) == 0


def run_concat(gpu, parts, expect=0):
    n = parts[0].shape[0]
    d_in = [gpu.to_device(p) for p in parts]
    counts = [p.size // n for p in parts]
    total = sum(counts) * n
    d_out = gpu.torch.full((total,), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    rc = gpu.lib.nnf_hip_concat_forward(gpu.stream, d_out.data_ptr(), capi.pointer_array([t.data_ptr() for t in d_in]),
                                        u32(counts), len(parts), n)
    assert rc == expect, capi.error_string(rc)
    return gpu.to_host(d_out, (n, sum(p.shape[1] for p in parts)) + parts[0].shape[2:])


@pytest.mark.parametrize("n,fms,spatial", [
    (32, (64, 128, 32, 32), (28, 28)),     # an inception-style join
    (5, (3, 7), (5, 3)),                   # lengths not multiples of 4: scalar path
    (2, (1,), (1,)),
    (70000, (2, 2), (2,)),                 # more entries than grid rows
    (3, tuple(range(1, 12)), (4,)),        # 11 inputs: two launches
    (4, (8, 0, 8), (4, 4)),                # an input without feature maps
])
def test_concat(gpu, n, fms, spatial):
    gen = T.rng(62, n + len(fms))
    parts = [spiced(gen, (n, c) + spatial) if c else np.zeros((n, 0) + spatial, F) for c in fms]
    got = run_concat(gpu, parts)
    want = oracle.concat(parts)
    assert got.shape == want.shape
    assert T.bit_mismatches(got, want) == 0


def run_maxout(gpu, x, k, expect=0):
    n, c = x.shape[:2]
    plane = int(np.prod(x.shape[2:], dtype=np.int64))
    d_in = gpu.to_device(x)
    out_shape = (n, c // k) + x.shape[2:]
    d_out = gpu.torch.full((int(np.prod(out_shape)),), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    rc = gpu.lib.nnf_hip_maxout_forward(gpu.stream, d_out.data_ptr(), d_in.data_ptr(), n, c // k, plane, k)
    assert rc == expect, capi.error_string(rc)
    return gpu.to_host(d_out, out_shape)


@pytest.mark.parametrize("shape,k", [
    ((32, 256, 14, 14), 2),
    ((8, 96, 7, 7), 3),        # group 32*49 is a multiple of 4
    ((5, 15, 3, 3), 5),        # scalar path
    ((1, 2, 1), 2),
    ((66000, 4, 2), 2),        # more entries than grid rows
])
def test_maxout(gpu, shape, k):
    x = spiced(T.rng(63, sum(shape)), shape)
    got = run_maxout(gpu, x, k)
    want = oracle.maxout(x, k)
    assert T.bit_mismatches(got, want) == 0


def run_max_subsampling(gpu, x, windows, strides=None, round_ups=None, fm=1, en=1, is_min=False, expect=0):
    """windows / strides / round_ups in nnForge order (x first)."""
    dims = list(x.shape[2:])[::-1]
    want_shape = None
    d_in = gpu.to_device(x)
    out_dims = oracle.max_subsampling_output_sizes(dims, windows, strides, round_ups)
    want_shape = (x.shape[0] // en, x.shape[1] // fm) + tuple(out_dims[::-1])
    d_out = gpu.torch.full((max(1, int(np.prod(want_shape))),), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    rc = gpu.lib.nnf_hip_max_subsampling_forward(
        gpu.stream, d_out.data_ptr(), d_in.data_ptr(), x.shape[0] // en, x.shape[1], len(dims), u32(dims), u32(windows),
        u32(strides) if strides else None, u32([int(r) for r in round_ups]) if round_ups else None, fm, en, int(is_min))
    assert rc == expect, capi.error_string(rc)
    if expect != 0:
        return None
    return gpu.to_host(d_out, want_shape)


POOL_CASES = [
    # shape, windows (x first), strides, round_ups
    ((32, 64, 112, 112), [3, 3], [2, 2], None),              # ResNet pool1 as nnForge computes it: 55x55
    ((4, 64, 112, 112), [3, 3], [2, 2], [True, True]),       # 56x56, the last window cut off
    ((8, 96, 55, 55), [3, 3], [2, 2], None),                 # AlexNet-style overlapping pooling
    ((16, 32, 28, 28), [2, 2], None, None),                  # whole planes per workgroup
    ((7, 5, 13, 13), [3, 3], [2, 2], [True, True]),          # many small planes per workgroup, odd counts
    ((3, 3, 9, 31), [5, 2], [3, 1], [True, False]),          # run-time window sizes
    ((2, 2, 300, 200), [4, 7], [4, 5], None),                # bands of a large plane
    ((2, 3, 4, 4000), [3, 2], [2, 2], None),                 # very wide rows: one output row per band
    ((2, 2, 3, 20000), [2, 3], [2, 1], None),                # rows too wide for LDS: general kernel
    ((5, 6, 37), [4], [3], [True]),                          # 1-D
    ((1, 1, 1, 1), [1, 1], None, None),
    ((2, 3, 6, 7, 8), [2, 3, 2], [2, 2, 1], None),           # 3-D: general kernel
    ((2, 2, 3, 4, 5, 6), [2, 2, 2, 2], [1, 2, 1, 2], [True, False, True, False]),  # 4-D
]


@pytest.mark.parametrize("is_min", [False, True])
@pytest.mark.parametrize("shape,windows,strides,round_ups", POOL_CASES)
def test_max_subsampling(gpu, shape, windows, strides, round_ups, is_min):
    x = spiced(T.rng(64, sum(shape)), shape)
    got = run_max_subsampling(gpu, x, windows, strides, round_ups, is_min=is_min)
    want = oracle.max_subsampling(x, windows, strides=strides, round_ups=round_ups, is_min=is_min)
    assert got.shape == want.shape
    assert T.bit_mismatches(got, want) == 0


@pytest.mark.parametrize("fm,en", [(3, 1), (1, 2), (2, 3)])
def test_max_subsampling_over_feature_maps_and_entries(gpu, fm, en):
    x = spiced(T.rng(65, fm * 10 + en), (6, 12, 9, 10))
    got = run_max_subsampling(gpu, x, [2, 3], [2, 2], None, fm=fm, en=en)
    want = oracle.max_subsampling(x, [2, 3], strides=[2, 2], feature_map_window=fm, entry_window=en)
    assert got.shape == want.shape
    assert T.bit_mismatches(got, want) == 0


def test_neighbour_entry_points_reject_bad_arguments(gpu):
    lib, s = gpu.lib, gpu.stream
    d = gpu.to_device(np.zeros(256, F))
    e = gpu.to_device(np.zeros(256, F))
    # max subsampling: 5 dimensions, zero stride, window larger than the input, in place
    assert lib.nnf_hip_max_subsampling_forward(s, e.data_ptr(), d.data_ptr(), 1, 1, 5, u32([2] * 5), u32([1] * 5), None, None, 1, 1, 0) == capi.E_UNSUPPORTED
    assert lib.nnf_hip_max_subsampling_forward(s, e.data_ptr(), d.data_ptr(), 1, 1, 2, u32([8, 8]), u32([2, 2]), u32([0, 2]), None, 1, 1, 0) == capi.E_INVAL
    assert lib.nnf_hip_max_subsampling_forward(s, e.data_ptr(), d.data_ptr(), 1, 1, 2, u32([4, 4]), u32([5, 2]), u32([7, 2]), None, 1, 1, 0) == capi.E_INVAL
    assert lib.nnf_hip_max_subsampling_forward(s, d.data_ptr(), d.data_ptr(), 1, 1, 2, u32([8, 8]), u32([2, 2]), None, None, 1, 1, 0) == capi.E_OVERLAP
    assert lib.nnf_hip_max_subsampling_forward(s, e.data_ptr() + 4, d.data_ptr(), 1, 1, 2, u32([8, 8]), u32([2, 2]), None, None, 1, 1, 0) == capi.E_ALIGN
    # maxout: group size below 2, in place
    assert lib.nnf_hip_maxout_forward(s, e.data_ptr(), d.data_ptr(), 1, 4, 4, 1) == capi.E_INVAL
    assert lib.nnf_hip_maxout_forward(s, d.data_ptr(), d.data_ptr(), 1, 4, 4, 2) == capi.E_OVERLAP
    # concat: no inputs, output overlapping an input
    assert lib.nnf_hip_concat_forward(s, e.data_ptr(), capi.pointer_array([]), u32([]), 0, 1) == capi.E_INVAL
    assert lib.nnf_hip_concat_forward(s, d.data_ptr(), capi.pointer_array([d.data_ptr()]), u32([16]), 1, 2) == capi.E_OVERLAP
    # zero entries: nothing to do
    assert lib.nnf_hip_concat_forward(s, e.data_ptr(), capi.pointer_array([d.data_ptr()]), u32([16]), 1, 0) == 0
    assert lib.nnf_hip_maxout_forward(s, e.data_ptr(), d.data_ptr(), 0, 4, 4, 2) == 0
    gpu.torch.cuda.synchronize()
