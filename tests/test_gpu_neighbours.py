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


@pytest.mark.parametrize("flags", [(1, 0, 1, 0), (0, 0, 0, 1), (1, 1, 1, 1), (0, 0, 0, 0), (0, 1, 1, 0, 1, 0, 1, 1, 0, 1)])
def test_concat_with_inputs_already_in_place(gpu, flags):
    """nnf_hip_concat_forward_partial: the inputs flagged as in place are not copied (their pointers are null here) and keep
    what lies in their parts of the output; the others are copied to theirs."""
    gen = T.rng(62, sum(flags) + len(flags))
    n, plane = 7, 36
    fms = [int(gen.integers(1, 9)) for _ in flags]
    parts = [spiced(gen, (n, c, plane)) for c in fms]
    want = oracle.concat(parts)
    there = np.full_like(want, np.float32(-3.5))
    offset = 0
    for part, flag, c in zip(parts, flags, fms):
        if flag:
            there[:, offset:offset + c] = part
        offset += c
    d_out = gpu.to_device(there)
    d_parts = [gpu.to_device(p) for p in parts]
    ptrs = capi.pointer_array([0 if flag else t.data_ptr() for t, flag in zip(d_parts, flags)])
    rc = gpu.lib.nnf_hip_concat_forward_partial(gpu.stream, d_out.data_ptr(), ptrs, u32([c * plane for c in fms]),
                                                (ctypes.c_uint8 * len(flags))(*flags), len(flags), n)
    assert rc == 0, capi.error_string(rc)
    assert T.bit_mismatches(gpu.to_host(d_out, want.shape), want) == 0


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
    ((64, 512, 14, 14), 2),    # the benchmark's shape
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
    ((64, 64, 112, 112), [3, 3], [2, 2], [True, True]),      # ... at the size of the ResNet-50 stem with 64 entries
    ((8, 96, 55, 55), [3, 3], [2, 2], None),                 # AlexNet-style overlapping pooling
    ((16, 32, 28, 28), [2, 2], None, None),                  # whole planes per workgroup
    ((7, 5, 13, 13), [3, 3], [2, 2], [True, True]),          # many small planes per workgroup, odd counts
    ((6, 5, 10, 12), [3, 3], [2, 2], [True, True]),          # ... with rows of whole float4s: two outputs per lane at a time, the last pair's window cut off
    ((3, 7, 9, 8), [2, 2], None, None),                      # ... 2x2 windows, an input row left over
    ((2, 3, 6, 16), [3, 3], [2, 2], [True, False]),          # rounded up in x only
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


TILING_CASES = [
    # shape, windows (x first)
    ((3, 4, 9, 11), [2, 3]),              # 6 output entries per input entry
    ((2, 3, 7, 5), [2, 2]),               # the smallest sizes some windows allow: 5 >= 2 * 2 - 1... and margins left over
    ((5, 2, 23), [4]),                    # 1-D
    ((2, 2, 5, 6, 9), [3, 2, 2]),         # 3-D
    ((1, 2, 3, 5, 4, 7), [2, 2, 2, 1]),   # 4-D, a window of 1 in one dimension
    ((4, 8, 28, 28), [2, 2]),             # four planes of an entry per workgroup, one run per grid
    ((2, 6, 30, 30), [2, 2]),             # three of six
    ((3, 4, 21, 19), [3, 2]),             # planes of an odd number of floats: staged from an unaligned start
    ((5, 12, 56, 56), [2, 2]),            # one plane per workgroup, neighbouring planes on one die
    ((2, 1, 3, 3), [1, 1]),               # one tile: plain copy
    ((7, 37, 6, 5), [2, 2]),              # 259 small planes: 256 in the first workgroup, 3 in the second
    ((1, 2, 200, 300), [3, 2]),           # bands of a large plane
    ((2, 3, 112, 112), [3, 3]),           # a whole plane per workgroup
    ((64, 64, 112, 112), [2, 2]),         # the benchmark's shape: 256 output entries of 55 x 55
    ((2, 5, 112, 112), [2, 2]),           # ten planes in five bands each: 40 workgroups regrouped by die, the last 10 in plain order
    ((1, 3, 100, 96), [2, 2]),            # strips of four columns, bands of unequal height
    ((3, 7, 90, 120), [2, 2]),
    ((1, 1, 5000, 4), [2, 2]),            # rows of one strip
    ((2, 9, 200, 300), [3, 2]),           # bands regrouped by die in the general kernel
    ((2, 1, 5, 20000), [2, 2]),           # rows too wide to stage: one lane per output
    ((3, 2, 40000), [3]),                 # 1-D, wide
]


@pytest.mark.parametrize("is_min", [False, True])
@pytest.mark.parametrize("shape,windows", TILING_CASES)
def test_max_subsampling_with_tiling(gpu, shape, windows, is_min):
    """nnforge/plain/max_subsampling_layer_tester_plain.cpp:78-170: every shift of the window grid is an output entry."""
    x = spiced(T.rng(66, sum(shape) + len(windows)), shape)
    want = oracle.max_subsampling(x, windows, tiling=True, is_min=is_min)
    assert want.shape[0] == shape[0] * int(np.prod(windows))
    dims = list(shape[2:])[::-1]
    d_in = gpu.to_device(x)
    d_out = gpu.torch.full((want.size,), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    rc = gpu.lib.nnf_hip_max_subsampling_tiling_forward(gpu.stream, d_out.data_ptr(), d_in.data_ptr(), shape[0], shape[1], len(dims),
                                                        u32(dims), u32(windows), int(is_min))
    assert rc == 0, capi.error_string(rc)
    got = gpu.to_host(d_out, want.shape)
    assert T.bit_mismatches(got, want) == 0
    # tile 0 is the plain layer with the window as its stride, cut to the tiling's output sizes
    plain = oracle.max_subsampling(x, windows, is_min=is_min)
    tile0 = got.reshape((shape[0], -1) + got.shape[1:])[:, 0]
    cut = (slice(None), slice(None)) + tuple(slice(0, n) for n in got.shape[2:])
    assert T.bit_mismatches(tile0, plain[cut]) == 0


@pytest.mark.parametrize("is_min", [False, True])
@pytest.mark.parametrize("shape,fm,en", [
    ((8, 6, 16, 16, 2), 1, 4),       # 3-D so that the staged 2-D kernel stays out: entries folded as rows of float4
    ((4, 13, 16, 20, 1), 3, 2),      # planes as rows, a feature map left over
    ((6, 12, 9, 10, 1), 1, 3),       # planes of 90 values, entries of 1080
    ((6, 12, 9, 10, 1), 4, 1),       # planes of 90 values with a window over feature maps: one lane per output
    ((6, 12, 16, 16), 2, 3),         # 2-D
])
def test_max_subsampling_over_feature_maps_and_entries_only(gpu, shape, fm, en, is_min):
    x = spiced(T.rng(67, sum(shape) + fm), shape)
    ones = [1] * (len(shape) - 2)
    got = run_max_subsampling(gpu, x, ones, None, None, fm=fm, en=en, is_min=is_min)
    want = oracle.max_subsampling(x, ones, feature_map_window=fm, entry_window=en, is_min=is_min)
    assert got.shape == want.shape
    assert T.bit_mismatches(got, want) == 0
    # the same thing said with numpy: fold over the entry and feature-map axes
    c_out = shape[1] // fm
    folded = x[:, :c_out * fm].reshape((shape[0] // en, en, c_out, fm) + shape[2:])
    with np.errstate(invalid="ignore"):
        # the fold starts at -+1.0e37F, which bounds the result
        ref = np.minimum(folded.min(axis=(1, 3)), F(1.0e37)) if is_min else np.maximum(folded.max(axis=(1, 3)), F(-1.0e37))
    plain = ~np.isnan(ref)    # windows without NaN (the reference's fold skips NaN, numpy's does not)
    assert np.array_equal(got[plain], ref[plain])


def test_neighbour_entry_points_reject_bad_arguments(gpu):
    lib, s = gpu.lib, gpu.stream
    d = gpu.to_device(np.zeros(256, F))
    e = gpu.to_device(np.zeros(256, F))
    # tiling: an input below 2 * window - 1, 5 dimensions, in place
    assert lib.nnf_hip_max_subsampling_tiling_forward(s, e.data_ptr(), d.data_ptr(), 1, 1, 2, u32([8, 4]), u32([2, 3]), 0) == capi.E_INVAL
    assert lib.nnf_hip_max_subsampling_tiling_forward(s, e.data_ptr(), d.data_ptr(), 1, 1, 5, u32([2] * 5), u32([1] * 5), 0) == capi.E_UNSUPPORTED
    assert lib.nnf_hip_max_subsampling_tiling_forward(s, d.data_ptr(), d.data_ptr(), 1, 1, 2, u32([8, 8]), u32([2, 2]), 0) == capi.E_OVERLAP
    assert lib.nnf_hip_max_subsampling_tiling_forward(s, e.data_ptr(), d.data_ptr(), 0, 1, 2, u32([8, 8]), u32([2, 2]), 0) == 0
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


# ---------------------------------------------------------------------------------------------
# subsampling with the element-wise layers in front of it folded in
# ---------------------------------------------------------------------------------------------

def zero_heavy(gen, shape, negative_share=0.0):
    """Data on which the hardware's maximum and the reference's fold part ways unless the kernels repair it: most
    windows hold nothing above zero, so which zero comes first decides the sign of the result; signalling and
    negative NaNs, denormals (a flushed one would be a zero), values under the fold's start value and infinities
    are mixed in. negative_share: that part of the values is drawn negative normal instead (for data in front of
    a rectified_linear with slope 0, whose results are the -0.0s)."""
    zeros = [0x00000000, 0x80000000]
    nans = [0x7FA00000, 0xFFA00000, 0x7FC00000, 0xFFC00001]                 # signalling and quiet, both signs
    below = [0x80000001, 0x807FFFFF, 0xBF800000, 0xFF800000, 0xFE967699,    # negative denormals, -1.0, -inf, -1.0e38,
             0xFCF0BDC2, 0xFCF0BDC3]                                        # the start value -1.0e37F and one step under it
    above = [0x00000001, 0x007FFFFF, 0x7CF0BDC2, 0x7E967699, 0x7F800000]    # denormals, 1.0e37F, 1.0e38, +inf
    count = int(np.prod(shape))
    kind = gen.random(count)
    pick = lambda values: np.array(values, np.uint32)[gen.integers(0, len(values), size=count)]
    bits = np.where(kind < 0.5, pick(zeros), np.where(kind < 0.65, pick(nans), np.where(kind < 0.92, pick(below), pick(above))))
    x = bits.view(F).copy()
    rare = gen.random(count) < 0.02
    x[rare] = T.normal(gen, (count,), 2.0)[rare]
    if negative_share > 0.0:
        negative = gen.random(count) < negative_share
        x[negative] = -np.abs(T.normal(gen, (count,), 2.0))[negative] - F(1.0e-3)
    return x.reshape(shape)


ZERO_HEAVY_POOL_CASES = [
    ((8, 64, 112, 112), [3, 3], [2, 2], [True, True]),       # two outputs per lane at a time, bands of a plane
    ((8, 16, 55, 55), [3, 3], [2, 2], None),                 # one output per lane, window size known
    ((16, 32, 28, 28), [2, 2], None, None),                  # whole planes per workgroup, pairs of 2x2 windows
    ((3, 3, 9, 31), [5, 2], [3, 1], [True, False]),          # run-time window sizes
    ((5, 6, 37), [4], [3], [True]),                          # 1-D
]


@pytest.mark.parametrize("is_min", [False, True])
@pytest.mark.parametrize("shape,windows,strides,round_ups", ZERO_HEAVY_POOL_CASES)
def test_max_subsampling_where_the_first_zero_decides(gpu, shape, windows, strides, round_ups, is_min):
    """The kernels fold with the hardware's maximum and fold a window again in the reference's order when its result
    is a zero: here most windows need that, and signalling NaNs and denormals lie in between."""
    x = zero_heavy(T.rng(71, sum(shape)), shape)
    if is_min:
        x = -x
    got = run_max_subsampling(gpu, x, windows, strides, round_ups, is_min=is_min)
    want = oracle.max_subsampling(x, windows, strides=strides, round_ups=round_ups, is_min=is_min)
    zeros = float(np.mean(want == 0.0))
    assert zeros > 0.2, zeros  # the case is what it says
    assert T.bit_mismatches(got, want) == 0


@pytest.mark.parametrize("is_min", [False, True])
@pytest.mark.parametrize("shape,windows", [((4, 16, 112, 112), [2, 2]), ((1, 3, 100, 96), [2, 2]), ((2, 3, 60, 60), [3, 3]), ((7, 37, 6, 5), [2, 2]),
                                           ((4, 8, 28, 28), [2, 2]), ((3, 4, 21, 19), [3, 2]),
                                           ((3, 4, 9, 11), [2, 3]), ((5, 2, 23), [4])])
def test_max_subsampling_with_tiling_where_the_first_zero_decides(gpu, shape, windows, is_min):
    x = zero_heavy(T.rng(72, sum(shape)), shape)
    if is_min:
        x = -x
    want = oracle.max_subsampling(x, windows, tiling=True, is_min=is_min)
    assert float(np.mean(want == 0.0)) > 0.2
    dims = list(shape[2:])[::-1]
    d_in = gpu.to_device(x)
    d_out = gpu.torch.full((want.size,), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    rc = gpu.lib.nnf_hip_max_subsampling_tiling_forward(gpu.stream, d_out.data_ptr(), d_in.data_ptr(), shape[0], shape[1], len(dims),
                                                        u32(dims), u32(windows), int(is_min))
    assert rc == 0, capi.error_string(rc)
    assert T.bit_mismatches(gpu.to_host(d_out, want.shape), want) == 0


def prologue_case(kind, gen, c):
    """-> (ops of the single arm, weight chunks, oracle steps) of a group in front of a subsampling layer"""
    if kind == "bn_relu":
        g, b, m, s = T.bn_params(gen, c)
        return ([(capi.OP_BATCH_NORM, 0), (capi.OP_RELU, 0, 0.0)], [g, b, m, s],
                [lambda v: oracle.batch_norm(v, g, b, m, s), lambda v: oracle.rectified_linear(v, 0.0)])
    if kind == "tanh_abs":
        return ([(capi.OP_TANH, 0, 1.7159, 0.6666), (capi.OP_ABSOLUTE,)], [],
                [lambda v: oracle.hyperbolic_tangent(v, 1.7159, 0.6666), oracle.absolute])
    if kind == "bn_prelu_elu_sigmoid":
        g, b, m, s = T.bn_params(gen, c)
        a = T.uniform(gen, c, -0.5, 0.5)
        return ([(capi.OP_BATCH_NORM, 0), (capi.OP_PRELU, 4), (capi.OP_DROPOUT,), (capi.OP_ELU,), (capi.OP_SIGMOID,)], [g, b, m, s, a],
                [lambda v: oracle.batch_norm(v, g, b, m, s), lambda v: oracle.parametric_rectified_linear(v, a),
                 oracle.exponential_linear, oracle.sigmoid])
    if kind == "prelu_bn":
        g, b, m, s = T.bn_params(gen, c)
        a = T.uniform(gen, c, -0.5, 0.5)
        return ([(capi.OP_PRELU, 0), (capi.OP_ABSOLUTE,), (capi.OP_BATCH_NORM, 1)], [a, g, b, m, s],
                [lambda v: oracle.parametric_rectified_linear(v, a), oracle.absolute, lambda v: oracle.batch_norm(v, g, b, m, s)])
    if kind == "leaky":
        return ([(capi.OP_RELU, 0, 0.1)], [], [lambda v: oracle.rectified_linear(v, 0.1)])
    raise ValueError(kind)


def prologue_input(gen, shape):
    """Values across the activations' ranges, with the exp range edges, zeros and infinities in."""
    x = T.normal(gen, shape, 3.0)
    flat = x.reshape(-1)
    idx = gen.integers(0, flat.size, size=max(4, flat.size // 50))
    flat[idx] = gen.choice(np.array([0.0, -0.0, np.inf, -np.inf, 88.8, -88.8, -104.0, 3.0e38, -3.0e38, 1.0e-40], F), size=idx.size)
    return x


FUSED_MAX_CASES = [
    # shape, windows (x first), strides, round_ups, group
    ((4, 64, 112, 112), [3, 3], [2, 2], [True, True], "bn_relu"),       # ResNet stem: bands of a plane per workgroup
    ((64, 64, 112, 112), [3, 3], [2, 2], [True, True], "bn_relu"),      # ... with 64 entries
    ((2, 6, 112, 112), [3, 3], [2, 2], None, "bn_prelu_elu_sigmoid"),
    ((8, 96, 55, 55), [3, 3], [2, 2], None, "bn_relu"),                # planes of 3025 floats, several per workgroup
    ((16, 32, 28, 28), [2, 2], None, None, "tanh_abs"),                # several planes per workgroup
    ((9, 3, 12, 12), [2, 2], None, None, "bn_prelu_elu_sigmoid"),      # more planes per workgroup than feature maps
    ((6, 5, 10, 12), [3, 3], [2, 2], [True, True], "bn_relu"),         # two outputs per lane at a time, small planes
    ((2, 4, 57, 56), [3, 3], [2, 2], [True, True], "prelu_bn"),        # ... a plane per workgroup
    ((5, 7, 6, 10), [3, 2], [2, 2], [True, False], "bn_relu"),         # run-time window, odd plane counts
    ((6, 10, 7, 7), [3, 3], [2, 2], None, "bn_prelu_elu_sigmoid"),     # planes of 49 floats: float4s straddle planes
    ((4, 3, 13, 13), [3, 3], [2, 2], [True, True], "bn_relu"),         # ... with more planes per workgroup than feature maps
    ((3, 5, 2, 3), [2, 1], [1, 1], None, "bn_relu"),                   # planes of 6 floats
    ((40, 30, 3, 3), [2, 2], [1, 1], None, "prelu_bn"),                # more planes than a workgroup takes coefficients for
    ((2, 3, 112, 112), [3, 3], [2, 2], None, "prelu_bn"),
    ((2, 2, 300, 200), [4, 7], [4, 5], None, "leaky"),
    ((1, 3, 4, 4000), [3, 2], [2, 2], None, "bn_relu"),                # one output row per band
    # BatchNorm -> ReLU as straight code with several planes per workgroup (coefficients in LDS, float4s between planes) ...
    ((5, 12, 27, 27), [3, 3], [2, 2], [True, True], "bn_relu"),
    ((3, 10, 35, 35), [3, 3], [2, 2], [True, True], "bn_relu"),
    ((4, 9, 28, 28), [2, 2], None, None, "bn_relu"),
    ((2, 7, 40, 40), [2, 2], None, None, "bn_relu"),
    ((7, 5, 9, 11), [2, 3], [1, 2], [False, True], "bn_relu"),
    # ... and planes large enough to get a workgroup each although several would fit (weights through the scalar cache)
    ((3, 5, 51, 51), [3, 3], [2, 2], [True, True], "bn_relu"),
    ((2, 3, 45, 45), [3, 3], [2, 2], None, "prelu_bn"),
    ((2, 7, 48, 48), [2, 2], None, None, "bn_prelu_elu_sigmoid"),
    ((2, 6, 56, 56), [2, 2], None, None, "bn_relu"),
]


def run_fused_max(gpu, x, ops, chunks, windows, strides, round_ups, is_min=False, fm=1, en=1, expect=0):
    n, c = x.shape[0], x.shape[1]
    dims = list(x.shape[2:])[::-1]
    plane = int(np.prod(dims))
    out_dims = oracle.max_subsampling_output_sizes(dims, windows, strides, round_ups)
    want_shape = (n // en, c // fm) + tuple(out_dims[::-1])
    desc = capi.make_desc(n, c, plane, [ops], [])
    d_in = gpu.to_device(x)
    d_chunks = [gpu.to_device(a) for a in chunks]
    chk = capi.pointer_array([t.data_ptr() for t in d_chunks])
    d_out = gpu.torch.full((max(1, int(np.prod(want_shape))),), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    shape_args = (n // en, c, len(dims), u32(dims), u32(windows), u32(strides) if strides else None,
                  u32([int(r) for r in round_ups]) if round_ups else None, fm, en)
    assert gpu.lib.nnf_hip_max_subsampling_fusable(*shape_args) == expect
    rc = gpu.lib.nnf_hip_max_subsampling_fused_forward(gpu.stream, d_out.data_ptr(), d_in.data_ptr(), ctypes.byref(desc),
                                                       chk if d_chunks else None, *(shape_args + (int(is_min),)))
    assert rc == expect, capi.error_string(rc)
    if expect != 0:
        gpu.torch.cuda.synchronize()
        return None
    return gpu.to_host(d_out, want_shape)


@pytest.mark.parametrize("is_min", [False, True])
@pytest.mark.parametrize("shape,windows,strides,round_ups,group", FUSED_MAX_CASES)
def test_max_subsampling_with_group_folded_in(gpu, shape, windows, strides, round_ups, group, is_min):
    gen = T.rng(66, sum(shape))
    ops, chunks, steps = prologue_case(group, gen, shape[1])
    x = prologue_input(gen, shape)
    v = x
    for step in steps:
        v = step(v)
    want = oracle.max_subsampling(v, windows, strides=strides, round_ups=round_ups, is_min=is_min)
    got = run_fused_max(gpu, x, ops, chunks, windows, strides, round_ups, is_min=is_min)
    assert got.shape == want.shape
    assert T.bit_mismatches(got, want) == 0


@pytest.mark.parametrize("shape,windows,strides,round_ups,group", [
    ((8, 64, 112, 112), [3, 3], [2, 2], [True, True], "relu"),      # a ResNet stem's pooling behind ReLU: all-negative windows give -0.0
    ((8, 64, 112, 112), [3, 3], [2, 2], [True, True], "bn_relu"),
    ((16, 32, 28, 28), [2, 2], None, None, "relu"),
    ((6, 10, 7, 7), [3, 3], [2, 2], None, "bn_relu"),
    ((5, 7, 6, 10), [3, 2], [2, 2], [True, False], "relu"),
])
def test_max_subsampling_behind_relu_where_many_windows_hold_only_zeros(gpu, shape, windows, strides, round_ups, group):
    """rectified_linear with slope 0 turns every negative value into -0.0 and keeps +0.0: with three values in four
    negative about one window in eight (3x3) holds nothing but zeros and the first of them decides the sign."""
    gen = T.rng(73, sum(shape))
    if group == "relu":
        ops, chunks, steps = [(capi.OP_RELU, 0, 0.0)], [], [lambda v: oracle.rectified_linear(v, 0.0)]
        x = zero_heavy(gen, shape, negative_share=0.75)
    else:
        ops, chunks, steps = prologue_case("bn_relu", gen, shape[1])
        x = T.normal(gen, shape, 1.0) - F(0.9)
        flat = x.reshape(-1)
        idx = gen.integers(0, flat.size, size=flat.size // 20)
        flat[idx] = chunks[2][(idx // int(np.prod(shape[2:]))) % shape[1]]  # the feature map's mean: BatchNorm gives beta, often +-0 after ReLU
    v = x
    for step in steps:
        v = step(v)
    want = oracle.max_subsampling(v, windows, strides=strides, round_ups=round_ups)
    assert float(np.mean(want == 0.0)) > 0.03
    got = run_fused_max(gpu, x, ops, chunks, windows, strides, round_ups)
    assert T.bit_mismatches(got, want) == 0


def run_fused_pool(gpu, x, ops, chunks, ww, wh, mult, expect=0):
    n, c, h, w = x.shape
    desc = capi.make_desc(n, c, h * w, [ops], [])
    d_in = gpu.to_device(x)
    d_chunks = [gpu.to_device(a) for a in chunks]
    chk = capi.pointer_array([t.data_ptr() for t in d_chunks])
    out_shape = (n, c, h // wh, w // ww)
    d_out = gpu.torch.full((int(np.prod(out_shape)),), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    assert gpu.lib.nnf_hip_average_subsampling_fusable(n, c, w, h, ww, wh) == expect
    rc = gpu.lib.nnf_hip_average_subsampling_fused_forward(gpu.stream, d_out.data_ptr(), d_in.data_ptr(), ctypes.byref(desc),
                                                           chk if d_chunks else None, n, c, w, h, ww, wh, mult)
    assert rc == expect, capi.error_string(rc)
    if expect != 0:
        gpu.torch.cuda.synchronize()
        return None
    return gpu.to_host(d_out, out_shape)


@pytest.mark.parametrize("shape,ww,wh,group", [
    ((8, 38, 28, 28), 2, 2, "tanh_abs"),               # the GTSRB stages: TanH -> Absolute -> AverageSubsampling
    ((3, 5, 12, 12), 2, 2, "tanh_abs"),
    ((2, 64, 56, 56), 2, 2, "bn_relu"),
    ((1, 2, 120, 100), 2, 2, "bn_prelu_elu_sigmoid"),  # bands of rows
    ((2, 3, 113, 115), 3, 3, "bn_relu"),               # leftover margins, plane not a multiple of 4
    ((1, 4, 9, 7), 3, 2, "leaky"),                     # small planes of 63 floats
    ((7, 9, 5, 5), 2, 2, "bn_prelu_elu_sigmoid"),      # planes of 25 floats, margins
    # whole-plane windows: the global pooling kernel
    ((64, 128, 7, 7), 7, 7, "bn_relu"),                # a ResNet-like tail: 49 floats per plane, float4s straddle planes
    ((3, 5, 7, 7), 7, 7, "bn_prelu_elu_sigmoid"),      # the last workgroup holds 15 planes: 735 floats, three behind the last float4
    ((9, 70, 8, 8), 8, 8, "tanh_abs"),
    ((5, 33, 14, 14), 14, 14, "prelu_bn"),
    ((2, 7, 15, 15), 15, 15, "bn_relu"),               # 225 floats per plane
    ((6, 11, 3, 5), 5, 3, "leaky"),
    ((1, 1, 2, 2), 2, 2, "bn_relu"),
    # odd planes: every wavefront on its own 32 planes, the layers applied per plane on the way out of LDS
    ((1, 37, 7, 7), 7, 7, "bn_prelu_elu_sigmoid"),     # 37 planes: a full wavefront and one with 5 planes (245 floats: one behind the last float4)
    ((70, 3, 3, 3), 3, 3, "bn_relu"),                  # 210 planes of 9 floats: the last wavefront holds 18 of them
    ((5, 33, 5, 5), 5, 5, "prelu_bn"),
    ((3, 7, 9, 9), 9, 9, "tanh_abs"),
    ((2, 3, 11, 11), 11, 11, "bn_prelu_elu_sigmoid"),  # 121 floats per plane: 62 KB of LDS per workgroup
    ((2, 5, 13, 13), 13, 13, "bn_relu"),               # 169 floats per plane: beyond that kernel, odd all the same
    # BatchNorm -> ReLU on odd planes: straight code, rounds of two float4s per lane with the next round in flight
    ((1, 37, 7, 7), 7, 7, "bn_relu"),                  # a wavefront with 5 planes: one round and a half, one float behind
    ((3, 5, 7, 7), 7, 7, "bn_relu"),                   # 15 planes: 183 float4s (three rounds, the last one half) and three floats
    ((5, 33, 5, 5), 5, 5, "bn_relu"),
    ((3, 7, 9, 9), 9, 9, "bn_relu"),
    ((2, 3, 11, 11), 11, 11, "bn_relu"),
    ((1, 2, 3, 3), 3, 3, "bn_relu"),                   # 18 floats: four float4s and two floats in one wavefront
    ((7, 96, 7, 7), 7, 7, "bn_relu"),                  # 672 planes: 21 whole wavefronts
    # ... and on the planes the workgroup-wide kernel takes (even sizes, odd ones beyond 127 floats): straight code there too
    ((9, 70, 8, 8), 8, 8, "bn_relu"),
    ((5, 33, 14, 14), 14, 14, "bn_relu"),
    ((3, 5, 4, 4), 4, 4, "bn_relu"),
    ((2, 9, 6, 3), 3, 6, "bn_relu"),                   # 18 floats per plane: float4s that straddle two planes
    ((1, 3, 2, 3), 3, 2, "bn_relu"),                   # 18 floats in all: four float4s and two floats behind them
])
def test_average_subsampling_with_group_folded_in(gpu, shape, ww, wh, group):
    gen = T.rng(67, sum(shape) + ww)
    ops, chunks, steps = prologue_case(group, gen, shape[1])
    x = T.normal(gen, shape, 2.0)
    v = x
    for step in steps:
        v = step(v)
    mult = oracle.average_subsampling_full_mult([ww, wh])
    want = oracle.average_subsampling(v, [ww, wh], mult=mult)
    got = run_fused_pool(gpu, x, ops, chunks, ww, wh, mult)
    assert got.shape == want.shape
    assert T.bit_mismatches(got, want) == 0


JOINED_POOL_CASES = [
    # shape, arms ("bn": BatchNorm, "-": nothing, "leaky": ReLU 0.1, "elu"), alpha, tail
    ((64, 128, 7, 7), ("-", "bn"), 1.0, "relu"),        # residual + BatchNorm(main) -> Add -> ReLU: the last block of a ResNet
    ((64, 2048, 7, 7), ("-", "bn"), 1.0, "relu"),       # ... at ResNet-50's size with 64 entries
    ((5, 24, 7, 7), ("bn", "bn"), 1.0, "relu"),         # BatchNorm on both arms (a block with a projection shortcut)
    ((3, 5, 7, 7), ("bn", "elu"), 0.5, "sigmoid"),      # 15 planes in the last workgroup, three floats behind the last float4
    ((9, 70, 8, 8), ("leaky", "-"), 2.0, "none"),       # planes that are multiples of 4 floats, nothing behind the Add
    ((2, 7, 15, 15), ("bn", "-"), 1.0, "prelu"),        # 225 floats per plane, weights on an arm and behind the join
    ((1, 1, 2, 2), ("-", "-"), 1.0, "relu"),
    ((1, 37, 7, 7), ("bn", "elu"), 1.0, "sigmoid"),     # a wavefront with 5 planes: 245 floats, one behind the last float4
    ((70, 3, 3, 3), ("bn", "leaky"), 1.0, "relu"),      # 210 planes of 9 floats
    ((4, 9, 5, 5), ("-", "bn"), 0.25, "prelu"),
    ((2, 3, 11, 11), ("bn", "-"), 1.0, "relu"),         # 121 floats per plane: two staged tensors do not fit the odd-plane kernel
    # the two residual groups compiled as straight code (BatchNorm on either input, ReLU behind the Add), ragged ends
    ((5, 24, 7, 7), ("bn", "-"), 1.0, "relu"),
    ((1, 37, 7, 7), ("bn", "-"), 0.5, "relu"),
    ((3, 5, 7, 7), ("bn", "-"), 1.0, "relu"),
    ((70, 3, 3, 3), ("bn", "-"), 1.0, "relu"),
    ((3, 7, 9, 9), ("bn", "-"), 2.0, "relu"),
    ((7, 96, 7, 7), ("bn", "-"), 1.0, "relu"),
    ((1, 37, 7, 7), ("-", "bn"), 1.0, "relu"),
    ((3, 5, 7, 7), ("-", "bn"), 0.25, "relu"),
    ((70, 3, 3, 3), ("-", "bn"), 1.0, "relu"),
    ((2, 5, 5, 5), ("-", "bn"), 1.0, "relu"),
    ((1, 2, 3, 3), ("-", "bn"), 1.0, "relu"),
    # ... on the planes of the workgroup-wide kernel
    ((9, 70, 8, 8), ("bn", "-"), 1.0, "relu"),
    ((5, 33, 14, 14), ("-", "bn"), 1.0, "relu"),
    ((3, 5, 4, 4), ("bn", "-"), 0.5, "relu"),
    ((2, 7, 15, 15), ("-", "bn"), 1.0, "relu"),         # 225 floats per plane, float4s that straddle two planes
    ((2, 9, 3, 6), ("bn", "-"), 1.0, "relu"),
    ((1, 3, 2, 3), ("-", "bn"), 2.0, "relu"),
]


def joined_arm(kind, gen, c, chunks):
    """-> (ops, oracle function) of one arm; weight chunks are appended to chunks"""
    if kind == "bn":
        g, b, m, s = T.bn_params(gen, c)
        first = len(chunks)
        chunks += [g, b, m, s]
        return [(capi.OP_BATCH_NORM, first)], lambda v: oracle.batch_norm(v, g, b, m, s)
    if kind == "leaky":
        return [(capi.OP_RELU, 0, 0.1)], lambda v: oracle.rectified_linear(v, 0.1)
    if kind == "elu":
        return [(capi.OP_ELU,)], oracle.exponential_linear
    return [], lambda v: v


@pytest.mark.parametrize("shape,arms,alpha,tail", JOINED_POOL_CASES)
def test_whole_plane_average_with_a_joined_group_folded_in(gpu, shape, arms, alpha, tail):
    """Two inputs, each with its own layers, an Add, the layers behind it and the average over whole planes in one
    launch: the bits of the layers run one after another by the oracle."""
    gen = T.rng(69, sum(shape) + len(tail))
    n, c, h, w = shape
    chunks = []
    arm_ops, arm_fns = zip(*[joined_arm(kind, gen, c, chunks) for kind in arms])
    if tail == "relu":
        tail_ops, tail_fn = [(capi.OP_RELU, 0, 0.0)], lambda v: oracle.rectified_linear(v, 0.0)
    elif tail == "sigmoid":
        tail_ops, tail_fn = [(capi.OP_SIGMOID,)], oracle.sigmoid
    elif tail == "prelu":
        a = T.uniform(gen, c, -0.5, 0.5)
        tail_ops, tail_fn = [(capi.OP_PRELU, len(chunks))], lambda v: oracle.parametric_rectified_linear(v, a)
        chunks.append(a)
    else:
        tail_ops, tail_fn = [], lambda v: v
    xs = [prologue_input(gen, shape) if i == 0 else T.normal(gen, shape, 2.0) for i in range(2)]
    joined = tail_fn(oracle.add([fn(x) for fn, x in zip(arm_fns, xs)], alpha))
    mult = oracle.average_subsampling_full_mult([w, h])
    want = oracle.average_subsampling(joined, [w, h], mult=mult)

    desc = capi.make_desc(n, c, h * w, [list(ops) for ops in arm_ops], tail_ops, add_alpha=alpha)
    d_ins = [gpu.to_device(x) for x in xs]
    d_chunks = [gpu.to_device(a) for a in chunks]
    chk = capi.pointer_array([t.data_ptr() for t in d_chunks])
    ins = capi.pointer_array([t.data_ptr() for t in d_ins])
    d_out = gpu.torch.full((n * c,), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    assert gpu.lib.nnf_hip_average_subsampling_joinable(n, c, w, h, w, h) == 0
    rc = gpu.lib.nnf_hip_average_subsampling_joined_forward(gpu.stream, d_out.data_ptr(), ins, ctypes.byref(desc), chk if d_chunks else None,
                                                            n, c, w, h, w, h, mult)
    assert rc == 0, capi.error_string(rc)
    got = gpu.to_host(d_out, want.shape)
    assert T.bit_mismatches(got, want) == 0


def test_joined_groups_the_average_cannot_take_are_refused(gpu):
    gen = T.rng(70, 0)
    n, c, h, w = 2, 6, 8, 8
    d_ins = [gpu.to_device(T.normal(gen, (n, c, h, w))) for _ in range(2)]
    ins = capi.pointer_array([t.data_ptr() for t in d_ins])
    d_out = gpu.torch.zeros(n * c * 16, dtype=gpu.torch.float32, device=gpu.device)
    desc = capi.make_desc(n, c, h * w, [[], []], [(capi.OP_RELU, 0, 0.0)])
    call = gpu.lib.nnf_hip_average_subsampling_joined_forward
    # windows smaller than the plane
    assert gpu.lib.nnf_hip_average_subsampling_joinable(n, c, w, h, 2, 2) == capi.E_UNSUPPORTED
    assert call(gpu.stream, d_out.data_ptr(), ins, ctypes.byref(desc), None, n, c, w, h, 2, 2, 0.25) == capi.E_UNSUPPORTED
    # a single-input description, a missing second input, a shape that is not the description's
    single = capi.make_desc(n, c, h * w, [[(capi.OP_RELU, 0, 0.0)]], [])
    assert call(gpu.stream, d_out.data_ptr(), ins, ctypes.byref(single), None, n, c, w, h, w, h, 1.0) == capi.E_INVAL
    one = capi.pointer_array([d_ins[0].data_ptr(), 0])
    assert call(gpu.stream, d_out.data_ptr(), one, ctypes.byref(desc), None, n, c, w, h, w, h, 1.0) == capi.E_INVAL
    assert call(gpu.stream, d_out.data_ptr(), ins, ctypes.byref(desc), None, n, c + 1, w, h, w, h, 1.0) == capi.E_INVAL
    # the output may not lie inside an input
    assert call(gpu.stream, d_ins[1].data_ptr(), ins, ctypes.byref(desc), None, n, c, w, h, w, h, 1.0) == capi.E_OVERLAP
    gpu.torch.cuda.synchronize()


@pytest.mark.parametrize("shape", [(4, 16, 128, 128), (64, 256, 8, 8)])
def test_exp_layers_folded_into_subsampling_over_a_sweep_of_all_exponents(gpu, shape):
    """ELU, Sigmoid and TanH inside the subsampling kernels (their own expf batches and range repair) on a regular
    sweep of fp32 bit patterns - every 4099th, so every exponent and both signs, NaNs and infinities included. A 1x1
    average window passes each value through (0.0F + x, times 1), so the output is the layer's result element by
    element: bit for bit the oracle's. One plane per workgroup (bands) and many small planes per workgroup."""
    count = int(np.prod(shape))
    bits = (np.arange(count, dtype=np.uint64) * 4099 % (1 << 32)).astype(np.uint32)
    x = bits.view(F).reshape(shape)
    for op, fn in (((capi.OP_ELU,), oracle.exponential_linear), ((capi.OP_SIGMOID,), oracle.sigmoid),
                   ((capi.OP_TANH, 0, 1.7159, 0.6666), lambda v: oracle.hyperbolic_tangent(v, 1.7159, 0.6666))):
        want = oracle.average_subsampling(fn(x), [1, 1], mult=1.0)
        got = run_fused_pool(gpu, x, [op], [], 1, 1, 1.0)
        assert T.bit_mismatches(got, want) == 0, "layer kind %d" % op[0]


def test_subsampling_that_cannot_fold_a_group_in_says_so(gpu):
    gen = T.rng(68, 0)
    ops, chunks, _ = prologue_case("bn_relu", gen, 6)
    # several planes of 3 floats per workgroup (a float4 would straddle three planes), windows over feature
    # maps, 3-D, rows too wide for the staging buffer
    run_fused_max(gpu, T.normal(gen, (4, 6, 1, 3)), ops, chunks, [1, 1], None, None, expect=capi.E_UNSUPPORTED)
    run_fused_max(gpu, T.normal(gen, (4, 6, 8, 8)), ops, chunks, [2, 2], None, None, fm=2, expect=capi.E_UNSUPPORTED)
    run_fused_max(gpu, T.normal(gen, (2, 6, 4, 6, 8)), ops, chunks, [2, 2, 2], None, None, expect=capi.E_UNSUPPORTED)
    run_fused_max(gpu, T.normal(gen, (1, 6, 3, 20000)), ops, chunks, [2, 3], [2, 1], None, expect=capi.E_UNSUPPORTED)
    # whole-plane average windows over planes of fewer than four floats
    run_fused_pool(gpu, T.normal(gen, (4, 6, 1, 3)), ops, chunks, 3, 1, 1.0, expect=capi.E_UNSUPPORTED)
    # a group with an Add, a group of another shape, a missing weight pointer
    x = gpu.to_device(T.normal(gen, (2, 6, 8, 8)))
    out = gpu.torch.empty(2 * 6 * 16, dtype=gpu.torch.float32, device=gpu.device)
    d_chunks = [gpu.to_device(a) for a in chunks]
    chk = capi.pointer_array([t.data_ptr() for t in d_chunks])
    shape_args = (2, 6, 2, u32([8, 8]), u32([2, 2]), None, None, 1, 1, 0)
    call = gpu.lib.nnf_hip_max_subsampling_fused_forward
    with_add = capi.make_desc(2, 6, 64, [[], ops], [])
    assert call(gpu.stream, out.data_ptr(), x.data_ptr(), ctypes.byref(with_add), chk, *shape_args) == capi.E_INVAL
    other_fm = capi.make_desc(2, 5, 64, [ops], [])
    assert call(gpu.stream, out.data_ptr(), x.data_ptr(), ctypes.byref(other_fm), chk, *shape_args) == capi.E_INVAL
    other_plane = capi.make_desc(2, 6, 63, [ops], [])
    assert call(gpu.stream, out.data_ptr(), x.data_ptr(), ctypes.byref(other_plane), chk, *shape_args) == capi.E_INVAL
    good = capi.make_desc(2, 6, 64, [ops], [])
    assert call(gpu.stream, out.data_ptr(), x.data_ptr(), None, chk, *shape_args) == capi.E_INVAL
    assert call(gpu.stream, out.data_ptr(), x.data_ptr(), ctypes.byref(good), None, *shape_args) == capi.E_INVAL
    assert call(gpu.stream, out.data_ptr(), x.data_ptr(), ctypes.byref(good), chk, *shape_args) == 0
    # two layers with weights are applied, a third is one too many
    two = capi.make_desc(2, 6, 64, [[(capi.OP_BATCH_NORM, 0)] * 2], [])
    three = capi.make_desc(2, 6, 64, [[(capi.OP_BATCH_NORM, 0)] * 3], [])
    assert call(gpu.stream, out.data_ptr(), x.data_ptr(), ctypes.byref(two), chk, *shape_args) == 0
    assert call(gpu.stream, out.data_ptr(), x.data_ptr(), ctypes.byref(three), chk, *shape_args) == capi.E_UNSUPPORTED
    gpu.torch.cuda.synchronize()


class Guarded:
    """An output of `count` floats with 256 sentinel floats on either side of it (the inner pointer keeps the 1 KB
    alignment of the allocation): a kernel that stores in front of its output or behind it changes a sentinel."""

    margin = 256
    sentinel = F(-123456.0)

    def __init__(self, gpu, count):
        self.gpu, self.count = gpu, count
        self.whole = gpu.torch.full((count + 2 * self.margin,), float(self.sentinel), dtype=gpu.torch.float32, device=gpu.device)
        self.ptr = self.whole.data_ptr() + 4 * self.margin

    def check(self, want, what):
        host = self.gpu.to_host(self.whole, (self.count + 2 * self.margin,))
        assert np.all(host[:self.margin] == self.sentinel), what + ": stores in front of the output"
        assert np.all(host[self.margin + self.count:] == self.sentinel), what + ": stores behind the output"
        assert T.bit_mismatches(host[self.margin:self.margin + self.count].reshape(want.shape), want) == 0, what


@pytest.mark.parametrize("shape,windows", [
    ((2, 5, 112, 112), [2, 2]), ((1, 3, 100, 96), [2, 2]), ((4, 8, 28, 28), [2, 2]), ((3, 4, 21, 19), [3, 2]), ((7, 37, 6, 5), [2, 2]),
    ((5, 12, 56, 56), [2, 2]), ((2, 3, 57, 57), [3, 3]), ((1, 2, 200, 300), [3, 2]), ((5, 2, 23), [4]), ((1, 1, 5000, 4), [2, 2])])
def test_tiling_kernels_store_nothing_outside_their_output(gpu, shape, windows):
    """Every way the tiling kernel leaves its results - runs of bands, runs of whole planes (one or several to a workgroup),
    stores from the scan loop - with the output between sentinels: the runs' scalar heads and tails stop where the output does."""
    x = spiced(T.rng(90, sum(shape)), shape)
    want = oracle.max_subsampling(x, windows, tiling=True)
    dims = list(shape[2:])[::-1]
    out = Guarded(gpu, want.size)
    rc = gpu.lib.nnf_hip_max_subsampling_tiling_forward(gpu.stream, out.ptr, gpu.to_device(x).data_ptr(), shape[0], shape[1], len(dims), u32(dims), u32(windows), 0)
    assert rc == 0, capi.error_string(rc)
    out.check(want, "tiling %r %r" % (shape, windows))


@pytest.mark.parametrize("shape,windows,strides,round_ups", [
    ((3, 5, 112, 112), [3, 3], [2, 2], [True, True]), ((2, 7, 55, 55), [3, 3], [2, 2], None), ((5, 3, 28, 28), [2, 2], None, None),
    ((7, 5, 13, 13), [3, 3], [2, 2], [True, True]), ((6, 5, 10, 12), [3, 3], [2, 2], [True, True]), ((1, 3, 4, 4000), [3, 2], [2, 2], None)])
def test_pooling_kernels_store_nothing_outside_their_output(gpu, shape, windows, strides, round_ups):
    """The staged pooling kernels - alone, and with BatchNorm -> ReLU folded in (the kernel of its own for one plane per
    workgroup and the general one) - with the output between sentinels."""
    gen = T.rng(91, sum(shape))
    x = spiced(gen, shape)
    dims = list(shape[2:])[::-1]
    want = oracle.max_subsampling(x, windows, strides=strides, round_ups=round_ups)
    out = Guarded(gpu, want.size)
    d_in = gpu.to_device(x)
    args = (shape[0], shape[1], len(dims), u32(dims), u32(windows), u32(strides) if strides else None,
            u32([int(r) for r in round_ups]) if round_ups else None, 1, 1, 0)
    rc = gpu.lib.nnf_hip_max_subsampling_forward(gpu.stream, out.ptr, d_in.data_ptr(), *args)
    assert rc == 0, capi.error_string(rc)
    out.check(want, "pooling %r" % (shape,))
    # the same with BatchNorm -> ReLU in front (values without NaN: ReLU of NaN is the reference's own matter)
    c = shape[1]
    y = T.normal(gen, shape, 2.0)
    gamma, beta, mean, inv_sigma = T.bn_params(gen, c)
    chunks = [gpu.to_device(a) for a in (gamma, beta, mean, inv_sigma)]
    chk = capi.pointer_array([t.data_ptr() for t in chunks])
    desc = capi.make_desc(shape[0], c, int(np.prod(dims)), [[(capi.OP_BATCH_NORM, 0), (capi.OP_RELU, 0, 0.0)]], [])
    staged = oracle.rectified_linear(oracle.batch_norm(y.reshape(shape[0], c, -1), gamma, beta, mean, inv_sigma)).reshape(shape)
    want = oracle.max_subsampling(staged, windows, strides=strides, round_ups=round_ups)
    out = Guarded(gpu, want.size)
    rc = gpu.lib.nnf_hip_max_subsampling_fused_forward(gpu.stream, out.ptr, gpu.to_device(y).data_ptr(), ctypes.byref(desc), chk, *args)
    assert rc == 0, capi.error_string(rc)
    out.check(want, "BatchNorm -> ReLU -> pooling %r" % (shape,))
