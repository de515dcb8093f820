"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle on identical seeded inputs.

Bars: batch norm and element-wise layers within max(2 ULP, 1e-6 relative) of
the plain CPU tester; softmax within 1e-5 relative. On top of that the tests demand what the
design promises: bit-for-bit equality wherever the operation order is the reference's own (every
kernel except the row softmax, whose sum is a tree instead of a left-to-right loop).
"""

import ctypes
import os

import numpy as np
import pytest

import nnf_testing as T
import oracle
from nnforge_amd import capi

pytestmark = pytest.mark.gpu

BN, RELU, PRELU, ELU, SIGMOID, TANH = (capi.OP_BATCH_NORM, capi.OP_RELU, capi.OP_PRELU, capi.OP_ELU,
                                       capi.OP_SIGMOID, capi.OP_TANH)


def oracle_chain(x, steps):
    """Runs the oracle layer by layer the way forward_propagation_plain drives the testers."""
    v = x
    for step in steps:
        v = step(v)
    return v


def check_exact(got, want, what):
    got = np.asarray(got, dtype=np.float32).reshape(-1)
    want = np.asarray(want, dtype=np.float32).reshape(-1)
    T.assert_close_elementwise(got, want, ulps=2, rel=1e-6, what=what)
    mism = T.bit_mismatches(got, want)
    assert mism == 0, "%s: %d of %d elements differ in bits (max %d ulp)" % (
        what, mism, got.size, int(T.ulp_distance(got, want).max()))


# ---------------------------------------------------------------------------------------------
# benchmark configurations at their real sizes
# ---------------------------------------------------------------------------------------------

def test_config0_bn_relu_full_size(gpu):
    n, c, h, w = 32, 64, 56, 56
    x = T.normal(T.rng(0, 0), (n, c, h, w))
    g, b, m, s = T.bn_params(T.rng(0, 1), c)
    want = oracle.rectified_linear(oracle.batch_norm(x, g, b, m, s), 0.0)
    got = gpu.chain((n, c, h * w), [[(BN, 0)]], [(RELU, 0, 0.0)], [x], [g, b, m, s])
    check_exact(got, want, "config 0")
    # -0.0 for negative pre-activations, as x * 0.0F gives in the reference
    assert np.signbit(got[(want.reshape(-1) == 0)]).any()


def test_config2_bn_add_prelu_full_size(gpu):
    n, c, h, w = 128, 256, 56, 56
    main = T.normal(T.rng(2, 0), (n, c, h, w))
    residual = T.normal(T.rng(2, 1), (n, c, h, w))
    g, b, m, s = T.bn_params(T.rng(2, 2), c)
    slopes = T.uniform(T.rng(2, 3), c, 0.0, 0.25)
    bn = oracle.batch_norm(main, g, b, m, s)
    want = oracle.parametric_rectified_linear(oracle.add([residual, bn]), slopes)
    del bn
    # Add's inputs in schema order: [residual, batch-normed main path]
    got = gpu.chain((n, c, h * w), [[], [(BN, 0)]], [(PRELU, 4)], [residual, main], [g, b, m, s, slopes])
    check_exact(got, want, "config 2")


def config3_input(shape):
    gen = T.rng(3, 0)
    x = T.normal(gen, shape, 2.0)
    spikes = gen.random(shape) < 0.001
    signs = np.where(gen.random(shape) < 0.5, np.float32(-50.0), np.float32(50.0))
    return np.where(spikes, signs, x).astype(np.float32)


def test_config3_activation_chain_full_size(gpu):
    n, c, h, w = 64, 512, 28, 28
    x = config3_input((n, c, h, w))
    g, b, m, s = T.bn_params(T.rng(3, 1), c)
    want = oracle_chain(x, [
        lambda v: oracle.batch_norm(v, g, b, m, s),
        oracle.exponential_linear,
        oracle.sigmoid,
        lambda v: oracle.hyperbolic_tangent(v, T.TANH_SCALE, T.TANH_STEEPNESS)])
    got = gpu.chain((n, c, h * w), [[(BN, 0), (ELU,), (SIGMOID,), (TANH, 0, T.TANH_SCALE, T.TANH_STEEPNESS)]], [], [x], [g, b, m, s])
    T.assert_close_elementwise(got, want.reshape(-1), 2, 1e-6, "config 3")
    mism = T.bit_mismatches(got, want.reshape(-1))
    print("config 3: %d of %d elements differ in bits from the oracle" % (mism, got.size))
    assert mism == 0


def config1_input(n, c):
    gen = T.rng(1, 0)
    x = T.normal(gen, (n, c), 4.0)
    return np.where(gen.random((n, c)) < 0.01, np.float32(30.0), x).astype(np.float32)


def run_softmax(gpu, x3, in_place=False, expect=0):
    n, c, plane = x3.shape
    d_in = gpu.to_device(x3)
    d_out = d_in if in_place else gpu.torch.full((x3.size,), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    rc = gpu.lib.nnf_hip_softmax_forward(gpu.stream, d_out.data_ptr(), d_in.data_ptr(), n, c, plane)
    assert rc == expect, capi.error_string(rc)
    return gpu.to_host(d_out, x3.shape)


def assert_softmax_close(got, want, what):
    """1e-5 relative (north_star); an absolute floor of one denormal step covers flushed tails."""
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    tol = 1e-5 * np.abs(want.astype(np.float64)) + 1e-45
    bad = ~(err <= tol) & ~(np.isnan(got) & np.isnan(want))
    assert not bad.any(), "%s: %d elements outside 1e-5 relative, worst %g" % (
        what, int(bad.sum()), float((err / np.maximum(np.abs(want), 1e-300)).max()))


def test_config1_softmax_full_size(gpu):
    n, c = 256, 1000
    x = config1_input(n, c).reshape(n, c, 1)
    want = oracle.softmax(x)
    got = run_softmax(gpu, x)
    assert_softmax_close(got, want, "config 1")
    # rows sum to one within C * 2^-24 and the exponentials themselves are the oracle's bit for bit:
    # value / row-multiplier reproduces them up to the last place
    assert np.abs(got.astype(np.float64).sum(axis=1) - 1.0).max() < c * 2.0 ** -24
    worst = float((np.abs(got.astype(np.float64) - want) / want.astype(np.float64)).max())
    print("config 1: worst relative difference from the oracle %.3g" % worst)
    assert worst < 2e-6


# ---------------------------------------------------------------------------------------------
# one-input groups with more tiles than the device holds workgroups at once (33 to 67 MB per tensor): these
# take the grid that stays put, every workgroup walking over several tiles
# ---------------------------------------------------------------------------------------------

def test_groups_on_the_walking_grid_full_size(gpu):
    # batch_norm -> rectified_linear on a ResNet-50 shape at N=64: 64 feature maps of 56x56 (51 MB)
    n, c, hw = 64, 64, 56
    gen = T.rng(13, 0)
    x = T.normal(gen, (n, c, hw * hw))
    g, b, m, s = T.bn_params(gen, c)
    bn = oracle.batch_norm(x, g, b, m, s)
    got = gpu.chain((n, c, hw * hw), [[(BN, 0)]], [(RELU, 0, 0.0)], [x], [g, b, m, s])
    check_exact(got, oracle.rectified_linear(bn), "BN+ReLU 64x64x56^2")
    # in place, with a per-feature-map slope behind the batch norm
    slopes = T.uniform(gen, c, 0.0, 0.25)
    got = gpu.chain((n, c, hw * hw), [[(BN, 0), (PRELU, 4)]], [], [x], [g, b, m, s, slopes], in_place=True)
    check_exact(got, oracle.parametric_rectified_linear(bn, slopes), "BN+PReLU 64x64x56^2 in place")
    # a group that calls expf and is not one of the compile-time programs: the layer list is interpreted
    y = config3_input((9, 256, 4096))   # 37.7 MB
    g, b, m, s = T.bn_params(gen, 256)
    want = oracle.sigmoid(oracle.rectified_linear(oracle.batch_norm(y, g, b, m, s), 0.1))
    got = gpu.chain((9, 256, 4096), [[(BN, 0), (RELU, 0, 0.1), (SIGMOID,)]], [], [y], [g, b, m, s])
    check_exact(got, want, "BN+ReLU+Sigmoid 9x256x4096")


@pytest.mark.parametrize("total", [9000001, 9000002, 9000003, 8650752 + 4096 * 3 + 5, 16777215])
def test_walking_grid_with_a_partial_last_vector(gpu, total):
    """No weights: any element count goes. The last float4 of the tensor is partial, in the last tile, which one of the
    workgroups reaches on its last round (or its first: 8650752 + ... puts it a few tiles behind one round of 2048 + 64)."""
    x = T.normal(T.rng(14, total % 97), total)
    got = gpu.chain((1, 1, total), [[(RELU, 0, 0.25), (capi.OP_ABSOLUTE,)]], [], [x])
    check_exact(got, np.abs(oracle.rectified_linear(x, 0.25)), "ReLU+Absolute on %d elements" % total)
    assert gpu.lib.nnf_hip_rectified_linear_forward  # the single-layer entry point takes the same path:
    d_in = gpu.to_device(x)
    d_out = gpu.torch.full((total + 1,), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    assert gpu.lib.nnf_hip_rectified_linear_forward(gpu.stream, d_out.data_ptr(), d_in.data_ptr(), 0.0, total) == 0
    out = gpu.to_host(d_out)
    check_exact(out[:total], oracle.rectified_linear(x, 0.0), "rectified_linear on %d elements" % total)
    assert np.isnan(out[total]), "wrote past the end"


# ---------------------------------------------------------------------------------------------
# every fused group shape of the ResNet-50 stack (config 4), reduced entry count
# ---------------------------------------------------------------------------------------------

RESNET_SHAPES = [(64, 112), (64, 56), (128, 56), (128, 28), (256, 28), (256, 14), (512, 14), (512, 7),
                 (256, 56), (512, 28), (1024, 14), (2048, 7)]


@pytest.mark.parametrize("c,hw", RESNET_SHAPES)
def test_resnet_group_shapes(gpu, c, hw):
    n = 3
    gen = T.rng(4, c * 1000 + hw)
    x = T.normal(gen, (n, c, hw, hw))
    r = T.normal(gen, (n, c, hw, hw))
    g, b, m, s = T.bn_params(gen, c)
    g2, b2, m2, s2 = T.bn_params(gen, c)
    bn = oracle.batch_norm(x, g, b, m, s)
    # BN + ReLU
    got = gpu.chain((n, c, hw * hw), [[(BN, 0)]], [(RELU, 0, 0.0)], [x], [g, b, m, s])
    check_exact(got, oracle.rectified_linear(bn), "BN+ReLU %dx%d^2" % (c, hw))
    # BN + Add(residual) + ReLU, Add inputs = [residual, BN(main)]
    got = gpu.chain((n, c, hw * hw), [[], [(BN, 0)]], [(RELU, 0, 0.0)], [r, x], [g, b, m, s])
    check_exact(got, oracle.rectified_linear(oracle.add([r, bn])), "BN+Add+ReLU %dx%d^2" % (c, hw))
    # BN(shortcut) + BN(main) + Add + ReLU
    bn2 = oracle.batch_norm(r, g2, b2, m2, s2)
    got = gpu.chain((n, c, hw * hw), [[(BN, 4)], [(BN, 0)]], [(RELU, 0, 0.0)], [r, x], [g, b, m, s, g2, b2, m2, s2])
    check_exact(got, oracle.rectified_linear(oracle.add([bn2, bn])), "BN+BN+Add+ReLU %dx%d^2" % (c, hw))


# ---------------------------------------------------------------------------------------------
# single-layer entry points, awkward shapes, special values
# ---------------------------------------------------------------------------------------------

SPECIALS = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1e-38, -1e-38, 1.1754944e-38,
                     3.4028235e38, -3.4028235e38, 50.0, -50.0, 88.0, 88.7, 88.72, 88.73, 89.0, -87.0, -88.0, -103.0,
                     -103.9, -103.97, -103.98, -104.0, -150.0, 1e-6, -1e-6, 0.5, -0.5, 17.0, -17.0, 30.0, -30.0],
                    dtype=np.float32)


def awkward_input(shape, seed):
    gen = T.rng(9, seed)
    x = T.normal(gen, shape, 4.0)
    flat = x.reshape(-1)
    k = min(flat.size, SPECIALS.size)
    pos = gen.permutation(flat.size)[:k]
    flat[pos] = SPECIALS[:k]
    return x


AWKWARD_SHAPES = [(1, 1, 1), (1, 1, 3), (2, 3, 1), (1, 5, 2), (3, 7, 3), (2, 3, 49), (5, 13, 49), (1, 3, 5 * 5), (2, 2, 4),
                  (1, 64, 4097), (3, 5, 1023), (2, 4100, 1), (7, 3, 3136), (1, 2, 20000), (4, 1, 12544)]


@pytest.mark.parametrize("shape", AWKWARD_SHAPES)
def test_batch_norm_entry_point_awkward_shapes(gpu, shape):
    n, c, plane = shape
    x = awkward_input(shape, 1)
    g, b, m, s = T.bn_params(T.rng(9, 2), c)
    d_x = gpu.to_device(x)
    d_p = [gpu.to_device(v) for v in (g, b, m, s)]
    d_out = gpu.torch.full((x.size,), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    rc = gpu.lib.nnf_hip_batch_norm_forward(gpu.stream, d_out.data_ptr(), d_x.data_ptr(), *[t.data_ptr() for t in d_p], n, c, plane)
    assert rc == 0, capi.error_string(rc)
    check_exact(gpu.to_host(d_out), oracle.batch_norm(x, g, b, m, s), "batch_norm %s" % (shape,))


@pytest.mark.parametrize("shape", AWKWARD_SHAPES)
def test_prelu_entry_point_awkward_shapes(gpu, shape):
    n, c, plane = shape
    x = awkward_input(shape, 3)
    a = T.uniform(T.rng(9, 4), c, -0.5, 0.5)
    d_x, d_a = gpu.to_device(x), gpu.to_device(a)
    d_out = gpu.torch.full((x.size,), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    rc = gpu.lib.nnf_hip_parametric_rectified_linear_forward(gpu.stream, d_out.data_ptr(), d_x.data_ptr(), d_a.data_ptr(), n, c, plane)
    assert rc == 0, capi.error_string(rc)
    check_exact(gpu.to_host(d_out), oracle.parametric_rectified_linear(x, a), "prelu %s" % (shape,))


FLAT_SIZES = [1, 2, 3, 4, 5, 63, 64, 65, 1023, 1024, 1025, 4095, 4096, 4097, 100003, 1 << 20]


def run_flat(gpu, fn, x, *args, in_place=False):
    d_x = gpu.to_device(x)
    d_out = d_x if in_place else gpu.torch.full((x.size,), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    rc = fn(gpu.stream, d_out.data_ptr(), d_x.data_ptr(), *args, x.size)
    assert rc == 0, capi.error_string(rc)
    return gpu.to_host(d_out)


@pytest.mark.parametrize("size", FLAT_SIZES)
def test_flat_activation_entry_points(gpu, size):
    x = awkward_input((size,), size)
    lib = gpu.lib
    for slope in (0.0, 0.1, -2.0):
        check_exact(run_flat(gpu, lib.nnf_hip_rectified_linear_forward, x, slope), oracle.rectified_linear(x, slope), "relu slope %g" % slope)
    check_exact(run_flat(gpu, lib.nnf_hip_exponential_linear_forward, x), oracle.exponential_linear(x), "elu")
    check_exact(run_flat(gpu, lib.nnf_hip_sigmoid_forward, x), oracle.sigmoid(x), "sigmoid")
    for scale, steep in ((1.0, 1.0), (T.TANH_SCALE, T.TANH_STEEPNESS), (1.7159, 0.666666)):
        check_exact(run_flat(gpu, lib.nnf_hip_hyperbolic_tangent_forward, x, scale, steep),
                    oracle.hyperbolic_tangent(x, scale, steep), "tanh %g %g" % (scale, steep))
    # in place, as every tester on the path allows
    check_exact(run_flat(gpu, lib.nnf_hip_sigmoid_forward, x, in_place=True), oracle.sigmoid(x), "sigmoid in place")


def test_expf_dense_sweep_through_elu_and_sigmoid(gpu):
    """Every fp32 in a few dense bit-pattern windows plus a coarse sweep of all negative floats:
    expf on the device is the oracle's expf bit for bit."""
    windows = []
    for start in (np.float32(-1e-3), np.float32(-0.7), np.float32(-12.0), np.float32(-87.3), np.float32(-103.5)):
        first = int(np.array(start, dtype=np.float32).view(np.uint32))
        windows.append(np.arange(first, first + (1 << 18), dtype=np.uint32))
    windows.append(np.arange(0x80000000, 0xFF800000, 4099, dtype=np.uint32))  # all negative floats, strided
    x = np.concatenate(windows).view(np.float32)
    check_exact(run_flat(gpu, gpu.lib.nnf_hip_exponential_linear_forward, x), oracle.exponential_linear(x), "elu sweep")
    check_exact(run_flat(gpu, gpu.lib.nnf_hip_sigmoid_forward, x), oracle.sigmoid(x), "sigmoid sweep (negative)")
    check_exact(run_flat(gpu, gpu.lib.nnf_hip_sigmoid_forward, -x), oracle.sigmoid(-x), "sigmoid sweep (positive)")


def test_exp_range_edges_dense(gpu):
    """Every fp32 in windows around the arguments where the device code changes path: |x| = 87 (range
    repair branch), expf(x) + 1 = 2^126 (x = 87.34: the short division sequences end), log(2^128)
    (expf overflows, TanH turns NaN), log(2^-126) and log(2^-150) (expf results go subnormal, then 0) -
    with ordinary values in the same wavefronts, so that both sides of every wavefront-uniform
    branch hold live lanes."""
    windows = []
    for centre in (87.0, 87.336, 88.7228, -87.0, -87.3365, -103.972):
        first = int(np.array(centre, dtype=np.float32).view(np.uint32)) - (1 << 15)
        windows.append(np.arange(first, first + (1 << 16), dtype=np.uint32))
    edge = np.concatenate(windows).view(np.float32)
    x = np.empty(edge.size * 2, np.float32)
    x[0::2] = edge
    x[1::2] = T.normal(T.rng(17, 0), edge.size, 2.0)  # every other lane holds an ordinary value
    with np.errstate(all="ignore"):
        for sign in (1.0, -1.0):
            v = (x * np.float32(sign)).astype(np.float32)
            check_exact(run_flat(gpu, gpu.lib.nnf_hip_exponential_linear_forward, v), oracle.exponential_linear(v), "elu edges")
            check_exact(run_flat(gpu, gpu.lib.nnf_hip_sigmoid_forward, v), oracle.sigmoid(v), "sigmoid edges")
            check_exact(run_flat(gpu, gpu.lib.nnf_hip_hyperbolic_tangent_forward, v, 1.0, 0.5), oracle.hyperbolic_tangent(v, 1.0, 0.5), "tanh edges")
            check_exact(run_flat(gpu, gpu.lib.nnf_hip_hyperbolic_tangent_forward, v, T.TANH_SCALE, T.TANH_STEEPNESS),
                        oracle.hyperbolic_tangent(v, T.TANH_SCALE, T.TANH_STEEPNESS), "tanh edges, scaled")
        rows = edge[: (edge.size // 1000) * 1000].reshape(-1, 1000, 1)  # row softmax: x - max crosses the same edges
        got = run_softmax(gpu, np.ascontiguousarray(-np.abs(rows)))
        assert_softmax_close(got, oracle.softmax(np.ascontiguousarray(-np.abs(rows))), "softmax edges")


@pytest.mark.parametrize("input_count", [1, 2, 3, 4, 5, 8, 9])
@pytest.mark.parametrize("size,alpha", [(5, 1.0), (4099, 0.5), (1 << 18, -1.25)])
def test_add_entry_point(gpu, input_count, size, alpha):
    gen = T.rng(10, input_count * 31 + size)
    xs = [T.normal(gen, (size,), 3.0) for _ in range(input_count)]
    for x in xs:  # signed zeros meet in the sum
        x[:: max(1, size // 7)] = -0.0
    d_in = [gpu.to_device(x) for x in xs]
    d_out = gpu.torch.full((size,), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    ptrs = capi.pointer_array([t.data_ptr() for t in d_in])
    rc = gpu.lib.nnf_hip_add_forward(gpu.stream, d_out.data_ptr(), ptrs, input_count, alpha, size)
    assert rc == 0, capi.error_string(rc)
    check_exact(gpu.to_host(d_out), oracle.add(xs, alpha), "add k=%d" % input_count)


def test_fused_equals_unfused_bitwise(gpu):
    """A fused group is the same arithmetic as its layers launched one by one."""
    n, c, plane = 4, 24, 196
    gen = T.rng(11, 0)
    x = T.normal(gen, (n, c, plane), 2.0)
    r = T.normal(gen, (n, c, plane))
    g, b, m, s = T.bn_params(gen, c)
    a = T.uniform(gen, c, 0.0, 0.25)
    fused = gpu.chain((n, c, plane), [[], [(BN, 0), (ELU,)]], [(PRELU, 4), (SIGMOID,), (TANH, 0, 1.7159, 0.6666)], [r, x], [g, b, m, s, a], alpha=0.5)
    v = gpu.chain((n, c, plane), [[(BN, 0)]], [], [x], [g, b, m, s])
    v = gpu.chain((n, c, plane), [[(ELU,)]], [], [v])
    v = gpu.chain((n, c, plane), [[], []], [], [r, v.reshape(n, c, plane)], alpha=0.5)
    v = gpu.chain((n, c, plane), [[(PRELU, 0)]], [], [v], [a])
    v = gpu.chain((n, c, plane), [[(SIGMOID,)]], [], [v])
    v = gpu.chain((n, c, plane), [[(TANH, 0, 1.7159, 0.6666)]], [], [v])
    assert T.bit_mismatches(fused, v) == 0
    want = oracle.hyperbolic_tangent(oracle.sigmoid(oracle.parametric_rectified_linear(
        oracle.add([r, oracle.exponential_linear(oracle.batch_norm(x, g, b, m, s))], 0.5), a)), 1.7159, 0.6666)
    check_exact(fused, want, "fused group")


def random_layer(gen, c, chunks, allow_exp=True):
    """-> (op tuple, oracle step) of one random element-wise layer; weights are appended to chunks"""
    kinds = [BN, RELU, PRELU, capi.OP_ABSOLUTE, capi.OP_DROPOUT] + ([ELU, SIGMOID, TANH] if allow_exp else [])
    kind = kinds[int(gen.integers(0, len(kinds)))]
    if kind == BN:
        g, b, m, s = T.bn_params(gen, c)
        first = len(chunks)
        chunks.extend([g, b, m, s])
        return (BN, first), lambda v: oracle.batch_norm(v, g, b, m, s)
    if kind == RELU:
        slope = float(gen.choice(np.array([0.0, 0.1, -0.5, 1.0], np.float32)))
        return (RELU, 0, slope), lambda v: oracle.rectified_linear(v, slope)
    if kind == PRELU:
        a = T.uniform(gen, c, -0.5, 0.5)
        first = len(chunks)
        chunks.append(a)
        return (PRELU, first), lambda v: oracle.parametric_rectified_linear(v, a)
    if kind == capi.OP_ABSOLUTE:
        return (capi.OP_ABSOLUTE,), oracle.absolute
    if kind == capi.OP_DROPOUT:
        return (capi.OP_DROPOUT,), oracle.dropout
    if kind == ELU:
        return (ELU,), oracle.exponential_linear
    if kind == SIGMOID:
        return (SIGMOID,), oracle.sigmoid
    scale, steepness = float(gen.uniform(0.5, 2.0)), float(gen.uniform(0.2, 1.5))
    return (TANH, 0, scale, steepness), lambda v: oracle.hyperbolic_tangent(v, scale, steepness)


def random_group(seed, allow_exp=True):
    """A group drawn at random - 1 to 4 inputs, any split of up to 8 layers over the arms and the tail, any layer kinds,
    shapes with odd planes and element counts - and what the oracle, run layer by layer, makes of it.
    -> (shape3, arms, tail, inputs, chunks, has_add, alpha, want)"""
    gen = T.rng(13, seed)
    n = int(gen.integers(1, 6))
    c = int(gen.choice([1, 3, 8, 17, 64, 130]))
    plane = int(gen.choice([1, 2, 7, 49, 196, 225, 784, 1000, 3136]))
    input_count = int(gen.choice([1, 1, 2, 2, 3, 4]))
    has_add = (input_count > 1) or bool(gen.integers(0, 2))
    budget = capi.MAX_OPS
    chunks, arms, arm_steps = [], [], []
    for _ in range(input_count):
        count = int(gen.integers(0, min(3, budget) + 1))
        budget -= count
        ops, steps = [], []
        for _ in range(count):
            op, step = random_layer(gen, c, chunks, allow_exp)
            ops.append(op)
            steps.append(step)
        arms.append(ops)
        arm_steps.append(steps)
    tail, tail_steps = [], []
    if has_add:
        for _ in range(int(gen.integers(0, min(3, budget) + 1))):
            op, step = random_layer(gen, c, chunks, allow_exp)
            tail.append(op)
            tail_steps.append(step)
    elif not arms[0]:
        op, step = random_layer(gen, c, chunks, allow_exp)
        arms[0].append(op)
        arm_steps[0].append(step)
    alpha = float(gen.choice(np.array([1.0, 0.5, -1.25], np.float32)))
    inputs = [awkward_input((n, c, plane), 100 * seed + j) if j == 0 else T.normal(gen, (n, c, plane), 2.0) for j in range(input_count)]
    values = []
    for x, steps in zip(inputs, arm_steps):
        v = x
        for step in steps:
            v = step(v)
        values.append(v)
    want = oracle.add(values, alpha).reshape(inputs[0].shape) if has_add else values[0]
    for step in tail_steps:
        want = step(want)
    return (n, c, plane), arms, tail, inputs, chunks, has_add, alpha, want


# NNF_EXHAUSTIVE=1: 360 more groups
@pytest.mark.parametrize("seed", range(400 if os.environ.get("NNF_EXHAUSTIVE") == "1" else 40))
def test_random_groups_equal_the_layers_one_by_one(gpu, seed):
    """Random groups against the oracle run layer by layer, bit for bit."""
    shape3, arms, tail, inputs, chunks, has_add, alpha, want = random_group(seed)
    got = gpu.chain(shape3, arms, tail, inputs, chunks, has_add=has_add, alpha=alpha)
    check_exact(got, want, "random group %d: %d inputs, arms %s, tail %s" % (seed, len(inputs), arms, tail))


@pytest.mark.parametrize("first_seed,count", [(0, 40), (40, 17), (100, 2), (200, 7)])
def test_independent_groups_in_one_call_equal_the_groups_one_by_one(gpu, first_seed, count):
    """nnf_hip_chain_forward_batch: groups that share a kernel instance go several to a launch. Random groups of all
    kinds in one call (among them groups without elements, groups that work in place and one of the compile-time expf
    programs, which keeps a launch of its own) against the oracle, bit for bit."""
    groups = [random_group(first_seed + i, allow_exp=(i % 3 == 0)) for i in range(count)]
    n, c, plane = 3, 16, 196
    x = config3_input((n, c, plane))
    g, b, m, s = T.bn_params(T.rng(15, first_seed), c)
    groups.append(((n, c, plane), [[(BN, 0), (ELU,), (SIGMOID,), (TANH, 0, T.TANH_SCALE, T.TANH_STEEPNESS)]], [], [x], [g, b, m, s], False, 1.0,
                   oracle.hyperbolic_tangent(oracle.sigmoid(oracle.exponential_linear(oracle.batch_norm(x, g, b, m, s))), T.TANH_SCALE, T.TANH_STEEPNESS)))
    groups.append(((0, 4, 49), [[(RELU, 0, 0.0)]], [], [np.zeros((0, 4, 49), np.float32)], [], False, 1.0, np.zeros((0, 4, 49), np.float32)))
    in_place = [i % 4 == 1 for i in range(len(groups))]
    got = gpu.chain_batch([(sh, arms, tail, ins, chunks, has_add, alpha) for sh, arms, tail, ins, chunks, has_add, alpha, _ in groups], in_place)
    for i, (out, group) in enumerate(zip(got, groups)):
        check_exact(out, group[7], "group %d of the call (seed %d)" % (i, first_seed + i))


@pytest.mark.parametrize("n,c,plane,before,after,kind", [
    (5, 64, 784, 32 * 784, 96 * 784, "bn_relu"),        # an Inception branch among others: weights straight from memory
    (3, 8, 49, 12 * 49, 0, "bn_relu"),                  # planes of 49 floats: coefficients through LDS, last part of the wide tensor
    (4, 16, 196, 0, 4 * 196, "bn_add_relu"),            # two inputs joined by an Add, first part
    (70000, 4, 1, 8, 4, "prelu"),                       # more entries than the grid has rows: workgroups take several
    (2, 6, 1000, 6000, 2000, "elu_tanh"),               # expf layers, one partly filled tile per entry
    (0, 8, 16, 64, 64, "bn_relu"),                      # no entries
])
def test_group_written_into_a_wider_tensor(gpu, n, c, plane, before, after, kind):
    """nnf_hip_chain_forward_strided: the group's result lands where a Concat layer would copy it, entry by entry, and
    nothing around it is touched."""
    gen = T.rng(18, n % 97 + c + plane)
    per_entry = c * plane
    stride = before + per_entry + after
    x = config3_input((n, c, plane)) if kind == "elu_tanh" else T.normal(gen, (n, c, plane), 1.5)
    inputs, chunks = [x], []
    if kind == "bn_relu":
        g, b, m, s = T.bn_params(gen, c)
        arms, tail, chunks = [[(BN, 0), (RELU, 0, 0.0)]], [], [g, b, m, s]
        want = oracle.rectified_linear(oracle.batch_norm(x, g, b, m, s))
    elif kind == "bn_add_relu":
        g, b, m, s = T.bn_params(gen, c)
        r = T.normal(gen, (n, c, plane), 1.5)
        inputs = [r, x]
        arms, tail, chunks = [[], [(BN, 0)]], [(RELU, 0, 0.1)], [g, b, m, s]
        want = oracle.rectified_linear(oracle.add([r, oracle.batch_norm(x, g, b, m, s)]).reshape(x.shape), 0.1)
    elif kind == "prelu":
        a = T.uniform(gen, c, -0.5, 0.5)
        arms, tail, chunks = [[(PRELU, 0)]], [], [a]
        want = oracle.parametric_rectified_linear(x, a)
    else:
        arms, tail = [[(ELU,), (TANH, 0, T.TANH_SCALE, T.TANH_STEEPNESS)]], []
        want = oracle.hyperbolic_tangent(oracle.exponential_linear(x), T.TANH_SCALE, T.TANH_STEEPNESS)
    desc = capi.make_desc(n, c, plane, arms, tail)
    assert gpu.lib.nnf_hip_chain_forward_strided_status(ctypes.byref(desc), stride) == 0
    sentinel = np.float32(-12345.5)
    wide = gpu.torch.full((max(1, n * stride),), float(sentinel), dtype=gpu.torch.float32, device=gpu.device)
    d_in = [gpu.to_device(a if a.size else np.zeros(4, np.float32)) for a in inputs]
    d_chunks = [gpu.to_device(a) for a in chunks]
    ins = capi.pointer_array([t.data_ptr() for t in d_in])
    chk = capi.pointer_array([t.data_ptr() for t in d_chunks])
    rc = gpu.lib.nnf_hip_chain_forward_strided(gpu.stream, ctypes.byref(desc), wide.data_ptr() + 4 * before, stride, ins, chk if d_chunks else None)
    assert rc == 0, capi.error_string(rc)
    got = gpu.to_host(wide)[:n * stride].reshape(n, stride)
    check_exact(got[:, before:before + per_entry], want, "the group's part of the wide tensor")
    assert (got[:, :before] == sentinel).all() and (got[:, before + per_entry:] == sentinel).all(), "the rest of the wide tensor is untouched"


def test_groups_written_side_by_side_into_a_wider_tensor_in_one_call(gpu):
    """nnf_hip_chain_forward_strided_batch: the branches in front of a Concat - a two-input group, a group on 7 x 7 planes
    (coefficients through LDS), two plain ones, eight groups in all so that the call takes two launches - write their parts
    of the wide tensor; the result is the oracle's groups concatenated, the room left between two parts stays untouched."""
    gen = T.rng(19, 1)
    n, plane = 6, 49
    widths = [8, 12, 4, 16, 8, 4, 8, 12]
    gap_after = 3   # leave 16 floats unused behind the third part
    parts, descs, keep, outs, ins_list, chk_list, offsets = [], [], [], [], [], [], []
    stride = sum(widths) * plane + 16
    wide = gpu.torch.full((n * stride,), -777.25, dtype=gpu.torch.float32, device=gpu.device)
    offset = 0
    for i, c in enumerate(widths):
        x = T.normal(gen, (n, c, plane), 1.5)
        g, b, m, s_ = T.bn_params(gen, c)
        if i == 1:
            r = T.normal(gen, (n, c, plane), 1.5)
            arms, tail, inputs = [[], [(BN, 0)]], [(RELU, 0, 0.0)], [r, x]
            want = oracle.rectified_linear(oracle.add([r, oracle.batch_norm(x, g, b, m, s_)]).reshape(x.shape))
        else:
            arms, tail, inputs = [[(BN, 0), (RELU, 0, 0.125)]], [], [x]
            want = oracle.rectified_linear(oracle.batch_norm(x, g, b, m, s_), 0.125)
        descs.append(capi.make_desc(n, c, plane, arms, tail))
        d_in = [gpu.to_device(a) for a in inputs]
        d_chunks = [gpu.to_device(a) for a in (g, b, m, s_)]
        keep += d_in + d_chunks
        ins_list.append(capi.pointer_array([t.data_ptr() for t in d_in]))
        chk_list.append(capi.pointer_array([t.data_ptr() for t in d_chunks]))
        outs.append(wide.data_ptr() + 4 * offset)
        offsets.append(offset)
        parts.append(want.reshape(n, -1))
        offset += c * plane + (16 if i == gap_after - 1 else 0)
    count = len(widths)
    desc_array = (capi.ChainDesc * count)(*descs)
    out_array = (ctypes.c_void_p * count)(*outs)
    strides = (ctypes.c_uint32 * count)(*([stride] * count))
    in_array = (ctypes.POINTER(ctypes.c_void_p) * count)(*[ctypes.cast(p, ctypes.POINTER(ctypes.c_void_p)) for p in ins_list])
    chk_array = (ctypes.POINTER(ctypes.c_void_p) * count)(*[ctypes.cast(p, ctypes.POINTER(ctypes.c_void_p)) for p in chk_list])
    before = ctypes.c_uint64()
    after = ctypes.c_uint64()
    gpu.lib.nnf_hip_launch_count(ctypes.byref(before))
    rc = gpu.lib.nnf_hip_chain_forward_strided_batch(gpu.stream, count, desc_array, out_array, strides, in_array, chk_array)
    assert rc == 0, capi.error_string(rc)
    gpu.lib.nnf_hip_launch_count(ctypes.byref(after))
    assert after.value - before.value == 2   # six groups to a launch
    got = gpu.to_host(wide).reshape(n, stride)
    for i, c in enumerate(widths):
        check_exact(got[:, offsets[i]:offsets[i] + c * plane], parts[i], "part %d" % i)
    gap = offsets[gap_after] - 16
    assert (got[:, gap:gap + 16] == np.float32(-777.25)).all()
    # parts that meet are refused, whichever way: the second group moved 4 floats into the first one's part
    out_array[1] = outs[1] - 16
    assert gpu.lib.nnf_hip_chain_forward_strided_batch(gpu.stream, count, desc_array, out_array, strides, in_array, chk_array) == capi.E_OVERLAP
    out_array[1] = outs[1]
    strides[2] = stride + 4
    assert gpu.lib.nnf_hip_chain_forward_strided_batch(gpu.stream, count, desc_array, out_array, strides, in_array, chk_array) == capi.E_OVERLAP
    gpu.torch.cuda.synchronize()


def test_group_written_into_a_wider_tensor_refuses_what_it_cannot_do(gpu):
    desc = capi.make_desc(2, 3, 5, [[(RELU, 0, 0.0)]], [])           # 15 floats per entry: entries would not start on 16 bytes
    assert gpu.lib.nnf_hip_chain_forward_strided_status(ctypes.byref(desc), 32) == capi.E_UNSUPPORTED
    desc = capi.make_desc(2, 4, 4, [[(RELU, 0, 0.0)]], [])
    assert gpu.lib.nnf_hip_chain_forward_strided_status(ctypes.byref(desc), 18) == capi.E_UNSUPPORTED   # stride not a multiple of 4
    assert gpu.lib.nnf_hip_chain_forward_strided_status(ctypes.byref(desc), 12) == capi.E_INVAL         # narrower than the group
    desc = capi.make_desc(2, 4, 4, [[], [], []], [(RELU, 0, 0.0)])
    assert gpu.lib.nnf_hip_chain_forward_strided_status(ctypes.byref(desc), 32) == capi.E_UNSUPPORTED   # three inputs
    # the written range may not reach into an input
    desc = capi.make_desc(2, 4, 4, [[(RELU, 0, 0.0)]], [])
    buf = gpu.torch.zeros(256, dtype=gpu.torch.float32, device=gpu.device)
    ins = capi.pointer_array([buf.data_ptr() + 4 * 40])
    assert gpu.lib.nnf_hip_chain_forward_strided(gpu.stream, ctypes.byref(desc), buf.data_ptr(), 32, ins, None) == capi.E_OVERLAP
    gpu.torch.cuda.synchronize()


def test_recorded_launches_replay_with_the_results_of_launching(gpu):
    """nnf_hip_stream_begin_capture / nnf_hip_stream_end_capture / nnf_hip_graph_launch: a fused group, a softmax and a whole-plane
    average recorded once on a stream of their own, then replayed four times with new values in the same input
    buffers each time and the program's ordinary work (copies, synchronisations) in between: every replay gives the
    bits the oracle gives (softmax to 1e-5)."""
    lib, torch = gpu.lib, gpu.torch
    n, c, plane = 5, 24, 49
    gamma, beta, mean, inv_sigma = T.bn_params(T.rng(16, 1), c)
    d_chunks = [gpu.to_device(a) for a in (gamma, beta, mean, inv_sigma)]
    chk = capi.pointer_array([t.data_ptr() for t in d_chunks])
    desc = capi.make_desc(n, c, plane, [[], [(BN, 0)]], [(RELU, 0, 0.0)])
    d_x, d_r = gpu.to_device(np.zeros((n, c, plane), np.float32)), gpu.to_device(np.zeros((n, c, plane), np.float32))
    d_y = torch.empty_like(d_x)
    d_pool = torch.empty(n * c, dtype=torch.float32, device=gpu.device)
    d_prob = torch.empty(n * c, dtype=torch.float32, device=gpu.device)
    ins = capi.pointer_array([d_r.data_ptr(), d_x.data_ptr()])
    stream = ctypes.c_void_p()
    capi.check(lib.nnf_hip_stream_create(ctypes.byref(stream)))
    torch.cuda.synchronize()
    capi.check(lib.nnf_hip_stream_begin_capture(stream))
    capi.check(lib.nnf_hip_chain_forward(stream, ctypes.byref(desc), d_y.data_ptr(), ins, chk))
    capi.check(lib.nnf_hip_average_subsampling_forward(stream, d_pool.data_ptr(), d_y.data_ptr(), n, c, 7, 7, 7, 7, 1.0 / 49.0))
    capi.check(lib.nnf_hip_softmax_forward(stream, d_prob.data_ptr(), d_pool.data_ptr(), n, c, 1))
    graph = ctypes.c_void_p()
    capi.check(lib.nnf_hip_stream_end_capture(stream, ctypes.byref(graph)))
    assert graph.value
    for replay in range(4):
        gen = T.rng(17, replay)
        x, r = T.normal(gen, (n, c, plane), 2.0), T.normal(gen, (n, c, plane), 2.0)
        d_x.copy_(torch.from_numpy(x).reshape(d_x.shape))
        d_r.copy_(torch.from_numpy(r).reshape(d_r.shape))
        d_y.fill_(float("nan"))
        torch.cuda.synchronize()
        capi.check(lib.nnf_hip_graph_launch(graph, stream))
        capi.check(lib.nnf_hip_stream_synchronize(stream))
        want_y = oracle.rectified_linear(oracle.add([r, oracle.batch_norm(x, gamma, beta, mean, inv_sigma)]).reshape(x.shape))
        want_pool = oracle.average_subsampling(want_y.reshape(n, c, 7, 7), [7, 7], mult=1.0 / 49.0)
        check_exact(gpu.to_host(d_y, x.shape), want_y, "replay %d: group" % replay)
        check_exact(gpu.to_host(d_pool, want_pool.shape), want_pool, "replay %d: average" % replay)
        assert_softmax_close(gpu.to_host(d_prob, (n, c, 1)), oracle.softmax(want_pool.reshape(n, c, 1)), "replay %d: softmax" % replay)
    capi.check(lib.nnf_hip_graph_destroy(graph))
    capi.check(lib.nnf_hip_stream_destroy(stream))


@pytest.mark.parametrize("planes", [(784, 3136), (49, 9), (784, 49), (49, 196, 7, 3136)])
def test_groups_of_one_and_of_two_inputs_share_launches(gpu, planes):
    """A residual network's groups as the driver hands them over: BatchNorm -> ReLU over one tensor and BatchNorm
    (-> BatchNorm on the shortcut) -> Add -> ReLU over two, thirteen of them in one call - more than one launch holds -
    with planes whose weights are read straight from memory, planes that need staged coefficients, and both in one call."""
    groups = []
    for i in range(13):
        gen = T.rng(17, 100 * len(planes) + i)
        plane = planes[i % len(planes)]
        n, c = 1 + i % 3, (5, 16, 64)[(i // 2) % 3]
        x = T.normal(gen, (n, c, plane), 1.5)
        g, b, m, s = T.bn_params(gen, c)
        if i % 2 == 0:
            groups.append(((n, c, plane), [[(BN, 0), (RELU, 0, 0.0)]], [], [x], [g, b, m, s], False, 1.0,
                           oracle.rectified_linear(oracle.batch_norm(x, g, b, m, s))))
        elif i % 4 == 1:
            r = T.normal(gen, (n, c, plane))
            groups.append(((n, c, plane), [[], [(BN, 0)]], [(RELU, 0, 0.0)], [r, x], [g, b, m, s], True, 1.0,
                           oracle.rectified_linear(oracle.add([r, oracle.batch_norm(x, g, b, m, s)]))))
        else:
            y = T.normal(gen, (n, c, plane))
            g2, b2, m2, s2 = T.bn_params(gen, c)
            groups.append(((n, c, plane), [[(BN, 0)], [(BN, 4)]], [(RELU, 0, 0.0)], [y, x], [g2, b2, m2, s2, g, b, m, s], True, 1.0,
                           oracle.rectified_linear(oracle.add([oracle.batch_norm(y, g2, b2, m2, s2), oracle.batch_norm(x, g, b, m, s)]))))
    got = gpu.chain_batch([group[:7] for group in groups])
    for i, (out, group) in enumerate(zip(got, groups)):
        check_exact(out, group[7], "group %d of the call (plane %d, %d inputs)" % (i, group[0][2], len(group[3])))


def test_groups_of_one_call_must_not_touch_each_other(gpu):
    x = gpu.to_device(T.normal(T.rng(16, 0), 4096))
    y = gpu.torch.empty(8192, dtype=gpu.torch.float32, device=gpu.device)
    descs = (capi.ChainDesc * 2)(capi.make_desc(1, 1, 4096, [[(RELU, 0, 0.0)]]), capi.make_desc(1, 1, 4096, [[(capi.OP_ABSOLUTE,)]]))

    def call(outs, ins):
        in_arrays = [capi.pointer_array([a]) for a in ins]
        in_ptrs = (ctypes.POINTER(ctypes.c_void_p) * 2)(*[ctypes.cast(a, ctypes.POINTER(ctypes.c_void_p)) for a in in_arrays])
        return gpu.lib.nnf_hip_chain_forward_batch(gpu.stream, 2, descs, capi.pointer_array(outs), in_ptrs, None)

    base = y.data_ptr()
    assert call([base, base + 16384], [x.data_ptr(), x.data_ptr()]) == 0                       # a shared input is fine
    assert call([base, base + 8192], [x.data_ptr(), x.data_ptr()]) == capi.E_OVERLAP           # two outputs overlap
    assert call([base, base + 16384], [x.data_ptr(), base]) == capi.E_OVERLAP                  # one reads what the other writes
    assert call([base, base + 16384], [base, x.data_ptr()]) == 0                               # in place within a group
    assert gpu.lib.nnf_hip_chain_forward_batch(gpu.stream, 0, None, None, None, None) == 0
    assert gpu.lib.nnf_hip_chain_forward_batch(gpu.stream, 2, None, None, None, None) == capi.E_INVAL
    gpu.torch.cuda.synchronize()


def test_in_place_group(gpu):
    n, c, plane = 2, 8, 49
    gen = T.rng(12, 0)
    x = T.normal(gen, (n, c, plane))
    r = T.normal(gen, (n, c, plane))
    g, b, m, s = T.bn_params(gen, c)
    want = oracle.rectified_linear(oracle.add([oracle.batch_norm(x, g, b, m, s), r]))
    got = gpu.chain((n, c, plane), [[(BN, 0)], []], [(RELU, 0, 0.0)], [x, r], [g, b, m, s], in_place=True)
    check_exact(got, want, "in-place group")


def test_identity_batch_norm_and_zero_entries(gpu):
    x = awkward_input((2, 5, 33), 5)
    one, zero = np.ones(5, np.float32), np.zeros(5, np.float32)
    got = gpu.chain((2, 5, 33), [[(BN, 0)]], [], [x], [one, zero, zero, one])
    # identity parameters: x * 1 + 0 (signed zero aside, -0 + 0 = +0, as in the reference)
    check_exact(got, oracle.batch_norm(x, one, zero, zero, one), "identity BN")
    # zero entries: nothing is launched, nothing is touched
    d = gpu.to_device(np.full(8, 7.0, np.float32))
    desc = capi.make_desc(0, 5, 33, [[(RELU, 0, 0.0)]])
    ins = capi.pointer_array([d.data_ptr()])
    assert gpu.lib.nnf_hip_chain_forward(gpu.stream, ctypes.byref(desc), d.data_ptr(), ins, None) == 0
    assert (gpu.to_host(d) == 7.0).all()


def test_argument_errors(gpu):
    lib = gpu.lib
    d = gpu.to_device(np.zeros(64, np.float32))
    e = gpu.to_device(np.zeros(64, np.float32))
    base = d.data_ptr()
    s = gpu.stream
    assert lib.nnf_hip_rectified_linear_forward(s, base + 4, base + 64, 0.0, 8) == capi.E_ALIGN
    assert lib.nnf_hip_rectified_linear_forward(s, base + 16, base, 0.0, 8) == capi.E_OVERLAP
    assert lib.nnf_hip_rectified_linear_forward(s, None, base, 0.0, 8) == capi.E_INVAL
    assert lib.nnf_hip_rectified_linear_forward(s, base, base, 0.0, 1 << 33) == capi.E_TOOBIG
    desc = capi.make_desc(1, 4, 4, [[], []], has_add=False)
    ins = capi.pointer_array([d.data_ptr(), e.data_ptr()])
    assert lib.nnf_hip_chain_forward(s, ctypes.byref(desc), d.data_ptr(), ins, None) == capi.E_INVAL
    desc = capi.make_desc(1, 4, 4, [[(BN, 0)]])
    assert lib.nnf_hip_chain_forward(s, ctypes.byref(desc), d.data_ptr(), ins, None) == capi.E_INVAL  # BN without chunks
    desc = capi.make_desc(1, 4, 4, [[(99,)]])
    assert lib.nnf_hip_chain_forward(s, ctypes.byref(desc), d.data_ptr(), ins, None) == capi.E_INVAL
    # second input overlapping the output
    desc = capi.make_desc(1, 4, 4, [[], []])
    ins = capi.pointer_array([e.data_ptr(), d.data_ptr()])
    assert lib.nnf_hip_chain_forward(s, ctypes.byref(desc), d.data_ptr(), ins, None) == capi.E_OVERLAP
    assert lib.nnf_hip_softmax_forward(s, base, base + 16, 1, 8, 1) == capi.E_OVERLAP
    assert lib.nnf_hip_average_subsampling_forward(s, e.data_ptr(), d.data_ptr(), 1, 1, 4, 4, 5, 2, 1.0) == capi.E_INVAL
    assert b"aligned" in lib.nnf_hip_error_string(capi.E_ALIGN)
    gpu.torch.cuda.synchronize()


# ---------------------------------------------------------------------------------------------
# softmax
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("n,c", [(1, 1), (3, 2), (5, 3), (2, 4), (7, 10), (4, 64), (9, 255), (3, 256), (2, 257), (5, 1000), (64, 1000),
                                 (3, 1001), (2, 2048), (2, 2049), (3, 4096), (2, 8200), (2, 32768), (1, 40000), (2, 33001), (5000, 12),
                                 # many rows that are no multiple of four floats long: a wavefront per row, up to sixteen floats per lane
                                 (2048, 1001), (2100, 1023), (2049, 513), (2500, 999), (4099, 1021), (2048, 1025), (3000, 130),
                                 # 4096 rows or more of up to 32 vectors: four rows to a wavefront
                                 (4096, 100), (4097, 128), (5000, 10), (4500, 31), (4100, 33), (4099, 1), (4111, 5), (70000, 100), (4096, 124)])
def test_softmax_rows(gpu, n, c):
    gen = T.rng(13, n * 100000 + c)
    x = T.normal(gen, (n, c, 1), 4.0)
    x[gen.random((n, c, 1)) < 0.01] = 30.0
    want = oracle.softmax(x)
    got = run_softmax(gpu, x)
    assert_softmax_close(got, want, "softmax rows %dx%d" % (n, c))
    got2 = run_softmax(gpu, x, in_place=True)
    assert T.bit_mismatches(got, got2) == 0


@pytest.mark.parametrize("n,c,plane", [(2, 1, 5), (2, 2, 777), (2, 3, 2), (3, 4, 130), (1, 10, 49), (3, 16, 5), (2, 17, 64), (2, 21, 1000),
                                       (3, 33, 300), (2, 64, 129), (1, 1100, 70001), (4, 5, 4096),
                                       # four positions per lane (plane a multiple of 4, at least 262144 columns, up to 16 feature maps)
                                       (1, 2, 262144), (1, 3, 262148), (2, 8, 131072), (1, 16, 262144), (1, 17, 262144)])
def test_softmax_columns_bit_exact(gpu, n, c, plane):
    """One lane per column (up to 64 feature maps, or columns too many and too long for the shared-out
    kernel): the reference's own left-to-right sum, so the bits are the oracle's."""
    gen = T.rng(14, n * 100000 + c * 100 + plane)
    x = T.normal(gen, (n, c, plane), 4.0)
    x[gen.random((n, c, plane)) < 0.01] = 30.0
    want = oracle.softmax(x)
    got = run_softmax(gpu, x)
    assert_softmax_close(got, want, "softmax columns")
    assert T.bit_mismatches(got, want) == 0  # same left-to-right sum as the reference
    assert T.bit_mismatches(run_softmax(gpu, x, in_place=True), want) == 0


@pytest.mark.parametrize("n,c,plane", [(1, 150, 333), (4, 1000, 49), (2, 65, 7), (3, 257, 100), (1, 4100, 3), (1, 66, 65536),
                                       # values staged in LDS: 64 positions x up to 240 feature maps, 32 x up to 480, 16 x up to 960
                                       (1, 70, 70001), (2, 150, 40000), (1, 240, 33000), (1, 241, 33000), (3, 960, 50), (3, 961, 50),
                                       (1, 300, 65536), (1, 300, 65537), (1, 480, 33000), (1, 481, 33000),
                                       # up to 65536 columns: 8 positions x up to 1920 feature maps staged; 32 positions from 97 feature maps on in large tensors
                                       (64, 1000, 49), (2, 1920, 70), (2, 1921, 70), (3, 1500, 9), (1, 1100, 65536),
                                       (1, 96, 33000), (1, 97, 33000), (2, 128, 20000)])
def test_softmax_columns_sliced(gpu, n, c, plane):
    """More than 64 feature maps: a column is shared out over 4 to 32 lanes whose partial sums are
    added in slice order, so the bar is the one stated for softmax, 1e-5 relative."""
    gen = T.rng(15, n * 100000 + c * 100 + plane)
    x = T.normal(gen, (n, c, plane), 4.0)
    x[gen.random((n, c, plane)) < 0.01] = 30.0
    want = oracle.softmax(x)
    got = run_softmax(gpu, x)
    assert_softmax_close(got, want, "softmax sliced columns")
    assert np.abs(got.astype(np.float64).sum(axis=1) - 1.0).max() < c * 2.0 ** -24
    assert T.bit_mismatches(run_softmax(gpu, x, in_place=True), got) == 0


def test_softmax_special_rows(gpu):
    c = 100
    rows = np.zeros((7, c, 1), np.float32)
    rows[0] = 5.0                      # uniform -> exactly 1/C up to rounding
    rows[1, 3] = np.nan                # NaN poisons the row (max skips it, expf does not)
    rows[2] = -3.0e38                  # below the -1e37 start value of the max: sum 0 -> 0 * inf = NaN
    rows[3, 7] = 30.0                  # one-hot limit
    rows[4] = ((np.arange(c, dtype=np.float32) - 50.0) * 0.5).reshape(c, 1)
    rows[5] = rows[4] + 64.0           # shift invariance (the shift is exact in fp32)
    rows[6, 0] = np.inf                # inf - inf = NaN at the maximum
    want = oracle.softmax(rows)
    got = run_softmax(gpu, rows)
    assert_softmax_close(got, want, "softmax special rows")
    assert np.isnan(got[1]).all() and np.isnan(got[2]).all()
    assert abs(float(got[0, 0, 0]) - 1.0 / c) < 1e-9
    assert got[3, 7, 0] > 0.999999
    assert T.bit_mismatches(got[4], got[5]) == 0  # x - max is the same number in both rows
    cols = np.repeat(rows.transpose(2, 1, 0), 3, axis=0).copy()  # the same data laid out as columns (sliced kernel)
    got_cols = run_softmax(gpu, cols)
    assert_softmax_close(got_cols, oracle.softmax(cols), "softmax special columns")
    assert T.bit_mismatches(np.isnan(got_cols), np.isnan(oracle.softmax(cols))) == 0
    narrow = np.ascontiguousarray(cols[:, :60, :])                # 60 feature maps: one lane per column, bit-exact
    assert T.bit_mismatches(run_softmax(gpu, narrow), oracle.softmax(narrow)) == 0


# ---------------------------------------------------------------------------------------------
# average subsampling
# ---------------------------------------------------------------------------------------------

def run_pool(gpu, x, ww, wh, mult, expect=0):
    n, c, h, w = x.shape
    d_in = gpu.to_device(x)
    out_shape = (n, c, h // wh, w // ww)
    d_out = gpu.torch.full((int(np.prod(out_shape)),), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    rc = gpu.lib.nnf_hip_average_subsampling_forward(gpu.stream, d_out.data_ptr(), d_in.data_ptr(), n, c, w, h, ww, wh, mult)
    assert rc == expect, capi.error_string(rc)
    return gpu.to_host(d_out, out_shape)


@pytest.mark.parametrize("n,c", [(64, 2048), (3, 5), (1, 1), (2, 300)])
def test_global_average_7x7(gpu, n, c):
    x = T.normal(T.rng(15, n + c), (n, c, 7, 7))
    plain_mult = 1.0  # what the plain tester uses when the schema sets no alpha: the window SUM
    full_mult = oracle.average_subsampling_full_mult([7, 7])  # 1/49, the CUDA tester's / explicit alpha
    for mult in (plain_mult, full_mult):
        want = oracle.average_subsampling(x, [7, 7], mult=mult)
        got = run_pool(gpu, x, 7, 7, mult)
        assert T.bit_mismatches(got, want) == 0


@pytest.mark.parametrize("shape,ww,wh", [((2, 3, 8, 8), 2, 2), ((1, 4, 9, 7), 3, 2), ((2, 2, 6, 10), 5, 3), ((1, 2, 4, 4), 4, 4),
                                         ((3, 3, 5, 12), 12, 5), ((1, 1, 30, 30), 30, 30), ((2, 5, 16, 16), 1, 1), ((1, 3, 7, 9), 2, 3),
                                         # planes larger than a workgroup's staging buffer (bands of rows), leftover margins
                                         ((1, 2, 120, 100), 2, 2), ((2, 3, 113, 115), 3, 3), ((1, 1, 300, 70), 7, 5), ((2, 2, 56, 56), 2, 2),
                                         ((1, 2, 97, 4100), 4, 3),
                                         # whole-plane windows of several sizes (global pooling kernel up to 240 floats per plane)
                                         ((5, 70, 14, 14), 14, 14), ((3, 9, 15, 15), 15, 15), ((2, 5, 15, 16), 16, 15), ((2, 3, 16, 16), 16, 16),
                                         ((70, 3, 8, 8), 8, 8),
                                         # odd planes: every wavefront on its own 32 planes (37 planes: a wavefront with 5; 210 planes of 9 floats;
                                         # 121 floats per plane; 169 and 225 are beyond that kernel)
                                         ((1, 37, 7, 7), 7, 7), ((70, 3, 3, 3), 3, 3), ((5, 33, 5, 5), 5, 5), ((3, 7, 9, 9), 9, 9), ((2, 3, 11, 11), 11, 11),
                                         ((2, 5, 13, 13), 13, 13), ((9, 1, 3, 1), 1, 3),
                                         # more than 65535 outputs per plane: the one-lane-per-output kernel
                                         ((1, 1, 300, 300), 1, 1), ((1, 1, 520, 260), 2, 1)])
def test_average_subsampling_windows(gpu, shape, ww, wh):
    x = T.normal(T.rng(16, sum(shape) + ww), shape)
    mult = oracle.average_subsampling_full_mult([ww, wh])
    want = oracle.average_subsampling(x, [ww, wh], mult=mult)
    got = run_pool(gpu, x, ww, wh, mult)
    assert got.shape == want.shape
    assert T.bit_mismatches(got, want) == 0


def run_pool_nd(gpu, x, windows, fm_window=1, entry_window=1, mult=1.0, expect=0):
    """windows: per spatial dimension, x first"""
    dims = list(x.shape[2:])[::-1]
    out_dims = [d // w for d, w in zip(dims, windows)]
    out_shape = (x.shape[0] // entry_window, x.shape[1] // fm_window) + tuple(out_dims[::-1])
    d_in = gpu.to_device(x)
    d_out = gpu.torch.full((max(1, int(np.prod(out_shape))),), float("nan"), dtype=gpu.torch.float32, device=gpu.device)
    u32 = lambda v: (ctypes.c_uint32 * len(v))(*v)
    rc = gpu.lib.nnf_hip_average_subsampling_nd_forward(gpu.stream, d_out.data_ptr(), d_in.data_ptr(), x.shape[0] // entry_window, x.shape[1],
                                                        len(dims), u32(dims), u32(windows), fm_window, entry_window, mult)
    assert rc == expect, capi.error_string(rc)
    return gpu.to_host(d_out, out_shape) if expect == 0 else None


@pytest.mark.parametrize("shape,windows,fm_window,entry_window", [
    ((3, 4, 37), [4], 1, 1),                        # 1-D: the staged 2-D kernel
    ((2, 3, 12, 10), [2, 3], 1, 1),                 # 2-D: the staged 2-D kernel
    ((2, 6, 12, 10), [2, 3], 3, 1),                 # windows over feature maps
    ((6, 4, 8, 8), [2, 2], 1, 2),                   # windows over entries
    ((6, 9, 5, 7), [2, 2], 3, 3),                   # both, with margins
    ((2, 3, 6, 7, 8), [2, 3, 2], 1, 1),             # 3-D
    ((4, 4, 3, 4, 5, 6), [2, 2, 2, 3], 2, 2),       # 4-D with feature-map and entry windows
    ((2, 8, 9), [3], 4, 1),                         # 1-D with feature-map windows
    ((3, 5, 1, 1), [1, 1], 5, 3),                   # pure feature-map / entry averaging
    ((8, 6, 16, 16), [1, 1], 1, 4),                 # windows over entries only: whole entries folded as rows of float4
    ((4, 13, 16, 20), [1, 1], 3, 2),                # planes as rows, a feature map left over
    ((6, 12, 9, 10), [1, 1], 1, 3),                 # planes of 90 values, entries of 1080: rows of float4 all the same
    ((6, 12, 9, 10), [1, 1], 4, 1),                 # ... but not with a window over feature maps: one lane per output
    ((2, 4, 4, 4, 4, 4), [1, 1, 1, 1], 2, 2),       # 4-D, windows of 1
])
def test_average_subsampling_in_the_full_form(gpu, shape, windows, fm_window, entry_window):
    x = T.normal(T.rng(17, sum(shape) + fm_window), shape)
    mult = oracle.average_subsampling_full_mult(windows, fm_window, entry_window)
    want = oracle.average_subsampling(x, windows, feature_map_window=fm_window, entry_window=entry_window, mult=mult)
    got = run_pool_nd(gpu, x, windows, fm_window, entry_window, mult)
    assert got.shape == want.shape
    assert T.bit_mismatches(got, want) == 0


def test_average_subsampling_full_form_rejects_bad_arguments(gpu):
    x = T.normal(T.rng(17, 99), (2, 4, 6, 6, 6))
    run_pool_nd(gpu, x, [7, 2, 2], expect=capi.E_INVAL)          # window larger than the input
    run_pool_nd(gpu, x, [2, 2, 2], fm_window=5, expect=capi.E_INVAL)   # more feature maps per window than there are
    d = gpu.to_device(x)
    u32 = lambda v: (ctypes.c_uint32 * len(v))(*v)
    call = gpu.lib.nnf_hip_average_subsampling_nd_forward
    assert call(gpu.stream, d.data_ptr(), d.data_ptr(), 2, 4, 3, u32([6, 6, 6]), u32([2, 2, 2]), 1, 1, 1.0) == capi.E_OVERLAP
    assert call(gpu.stream, d.data_ptr(), d.data_ptr(), 2, 4, 5, u32([6] * 5), u32([2] * 5), 1, 1, 1.0) == capi.E_UNSUPPORTED
    assert call(gpu.stream, None, d.data_ptr(), 2, 4, 3, u32([6, 6, 6]), u32([2, 2, 2]), 1, 1, 1.0) == capi.E_INVAL
    gpu.torch.cuda.synchronize()


# ---------------------------------------------------------------------------------------------
# every fp32 input through the layers that call expf and divide
# ---------------------------------------------------------------------------------------------

def test_exp_layers_over_the_whole_fp32_range(gpu):
    """ELU, Sigmoid and TanH against the oracle on a regular sweep of ALL fp32 bit patterns (every
    61st by default, every single one with NNF_EXHAUSTIVE=1): the device expf and the device's
    short division sequence must reproduce libm's expf and IEEE division bit for bit, including
    the inputs where expf under- or overflows and where the quotient is subnormal."""
    import os

    stride = 1 if os.environ.get("NNF_EXHAUSTIVE") == "1" else 61
    chunk = 1 << 26
    lib = gpu.lib
    total_bad = 0
    checked = 0
    for start in range(0, 1 << 32, chunk * stride):
        bits = np.arange(start, min(start + chunk * stride, 1 << 32), stride, dtype=np.uint64).astype(np.uint32)
        x = bits.view(np.float32)
        with np.errstate(all="ignore"):
            cases = [
                (run_flat(gpu, lib.nnf_hip_exponential_linear_forward, x), oracle.exponential_linear(x), "elu"),
                (run_flat(gpu, lib.nnf_hip_sigmoid_forward, x), oracle.sigmoid(x), "sigmoid"),
                # steepness 0.5: the exponent argument is x itself, so e runs over the whole image of expf
                (run_flat(gpu, lib.nnf_hip_hyperbolic_tangent_forward, x, 1.0, 0.5), oracle.hyperbolic_tangent(x, 1.0, 0.5), "tanh"),
            ]
        for got, want, what in cases:
            bad = T.bit_mismatches(got, want)
            assert bad == 0, "%s: %d mismatches in the chunk starting at bit pattern 0x%08x" % (what, bad, start)
            total_bad += bad
        checked += x.size
    print("exp layers: %d inputs per layer checked, %d mismatches" % (checked, total_bad))


def test_device_expf_against_the_golden_vectors(gpu):
    """The device's ELU, Sigmoid and TanH on the 8192 inputs of tests/golden/expf_vectors.npy against the reference's
    formulas applied to the recorded glibc expf values: no host libm is involved when this runs."""
    x, e = T.golden_expf()
    elu, sig, tanh = T.layers_from_golden_expf(x, e)
    shape = (1, 1, x.size)
    assert T.bit_mismatches(gpu.chain(shape, [[(ELU,)]], [], [x.reshape(shape)]), elu) == 0
    assert T.bit_mismatches(gpu.chain(shape, [[(SIGMOID,)]], [], [(-x).reshape(shape)]), sig) == 0
    assert T.bit_mismatches(gpu.chain(shape, [[(TANH, 0, 1.0, 0.5)]], [], [x.reshape(shape)]), tanh) == 0


def test_short_division_sequences_equal_ieee_division_for_every_denominator(gpu):
    """The device's own sweep over every non-negative float e with e + 1 <= 2^126 (2^31 values): the
    reciprocal sequence of Sigmoid and the quotient sequence of TanH return the bits of IEEE division."""
    counts = gpu.torch.zeros(2, dtype=gpu.torch.int64, device=gpu.device)
    rc = gpu.lib.nnf_hip_check_division_sequences(gpu.stream, counts.data_ptr())
    assert rc == 0, capi.error_string(rc)
    gpu.torch.cuda.synchronize()
    assert counts.tolist() == [0, 0]


def test_largest_tensor_the_kernels_index(gpu):
    """0xFFFF0000 elements (65535 x 256 x 256, 17 GB): the largest count the 32-bit tile arithmetic
    accepts. The CPU oracle would need minutes and tens of GB for it, so the check is a size-independent
    one: batch norm -> ReLU is two fp32 roundings per element, which plain device tensor arithmetic
    reproduces exactly (multiply, add and maximum as separate operations), compared on the device
    over the whole tensor, in place, plus the oracle on the first and the last entries."""
    torch = gpu.torch
    free, _ = torch.cuda.mem_get_info()
    n, c, plane = 65535, 256, 256
    total = n * c * plane
    assert total == 0xFFFF0000
    if free < 3.2 * 4 * total:
        pytest.skip("needs about 55 GB of free device memory")
    gen = torch.Generator(device=gpu.device)
    gen.manual_seed(20)
    x = torch.randn(total, generator=gen, device=gpu.device, dtype=torch.float32)
    g, b, m, s = T.bn_params(T.rng(20, 1), c)
    head = x[: 2 * c * plane].cpu().numpy().reshape(2, c, plane)
    tail = x[-2 * c * plane:].cpu().numpy().reshape(2, c, plane)
    d_w = [gpu.to_device(v) for v in (g, b, m, s)]
    mult = d_w[0] * d_w[3]
    add = d_w[1] - mult * d_w[2]
    want = x.view(n, c, plane) * mult.view(1, c, 1)
    want += add.view(1, c, 1)
    want = torch.where(want >= 0, want, want * 0.0)  # -0.0 for negative values, as the reference's x * 0.0F
    desc = capi.make_desc(n, c, plane, [[(BN, 0), (RELU, 0, 0.0)]], [])
    rc = gpu.lib.nnf_hip_chain_forward(gpu.stream, ctypes.byref(desc), x.data_ptr(), capi.pointer_array([x.data_ptr()]),
                                       capi.pointer_array([t.data_ptr() for t in d_w]))
    assert rc == 0, capi.error_string(rc)
    torch.cuda.synchronize()
    differing = int((x.view(torch.int32) != want.view(-1).view(torch.int32)).sum().item())
    assert differing == 0, "%d of %d elements differ from the device-side evaluation" % (differing, total)
    del want
    for got, src in ((x[: 2 * c * plane], head), (x[-2 * c * plane:], tail)):
        ref = oracle.rectified_linear(oracle.batch_norm(src, g, b, m, s), 0.0)
        assert T.bit_mismatches(got.cpu().numpy(), ref.reshape(-1)) == 0
    # one element more is refused before anything is launched
    desc = capi.make_desc(n, c, plane + 1, [[(RELU, 0, 0.0)]], [])
    assert gpu.lib.nnf_hip_chain_forward(gpu.stream, ctypes.byref(desc), x.data_ptr(), capi.pointer_array([x.data_ptr()]), None) == capi.E_TOOBIG
