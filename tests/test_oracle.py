"""Pins the CPU oracle (oracle/nnf_oracle.c) without the reference running.

The reference has no tests, golden vectors or fixtures, and its sources do not compile in this
image (Boost and protobuf-generated headers are absent). Each oracle function is therefore pinned
against an independent evaluation chosen so that a plausible slip (dropped term, wrong sign or
index, transposed layout, fused multiply-add, wrong summation order) fails:
  * numpy fp32 arithmetic, one rounding per operation, for batch norm / ReLU / PReLU / Add /
    average subsampling: bit-for-bit equality;
  * fp64 closed forms (expm1, logistic, tanh, softmax) with explicit error budgets for the layers
    that call expf;
  * identities and brute-force index checks with a distinct value in every element.
"""

import numpy as np
import pytest

import nnf_testing as T
import oracle

F = np.float32


def bits_equal(a, b):
    return T.bit_mismatches(a, b) == 0


def test_batch_norm_matches_per_operation_fp32_and_layout():
    gen = T.rng(20, 0)
    n, c, plane = 3, 5, 7
    x = T.normal(gen, (n, c, plane), 3.0)
    g, b, m, s = T.bn_params(gen, c)
    got = oracle.batch_norm(x, g, b, m, s)
    mult = (g * s).astype(F)                      # one rounding
    add = (b - (mult * m).astype(F)).astype(F)    # product rounded, then the difference
    want = ((x * mult[None, :, None]).astype(F) + add[None, :, None]).astype(F)
    assert bits_equal(got, want)
    # a fused multiply-add would differ somewhere on this much data
    big = T.normal(gen, (4, c, 4096), 3.0)
    fused = (big.astype(np.float64) * mult[None, :, None].astype(np.float64) + add[None, :, None].astype(np.float64)).astype(F)
    assert T.bit_mismatches(oracle.batch_norm(big, g, b, m, s), fused) > 0
    # the fourth chunk is used as an inverse standard deviation as is: doubling it doubles mult
    got2 = oracle.batch_norm(x, g, b, np.zeros(c, F), (2 * s).astype(F))
    assert bits_equal(got2, ((x * (g * (2 * s).astype(F)).astype(F)[None, :, None]).astype(F) + b[None, :, None]).astype(F))


def test_batch_norm_identity_and_gamma_zero():
    x = T.normal(T.rng(20, 1), (2, 4, 9), 5.0)
    one, zero = np.ones(4, F), np.zeros(4, F)
    assert np.array_equal(oracle.batch_norm(x, one, zero, zero, one), x)
    beta = np.array([1.5, -2.0, 0.25, 7.0], F)
    got = oracle.batch_norm(x, zero, beta, T.normal(T.rng(20, 2), 4), one)
    assert np.array_equal(got, np.broadcast_to(beta[None, :, None], x.shape))


def test_batch_norm_feature_map_indexing_brute_force():
    n, c, plane = 2, 3, 4
    x = np.arange(n * c * plane, dtype=F).reshape(n, c, plane)
    g = np.array([1, 10, 100], F)
    b = np.array([0.5, 0.25, 0.125], F)
    m = np.array([1, 2, 3], F)
    s = np.array([1, 0.5, 0.25], F)
    got = oracle.batch_norm(x, g, b, m, s)
    for e in range(n):
        for f in range(c):
            for p in range(plane):
                mult = F(g[f] * s[f])
                assert got[e, f, p] == F(F(x[e, f, p] * mult) + F(b[f] - F(mult * m[f])))


def test_rectified_linear():
    x = np.array([-2.0, -0.0, 0.0, 3.0, np.nan, -np.inf, np.inf, -1e-45], F)
    got = oracle.rectified_linear(x, 0.0)
    assert np.array_equal(got[[2, 3, 6]], x[[2, 3, 6]])
    assert got[0] == 0 and np.signbit(got[0])            # x * 0.0F keeps the sign: -0.0
    assert got[1] == 0 and np.signbit(got[1])            # -0.0 >= 0 is true: passes through
    assert np.isnan(got[4]) and np.isnan(got[5])         # -inf * 0 = NaN, as in the reference
    y = T.normal(T.rng(21, 0), 1000, 2.0)
    assert bits_equal(oracle.rectified_linear(y, 0.1), np.where(y >= 0, y, (y * F(0.1)).astype(F)))
    once = oracle.rectified_linear(y, 0.0)
    assert bits_equal(oracle.rectified_linear(once, 0.0), once)  # idempotent


def test_parametric_rectified_linear():
    gen = T.rng(22, 0)
    n, c, plane = 3, 4, 5
    x = T.normal(gen, (n, c, plane), 2.0)
    a = np.array([0.25, 0.0, 1.0, -0.5], F)
    got = oracle.parametric_rectified_linear(x, a)
    want = (x * np.where(x >= 0, F(1.0), a[None, :, None])).astype(F)
    assert bits_equal(got, want)
    assert np.array_equal(got[:, 2], x[:, 2])                                  # a = 1: identity
    relu = oracle.rectified_linear(x, 0.0)
    assert np.array_equal(got[:, 1], relu[:, 1])                                # a = 0: ReLU (signed zeros compare equal)


def test_exponential_linear_against_fp64():
    x = np.concatenate([T.normal(T.rng(23, 0), 20000, 9.0), np.array([0.0, -0.0, 50.0, -50.0, -1e-8, -104.0, -200.0], F)]).astype(F)
    got = oracle.exponential_linear(x).astype(np.float64)
    x64 = x.astype(np.float64)
    truth = np.where(x64 >= 0, x64, np.expm1(x64))
    # expf is within 1 ULP of exp; expf(x) - 1 then rounds once more: error <= ulp(1)/2 + ulp(result)
    assert np.all(np.abs(got - truth) <= 2.0 ** -24 * 1.5 + 2.0 ** -23 * np.abs(truth))
    assert oracle.exponential_linear(np.array([-50.0], F))[0] == -1.0
    assert oracle.exponential_linear(np.array([0.0], F))[0] == 0.0
    pos = x[x >= 0]
    assert np.array_equal(oracle.exponential_linear(pos), pos)
    # expf(x) - 1, not expm1f: for tiny negative x the result is exactly 0 or -2^-24, never x itself
    assert oracle.exponential_linear(np.array([-1e-8], F))[0] in (0.0, F(-2.0 ** -24))


def test_sigmoid_against_fp64():
    x = np.concatenate([T.normal(T.rng(24, 0), 20000, 16.0), np.array([0.0, 50.0, -50.0, 88.0, -88.0, 104.0, -104.0], F)]).astype(F)
    got = oracle.sigmoid(x)
    truth = 1.0 / (1.0 + np.exp(-x.astype(np.float64)))
    assert np.all(np.abs(got.astype(np.float64) - truth) <= 3 * 2.0 ** -24 * np.maximum(truth, 2.0 ** -126))
    assert oracle.sigmoid(np.array([0.0], F))[0] == 0.5
    assert oracle.sigmoid(np.array([50.0], F))[0] == 1.0
    assert oracle.sigmoid(np.array([-104.0], F))[0] == 0.0       # expf overflows to inf: 1/inf
    # sigma(-x) = 1 - sigma(x) up to rounding
    s_pos, s_neg = oracle.sigmoid(x).astype(np.float64), oracle.sigmoid(-x).astype(np.float64)
    assert np.all(np.abs(s_pos + s_neg - 1.0) <= 2.0 ** -22)


def test_hyperbolic_tangent_against_fp64():
    x = np.concatenate([T.normal(T.rng(25, 0), 20000, 4.0), np.array([0.0, 1.0, -1.0, 20.0, -20.0], F)]).astype(F)
    for scale, steep in ((1.0, 1.0), (1.7159, 0.6666), (1.7159, 0.666666)):
        got = oracle.hyperbolic_tangent(x, scale, steep).astype(np.float64)
        steep2 = F(F(steep) * F(2.0))
        arg = (x * steep2).astype(F).astype(np.float64)
        truth = np.tanh(arg / 2.0) * float(F(scale))
        # (e - 1) loses relative accuracy near 0: absolute floor of a few ulp(1) times the scale
        assert np.all(np.abs(got - truth) <= 4 * 2.0 ** -24 * scale + 4 * 2.0 ** -24 * np.abs(truth))
        assert oracle.hyperbolic_tangent(np.array([0.0], F), scale, steep)[0] == 0.0
    # odd function up to rounding; saturates at +-scale; overflow of expf gives NaN (inf/inf) as in the reference
    y = oracle.hyperbolic_tangent(np.array([30.0, -30.0, 100.0], F), 1.7159, 0.6666)
    assert y[0] == F(1.7159) and y[1] == -F(1.7159) and np.isnan(y[2])


def test_add_order_alpha_and_signed_zero():
    gen = T.rng(26, 0)
    xs = [T.normal(gen, 5000, 100.0) for _ in range(4)]
    got = oracle.add(xs, 0.5)
    acc = np.zeros(5000, F)
    for x in xs:
        acc = (acc + x).astype(F)
    assert bits_equal(got, (acc * F(0.5)).astype(F))
    # summation is left to right: a different order changes bits somewhere
    assert T.bit_mismatches(oracle.add(xs[::-1], 0.5), got) > 0
    # two inputs commute; adding zeros is the identity times alpha
    assert bits_equal(oracle.add(xs[:2]), oracle.add(xs[1::-1]))
    assert bits_equal(oracle.add([xs[0], np.zeros(5000, F)], 3.0), (xs[0] * F(3.0)).astype(F))
    # the sum starts from +0.0F: -0 + -0 comes out as +0
    z = oracle.add([np.array([-0.0], F), np.array([-0.0], F)])
    assert z[0] == 0 and not np.signbit(z[0])


def softmax_truth(x):
    # x - max is an fp32 subtraction in the reference (its rounding is part of the definition);
    # everything after it in fp64
    d = (x - x.max(axis=1, keepdims=True)).astype(F).astype(np.float64)
    e = np.exp(d)
    return e / e.sum(axis=1, keepdims=True)


@pytest.mark.parametrize("shape", [(4, 1000, 1), (3, 7, 5), (2, 10, 4, 3), (1, 1, 6)])
def test_softmax_against_fp64(shape):
    gen = T.rng(27, sum(shape))
    x = T.normal(gen, shape, 4.0)
    x[gen.random(shape) < 0.01] = 30.0
    got = oracle.softmax(x)
    truth = softmax_truth(x)
    c = shape[1]
    assert np.all(np.abs(got - truth) <= (c + 8) * 2.0 ** -24 * truth + 1e-45)
    assert np.all(np.abs(got.astype(np.float64).sum(axis=1) - 1.0) <= c * 2.0 ** -24)


def test_softmax_layout_shift_and_special_cases():
    # feature maps are strided by the plane size: softmax of [n][c][p] equals row softmax of the transposed data
    x = T.normal(T.rng(27, 100), (3, 6, 5), 3.0)
    rows = np.ascontiguousarray(x.transpose(0, 2, 1)).reshape(15, 6, 1)
    assert bits_equal(oracle.softmax(x).transpose(0, 2, 1).reshape(15, 6, 1), oracle.softmax(rows))
    # shift invariance with an exactly representable shift
    r = ((np.arange(100, dtype=F) - 50) * F(0.5)).reshape(1, 100, 1)
    assert bits_equal(oracle.softmax(r), oracle.softmax(r + F(64.0)))
    # uniform input: every exponential is exactly 1, sum = C, result = fl(1/C)
    u = oracle.softmax(np.full((2, 100, 1), 5.0, F))
    assert np.all(u == F(1.0) / F(100.0))
    # the maximum starts from -1.0e37F: rows entirely below it give sum 0 -> 0 * inf = NaN
    assert np.isnan(oracle.softmax(np.full((1, 4, 1), -3.0e38, F))).all()
    # a NaN is skipped by the max but poisons the sum
    n = np.zeros((1, 5, 1), F)
    n[0, 2] = np.nan
    assert np.isnan(oracle.softmax(n)).all()
    # multiply by the reciprocal of a left-to-right fp32 sum: with exponentials that are exact powers
    # of two the whole computation can be redone by hand in fp32
    ln2 = F(0.6931472)
    k = np.array([0, -1, -2, -3, -1, -5, -2, 0, -7, -1], F)
    with np.errstate(all="ignore"):
        y = (k * ln2).astype(F).reshape(1, -1, 1)
    got = oracle.softmax(y).reshape(-1)
    e = oracle.exponential_linear(np.minimum(y.reshape(-1), F(-1e-30))) + F(1.0)  # expf(y) for y < 0 via the ELU oracle
    e = np.where(y.reshape(-1) < 0, e, F(1.0)).astype(F)
    acc = F(0.0)
    for v in e:
        acc = F(acc + v)
    want = (e * F(F(1.0) / acc)).astype(F)
    assert T.ulp_distance(got, want).max() <= 1


def test_average_subsampling_brute_force_and_multipliers():
    # distinct value per element, windows 3 (x) by 2 (y): every output is the ordered sum of its own window
    n, c, h, w = 2, 3, 4, 9
    x = T.normal(T.rng(28, 0), (n, c, h, w), 10.0)
    mult = F(0.7)
    got = oracle.average_subsampling(x, [3, 2], mult=float(mult))
    assert got.shape == (n, c, 2, 3)
    for e in range(n):
        for f in range(c):
            for oy in range(2):
                for ox in range(3):
                    s = F(0.0)
                    for wy in range(2):          # y outer, x inner: x is the fastest dimension of the window walk
                        for wx in range(3):
                            s = F(s + x[e, f, oy * 2 + wy, ox * 3 + wx])
                    assert got[e, f, oy, ox] == F(s * mult)
    # a leftover margin is ignored (output size = input size / window, rounded down)
    y = T.normal(T.rng(28, 1), (1, 1, 5, 7))
    g2 = oracle.average_subsampling(y, [3, 2], mult=1.0)
    assert g2.shape == (1, 1, 2, 2)
    assert g2[0, 0, 1, 1] == F(F(F(F(F(F(y[0, 0, 2, 3] + y[0, 0, 2, 4]) + y[0, 0, 2, 5]) + y[0, 0, 3, 3]) + y[0, 0, 3, 4]) + y[0, 0, 3, 5]))
    # constant input, 7x7 global window: 49 * v * mult
    const = np.full((2, 8, 7, 7), 0.5, F)
    assert np.all(oracle.average_subsampling(const, [7, 7], mult=1.0) == F(24.5))
    # the plain tester's own multiplier without an alpha is 1 (it returns the window SUM);
    # the full-configuration rule gives 1/49; an explicit alpha wins in both
    assert np.all(oracle.average_subsampling(const, [7, 7]) == F(24.5))
    assert oracle.average_subsampling_full_mult([7, 7]) == F(1.0) / F(49.0)
    assert oracle.average_subsampling_full_mult([7, 7], alpha=0.25) == F(0.25)
    assert np.all(oracle.average_subsampling(const, [7, 7], alpha=0.25) == F(24.5 * 0.25))


def test_average_subsampling_feature_map_and_entry_windows():
    n, c, h, w = 4, 6, 2, 2
    x = T.normal(T.rng(28, 2), (n, c, h, w), 3.0)
    got = oracle.average_subsampling(x, [2, 1], feature_map_window=3, entry_window=2, mult=1.0)
    assert got.shape == (2, 2, 2, 1)
    for oe in range(2):
        for of in range(2):
            for oy in range(2):
                s = F(0.0)
                for we in range(2):              # entries slowest, then feature maps, then x
                    for wf in range(3):
                        for wx in range(2):
                            s = F(s + x[oe * 2 + we, of * 3 + wf, oy, wx])
                assert got[oe, of, oy, 0] == s
    # plain multiplier without alpha: 1 / (feature-map window * entry window)
    got = oracle.average_subsampling(x, [2, 1], feature_map_window=3, entry_window=2)
    ref = oracle.average_subsampling(x, [2, 1], feature_map_window=3, entry_window=2, mult=float(F(1.0) / F(6.0)))
    assert bits_equal(got, ref)


# ---- neighbouring testers: absolute, dropout, concat, maxout, max subsampling ------------------

def fold_max(values, start=None, new_first=False):
    """std::max folded over values the way the testers write it. new_first: std::max(new, current)
    (maxout); otherwise std::max<float>(current, new) (max subsampling). std::max(a, b) = (a < b) ? b : a."""
    cur = start
    for v in values:
        if cur is None:
            cur = v
            continue
        a, b = (v, cur) if new_first else (cur, v)
        cur = b if a < b else a
    return cur


def test_absolute_dropout():
    x = T.normal(T.rng(40, 0), (3, 4, 5, 6), 5.0)
    x.reshape(-1)[:4] = [-0.0, 0.0, -np.inf, np.nan]
    got = oracle.absolute(x)
    assert bits_equal(got, np.abs(x))
    assert np.signbit(got).sum() == 0
    d = oracle.dropout(x)
    assert bits_equal(d, x) and d is not x
    y = x.copy()
    assert oracle.dropout(y, out=y) is y and bits_equal(y, x)   # in place: nothing moves


def test_concat_joins_feature_maps_per_entry():
    gen = T.rng(41, 0)
    parts = [T.normal(gen, (4, c, 3, 5)) for c in (2, 7, 1)]
    got = oracle.concat(parts)
    assert got.shape == (4, 10, 3, 5)
    assert bits_equal(got, np.concatenate(parts, axis=1))
    # no spatial dimensions, one input
    flat = [T.normal(gen, (6, 9))]
    assert bits_equal(oracle.concat(flat), flat[0])


def test_maxout_groups_strided_feature_maps():
    gen = T.rng(42, 0)
    n, c_out, k, h, w = 3, 4, 3, 2, 5
    x = T.normal(gen, (n, c_out * k, h, w), 2.0)
    got = oracle.maxout(x, k)
    assert got.shape == (n, c_out, h, w)
    # output map o covers input maps o, o + c_out, o + 2 c_out (not o*k .. o*k + k - 1)
    want = x.reshape(n, k, c_out, h, w).max(axis=1)
    assert bits_equal(got, want)
    assert not bits_equal(got, x.reshape(n, c_out, k, h, w).max(axis=2))
    # ties and unordered values: std::max(new, current) keeps the NEW value unless new < current
    special = np.zeros((1, 3, 1, 4), F)
    special[0, :, 0, 0] = [0.0, -0.0, 0.0]          # -> last +0.0
    special[0, :, 0, 1] = [0.0, 0.0, -0.0]          # -> -0.0
    special[0, :, 0, 2] = [np.nan, 1.0, 0.5]        # nan replaced by 1.0, 0.5 < 1.0 keeps 1.0
    special[0, :, 0, 3] = [1.0, np.nan, 0.5]        # nan wins over 1.0, then 0.5 replaces nan
    g = oracle.maxout(special, 3)[0, 0, 0]
    for col in range(4):
        want_v = fold_max([F(v) for v in special[0, :, 0, col]], new_first=True)
        assert g[col].tobytes() == F(want_v).tobytes(), col
    assert np.signbit(g[1]) and not np.signbit(g[0]) and g[2] == 1.0 and g[3] == 0.5


def window_view_max(x, windows, strides, is_min=False):
    """Independent evaluation with numpy's sliding windows; windows/strides in numpy axis order
    (spatial axes of x after [N][C])."""
    from numpy.lib.stride_tricks import sliding_window_view
    axes = tuple(range(2, x.ndim))
    v = sliding_window_view(x, tuple(windows), axis=axes)
    index = (slice(None), slice(None)) + tuple(slice(None, None, s) for s in strides)
    v = v[index]
    red = tuple(range(x.ndim, x.ndim + len(windows)))
    return v.min(axis=red) if is_min else v.max(axis=red)


@pytest.mark.parametrize("shape,windows,strides", [
    ((2, 3, 9, 11), (3, 3), (2, 2)),      # the ResNet pool1 pattern: 3x3 every 2
    ((2, 3, 8, 12), (2, 2), (2, 2)),
    ((1, 2, 7, 10), (3, 2), (1, 3)),      # y window 3 stride 1, x window 2 stride 3
    ((2, 2, 13), (4,), (3,)),             # 1-D
    ((1, 2, 5, 6, 7), (2, 3, 2), (2, 2, 1)),   # 3-D
])
@pytest.mark.parametrize("is_min", [False, True])
def test_max_subsampling_against_sliding_windows(shape, windows, strides, is_min):
    x = T.normal(T.rng(43, len(shape)), shape, 3.0)
    # oracle takes nnForge order (x first): reverse
    got = oracle.max_subsampling(x, list(windows)[::-1], strides=list(strides)[::-1], is_min=is_min)
    want = window_view_max(x, windows, strides, is_min)
    assert got.shape == want.shape
    assert bits_equal(got, want)


def test_max_subsampling_default_stride_is_the_window_and_margin_is_dropped():
    x = T.normal(T.rng(43, 100), (2, 2, 7, 9))
    got = oracle.max_subsampling(x, [2, 3])         # x window 2, y window 3
    assert got.shape == (2, 2, 2, 4)
    assert bits_equal(got, window_view_max(x, (3, 2), (3, 2)))


def test_max_subsampling_round_up_skips_what_lies_outside():
    x = T.normal(T.rng(43, 101), (2, 3, 8, 8))
    got = oracle.max_subsampling(x, [3, 3], strides=[2, 2], round_ups=[True, True])
    assert got.shape == (2, 3, 4, 4)                # (8 + 2 - 3 + 2) / 2 = 4; without round up 3
    padded = np.full((2, 3, 9, 9), -np.inf, F)
    padded[:, :, :8, :8] = x
    assert bits_equal(got, window_view_max(padded, (3, 3), (2, 2)))
    assert oracle.max_subsampling(x, [3, 3], strides=[2, 2]).shape == (2, 3, 3, 3)
    # round up in x only
    got = oracle.max_subsampling(x, [3, 3], strides=[2, 2], round_ups=[True, False])
    assert got.shape == (2, 3, 3, 4)
    assert bits_equal(got, window_view_max(padded[:, :, :8, :], (3, 3), (2, 2)))


def test_max_subsampling_feature_map_and_entry_windows():
    x = T.normal(T.rng(43, 102), (4, 6, 4, 6))
    got = oracle.max_subsampling(x, [2, 2], feature_map_window=3, entry_window=2)
    assert got.shape == (2, 2, 2, 3)
    # neighbouring feature maps f*3 .. f*3+2 and entries e*2, e*2+1 join the window
    want = x.reshape(2, 2, 2, 3, 2, 2, 3, 2).max(axis=(1, 3, 5, 7))
    assert bits_equal(got, want)


def test_max_subsampling_start_value_ties_and_nan():
    # the fold starts at -1e37 / +1e37: smaller / larger inputs never show
    x = np.full((1, 1, 2, 2), -3.0e38, F)
    assert np.all(oracle.max_subsampling(x, [2, 2]) == F(-1.0e37))
    assert np.all(oracle.max_subsampling(-x, [2, 2], is_min=True) == F(1.0e37))
    # std::max<float>(current, new): the first of equal values stays, NaN never enters
    x = np.array([[[[0.0, -0.0], [-0.0, 0.0]]]], F)
    assert not np.signbit(oracle.max_subsampling(x, [2, 2])[0, 0, 0, 0])
    assert np.signbit(oracle.max_subsampling(-x, [2, 2])[0, 0, 0, 0])
    x = np.array([[[[np.nan, 2.0], [np.nan, -5.0]]]], F)
    assert oracle.max_subsampling(x, [2, 2])[0, 0, 0, 0] == 2.0
    assert oracle.max_subsampling(x, [2, 2], is_min=True)[0, 0, 0, 0] == -5.0
    x = np.full((1, 1, 2, 2), np.nan, F)
    assert oracle.max_subsampling(x, [2, 2])[0, 0, 0, 0] == F(-1.0e37)
    # scan order x fastest: with windows 2 (x) by 2 (y) over +-0 the first zero met decides the sign
    x = np.array([[[[-1.0, -0.0], [0.0, -2.0]]]], F)
    want = fold_max([F(-1.0), F(-0.0), F(0.0), F(-2.0)], start=F(-1.0e37))
    assert oracle.max_subsampling(x, [2, 2])[0, 0, 0, 0].tobytes() == F(want).tobytes()
    assert np.signbit(want)


def test_max_subsampling_tiling_brute_force():
    # every input entry gives 2*3 output entries, one per shift of the window grid (x shift fastest)
    n, c, h, w = 2, 2, 11, 7
    x = T.normal(T.rng(43, 103), (n, c, h, w))
    wx, wy = 2, 3
    got = oracle.max_subsampling(x, [wx, wy], tiling=True)
    oh, ow = (h - (wy - 1)) // wy, (w - (wx - 1)) // wx
    assert got.shape == (n * wx * wy, c, oh, ow)
    for e in range(n):
        for sy in range(wy):
            for sx in range(wx):
                j = sy * wx + sx
                for f in range(c):
                    for oy in range(oh):
                        for ox in range(ow):
                            win = x[e, f, oy * wy + sy: oy * wy + sy + wy, ox * wx + sx: ox * wx + sx + wx]
                            assert got[e * wx * wy + j, f, oy, ox] == win.max()


# ---- per-feature-map statistics and the batch norm refresh ---------------------------------------

def test_feature_map_stat_against_two_pass_fp64():
    gen = T.rng(44, 0)
    n, c, h, w = 7, 5, 6, 9
    x = (T.normal(gen, (n, c, h, w), 2.0) + np.arange(c, dtype=F)[None, :, None, None] * F(10.0)).astype(F)
    stat = oracle.FeatureMapStat(c).write(x)
    per_fm = x.transpose(1, 0, 2, 3).reshape(c, -1).astype(np.float64)
    st = stat.state
    assert np.all(st["n"] == n * h * w)
    assert np.allclose(st["mean"], per_fm.mean(axis=1), rtol=1e-13, atol=0)
    assert np.allclose(st["m2"], ((per_fm - per_fm.mean(axis=1, keepdims=True)) ** 2).sum(axis=1), rtol=1e-12, atol=0)
    got = stat.get()
    assert np.array_equal(got["min"], per_fm.min(axis=1).astype(F)) and np.array_equal(got["max"], per_fm.max(axis=1).astype(F))
    assert T.ulp_distance(got["average"], per_fm.mean(axis=1).astype(F)).max() <= 1
    # population deviation (divides by n, not n - 1), rounded to fp32 BEFORE the square root
    want_std = np.sqrt(per_fm.var(axis=1).astype(F))
    assert T.ulp_distance(got["std_dev"], want_std).max() <= 1
    assert not np.allclose(got["std_dev"], per_fm.std(axis=1, ddof=1), rtol=1e-4, atol=0)
    # feature map f of entry e is x[e, f]: a transposed layout would mix the shifted means
    assert np.all(np.abs(got["average"] - np.arange(c) * 10.0) < 1.0)


def test_feature_map_stat_is_sequential_and_stable():
    gen = T.rng(44, 1)
    x = T.normal(gen, (12, 3, 50))
    whole = oracle.FeatureMapStat(3).write(x)
    parts = oracle.FeatureMapStat(3).write(x[:5]).write(x[5:6]).write(x[6:])
    assert whole.state.tobytes() == parts.state.tobytes()     # packets do not change the result
    # a large offset with a small spread: the single-pass update keeps the deviation
    y = (F(1000.0) + T.normal(gen, (64, 2, 100), 0.01)).astype(F)
    st = oracle.FeatureMapStat(2).write(y).get()
    per_fm = y.transpose(1, 0, 2).reshape(2, -1).astype(np.float64)
    assert np.allclose(st["std_dev"], per_fm.std(axis=1), rtol=1e-6, atol=0)
    # one value: deviation 0; no value: 0/0
    one = oracle.FeatureMapStat(1).write(np.full((1, 1, 1), 3.5, F)).get()
    assert one["average"][0] == F(3.5) and one["std_dev"][0] == 0.0 and one["min"][0] == F(3.5) and one["max"][0] == F(3.5)
    with np.errstate(all="ignore"):
        empty = oracle.FeatureMapStat(1).get()
    assert np.isnan(empty["std_dev"][0]) and empty["min"][0] == np.finfo(F).max and empty["max"][0] == -np.finfo(F).max


def test_feature_map_stat_min_max_follow_std_min_max():
    x = np.array([[[np.nan, 2.0, -0.0, 0.0, -7.0, np.nan]]], F)
    st = oracle.FeatureMapStat(1).write(x)
    got = st.get()
    assert got["min"][0] == F(-7.0) and got["max"][0] == F(2.0)     # NaN never enters min / max ...
    assert np.isnan(got["average"][0])                               # ... but poisons the mean
    zeros = oracle.FeatureMapStat(1).write(np.array([[[-0.0, 0.0]]], F)).get()
    assert np.signbit(zeros["min"][0]) and np.signbit(zeros["max"][0])   # the first of equal values stays


def test_update_bn_weights_formula_and_effect():
    gen = T.rng(44, 2)
    c = 6
    _, _, mean, inv_sigma = T.bn_params(gen, c)
    average, std_dev = T.normal(gen, (c,), 0.3), T.uniform(gen, c, 0.5, 2.0)
    new_mean, new_inv = oracle.update_bn_weights(mean, inv_sigma, average, std_dev)
    assert bits_equal(new_inv, (inv_sigma / std_dev).astype(F))
    assert bits_equal(new_mean, (mean + (average / inv_sigma).astype(F)).astype(F))
    # closed loop: statistics of the output with gamma 1, beta 0 -> refreshed weights -> mean 0, deviation 1
    x = (T.normal(gen, (40, c, 64), 3.0) + F(5.0)).astype(F)
    ones, zeros = np.ones(c, F), np.zeros(c, F)
    st = oracle.FeatureMapStat(c).write(oracle.batch_norm(x, ones, zeros, mean, inv_sigma)).get()
    m2, s2 = oracle.update_bn_weights(mean, inv_sigma, st["average"], st["std_dev"])
    after = oracle.FeatureMapStat(c).write(oracle.batch_norm(x, ones, zeros, m2, s2)).get()
    assert np.abs(after["average"]).max() < 1e-5 and np.abs(after["std_dev"] - 1.0).max() < 1e-5


def test_host_expf_is_the_function_the_golden_vectors_were_taken_from():
    """tests/golden/expf_vectors.npy holds glibc 2.35's expf on 8192 inputs (all exponents, the underflow and overflow
    edges, zeros, infinities, NaN). The oracle's ELU, Sigmoid and TanH call the host's expf: on these inputs they must
    return what the reference's formulas give for the recorded expf values, bit for bit - so a host with another expf
    would show up here instead of as a mysterious GPU mismatch."""
    x, e = T.golden_expf()
    elu, sig, tanh = T.layers_from_golden_expf(x, e)
    assert T.bit_mismatches(oracle.exponential_linear(x), elu) == 0
    assert T.bit_mismatches(oracle.sigmoid(-x), sig) == 0
    assert T.bit_mismatches(oracle.hyperbolic_tangent(x, 1.0, 0.5), tanh) == 0

