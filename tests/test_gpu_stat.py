"""Per-feature-map statistics on the GPU (the state of nnForge's stat_data_bunch_writer) against the
oracle's sequential double-precision update. The device merges partial results instead of
updating value by value, so mean and m2 are compared as doubles with a tolerance of sqrt(n) units of
double rounding (what the sequential update itself accumulates), and the fp32 figures the reference derives from them (average,
std_dev) to one unit in the last place; count, min and max must be equal."""

import ctypes

import numpy as np
import pytest

import nnf_testing as T
import oracle
from nnforge_amd import capi

pytestmark = pytest.mark.gpu

F = np.float32


class DeviceStat:
    def __init__(self, gpu, c):
        self.gpu, self.c = gpu, c
        self.state = gpu.torch.zeros(c * 32, dtype=gpu.torch.uint8, device=gpu.device)
        assert gpu.lib.nnf_hip_feature_map_stat_init(gpu.stream, self.state.data_ptr(), c) == 0

    def write(self, x, expect=0):
        gpu = self.gpu
        n, c = x.shape[:2]
        plane = int(np.prod(x.shape[2:], dtype=np.int64))
        need = ctypes.c_size_t()
        assert gpu.lib.nnf_hip_feature_map_stat_workspace_bytes(n, c, plane, ctypes.byref(need)) == 0
        work = gpu.torch.empty(max(16, need.value), dtype=gpu.torch.uint8, device=gpu.device)
        d_x = gpu.to_device(x)
        rc = gpu.lib.nnf_hip_feature_map_stat_accumulate(gpu.stream, self.state.data_ptr(), work.data_ptr(), need.value, d_x.data_ptr(), n, c, plane)
        assert rc == expect, capi.error_string(rc)
        gpu.torch.cuda.synchronize()
        return self

    def host(self):
        self.gpu.torch.cuda.synchronize()
        return np.frombuffer(self.state.cpu().numpy().tobytes(), dtype=oracle.STAT_DTYPE)


def figures(state):
    with np.errstate(all="ignore"):
        return state["mean"].astype(F), np.sqrt((state["m2"] / state["n"]).astype(F))


def check(got, want, scale):
    assert np.array_equal(got["n"], want["n"])
    assert np.array_equal(got["min_val"], want["min_val"]) and np.array_equal(got["max_val"], want["max_val"])
    # Both sides round in double: the sequential update n times in a row (error growing like sqrt(n) roundings),
    # the device a handful of times per partial sum. Five orders of magnitude inside one fp32 rounding.
    n = want["n"]
    eps = 2.0 ** -53
    assert np.all(np.abs(got["mean"] - want["mean"]) <= 8 * np.sqrt(n) * eps * scale), np.abs(got["mean"] - want["mean"]).max()
    assert np.all(np.abs(got["m2"] - want["m2"]) <= 8 * np.sqrt(n) * eps * (want["m2"] + n * scale))
    g_avg, g_std = figures(got)
    w_avg, w_std = figures(want)
    assert T.ulp_distance(g_avg, w_avg).max() <= 1
    assert T.ulp_distance(g_std, w_std).max() <= 1


@pytest.mark.parametrize("shape", [
    (32, 64, 56, 56),      # config 0
    (64, 512, 7, 7),       # plane not a multiple of 4
    (256, 1000),           # no spatial dimensions
    (3, 5, 13, 3),
    (1, 1, 1),
    (2, 3, 300, 300),      # long planes: one entry per run, planes cut into segments
    (8, 3, 224, 224),      # statistics of input images: few planes, each cut into segments
    (1, 1, 100003),        # one long plane, not a multiple of 4: segments of single floats
    (3, 2, 16388),         # segments of unequal length
    (1000, 2, 4),          # many entries per run
])
def test_statistics_match_the_sequential_update(gpu, shape):
    gen = T.rng(70, sum(shape))
    c = shape[1]
    x = (T.normal(gen, shape, 2.0) + (np.arange(c, dtype=F) * F(3.0)).reshape((1, c) + (1,) * (len(shape) - 2))).astype(F)
    got = DeviceStat(gpu, c).write(x).host()
    want = oracle.FeatureMapStat(c).write(x).state
    check(got, want, scale=3.0 * c + 10.0)


def test_statistics_accumulate_over_packets(gpu):
    gen = T.rng(71, 0)
    c = 24
    x = T.normal(gen, (50, c, 14, 14), 1.5)
    dev = DeviceStat(gpu, c)
    for a, b in ((0, 16), (16, 17), (17, 50)):
        dev.write(x[a:b])
    want = oracle.FeatureMapStat(c).write(x).state
    check(dev.host(), want, scale=10.0)
    # zero entries change nothing
    before = dev.host().tobytes()
    dev.write(x[:0])
    assert dev.host().tobytes() == before


@pytest.mark.parametrize("c,plane,packet,n", [(256, 49, 12, 19), (64, 49, 29, 45), (512, 16, 20, 33)])
def test_short_last_packet_fits_the_workspace_of_a_full_one(gpu, c, plane, packet, n):
    """More workgroups than the device holds at once (feature maps x entries > 1792) and a last packet that would
    rather be cut into more runs than the full packet was: the workspace sized for the full packet must do."""
    gen = T.rng(74, c + n)
    x = T.normal(gen, (n, c, plane), 1.5)
    need = ctypes.c_size_t()
    assert gpu.lib.nnf_hip_feature_map_stat_workspace_bytes(packet, c, plane, ctypes.byref(need)) == 0
    work = gpu.torch.empty(need.value, dtype=gpu.torch.uint8, device=gpu.device)
    dev = DeviceStat(gpu, c)
    for first in range(0, n, packet):
        part = gpu.to_device(x[first:first + packet])
        rc = gpu.lib.nnf_hip_feature_map_stat_accumulate(gpu.stream, dev.state.data_ptr(), work.data_ptr(), need.value, part.data_ptr(),
                                                         min(packet, n - first), c, plane)
        assert rc == 0, capi.error_string(rc)
    want = oracle.FeatureMapStat(c).write(x).state
    check(dev.host(), want, scale=10.0)


def test_statistics_of_a_large_offset_and_of_constants(gpu):
    gen = T.rng(72, 0)
    x = (F(1000.0) + T.normal(gen, (64, 4, 28, 28), 0.01)).astype(F)
    got = DeviceStat(gpu, 4).write(x).host()
    want = oracle.FeatureMapStat(4).write(x).state
    # the deviation is 1e5 times smaller than the mean: sums of raw squares would lose it
    assert np.allclose(got["m2"], want["m2"], rtol=1e-9, atol=0)
    g_avg, g_std = figures(got)
    w_avg, w_std = figures(want)
    assert T.ulp_distance(g_avg, w_avg).max() <= 1 and T.ulp_distance(g_std, w_std).max() <= 1
    const = np.full((8, 3, 5, 5), -2.75, F)
    got = DeviceStat(gpu, 3).write(const).host()
    assert np.all(got["mean"] == -2.75) and np.all(got["m2"] == 0.0) and np.all(got["min_val"] == F(-2.75)) and np.all(got["max_val"] == F(-2.75))


def test_statistics_ignore_nan_in_min_max_only(gpu):
    x = T.normal(T.rng(73, 0), (4, 2, 8, 8))
    x[1, 0, 3, 3] = np.nan
    got = DeviceStat(gpu, 2).write(x).host()
    want = oracle.FeatureMapStat(2).write(x).state
    assert np.isnan(got["mean"][0]) and np.isnan(want["mean"][0])
    assert got["min_val"][0] == want["min_val"][0] and got["max_val"][0] == want["max_val"][0]
    assert abs(got["mean"][1] - want["mean"][1]) < 1e-13


def test_statistics_reject_bad_arguments(gpu):
    lib, s = gpu.lib, gpu.stream
    state = gpu.torch.zeros(64 * 32, dtype=gpu.torch.uint8, device=gpu.device)
    x = gpu.to_device(np.zeros(4096, F))
    work = gpu.torch.zeros(1 << 16, dtype=gpu.torch.uint8, device=gpu.device)
    assert lib.nnf_hip_feature_map_stat_init(s, None, 4) == capi.E_INVAL
    assert lib.nnf_hip_feature_map_stat_init(s, state.data_ptr(), 0) == capi.E_INVAL
    # workspace missing or too small
    assert lib.nnf_hip_feature_map_stat_accumulate(s, state.data_ptr(), None, 0, x.data_ptr(), 4, 4, 256) == capi.E_INVAL
    assert lib.nnf_hip_feature_map_stat_accumulate(s, state.data_ptr(), work.data_ptr(), 16, x.data_ptr(), 4, 4, 256) == capi.E_INVAL
    assert lib.nnf_hip_feature_map_stat_accumulate(s, state.data_ptr(), work.data_ptr(), 1 << 16, x.data_ptr() + 4, 4, 4, 255) == capi.E_ALIGN
    assert lib.nnf_hip_feature_map_stat_accumulate(s, state.data_ptr(), work.data_ptr(), 1 << 16, x.data_ptr(), 4, 0, 256) == capi.E_INVAL
    gpu.torch.cuda.synchronize()


def test_statistics_keep_subnormal_minimum_and_maximum(gpu):
    """min / max go through the hardware's fp32 minimum / maximum: subnormal values must come back as they are."""
    tiny = np.array([1, 5, 77, 0x7FFFFF, 0x80000003, 0x80000009], dtype=np.uint32).view(F)   # +-subnormals
    x = np.tile(tiny, 40).reshape(2, 1, 120).astype(F)
    got = DeviceStat(gpu, 1).write(x).host()
    want = oracle.FeatureMapStat(1).write(x).state
    assert got["min_val"].tobytes() == want["min_val"].tobytes() and got["max_val"].tobytes() == want["max_val"].tobytes()
    assert got["min_val"][0] == np.array([0x80000009], dtype=np.uint32).view(F)[0]
    assert got["max_val"][0] == np.array([0x7FFFFF], dtype=np.uint32).view(F)[0]
