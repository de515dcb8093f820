"""nnf_hip_feature_map_stat_accumulate_static: the statistics reduction with its partial states in the library's own
fixed device array instead of a caller's workspace, for callers that cannot allocate. It shares the kernels of
nnf_hip_feature_map_stat_accumulate; given a workspace of the array's size that entry point makes the same plan, so the
two must agree bit for bit. Against the workspace entry point with the workspace it asks for itself (another cut into
runs, another merge order) the bar is the one of the statistics tests: count, min, max equal, mean and m2 to double
rounding, the fp32 figures derived from them to one unit in the last place."""

import ctypes

import numpy as np
import pytest

import nnf_testing as T
import oracle
from nnforge_amd import capi
from test_gpu_stat import check

pytestmark = pytest.mark.gpu

F = np.float32
SCRATCH_BYTES = 262144


def fresh_state(gpu, c):
    """n = 0, mean = 0, m2 = 0, min = FLT_MAX, max = -FLT_MAX, written from the host: the library's own init call
    is left out on purpose, so that in a fresh process the first static call has to find the array by itself."""
    host = np.zeros(c, dtype=oracle.STAT_DTYPE)
    host["min_val"] = np.finfo(F).max
    host["max_val"] = -np.finfo(F).max
    return gpu.torch.from_numpy(np.frombuffer(host.tobytes(), dtype=np.uint8).copy()).to(gpu.device)


def read_state(gpu, state):
    gpu.torch.cuda.synchronize()
    return np.frombuffer(state.cpu().numpy().tobytes(), dtype=oracle.STAT_DTYPE)


def with_workspace(gpu, state, d_x, n, c, plane, workspace_bytes=None):
    need = ctypes.c_size_t()
    assert gpu.lib.nnf_hip_feature_map_stat_workspace_bytes(n, c, plane, ctypes.byref(need)) == 0
    size = need.value if workspace_bytes is None else workspace_bytes
    work = gpu.torch.empty(max(16, size), dtype=gpu.torch.uint8, device=gpu.device)
    rc = gpu.lib.nnf_hip_feature_map_stat_accumulate(gpu.stream, state.data_ptr(), work.data_ptr(), size, d_x.data_ptr(), n, c, plane)
    assert rc == 0, capi.error_string(rc)
    gpu.torch.cuda.synchronize()


def static(gpu, state, d_x, n, c, plane, expect=0):
    rc = gpu.lib.nnf_hip_feature_map_stat_accumulate_static(gpu.stream, state.data_ptr(), d_x.data_ptr(), n, c, plane)
    assert rc == expect, capi.error_string(rc)
    gpu.torch.cuda.synchronize()


# two calls in a row on one running state, the second with the smaller input
CASES = [
    ((40, 256, 7, 7), (9, 256, 7, 7)),        # more workgroups than the device holds at once, plane no multiple of 4
    ((32, 64, 56, 56), (5, 64, 56, 56)),      # config 0's shape
    ((6, 3, 224, 224), (1, 3, 224, 224)),     # few long planes: cut into segments
    ((300, 1000, 1), (17, 1000, 1)),          # no spatial dimensions
    ((64, 2048, 7, 7), (3, 2048, 7, 7)),      # 131072 planes: runs long enough to stay inside 8192 partial states
]


@pytest.mark.parametrize("first,second", CASES)
def test_static_scratch_equals_the_workspace_entry_point(gpu, first, second):
    c = first[1]
    gen = T.rng(75, sum(first))
    states = {k: fresh_state(gpu, c) for k in ("static", "same_plan", "own_plan")}
    for shape in (first, second):
        n, plane = shape[0], int(np.prod(shape[2:], dtype=np.int64))
        x = (T.normal(gen, (n, c, plane), 2.0) + (np.arange(c, dtype=F) % F(7.0)).reshape(1, c, 1)).astype(F)
        d_x = gpu.to_device(x)
        static(gpu, states["static"], d_x, n, c, plane)
        with_workspace(gpu, states["same_plan"], d_x, n, c, plane, SCRATCH_BYTES)
        with_workspace(gpu, states["own_plan"], d_x, n, c, plane)
        got = read_state(gpu, states["static"])
        assert got.tobytes() == read_state(gpu, states["same_plan"]).tobytes(), "same plan, same kernels: the bits must agree"
        check(got, read_state(gpu, states["own_plan"]), scale=20.0)
    assert np.all(got["n"] == float((first[0] + second[0]) * int(np.prod(first[2:], dtype=np.int64))))


def test_static_scratch_against_the_sequential_update(gpu):
    gen = T.rng(76, 0)
    c = 24
    x = T.normal(gen, (50, c, 14, 14), 1.5)
    state = fresh_state(gpu, c)
    for a, b in ((0, 33), (33, 50)):
        static(gpu, state, gpu.to_device(x[a:b]), b - a, c, 196)
    check(read_state(gpu, state), oracle.FeatureMapStat(c).write(x).state, scale=10.0)
    before = read_state(gpu, state).tobytes()
    static(gpu, state, gpu.to_device(x[:1]), 0, c, 196)   # zero entries change nothing
    assert read_state(gpu, state).tobytes() == before


def test_static_scratch_refuses_what_it_cannot_hold(gpu):
    lib, s = gpu.lib, gpu.stream
    x = gpu.to_device(np.zeros(1 << 16, F))
    state = fresh_state(gpu, 8200)
    before = read_state(gpu, state).tobytes()
    # one partial state per feature map is the least: 8193 feature maps do not fit 8192 states
    static(gpu, state, x, 2, 8193, 1, expect=capi.E_SCRATCH)
    assert b"static scratch" in lib.nnf_hip_error_string(capi.E_SCRATCH)
    # planes of 50000 float4 loads cannot share a run: 3 entries x 4000 feature maps would need 12000 states
    assert lib.nnf_hip_feature_map_stat_accumulate_static(s, state.data_ptr(), x.data_ptr(), 3, 4000, 200000) == capi.E_SCRATCH
    assert lib.nnf_hip_feature_map_stat_accumulate_static(s, None, x.data_ptr(), 1, 4, 4) == capi.E_INVAL
    assert lib.nnf_hip_feature_map_stat_accumulate_static(s, state.data_ptr(), x.data_ptr() + 4, 1, 4, 4) == capi.E_ALIGN
    assert read_state(gpu, state).tobytes() == before
    static(gpu, state, x, 2, 8192, 4)   # the largest feature map count it takes
    assert np.all(read_state(gpu, state)["n"][:8192] == 8.0)
