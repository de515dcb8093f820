"""Coarse speed guards, collected last: each workload must stay within twice the time it takes on an MI355X today.
They do not measure (bench.py does); they catch a change that makes a kernel grossly slower while it still
computes the right bits - a load loop that serialises, a launch shape that leaves the machine empty."""

import ctypes

import numpy as np
import pytest

from nnforge_amd import capi

pytestmark = pytest.mark.gpu

BN, RELU, PRELU = capi.OP_BATCH_NORM, capi.OP_RELU, capi.OP_PRELU


def u32(values):
    return (ctypes.c_uint32 * len(values))(*values)


def time_launches(gpu, launch, reps=60, warmup=6):
    """Microseconds per launch by HIP events on the launch stream."""
    lib = gpu.lib
    events = []
    for _ in range(2):
        p = ctypes.c_void_p()
        capi.check(lib.nnf_hip_event_create(ctypes.byref(p)))
        events.append(p)
    for i in range(warmup):
        launch(i)
    gpu.torch.cuda.synchronize()
    lib.nnf_hip_event_record(events[0], gpu.stream)
    for i in range(reps):
        launch(i)
    lib.nnf_hip_event_record(events[1], gpu.stream)
    capi.check(lib.nnf_hip_event_synchronize(events[1]))
    ms = ctypes.c_float()
    capi.check(lib.nnf_hip_event_elapsed_ms(ctypes.byref(ms), events[0], events[1]))
    for p in events:
        lib.nnf_hip_event_destroy(p)
    return ms.value / reps * 1e3


def buffers(gpu, count, sets):
    return [gpu.torch.randn(count, dtype=gpu.torch.float32, device=gpu.device) for _ in range(sets)]


def chain_launcher(gpu, n, c, plane, arms, tail, chunk_count, sets=4):
    total = n * c * plane
    ins = [[t for t in buffers(gpu, total, len(arms))] for _ in range(sets)]
    outs = [gpu.torch.empty(total, dtype=gpu.torch.float32, device=gpu.device) for _ in range(sets)]
    chunks = [gpu.torch.rand(c, dtype=gpu.torch.float32, device=gpu.device) + 0.5 for _ in range(chunk_count)]
    chk = capi.pointer_array([t.data_ptr() for t in chunks])
    desc = capi.make_desc(n, c, plane, arms, tail)
    in_ptrs = [capi.pointer_array([t.data_ptr() for t in group]) for group in ins]

    def launch(i):
        j = i % sets
        rc = gpu.lib.nnf_hip_chain_forward(gpu.stream, ctypes.byref(desc), outs[j].data_ptr(), in_ptrs[j], chk)
        assert rc == 0, capi.error_string(rc)

    launch.keep = (ins, outs, chunks, desc, in_ptrs)
    return launch


def test_config0_bn_relu_stays_fast(gpu):
    launch = chain_launcher(gpu, 32, 64, 56 * 56, [[(BN, 0)]], [(RELU, 0, 0.0)], 4, sets=16)
    us = time_launches(gpu, launch, reps=200, warmup=20)
    assert us < 19.0, "config 0 takes %.1f us per launch (about 9.2 us expected)" % us


def test_config2_bn_add_prelu_stays_fast(gpu):
    launch = chain_launcher(gpu, 128, 256, 56 * 56, [[], [(BN, 0)]], [(PRELU, 4)], 5, sets=2)
    us = time_launches(gpu, launch, reps=20, warmup=3)
    assert us < 390.0, "config 2 takes %.1f us per launch (about 192 us expected)" % us


def test_max_subsampling_alone_and_with_layers_folded_in_stays_fast(gpu):
    n, c, size = 64, 64, 112
    total_in, total_out = n * c * size * size, n * c * 56 * 56
    sets = 3
    ins = buffers(gpu, total_in, sets)
    outs = [gpu.torch.empty(total_out, dtype=gpu.torch.float32, device=gpu.device) for _ in range(sets)]
    dims, win, stride, up = u32([size, size]), u32([3, 3]), u32([2, 2]), u32([1, 1])
    chunks = [gpu.torch.rand(c, dtype=gpu.torch.float32, device=gpu.device) + 0.5 for _ in range(4)]
    chk = capi.pointer_array([t.data_ptr() for t in chunks])
    desc = capi.make_desc(n, c, size * size, [[(BN, 0), (RELU, 0, 0.0)]], [])

    def plain(i):
        j = i % sets
        assert gpu.lib.nnf_hip_max_subsampling_forward(gpu.stream, outs[j].data_ptr(), ins[j].data_ptr(), n, c, 2, dims, win, stride, up, 1, 1, 0) == 0

    def fused(i):
        j = i % sets
        assert gpu.lib.nnf_hip_max_subsampling_fused_forward(gpu.stream, outs[j].data_ptr(), ins[j].data_ptr(), ctypes.byref(desc), chk,
                                                             n, c, 2, dims, win, stride, up, 1, 1, 0) == 0

    us = time_launches(gpu, plain)
    assert us < 95.0, "max subsampling takes %.1f us per launch (about 47 us expected)" % us
    us = time_launches(gpu, fused)
    assert us < 120.0, "max subsampling with batch norm and ReLU folded in takes %.1f us per launch (about 59 us expected)" % us


def test_softmax_and_global_average_stay_fast(gpu):
    rows = gpu.torch.randn(256 * 1000, dtype=gpu.torch.float32, device=gpu.device)
    rows_out = gpu.torch.empty_like(rows)
    us = time_launches(gpu, lambda i: gpu.lib.nnf_hip_softmax_forward(gpu.stream, rows_out.data_ptr(), rows.data_ptr(), 256, 1000, 1), reps=200, warmup=20)
    assert us < 9.0, "softmax 256 x 1000 takes %.1f us per launch (about 3.7 us expected when issued from Python)" % us
    planes = gpu.torch.randn(64 * 2048 * 49, dtype=gpu.torch.float32, device=gpu.device)
    sums = gpu.torch.empty(64 * 2048, dtype=gpu.torch.float32, device=gpu.device)
    us = time_launches(gpu, lambda i: gpu.lib.nnf_hip_average_subsampling_forward(gpu.stream, sums.data_ptr(), planes.data_ptr(), 64, 2048, 7, 7, 7, 7, 1.0 / 49.0),
                       reps=100, warmup=10)
    assert us < 17.0, "the 7x7 global average takes %.1f us per launch (about 8.3 us expected)" % us


def test_tiling_and_entry_windows_stay_on_their_own_kernels(gpu):
    """Both have a general one-lane-per-output kernel to fall back on that is 2.5 to 3.5 times slower."""
    n, c, size = 64, 64, 112
    sets = 2
    ins = buffers(gpu, n * c * size * size, sets)
    outs = [gpu.torch.empty(4 * n * c * 55 * 55, dtype=gpu.torch.float32, device=gpu.device) for _ in range(sets)]

    def tiling(i):
        rc = gpu.lib.nnf_hip_max_subsampling_tiling_forward(gpu.stream, outs[i % sets].data_ptr(), ins[i % sets].data_ptr(), n, c, 2,
                                                            u32([size, size]), u32([2, 2]), 0)
        assert rc == 0, capi.error_string(rc)

    us = time_launches(gpu, tiling, reps=30, warmup=3)
    assert us < 165.0, "max subsampling with tiling takes %.1f us per launch (about 82 us expected)" % us

    def entry_window(i):
        rc = gpu.lib.nnf_hip_average_subsampling_nd_forward(gpu.stream, outs[i % sets].data_ptr(), ins[i % sets].data_ptr(), n // 4, c, 1,
                                                            u32([size * size]), u32([1]), 1, 4, 0.25)
        assert rc == 0, capi.error_string(rc)

    us = time_launches(gpu, entry_window, reps=30, warmup=3)
    assert us < 86.0, "the average over 4 entries takes %.1f us per launch (about 43 us expected)" % us
