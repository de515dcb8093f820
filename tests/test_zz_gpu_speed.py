"""Coarse speed guards, collected last. They do not measure (bench.py does); they catch a change that makes a kernel grossly
slower while it still computes the right bits - a load loop that serialises, a launch shape that leaves the machine empty.
Every bound is a ratio: the kernel's time against the library's plain copy kernel moving the same number of bytes, timed in
the same test on the same machine, with the launches of both queued behind a spin kernel so that neither the machine's
clocks of the day nor the host's launch calls enter. Today's ratios are between 0.76 and 1.12 (the expf chain: 1.5), the same
to two digits from run to run; the limits leave a quarter to a third on top. The last tests bound the driver's launch plan:
against the copy kernel moving the plan's bytes, and against the same network with one launch per group."""

import ctypes

import numpy as np
import pytest

from nnforge_amd import capi

pytestmark = pytest.mark.gpu

BN, RELU, PRELU, ELU, SIGMOID, TANH = capi.OP_BATCH_NORM, capi.OP_RELU, capi.OP_PRELU, capi.OP_ELU, capi.OP_SIGMOID, capi.OP_TANH


def u32(values):
    return (ctypes.c_uint32 * len(values))(*values)


def time_launches(gpu, launch, reps=60, warmup=6):
    """Microseconds per launch on the device: the stream is first held busy by a spin kernel, the launches queue up behind
    it, and HIP events bracket them on the stream."""
    lib = gpu.lib
    events = []
    for _ in range(2):
        p = ctypes.c_void_p()
        capi.check(lib.nnf_hip_event_create(ctypes.byref(p)))
        events.append(p)
    for i in range(warmup):
        launch(i)
    gpu.torch.cuda.synchronize()
    gpu.torch.cuda._sleep(int(5.0e-3 * 2.4e9))   # cycles: about 5 ms, longer than the host needs to issue the launches
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


def copy_time(gpu, traffic_bytes, reps=60):
    """Microseconds the plain copy kernel takes to move traffic_bytes (half read, half written), buffers rotating
    through more than the last-level cache holds."""
    count = max(4, (traffic_bytes // 8) & ~3)
    sets = int(max(2, min(16, (600 << 20) // (8 * count) + 1)))
    src = buffers(gpu, count, sets)
    dst = [gpu.torch.empty(count, dtype=gpu.torch.float32, device=gpu.device) for _ in range(sets)]

    def launch(i):
        assert gpu.lib.nnf_hip_copy_kernel(gpu.stream, dst[i % sets].data_ptr(), src[i % sets].data_ptr(), 4 * count) == 0

    return time_launches(gpu, launch, reps=reps, warmup=4)


def assert_ratio(gpu, what, us, traffic_bytes, limit, reps=60):
    yardstick = copy_time(gpu, traffic_bytes, reps)
    print("%s: %.1f us, %.2f times the copy's %.1f us (limit %.2f)" % (what, us, us / yardstick, yardstick, limit), flush=True)
    assert us < limit * yardstick, "%s takes %.1f us per launch, %.2f times the %.1f us of a plain copy of the same %.1f MB (limit %.1f)" % (
        what, us, us / yardstick, yardstick, traffic_bytes / 1e6, limit)


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
    assert_ratio(gpu, "config 0", us, 2 * 4 * 32 * 64 * 56 * 56, 1.35, reps=200)


def test_config2_bn_add_prelu_stays_fast(gpu):
    launch = chain_launcher(gpu, 128, 256, 56 * 56, [[], [(BN, 0)]], [(PRELU, 4)], 5, sets=2)
    us = time_launches(gpu, launch, reps=20, warmup=3)
    assert_ratio(gpu, "config 2", us, 3 * 4 * 128 * 256 * 56 * 56, 1.35, reps=20)


def test_config3_activation_chain_stays_fast(gpu):
    """Bound by the vector ALU, not by memory: 1.5 times the copy today (the limit leaves room for the clock the
    arithmetic is run at on the day)."""
    launch = chain_launcher(gpu, 64, 512, 28 * 28, [[(BN, 0), (ELU,), (SIGMOID,), (TANH, 0, 1.7159, 0.6666)]], [], 4, sets=4)
    us = time_launches(gpu, launch, reps=60, warmup=6)
    assert_ratio(gpu, "config 3", us, 2 * 4 * 64 * 512 * 28 * 28, 2.2)


def test_group_on_the_walking_grid_stays_fast(gpu):
    launch = chain_launcher(gpu, 64, 64, 56 * 56, [[(BN, 0)]], [(RELU, 0, 0.0)], 4, sets=8)
    us = time_launches(gpu, launch, reps=100, warmup=10)
    assert_ratio(gpu, "batch_norm -> rectified_linear on 64 x 64 x 56 x 56", us, 2 * 4 * 64 * 64 * 56 * 56, 1.35, reps=100)


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

    traffic = 4 * (total_in + total_out)
    assert_ratio(gpu, "max subsampling", time_launches(gpu, plain), traffic, 1.3)
    assert_ratio(gpu, "max subsampling with batch norm and ReLU folded in", time_launches(gpu, fused), traffic, 1.4)


def test_softmax_and_global_average_stay_fast(gpu):
    rows = [gpu.torch.randn(256 * 1000, dtype=gpu.torch.float32, device=gpu.device) for _ in range(32)]
    rows_out = gpu.torch.empty_like(rows[0])
    us = time_launches(gpu, lambda i: gpu.lib.nnf_hip_softmax_forward(gpu.stream, rows_out.data_ptr(), rows[i % 32].data_ptr(), 256, 1000, 1), reps=200, warmup=20)
    # 2 MB: both the softmax and the copy are bound by what a launch costs, about 2.7 against 2.2 us
    assert_ratio(gpu, "softmax 256 x 1000", us, 2 * 4 * 256 * 1000, 1.5, reps=200)
    # many rows: bound by memory, 1.02 to 1.2 times the copy depending on where the process's allocations lie
    many = [gpu.torch.randn(8192 * 1000, dtype=gpu.torch.float32, device=gpu.device) for _ in range(12)]
    many_out = [gpu.torch.empty_like(many[0]) for _ in range(12)]
    us = time_launches(gpu, lambda i: gpu.lib.nnf_hip_softmax_forward(gpu.stream, many_out[i % 12].data_ptr(), many[i % 12].data_ptr(), 8192, 1000, 1), reps=100, warmup=10)
    assert_ratio(gpu, "softmax 8192 x 1000", us, 2 * 4 * 8192 * 1000, 1.5, reps=100)
    del many, many_out
    planes = [gpu.torch.randn(64 * 2048 * 49, dtype=gpu.torch.float32, device=gpu.device) for _ in range(8)]
    sums = gpu.torch.empty(64 * 2048, dtype=gpu.torch.float32, device=gpu.device)
    us = time_launches(gpu, lambda i: gpu.lib.nnf_hip_average_subsampling_forward(gpu.stream, sums.data_ptr(), planes[i % 8].data_ptr(), 64, 2048, 7, 7, 7, 7, 1.0 / 49.0),
                       reps=100, warmup=10)
    assert_ratio(gpu, "the 7x7 global average", us, 4 * (64 * 2048 * 49 + 64 * 2048), 1.5, reps=100)
    # the last block of a residual network folded into it: 1.07 to 1.15 times the copy as straight code with the next round of
    # loads in flight, 1.4 times through the kernel's loop over the layer list (either order of the Add's inputs must take the former)
    shortcuts = [gpu.torch.randn(64 * 2048 * 49, dtype=gpu.torch.float32, device=gpu.device) for _ in range(8)]
    chunks = [gpu.torch.rand(2048, dtype=gpu.torch.float32, device=gpu.device) + 0.5 for _ in range(4)]
    chk = capi.pointer_array([t.data_ptr() for t in chunks])
    for arms in ([[], [(BN, 0)]], [[(BN, 0)], []]):
        desc = capi.make_desc(64, 2048, 49, arms, [(RELU, 0, 0.0)])
        pairs = [capi.pointer_array([shortcuts[j].data_ptr(), planes[j].data_ptr()]) for j in range(8)]

        def joined(i):
            rc = gpu.lib.nnf_hip_average_subsampling_joined_forward(gpu.stream, sums.data_ptr(), pairs[i % 8], ctypes.byref(desc), chk, 64, 2048, 7, 7, 7, 7, 1.0 / 49.0)
            assert rc == 0, capi.error_string(rc)

        assert_ratio(gpu, "the residual block and the 7x7 global average in one launch", time_launches(gpu, joined, reps=100, warmup=10),
                     4 * (2 * 64 * 2048 * 49 + 64 * 2048), 1.35, reps=100)


def test_tiling_and_entry_windows_stay_on_their_own_kernels(gpu):
    """Both have a general one-lane-per-output kernel to fall back on that is 2.5 to 4 times slower."""
    n, c, size = 64, 64, 112
    sets = 2
    ins = buffers(gpu, n * c * size * size, sets)
    outs = [gpu.torch.empty(4 * n * c * 55 * 55, dtype=gpu.torch.float32, device=gpu.device) for _ in range(sets)]

    def tiling(i):
        rc = gpu.lib.nnf_hip_max_subsampling_tiling_forward(gpu.stream, outs[i % sets].data_ptr(), ins[i % sets].data_ptr(), n, c, 2,
                                                            u32([size, size]), u32([2, 2]), 0)
        assert rc == 0, capi.error_string(rc)

    assert_ratio(gpu, "max subsampling with tiling", time_launches(gpu, tiling, reps=30, warmup=3), 4 * (n * c * size * size + 4 * n * c * 55 * 55), 1.25, reps=30)

    def entry_window(i):
        rc = gpu.lib.nnf_hip_average_subsampling_nd_forward(gpu.stream, outs[i % sets].data_ptr(), ins[i % sets].data_ptr(), n // 4, c, 1,
                                                            u32([size * size]), u32([1]), 1, 4, 0.25)
        assert rc == 0, capi.error_string(rc)

    assert_ratio(gpu, "the average over 4 entries", time_launches(gpu, entry_window, reps=30, warmup=3), 4 * (n * c * size * size * 5 // 4), 1.35, reps=30)


def resnet50_stack(seed):
    from nnforge_amd import schemas

    gen = np.random.Generator(np.random.MT19937(seed))
    layers, configs, outputs = schemas.resnet50_post_convolution()
    weights = {}
    for l in layers:
        if l["type"] == "BatchNorm":
            c = l["params"]["feature_map_count"]
            weights[l["name"]] = [gen.random(c, dtype=np.float32) + np.float32(0.5), gen.standard_normal(c, dtype=np.float32) * np.float32(0.3),
                                  gen.standard_normal(c, dtype=np.float32) * np.float32(0.3), gen.random(c, dtype=np.float32) + np.float32(0.6)]
    return schemas.schema_text(layers, "ResNet-50 post-convolution"), weights, configs, outputs, gen


def test_the_launch_plan_of_the_resnet50_stack_stays_near_the_copy_rate(gpu):
    """Config 4 through the driver at its 64 entries: a pass of the plan (eight launches, most of the bytes in four
    nnf::chain_batch_mixed_kernel grids of up to eleven groups each) against the copy kernel moving as many bytes as the
    plan's algorithmic 6.36 GB. Today's ratio is 0.98."""
    from nnforge_amd import backend, workloads

    text, weights, configs, outputs, gen = resnet50_stack(92)
    n = 64
    largest = max(fm * dims[0] * dims[1] for fm, dims in configs.values())
    pool = gen.standard_normal(n * largest, dtype=np.float32)
    rep = backend.time_kernels(text, weights, configs, outputs, warmup=2, passes=10, shared_input_pool=pool, entry_count=n, max_entry_count=n)
    assert rep["timed_entries"] == n and rep["launches"] == 8 and rep["plan_steps"] == 50, rep["raw"]
    plan_us = rep["device_seconds_per_pass"] * 1e6
    plan_bytes = sum(workloads.resnet50_algorithmic_bytes(n))
    piece = 512 << 20
    copy_us = copy_time(gpu, piece, reps=30) * plan_bytes / piece
    print("the ResNet-50 stack's plan: %.1f us per pass, %.2f times the %.1f us the copy kernel takes for its %.2f GB (limit 1.25)" % (
        plan_us, plan_us / copy_us, copy_us, plan_bytes / 1e9), flush=True)
    assert plan_us < 1.25 * copy_us


def test_groups_launched_together_stay_ahead_of_one_launch_per_group(gpu):
    """The ResNet-50 post-convolution stack through the driver at 8 entries per packet, where launches are what a pass
    costs: the default plan (8 kernel launches for 50 steps) against one launch per group on one stream, both timed by the
    driver on the same resident packet. Today's ratio is 1.5; a plan that fell back to a launch per group, or runs that
    ended early, would bring it to 1."""
    from nnforge_amd import backend

    text, weights, configs, outputs, gen = resnet50_stack(91)
    n = 8
    largest = max(fm * dims[0] * dims[1] for fm, dims in configs.values())
    pool = gen.standard_normal(n * largest, dtype=np.float32)

    def seconds(**options):
        rep = backend.time_kernels(text, weights, configs, outputs, warmup=3, passes=20, shared_input_pool=pool, entry_count=n, max_entry_count=n, **options)
        assert rep["timed_entries"] == n
        return rep["device_seconds_per_pass"], rep

    together, rep = seconds()
    one_by_one, _ = seconds(one_launch_per_group=True, kernel_stream_count=1)
    runs = {s["run"] for s in rep["steps"] if s["run"] is not None}
    assert len(runs) == 6, "the stack's groups in six runs, as many as its longest chain of blocks"
    assert one_by_one > 1.25 * together, "groups launched together: %.1f us per pass, one launch per group: %.1f us" % (together * 1e6, one_by_one * 1e6)
