"""The C++ hip backend end to end on the GPU: a text-format schema, nnForge-format weights and
host tensors go in through factory_generator_hip -> forward_propagation_hip; the outputs must equal
the CPU oracle run layer by layer the way the plain backend drives its testers."""

import os

import numpy as np
import pytest

import nnf_schemas as S
import nnf_testing as T
import oracle
from nnforge_amd import backend

F32 = np.float32

pytestmark = pytest.mark.gpu


def run(layers, weights, inputs, outputs, values, **kw):
    shapes = {n: values[n].shape for n in outputs}
    return backend.run_schema(S.schema_text(layers), weights, inputs, shapes, **kw)


def assert_bits(got, want, what):
    assert got.shape == want.shape
    assert T.bit_mismatches(got, want) == 0, "%s: %d of %d elements differ" % (what, T.bit_mismatches(got, want), got.size)


@pytest.mark.parametrize("fuse", [True, False])
@pytest.mark.parametrize("shortcut_bn", [True, False])
def test_resnet_block(fuse, shortcut_bn):
    gen = T.rng(50, int(fuse) * 2 + int(shortcut_bn))
    c, n = 16, 5
    layers = S.resnet_block(c, shortcut_bn)
    weights = S.make_weights(layers, gen)
    inputs = {"conv_main": T.normal(gen, (n, c, 14, 14)), "conv_shortcut": T.normal(gen, (n, c, 14, 14))}
    values = S.evaluate(layers, weights, inputs)
    got, rep = run(layers, weights, inputs, ["res_relu"], values, fuse=fuse)
    assert_bits(got["res_relu"], values["res_relu"], "resnet block")
    assert rep["entries"] == n
    assert len(rep["steps"]) == (1 if fuse else (4 if shortcut_bn else 3))


def test_classifier_tail_with_several_outputs_and_packets():
    gen = T.rng(51, 0)
    c, n = 12, 11
    layers = S.classifier_tail(c)
    weights = S.make_weights(layers, gen)
    inputs = {"conv_main": T.normal(gen, (n, c, 7, 7), 4.0), "conv_shortcut": T.normal(gen, (n, c, 7, 7), 4.0)}
    values = S.evaluate(layers, weights, inputs)
    # 11 entries in packets of 4: 4 + 4 + 3
    got, rep = run(layers, weights, inputs, ["prob", "pool", "res_relu"], values, max_entry_count=4, profile=True)
    assert rep["entries"] == n and rep["max_entry_count"] == 4
    assert_bits(got["res_relu"], values["res_relu"], "block output")
    assert_bits(got["pool"], values["pool"], "pool")
    rel = np.abs(got["prob"] - values["prob"]) / values["prob"]
    assert rel.max() < 1e-5
    assert set(rep["seconds"]) == {"shortcut_bn+main_bn+res+res_relu", "pool", "prob"}
    assert all(v > 0 for v in rep["seconds"].values())


@pytest.mark.parametrize("fuse,share", [(True, True), (False, True), (False, False)])
def test_activation_chain_and_branches(fuse, share):
    gen = T.rng(52, 0)
    c, n = 6, 7
    layers = S.activation_chain(c) + [S.L("PReLU", "p", ["bn"], feature_map_count=c), S.L("Add", "mix", ["tanh", "p", "x"], alpha=0.5),
                                      S.L("ReLU", "leaky", ["mix"], negative_slope=0.2)]
    weights = S.make_weights(layers, gen)
    x = T.normal(gen, (n, c, 9, 5), 2.0)
    x.reshape(-1)[::97] = 50.0
    x.reshape(-1)[5::89] = -50.0
    inputs = {"x": x}
    values = S.evaluate(layers, weights, inputs)
    got, rep = run(layers, weights, inputs, ["leaky", "tanh"], values, fuse=fuse, dont_share_buffers=not share)
    assert_bits(got["tanh"], values["tanh"], "tanh")
    assert_bits(got["leaky"], values["leaky"], "leaky")


def test_weights_from_nnforge_data_files(tmp_path):
    gen = T.rng(53, 0)
    layers = S.resnet_block(8)
    weights = S.make_weights(layers, gen)
    folder = str(tmp_path / "ann_trained_000")
    backend.write_weights(folder, weights)
    inputs = {"conv_main": T.normal(gen, (3, 8, 7, 7)), "conv_shortcut": T.normal(gen, (3, 8, 7, 7))}
    values = S.evaluate(layers, weights, inputs)
    got, _ = run(layers, {}, inputs, ["res_relu"], values, weights_folder=folder)
    assert_bits(got["res_relu"], values["res_relu"], "weights from .data files")


def test_run_errors():
    gen = T.rng(54, 0)
    layers = S.resnet_block(8)
    weights = S.make_weights(layers, gen)
    inputs = {"conv_main": T.normal(gen, (3, 8, 7, 7)), "conv_shortcut": T.normal(gen, (3, 8, 7, 7))}
    values = S.evaluate(layers, weights, inputs)
    with pytest.raises(backend.BackendError, match="No data found with layer name"):
        run(layers, {"main_bn": weights["main_bn"]}, inputs, ["res_relu"], values)
    bad = dict(weights)
    bad["main_bn"] = weights["main_bn"][:3]
    with pytest.raises(backend.BackendError, match="data weight vector count 3 doesn't satisfy layer configuration 4"):
        run(layers, bad, inputs, ["res_relu"], values)
    bad["main_bn"] = [w[:5] for w in weights["main_bn"]]
    with pytest.raises(backend.BackendError, match="data weight count 5 for vector 0 doesn't satisfy layer configuration 8"):
        run(layers, bad, inputs, ["res_relu"], values)


def test_cpp_application_uses_the_backend_like_a_reference_backend(tmp_path):
    """tests/cpp/backend_usage.cpp: factory_generator_hip -> forward_propagation_hip from C++ with
    a reader of unknown length, several packets, debug and profile switched on; then the same data through
    data set files written into the folder given."""
    import os
    import subprocess

    from nnforge_amd import build

    assert os.path.exists(build.USAGE_PROGRAM), "build it first: python -c 'import __graft_entry__ as g; g.build()'"
    proc = subprocess.run([build.USAGE_PROGRAM, str(tmp_path)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout
    lines = proc.stdout.strip().splitlines()
    assert lines[-1] == "ok", proc.stdout
    assert any("[fused] main_bn+res+res_prelu <- conv_shortcut, conv_main" in l for l in lines), proc.stdout
    # actions are keyed the reference's way (layer_name_with_action): a fused launch reports under its last layer
    assert any(l.startswith("action res_prelu forward (main_bn+res+res_prelu):") for l in lines), proc.stdout
    assert any("13 entries" in l for l in lines), proc.stdout


def test_many_packets_overlap_io_and_write_the_profile_report(tmp_path):
    """37 entries in packets of 3 (13 packets, the last one short): uploads, kernels and downloads of
    neighbouring packets overlap on two I/O slots, and every entry must still come out right. With a
    profile folder the run leaves the per-action report of nnforge/profile_util.cpp:25-105."""
    gen = T.rng(55, 0)
    c, n = 8, 37
    layers = S.classifier_tail(c)
    weights = S.make_weights(layers, gen)
    inputs = {"conv_main": T.normal(gen, (n, c, 7, 7), 4.0), "conv_shortcut": T.normal(gen, (n, c, 7, 7), 4.0)}
    values = S.evaluate(layers, weights, inputs)
    got, rep = run(layers, weights, inputs, ["prob", "pool", "res_relu"], values, max_entry_count=3, profile=True,
                   profile_folder=str(tmp_path))
    assert rep["entries"] == n
    assert_bits(got["res_relu"], values["res_relu"], "block output")
    assert_bits(got["pool"], values["pool"], "pool")
    assert (np.abs(got["prob"] - values["prob"]) / values["prob"]).max() < 1e-5

    lines = (tmp_path / "forward_prop_perf_per_layer_action_000.csv").read_text().splitlines()
    header = lines[0].split("\t")
    assert header[:3] == ["Layer", "Layer type", "Action"] and header[-2:] == ["GB/s", "Relative to peak bandwidth"]
    rows = {r.split("\t")[0]: r.split("\t") for r in lines[1:]}
    assert set(rows) == {"shortcut_bn+main_bn+res+res_relu", "pool", "prob"}
    assert rows["shortcut_bn+main_bn+res+res_relu"][1] == "BatchNorm+BatchNorm+Add+ReLU"
    assert all(r[2] == "forward" and len(r) == len(header) for r in rows.values())
    times = [float(r.split("\t")[5]) for r in lines[1:]]
    assert times == sorted(times, reverse=True) and times[-1] > 0
    # the fused step moves 2 inputs + 1 output of c*49 floats per entry
    fused = rows["shortcut_bn+main_bn+res+res_relu"]
    assert abs(float(fused[7]) - 3 * c * 49 * 4 * n / float(fused[5]) * 1e-9) < 1e-3 * float(fused[7])


@pytest.mark.parametrize("shortcut_bn", [True, False])
def test_last_block_of_a_residual_network_folded_into_its_global_average(shortcut_bn):
    """BatchNorm(main) [+ BatchNorm(shortcut)] -> Add -> ReLU -> 7x7 average with only the average (and what follows it)
    wanted: the average's kernel applies the joined group to the two tensors on their way in - one launch, the group's
    result never stored - and the outputs carry the bits of the layers run one by one."""
    gen = T.rng(58, int(shortcut_bn))
    c, n = 40, 11
    layers = S.classifier_tail(c, with_shortcut_bn=shortcut_bn)
    weights = S.make_weights(layers, gen)
    inputs = {"conv_main": T.normal(gen, (n, c, 7, 7), 4.0), "conv_shortcut": T.normal(gen, (n, c, 7, 7), 4.0)}
    values = S.evaluate(layers, weights, inputs)
    got, rep = run(layers, weights, inputs, ["prob", "pool"], values, max_entry_count=4)
    names = ["+".join(s["layers"]) for s in rep["steps"]]
    assert len(names) == 2 and names[0].endswith("+res+res_relu+pool") and names[1] == "prob", names
    assert len(rep["steps"][0]["inputs"]) == 2 and rep["steps"][0]["fused"]
    assert_bits(got["pool"], values["pool"], "average over the folded block")
    assert (np.abs(got["prob"] - values["prob"]) / values["prob"]).max() < 1e-5
    # without fusion: the same bits from six launches
    plain, rep = run(layers, weights, inputs, ["prob", "pool"], values, max_entry_count=4, fuse=False)
    assert len(rep["steps"]) == (6 if shortcut_bn else 5)
    assert_bits(plain["pool"], got["pool"], "fused against unfused")


@pytest.mark.parametrize("threads", [1, 3, 16])
def test_entries_read_by_the_job_runner_threads(threads):
    """The entries of a packet are read by the job runner's threads, one job per entry, while the packet before
    goes to the writer: whatever the number of threads, every entry lands in its own place (41 entries in
    packets of 6: full packets, a short last one, and reads asked beyond the last entry)."""
    gen = T.rng(57, 0)
    c, n = 5, 41
    layers = S.classifier_tail(c)
    weights = S.make_weights(layers, gen)
    inputs = {"conv_main": T.normal(gen, (n, c, 7, 7), 4.0), "conv_shortcut": T.normal(gen, (n, c, 7, 7), 4.0)}
    values = S.evaluate(layers, weights, inputs)
    got, rep = run(layers, weights, inputs, ["pool", "res_relu"], values, max_entry_count=6, host_thread_count=threads)
    assert rep["entries"] == n
    assert_bits(got["res_relu"], values["res_relu"], "block output with %d reading threads" % threads)
    assert_bits(got["pool"], values["pool"], "pool with %d reading threads" % threads)


def test_layer_in_place_on_a_data_layer_with_packets():
    """The only layer writes where the data layer was uploaded: the next upload into that slot has to
    wait for the download of the result."""
    gen = T.rng(56, 0)
    layers = [S.L("Data", "in"), S.L("TanH", "act", ["in"])]
    n = 50
    inputs = {"in": T.normal(gen, (n, 4, 10, 10))}
    values = S.evaluate(layers, {}, inputs)
    got, rep = run(layers, {}, inputs, ["act"], values, max_entry_count=7)
    assert_bits(got["act"], values["act"], "tanh in place over 8 packets")


@pytest.mark.parametrize("fuse", [True, False])
def test_inception_like_block_with_the_neighbouring_layers(fuse):
    """MaxSubsampling (rounded up, overlapping), Dropout, Absolute, PReLU, Concat of four inputs, Maxout,
    min pooling and TanH through the driver, in packets, against the oracle layer by layer."""
    gen = T.rng(57, int(fuse))
    c, n = 8, 21
    layers = S.inception_like(c)
    weights = S.make_weights(layers, gen)
    inputs = {"stem": T.normal(gen, (n, c, 29, 29), 2.0)}
    values = S.evaluate(layers, weights, inputs)
    assert values["pool1"].shape == (n, c, 15, 15) and values["join"].shape == (n, 4 * c, 15, 15)
    assert values["mo"].shape == (n, 2 * c, 15, 15) and values["out"].shape == (n, 2 * c, 7, 7)
    got, rep = run(layers, weights, inputs, ["out", "join", "drop"], values, fuse=fuse, max_entry_count=8)
    assert rep["entries"] == n
    assert_bits(got["join"], values["join"], "concat")
    assert_bits(got["drop"], values["drop"], "dropout behind maxout")
    assert_bits(got["out"], values["out"], "output")


@pytest.mark.parametrize("c,size,n,packet", [(16, 14, 23, 8), (32, 7, 9, 4), (16, 28, 5, 5)])
def test_inception_block_whose_concat_has_nothing_to_copy(c, size, n, packet):
    """Four branches that end in fused groups only the Concat reads: every group writes its feature maps into the Concat's
    output (a launch over tiles x entries, entry to entry by the Concat's neuron count) and the Concat launches nothing.
    Against the oracle layer by layer, bit for bit, in packets (the last one short); and the same bits with every input
    copied (hip_concat_in_place off). 7 x 7 planes take their weights through LDS coefficients."""
    gen = T.rng(65, size)
    layers = S.inception_block(c)
    weights = S.make_weights(layers, gen)
    inputs = {name: T.normal(gen, (n, fm, size, size), 1.5) for name, fm in (("conv_a", c), ("conv_b", 2 * c), ("conv_c", c), ("conv_d", c), ("conv_e", c))}
    values = S.evaluate(layers, weights, inputs)
    assert values["join"].shape == (n, 5 * c, size, size)
    got, rep = run(layers, weights, inputs, ["out", "mo"], values, max_entry_count=packet)
    join = [s for s in rep["steps"] if s["layers"] == ["join"]][0]
    assert join["inputs_in_place"] == ["a_relu", "b_relu", "c_prelu", "d_relu"], rep["raw"]
    assert_bits(got["mo"], values["mo"], "maxout behind the concat")
    assert_bits(got["out"], values["out"], "output")
    # the Concat's output as an output of the network: the groups write into the buffer that is copied back
    got, rep = run(layers, weights, inputs, ["join"], values, max_entry_count=packet)
    assert_bits(got["join"], values["join"], "concat as output")
    copied, rep = run(layers, weights, inputs, ["out", "join"], values, max_entry_count=packet, concat_copies_every_input=True)
    assert all(s["inputs_in_place"] == [] for s in rep["steps"])
    assert_bits(copied["join"], values["join"], "concat, every input copied")
    assert_bits(copied["out"], values["out"], "output, every input copied")


def test_concat_launches_nothing_when_every_input_is_in_place():
    gen = T.rng(66, 1)
    c, size, n = 16, 14, 6
    layers = S.inception_block(c)
    weights = S.make_weights(layers, gen)
    inputs = {name: T.normal(gen, (n, fm, size, size), 1.5) for name, fm in (("conv_a", c), ("conv_b", 2 * c), ("conv_c", c), ("conv_d", c), ("conv_e", c))}
    in_place = backend.time_kernels(S.schema_text(layers), weights, inputs, ["out"], warmup=1, passes=2, max_entry_count=n)
    copying = backend.time_kernels(S.schema_text(layers), weights, inputs, ["out"], warmup=1, passes=2, max_entry_count=n, concat_copies_every_input=True)
    # four groups, maxout, tanh: six steps, and three kernels - the four groups go to the kernels in one call (one launch),
    # the Concat is a step that launches nothing. Copying, it is a seventh step with a kernel of its own
    assert in_place["launches"] == 3 and in_place["plan_steps"] == 6, in_place["raw"]
    assert copying["plan_steps"] == 7 and 4 <= copying["launches"] <= 7, copying["raw"]


@pytest.mark.parametrize("fuse", [True, False])
@pytest.mark.parametrize("size", [28, 57])
def test_groups_folded_into_the_subsampling_layers_behind_them(fuse, size):
    """BatchNorm -> ReLU -> max pooling (3x3 every 2, rounded up), TanH -> Absolute -> 2x2 average pooling, ELU -> 7x7
    average: with fusion on, each pooling layer applies the layers in front of it to the values it reads (one launch,
    no intermediate tensor). Same bits either way."""
    gen = T.rng(62, size + int(fuse))
    c, n = 10, 13
    layers = [S.L("Data", "conv1"), S.L("BatchNorm", "bn", ["conv1"], feature_map_count=c), S.L("ReLU", "relu", ["bn"]),
              S.L("MaxSubsampling", "pool1", ["relu"], windows=[3, 3], strides=[2, 2], round_ups=[True, True]),
              S.L("TanH", "tanh", ["pool1"], scale=1.7159, steepness=0.6666), S.L("Absolute", "abs", ["tanh"]),
              S.L("AverageSubsampling", "pool2", ["abs"], windows=[2, 2]),
              S.L("ELU", "elu", ["pool2"]), S.L("AverageSubsampling", "global", ["elu"], windows=[7, 7], alpha=1.0 / 49.0)]
    weights = S.make_weights(layers, gen)
    inputs = {"conv1": T.normal(gen, (n, c, size, size), 2.0)}
    values = S.evaluate(layers, weights, inputs)
    got, rep = run(layers, weights, inputs, ["global", "pool2"], values, fuse=fuse, max_entry_count=5)
    assert rep["entries"] == n
    assert_bits(got["pool2"], values["pool2"], "average pooling behind TanH and Absolute")
    assert_bits(got["global"], values["global"], "global average behind ELU")
    names = ["+".join(s["layers"]) for s in rep["steps"]]
    if fuse:
        # 28: pool2 is 7x7 and the last window covers the whole plane (global pooling kernel); 57: pool2 is 14x14
        # (29x29 halved) and the 7x7 window is an ordinary one
        assert names == ["bn+relu+pool1", "tanh+abs+pool2", "elu+global"]
    else:
        assert len(names) == 8


# NNF_EXHAUSTIVE=1: 395 more networks (a few seconds on the device)
MORE_NETWORK_SEEDS = (list(range(12, 260)) + [-s for s in range(13, 160)]) if os.environ.get("NNF_EXHAUSTIVE") == "1" else []


@pytest.mark.parametrize("seed", list(range(12)) + [-s for s in range(1, 13)] + MORE_NETWORK_SEEDS)
def test_random_networks_equal_the_oracle_layer_by_layer(seed):
    """Random DAGs of every layer type the backend runs (the generator of the planner tests), in packets, with
    fusion and buffer sharing on: every output equals the oracle run layer by layer, bit for bit; the same
    network without fusion and with dedicated buffers gives the same bits. Negative seeds: networks with tiling
    layers and windows over entries, whose values hold different numbers of entries."""
    gen = T.rng(70 if seed >= 0 else 71, abs(seed))
    layers, shapes, outputs = S.random_network(gen, with_entry_factors=seed < 0)
    weights = S.make_weights(layers, gen)
    n = 7
    inputs = {k: T.normal(gen, (n, shapes[k][0]) + tuple(shapes[k][1][::-1]), 1.5) for k in ("in0", "in1")}
    values = S.evaluate(layers, weights, inputs)
    got, rep = run(layers, weights, inputs, outputs, values, fuse=True, max_entry_count=3)
    assert rep["entries"] == n
    for name in outputs:
        assert_bits(got[name], values[name], "seed %d, output %s, steps %s" % (seed, name, ["+".join(s["layers"]) for s in rep["steps"]]))
    plain, _ = run(layers, weights, inputs, outputs, values, fuse=False, dont_share_buffers=True)
    for name in outputs:
        assert_bits(plain[name], values[name], "seed %d unfused, output %s" % (seed, name))
    # fused, every group launched on its own, independent steps spread over the kernel streams, buffers shared
    spread, rep = run(layers, weights, inputs, outputs, values, fuse=True, max_entry_count=3, one_launch_per_group=True, kernel_stream_count=3)
    assert all(s["run"] is None for s in rep["steps"])
    for name in outputs:
        assert_bits(spread[name], values[name], "seed %d on kernel streams, output %s" % (seed, name))


def test_average_subsampling_in_the_full_form_through_the_driver():
    """3-D average subsampling with windows over feature maps, then one given by its output sizes, behind element-wise
    layers, in packets: equals the oracle layer by layer (the plain tester's multiplier: no division by the spatial
    window, only by the feature-map window, unless alpha is set)."""
    gen = T.rng(63, 0)
    c, n = 8, 9
    layers = [S.L("Data", "x"), S.L("BatchNorm", "bn", ["x"], feature_map_count=c), S.L("ReLU", "relu", ["bn"]),
              S.L("AverageSubsampling", "a3", ["relu"], windows=[2, 3, 2], fm_window=2),
              S.L("TanH", "tanh", ["a3"]),
              S.L("AverageSubsampling", "abs", ["tanh"], subsampled=[3, 1, 2], fm_subsampled=2, alpha=0.125)]
    weights = S.make_weights(layers, gen)
    inputs = {"x": T.normal(gen, (n, c, 9, 7, 6), 2.0)}
    values = S.evaluate(layers, weights, inputs)
    assert values["a3"].shape == (n, 4, 4, 2, 3) and values["abs"].shape == (n, 2, 2, 1, 3)
    got, rep = run(layers, weights, inputs, ["abs", "a3"], values, max_entry_count=4)
    assert_bits(got["a3"], values["a3"], "3-D average with feature-map windows")
    assert_bits(got["abs"], values["abs"], "average given by its output sizes")
    # these shapes have no staged kernel: the groups in front run on their own
    assert ["+".join(s["layers"]) for s in rep["steps"]] == ["bn+relu", "a3", "tanh", "abs"]


@pytest.mark.parametrize("fuse", [True, False])
def test_tiling_and_windows_over_entries_through_the_driver(fuse):
    """Max subsampling with tiling makes 4 entries of each entry read, the layers behind it run on all of them, and
    windows over entries fold them again (nnforge/plain/forward_propagation_plain.cpp:185-192: every tester gets
    entries read x the cumulative tiling factor of its layer, the writer every entry of the output layers). In packets of
    4 entries read; the outputs equal the oracle run layer by layer on the whole input."""
    gen = T.rng(62, int(fuse))
    c, n = 6, 9
    layers = [S.L("Data", "x"), S.L("BatchNorm", "bn", ["x"], feature_map_count=c), S.L("ReLU", "relu", ["bn"]),
              S.L("MaxSubsampling", "tiles", ["relu"], windows=[2, 2], tiling=True),
              S.L("BatchNorm", "bn2", ["tiles"], feature_map_count=c), S.L("TanH", "tanh", ["bn2"]),
              S.L("AverageSubsampling", "gap", ["tanh"], windows=[6, 5]),
              S.L("MaxSubsampling", "pairs_min", ["gap"], windows=[1, 1], entry_window=2, function="MIN"),
              S.L("AverageSubsampling", "mean", ["pairs_min"], windows=[1, 1], entry_window=2)]
    weights = S.make_weights(layers, gen)
    inputs = {"x": T.normal(gen, (n, c, 11, 13), 2.0)}
    values = S.evaluate(layers, weights, inputs)
    assert values["tiles"].shape == (4 * n, c, 5, 6) and values["pairs_min"].shape == (2 * n, c, 1, 1) and values["mean"].shape == (n, c, 1, 1)
    got, rep = run(layers, weights, inputs, ["mean"], values, max_entry_count=4, fuse=fuse)
    assert rep["entries"] == n
    assert_bits(got["mean"], values["mean"], "mean over the tiles")
    # outputs that hold 4 entries per entry read, in the order the tiles were made
    got, rep = run(layers, weights, inputs, ["tanh", "gap"], values, max_entry_count=4, fuse=fuse)
    assert_bits(got["tanh"], values["tanh"], "layers behind the tiling layer")
    assert_bits(got["gap"], values["gap"], "average over whole planes of the tiles")
    if fuse:
        assert ["+".join(s["layers"]) for s in rep["steps"]] == ["bn+relu", "tiles", "bn2+tanh", "gap"]
    # statistics over the tiled entries, reduced on the device
    stat, rep = backend.layer_statistics(S.schema_text(layers), weights, inputs, "tanh", c, max_entry_count=4, fuse=fuse)
    want = oracle.FeatureMapStat(c).write(values["tanh"]).get()
    assert rep["entries"] == n and rep["writer_entries"] == 4 * n
    assert np.array_equal(stat["min"], want["min"]) and np.array_equal(stat["max"], want["max"])
    assert T.ulp_distance(stat["average"], want["average"]).max() <= 1 and T.ulp_distance(stat["std_dev"], want["std_dev"]).max() <= 1


def test_inference_from_data_set_files_to_data_set_files(tmp_path):
    """The toolset's inference in its dump mode (nnforge/toolset.cpp:551-655) for one network: .dt files in through
    structured_data_bunch_stream_reader, outputs collected by neuron_value_set_data_bunch_writer, the four entries a
    tiling layer made of every input entry folded into their mean (neuron_value_set::compact), .dt files out."""
    gen = T.rng(61, 0)
    c, n = 5, 11
    layers = [S.L("Data", "images"), S.L("Data", "dataset_value"),
              S.L("BatchNorm", "bn", ["images"], feature_map_count=c), S.L("ReLU", "relu", ["bn"]),
              S.L("MaxSubsampling", "tiles", ["relu"], windows=[2, 2], tiling=True),
              S.L("Sigmoid", "sig", ["tiles"]),
              S.L("AverageSubsampling", "gap", ["sig"], windows=[4, 3]),
              S.L("Softmax", "prob", ["gap"]),
              S.L("ReLU", "flag", ["dataset_value"])]
    weights = S.make_weights(layers, gen)
    images = T.normal(gen, (n, c, 7, 9), 2.0)
    values = S.evaluate(layers, weights, {"images": images, "dataset_value": np.ones((n, 1), F32)})
    assert values["prob"].shape == (4 * n, c, 1, 1)
    backend.write_dataset(tmp_path / "images.dt", images)
    outputs = {"prob": tmp_path / "out_prob.dt", "sig": tmp_path / "out_sig.dt"}
    rep = backend.run_dataset(S.schema_text(layers), weights, {"images": tmp_path / "images.dt"}, outputs, compact_samples=4, max_entry_count=4)
    assert rep["entries"] == n
    for name in outputs:
        got = backend.read_dataset(outputs[name])
        # compact: left-to-right fp32 sum of the 4 tiles of an entry, times 0.25
        tiles = values[name].reshape((n, 4) + values[name].shape[1:])
        want = (((tiles[:, 0] + tiles[:, 1]) + tiles[:, 2]) + tiles[:, 3]) * F32(0.25)
        assert_bits(got, want.astype(F32), "compacted output " + name)
    # without compaction every tile is an entry of the file; the constant data layer reads 1
    outputs = {"prob": tmp_path / "all_prob.dt"}
    backend.run_dataset(S.schema_text(layers), weights, {"images": tmp_path / "images.dt"}, outputs, max_entry_count=3)
    assert_bits(backend.read_dataset(outputs["prob"]), values["prob"], "every tile")
    backend.run_dataset(S.schema_text(layers), weights, {"images": tmp_path / "images.dt"}, {"flag": tmp_path / "flag.dt"})
    assert_bits(backend.read_dataset(tmp_path / "flag.dt"), np.ones((n, 1), F32), "the dataset_value layer")
    with pytest.raises(backend.BackendError, match="Cannot open"):
        backend.run_dataset(S.schema_text(layers), weights, {"images": tmp_path / "nowhere.dt"}, outputs)


@pytest.mark.parametrize("mode", ["together", "streams", "plain"])
def test_resnet50_post_convolution_graph_layer_by_layer(mode):
    """Config 4 through the driver at a small entry count: every output of the 50 steps (48 groups, the last block's group
    with the 7x7 average behind it, the softmax) against the oracle run layer by layer (bit for bit; softmax to 1e-5) - with
    independent groups launched together (the default), with one launch per group spread over three kernel streams, and
    with one launch per group on one stream."""
    from nnforge_amd import schemas

    gen = T.rng(62, 0)
    n = 3
    layers, configs, outputs = schemas.resnet50_post_convolution()
    weights = S.make_weights(layers, gen)
    inputs = {name: T.normal(gen, (n, fm, dims[1], dims[0])) for name, (fm, dims) in sorted(configs.items())}
    inputs["logits"] = T.normal(gen, (n, 1000, 1, 1), 4.0)
    values = S.evaluate(layers, weights, inputs)
    options = {"together": {}, "streams": {"one_launch_per_group": True}, "plain": {"one_launch_per_group": True, "kernel_stream_count": 1}}[mode]
    got, rep = run(layers, weights, inputs, outputs, values, max_entry_count=2, **options)
    assert len(rep["steps"]) == 50 and rep["entries"] == n
    assert [s["layers"][-2:] for s in rep["steps"] if s["layers"][-1] == "pool5"] == [["res5c_relu", "pool5"]]
    assert len({s["stream"] for s in rep["steps"]}) == (3 if mode == "streams" else 1)
    assert len({s["run"] for s in rep["steps"]} - {None}) == (6 if mode == "together" else 0)
    for name in outputs:
        if name == "prob":
            assert np.all(np.abs(got[name] - values[name]) <= 1e-5 * np.abs(values[name])), name
        else:
            assert_bits(got[name], values[name], name)


def test_the_reference_example_schema_runs_around_its_convolutions(tmp_path):
    """examples/gtsrb/working_data/schema.txt of the reference, as it stands in the file, with keep_unregistered_layers: the
    results of its four convolutions come in as inputs (seeded values), and every layer the backend computes is compared
    with the oracle layer by layer, bit for bit - TanH -> Absolute -> AverageSubsampling as one launch each, the average
    being the plain tester's window sum (no alpha in the file)."""
    import os

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gtsrb_schema.txt"), "rb") as f:
        text = f.read().decode("ascii")
    _, parsed = S.parse_schema_text(text)
    layers = S.layers_for_the_oracle(parsed)
    gen = T.rng(64, 1)
    n = 37
    shapes = {"parameters_0": (n, 38, 28, 28), "parameters_1": (n, 96, 10, 10), "parameters_2": (n, 200, 1, 1), "parameters_3": (n, 43, 1, 1)}
    inputs = {name: T.normal(gen, shape, 1.5) for name, shape in shapes.items()}
    inputs["parameters_0"].reshape(-1)[::97] = np.array([0.0, -0.0, 70.0, -70.0, np.inf, -np.inf, 1.0e-40], np.float32)[np.arange(inputs["parameters_0"].size)[::97] % 7]
    # the oracle's turn: only what hangs on the supplied values (the other data layers are never looked at)
    needed = [l for l in layers if l["type"] == "Data" or all(i in inputs or i.startswith(("tanh", "abs", "avg", "dropout")) for i in l["inputs"])]
    values = S.evaluate([l for l in needed if l["name"] in inputs or l["type"] != "Data"], {}, inputs)
    outputs = ["avg_0_layer", "abs_0_layer", "avg_1_layer", "dropout_2_layer", "tanh_3_layer"]
    shapes_out = {name: values[name].shape for name in outputs}
    got, rep = backend.run_schema(text, {}, inputs, shapes_out, keep_unregistered_layers=True, max_entry_count=16)
    assert rep["entries"] == n
    # abs_0_layer is wanted as well here, so the first stretch cannot go into the average's kernel whole
    assert sorted("+".join(st["layers"]) for st in rep["steps"]) == sorted([
        "tanh_0_layer+abs_0_layer", "avg_0_layer", "tanh_1_layer+abs_1_layer+avg_1_layer", "tanh_2_layer+abs_2_layer+dropout_2_layer", "tanh_3_layer"])
    for name in outputs:
        assert_bits(got[name], values[name], name)
    assert got["avg_0_layer"].shape == (n, 38, 14, 14) and got["avg_1_layer"].shape == (n, 96, 5, 5)


def test_packets_under_the_staging_bound_keep_a_few_entries():
    """hip_max_io_staging_mb bounds the pinned staging of a packet, but not below eight entries: entries of 12.6 MB in and
    12.6 MB out would fit 64 MB two at a time. Twelve entries then go as packets of eight and four; with the bound lifted
    as one packet of twelve; with hip_max_entry_count = 5 as packets of five (the bound never raises a packet)."""
    gen = T.rng(63, 1)
    n, c, size = 12, 3, 1024
    layers = [S.L("Data", "x"), S.L("BatchNorm", "bn", ["x"], feature_map_count=c), S.L("ReLU", "act", ["bn"])]
    weights = S.make_weights(layers, gen)
    inputs = {"x": T.normal(gen, (n, c, size, size))}
    values = S.evaluate(layers, weights, inputs)
    for options, packet in (({}, 8), ({"max_io_staging_mb": -1}, 12), ({"max_entry_count": 5}, 5), ({"max_io_staging_mb": 1024}, 12)):
        got, rep = run(layers, weights, inputs, ["act"], values, **options)
        assert rep["packet_entries"] == packet, (options, rep["raw"])
        assert_bits(got["act"], values["act"], str(options))


def test_resnet50_post_convolution_graph_at_64_entries():
    """Config 4 at its full size through the driver, one packet of 64 entries (the bound on a packet's pinned staging is
    lifted for it: 54 data layers of 44 MB of input per entry would otherwise make packets of 8), the default launch
    plan (six runs of groups launched together, tiles of every ResNet-50 shape by the hundred thousand per launch):
    every output against the oracle run layer by layer, bit for bit (softmax to 1e-5). Inputs are cut out of one pool
    of normal values at offsets of their own (what is compared is arithmetic and indexing, not statistics)."""
    from nnforge_amd import schemas

    gen = T.rng(62, 64)
    n = 64
    layers, configs, outputs = schemas.resnet50_post_convolution()
    weights = S.make_weights(layers, gen)
    pool = T.normal(gen, 1 << 25, 1.5)
    inputs = {}
    for i, (name, (fm, dims)) in enumerate(sorted(configs.items())):
        count = n * fm * dims[0] * dims[1]
        start = (7919 * (i + 1)) % 65536
        inputs[name] = np.resize(pool[start:], count).reshape(n, fm, dims[1], dims[0])
    values = S.evaluate(layers, weights, inputs)
    got, rep = run(layers, weights, inputs, outputs, values, max_entry_count=n, max_io_staging_mb=-1)
    assert rep["entries"] == n and rep["max_entry_count"] == n and len(rep["steps"]) == 50
    assert rep["packet_entries"] == n  # the launches compared below are the launches of 64 entries, not 64 times those of one
    assert len({s["run"] for s in rep["steps"]} - {None}) == 6
    for name in outputs:
        if name == "prob":
            assert np.all(np.abs(got[name] - values[name]) <= 1e-5 * np.abs(values[name])), name
        else:
            assert_bits(got[name], values[name], name)


def test_dropout_only_network():
    """Dropout straight from the data layer to the output: in place there is nothing to launch."""
    gen = T.rng(58, 0)
    layers = [S.L("Data", "in"), S.L("Dropout", "d1", ["in"]), S.L("Dropout", "d2", ["d1"], dropout_rate=0.1)]
    inputs = {"in": T.normal(gen, (9, 3, 5, 5))}
    values = S.evaluate(layers, {}, inputs)
    got, rep = run(layers, {}, inputs, ["d2"], values, max_entry_count=4)
    assert_bits(got["d2"], inputs["in"], "dropout chain")


# ---- statistics of a layer's output and the batch norm refresh built on them -----------------------

def two_bn_net(c=6):
    """stem -> BatchNorm -> ReLU -> max pooling -> BatchNorm -> TanH: the second BatchNorm sees data shaped by the first."""
    return [S.L("Data", "stem"), S.L("BatchNorm", "bn1", ["stem"], feature_map_count=c), S.L("ReLU", "relu1", ["bn1"]),
            S.L("MaxSubsampling", "pool", ["relu1"], windows=[2, 2]), S.L("BatchNorm", "bn2", ["pool"], feature_map_count=c),
            S.L("TanH", "out", ["bn2"])]


@pytest.mark.parametrize("on_host", [False, True])
def test_layer_statistics_on_device_and_on_host(on_host):
    """forward_propagation::run into a stat_data_bunch_writer. On the host (outputs copied back, one value
    at a time) the figures equal the oracle's bit for bit; reduced on the device they agree to one fp32 ulp."""
    gen = T.rng(59, int(on_host))
    c, n = 6, 23
    layers = two_bn_net(c)
    weights = S.make_weights(layers, gen)
    inputs = {"stem": (T.normal(gen, (n, c, 12, 12), 2.0) + F32(1.5)).astype(F32)}
    values = S.evaluate(layers, weights, inputs)
    want = oracle.FeatureMapStat(c).write(values["bn2"]).get()
    got, rep = backend.layer_statistics(S.schema_text(layers), weights, inputs, "bn2", c, max_entry_count=5, stat_on_host=on_host)
    assert rep["entries"] == n and rep["writer_entries"] == n
    assert np.array_equal(got["min"], want["min"]) and np.array_equal(got["max"], want["max"])
    if on_host:
        assert T.bit_mismatches(got["average"], want["average"]) == 0 and T.bit_mismatches(got["std_dev"], want["std_dev"]) == 0
    else:
        assert T.ulp_distance(got["average"], want["average"]).max() <= 1
        assert T.ulp_distance(got["std_dev"], want["std_dev"]).max() <= 1


def test_layer_statistics_with_a_short_last_packet_and_more_workgroups_than_the_device_holds():
    """256 feature maps of 7x7 in packets of 12 entries, 19 entries in all: the last packet of 7 prefers another cut
    into runs than the full one, and feature maps x entries is beyond one round of resident workgroups."""
    gen = T.rng(61, 0)
    c, n = 256, 19
    layers = two_bn_net(c)
    weights = S.make_weights(layers, gen)
    inputs = {"stem": (T.normal(gen, (n, c, 14, 14), 2.0) + F32(0.5)).astype(F32)}
    values = S.evaluate(layers, weights, inputs)
    want = oracle.FeatureMapStat(c).write(values["bn2"]).get()
    got, rep = backend.layer_statistics(S.schema_text(layers), weights, inputs, "bn2", c, max_entry_count=12)
    assert rep["entries"] == n and rep["writer_entries"] == n
    assert np.array_equal(got["min"], want["min"]) and np.array_equal(got["max"], want["max"])
    assert T.ulp_distance(got["average"], want["average"]).max() <= 1
    assert T.ulp_distance(got["std_dev"], want["std_dev"]).max() <= 1


def test_update_bn_weights_refreshes_every_batch_norm_in_forward_order(tmp_path):
    """toolset::update_bn_weights: the oracle replays it layer by layer (statistics with gamma 1 / beta 0,
    then the two formulas); the backend must arrive at the same mean / inverse sigma to one ulp of what
    the statistics allow, leave gamma and beta alone, and the refreshed layers must then produce mean 0,
    deviation 1 on that data."""
    gen = T.rng(60, 0)
    c, n = 6, 40
    layers = two_bn_net(c)
    weights = S.make_weights(layers, gen)
    inputs = {"stem": (T.normal(gen, (n, c, 12, 12), 3.0) - F32(2.0)).astype(F32)}

    # the reference's procedure on the CPU
    ref = {k: [a.copy() for a in v] for k, v in weights.items()}
    ones, zeros = np.ones(c, F32), np.zeros(c, F32)
    for name in ("bn1", "bn2"):
        trial = {k: list(v) for k, v in ref.items()}
        trial[name] = [ones, zeros, ref[name][2], ref[name][3]]
        out = S.evaluate(layers, trial, inputs)[name]
        st = oracle.FeatureMapStat(c).write(out).get()
        new_mean, new_inv = oracle.update_bn_weights(ref[name][2], ref[name][3], st["average"], st["std_dev"])
        ref[name] = [ref[name][0], ref[name][1], new_mean, new_inv]

    log = backend.update_bn_weights(S.schema_text(layers), weights, inputs, str(tmp_path), max_entry_count=16)
    assert "Updating Batch Normalization weights for these layers: bn1, bn2" in log
    assert log.count("Average ") == 2 * c
    for name in ("bn1", "bn2"):
        gamma, beta, mean, inv = backend.read_weights(str(tmp_path), name, [c] * 4)
        assert T.bit_mismatches(gamma, weights[name][0]) == 0 and T.bit_mismatches(beta, weights[name][1]) == 0
        # one ulp in average / std_dev moves the results by about that much relative to their size
        assert np.allclose(inv, ref[name][3], rtol=3e-7, atol=0), name
        assert np.allclose(mean, ref[name][2], rtol=3e-7, atol=3e-7), name
        assert not np.allclose(inv, weights[name][3], rtol=1e-3)

    # closed loop with the refreshed weights: normalised outputs
    new_weights = {name: backend.read_weights(str(tmp_path), name, [c] * 4) for name in ("bn1", "bn2")}
    plain = {name: [ones, zeros, w[2], w[3]] for name, w in new_weights.items()}
    probe = dict(new_weights)
    probe["bn2"] = plain["bn2"]
    st2, _ = backend.layer_statistics(S.schema_text(layers), probe, inputs, "bn2", c)
    assert np.abs(st2["average"]).max() < 1e-5 and np.abs(st2["std_dev"] - 1.0).max() < 1e-5
