"""ctypes binding of the C bridge over the C++ hip backend (include/nnforge_hip_backend.h):
run or plan a text-format nnForge schema. Used by the tests; contains no arithmetic."""

import ctypes
import os

import numpy as np

from . import build as _build
from .capi import _share_hip_runtime_with_torch

_FP = ctypes.POINTER(ctypes.c_float)
_UP = ctypes.POINTER(ctypes.c_uint32)


class Weights(ctypes.Structure):
    _fields_ = [("layer_name", ctypes.c_char_p), ("chunk_count", ctypes.c_uint32), ("chunk_sizes", _UP),
                ("chunks", ctypes.POINTER(_FP))]


class Input(ctypes.Structure):
    _fields_ = [("layer_name", ctypes.c_char_p), ("feature_map_count", ctypes.c_uint32), ("dimension_count", ctypes.c_uint32),
                ("dimension_sizes", _UP), ("data", _FP)]


class Output(ctypes.Structure):
    _fields_ = [("layer_name", ctypes.c_char_p), ("data", _FP), ("capacity_floats", ctypes.c_size_t),
                ("written_floats", ctypes.c_size_t)]


class Options(ctypes.Structure):
    _fields_ = [("struct_size", ctypes.c_uint32), ("fuse", ctypes.c_int32), ("dont_share_buffers", ctypes.c_int32), ("max_entry_count", ctypes.c_int32),
                ("profile", ctypes.c_int32), ("weights_from_folder", ctypes.c_int32), ("weights_folder", ctypes.c_char_p),
                ("profile_folder", ctypes.c_char_p), ("stat_on_host", ctypes.c_int32), ("kernel_stream_count", ctypes.c_int32),
                ("one_launch_per_group", ctypes.c_int32), ("host_thread_count", ctypes.c_int32), ("max_io_staging_mb", ctypes.c_int32),
                ("resident_packets", ctypes.c_int32), ("concat_copies_every_input", ctypes.c_int32), ("replay_recorded_plan", ctypes.c_int32), ("keep_unregistered_layers", ctypes.c_int32)]


class DatasetFile(ctypes.Structure):
    _fields_ = [("layer_name", ctypes.c_char_p), ("path", ctypes.c_char_p)]


class BackendError(RuntimeError):
    def __init__(self, code, message):
        RuntimeError.__init__(self, message)
        self.code = code


_lib = None
REPORT_CAPACITY = 1 << 16


def load():
    global _lib
    if _lib is None:
        path = _build.BACKEND_LIBRARY
        if not os.path.exists(path):
            raise RuntimeError("%s is missing: build it first (python -c 'import __graft_entry__ as g; g.build()')" % path)
        _share_hip_runtime_with_torch()
        lib = ctypes.CDLL(path)
        lib.nnf_backend_run_schema.argtypes = [ctypes.c_char_p, ctypes.POINTER(Weights), ctypes.c_uint32, ctypes.POINTER(Input),
                                               ctypes.c_uint32, ctypes.c_uint32, ctypes.POINTER(Output), ctypes.c_uint32,
                                               ctypes.POINTER(Options), ctypes.c_char_p, ctypes.c_size_t]
        lib.nnf_backend_plan_schema.argtypes = [ctypes.c_char_p, ctypes.POINTER(Input), ctypes.c_uint32,
                                                ctypes.POINTER(ctypes.c_char_p), ctypes.c_uint32, ctypes.POINTER(Options),
                                                ctypes.c_uint64, ctypes.c_char_p, ctypes.c_size_t]
        lib.nnf_backend_time_kernels.argtypes = [ctypes.c_char_p, ctypes.POINTER(Weights), ctypes.c_uint32, ctypes.POINTER(Input),
                                                 ctypes.c_uint32, ctypes.c_uint32, ctypes.POINTER(ctypes.c_char_p), ctypes.c_uint32,
                                                 ctypes.POINTER(Options), ctypes.c_uint32, ctypes.c_uint32, ctypes.c_char_p, ctypes.c_size_t]
        lib.nnf_backend_rewrite_schema.argtypes = [ctypes.c_char_p, ctypes.c_int32, ctypes.c_char_p, ctypes.c_size_t]
        lib.nnf_backend_list_layers.argtypes = [ctypes.c_char_p, ctypes.c_int32, ctypes.c_char_p, ctypes.c_size_t]
        lib.nnf_backend_write_weights.argtypes = [ctypes.c_char_p, ctypes.POINTER(Weights), ctypes.c_uint32, ctypes.c_char_p, ctypes.c_size_t]
        lib.nnf_backend_read_weights.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_uint32, _UP, ctypes.POINTER(_FP),
                                                 ctypes.c_char_p, ctypes.c_size_t]
        lib.nnf_backend_layer_statistics.argtypes = [ctypes.c_char_p, ctypes.POINTER(Weights), ctypes.c_uint32, ctypes.POINTER(Input),
                                                     ctypes.c_uint32, ctypes.c_uint32, ctypes.c_char_p, ctypes.c_uint32, _FP, _FP, _FP, _FP,
                                                     ctypes.POINTER(Options), ctypes.c_char_p, ctypes.c_size_t]
        lib.nnf_backend_update_bn_weights.argtypes = [ctypes.c_char_p, ctypes.POINTER(Weights), ctypes.c_uint32, ctypes.POINTER(Input),
                                                      ctypes.c_uint32, ctypes.c_uint32, ctypes.POINTER(Options), ctypes.c_char_p,
                                                      ctypes.c_char_p, ctypes.c_size_t]
        lib.nnf_backend_run_dataset.argtypes = [ctypes.c_char_p, ctypes.POINTER(Weights), ctypes.c_uint32, ctypes.POINTER(DatasetFile),
                                                ctypes.c_uint32, ctypes.POINTER(DatasetFile), ctypes.c_uint32, ctypes.c_uint32,
                                                ctypes.POINTER(Options), ctypes.c_char_p, ctypes.c_size_t]
        lib.nnf_backend_rewrite_dataset.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32,
                                                    ctypes.c_char_p, ctypes.c_size_t]
        _lib = lib
    return _lib


def _options(fuse=True, dont_share_buffers=False, max_entry_count=0, profile=False, weights_folder=None,
             profile_folder=None, stat_on_host=False, kernel_stream_count=0, one_launch_per_group=False, host_thread_count=0,
             max_io_staging_mb=0, resident_packets=0, keep_unregistered_layers=False, replay_recorded_plan=False,
             concat_copies_every_input=False):
    o = Options()
    o.concat_copies_every_input = int(concat_copies_every_input)
    o.replay_recorded_plan = int(replay_recorded_plan)
    o.keep_unregistered_layers = int(keep_unregistered_layers)
    o.struct_size = ctypes.sizeof(Options)
    o.max_io_staging_mb = int(max_io_staging_mb)
    o.resident_packets = int(resident_packets)
    o.fuse = int(fuse)
    o.dont_share_buffers = int(dont_share_buffers)
    o.max_entry_count = int(max_entry_count)
    o.profile = int(profile)
    o.weights_from_folder = int(weights_folder is not None)
    o.weights_folder = weights_folder.encode() if weights_folder is not None else None
    o.profile_folder = profile_folder.encode() if profile_folder is not None else None
    o.stat_on_host = int(stat_on_host)
    o.kernel_stream_count = int(kernel_stream_count)
    o.one_launch_per_group = int(one_launch_per_group)
    o.host_thread_count = int(host_thread_count)
    return o


def _weights_array(weights, keep):
    """weights: {layer name: [numpy chunk, ...]}"""
    arr = (Weights * max(1, len(weights)))()
    for i, (name, chunks) in enumerate(sorted(weights.items())):
        chunks = [np.ascontiguousarray(c, dtype=np.float32) for c in chunks]
        sizes = (ctypes.c_uint32 * len(chunks))(*[c.size for c in chunks])
        ptrs = (_FP * len(chunks))(*[c.ctypes.data_as(_FP) for c in chunks])
        keep.extend([chunks, sizes, ptrs])
        arr[i].layer_name = name.encode()
        arr[i].chunk_count = len(chunks)
        arr[i].chunk_sizes = sizes
        arr[i].chunks = ptrs
    return arr


def _inputs_array(inputs, keep, with_data=True):
    """inputs: {data layer name: numpy array [entries][feature maps][...spatial, x last]} or, when
    only planning, {name: (feature_map_count, [dimension sizes, x first])}"""
    arr = (Input * max(1, len(inputs)))()
    entry_count = None
    for i, (name, value) in enumerate(sorted(inputs.items())):
        if with_data:
            a = np.ascontiguousarray(value, dtype=np.float32)
            fm = a.shape[1]
            dims = list(a.shape[2:])[::-1]
            entry_count = a.shape[0] if entry_count is None else entry_count
            assert a.shape[0] == entry_count
            keep.append(a)
            arr[i].data = a.ctypes.data_as(_FP)
        else:
            fm, dims = value
        dim_arr = (ctypes.c_uint32 * max(1, len(dims)))(*dims)
        keep.append(dim_arr)
        arr[i].layer_name = name.encode()
        arr[i].feature_map_count = fm
        arr[i].dimension_count = len(dims)
        arr[i].dimension_sizes = dim_arr
    return arr, entry_count


def parse_report(text):
    res = {"steps": [], "seconds": {}, "outputs": {}, "raw": text}
    for line in text.splitlines():
        key, _, rest = line.partition(": ")
        if key == "step":
            # "fused|single <layers> <- <inputs> @<kernel stream>[ #<run of groups launched together>]"
            kind, _, desc = rest.partition(" ")
            desc, _, placement = desc.rpartition(" @")
            placement, _, in_place = placement.partition(" =")
            placement, _, writes_into = placement.partition(" >")
            stream, _, run = placement.partition(" #")
            layers, _, sources = desc.partition(" <- ")
            res["steps"].append({"fused": kind == "fused", "layers": layers.split("+"), "inputs": sources.split(", "), "stream": int(stream),
                                 "run": int(run) if run else None, "writes_into": writes_into or None,
                                 "inputs_in_place": in_place.split(",") if in_place else []})
        elif key in ("per_entry_bytes", "max_entry_count", "entries", "writer_entries", "launches", "timed_entries", "packet_entries", "plan_steps", "resident_packets"):
            res[key] = int(rest)
        elif key in ("wall_seconds_per_pass", "device_seconds_per_pass", "host_seconds_per_pass"):
            res[key] = float(rest)
        elif key == "seconds":
            name, _, sec = rest.rpartition(" ")
            res["seconds"][name] = float(sec)
        elif key == "output":
            name, _, cfg = rest.partition(" ")
            res["outputs"][name] = cfg
        elif key == "stat":
            res["stat"] = rest
    return res


def run_schema(schema_text, weights, inputs, output_shapes, **options):
    """output_shapes: {output layer name: numpy shape of the whole result [entries][...]}.
    Returns ({name: array}, parsed report)."""
    lib = load()
    keep = []
    w = _weights_array(weights, keep)
    ins, entry_count = _inputs_array(inputs, keep)
    outs = (Output * len(output_shapes))()
    arrays = {}
    for i, (name, shape) in enumerate(sorted(output_shapes.items())):
        a = np.full(shape, np.nan, dtype=np.float32)
        arrays[name] = a
        outs[i].layer_name = name.encode()
        outs[i].data = a.ctypes.data_as(_FP)
        outs[i].capacity_floats = a.size
    report = ctypes.create_string_buffer(REPORT_CAPACITY)
    opt = _options(**options)
    rc = lib.nnf_backend_run_schema(schema_text.encode(), w, len(weights), ins, len(inputs), entry_count or 0, outs,
                                    len(output_shapes), ctypes.byref(opt), report, REPORT_CAPACITY)
    if rc != 0:
        raise BackendError(rc, report.value.decode(errors="replace"))
    for i, name in enumerate(sorted(output_shapes)):
        assert outs[i].written_floats == arrays[name].size, (name, outs[i].written_floats, arrays[name].size)
    return arrays, parse_report(report.value.decode())


def layer_statistics(schema_text, weights, inputs, layer_name, feature_map_count, **options):
    """Per-feature-map statistics of one layer's output: {'min', 'max', 'average', 'std_dev'} and the parsed report."""
    lib = load()
    keep = []
    w = _weights_array(weights, keep)
    ins, entry_count = _inputs_array(inputs, keep)
    res = {k: np.full(feature_map_count, np.nan, dtype=np.float32) for k in ("min", "max", "average", "std_dev")}
    report = ctypes.create_string_buffer(REPORT_CAPACITY)
    opt = _options(**options)
    rc = lib.nnf_backend_layer_statistics(schema_text.encode(), w, len(weights), ins, len(inputs), entry_count or 0, layer_name.encode(),
                                          feature_map_count, *[res[k].ctypes.data_as(_FP) for k in ("min", "max", "average", "std_dev")],
                                          ctypes.byref(opt), report, REPORT_CAPACITY)
    if rc != 0:
        raise BackendError(rc, report.value.decode(errors="replace"))
    return res, parse_report(report.value.decode())


def update_bn_weights(schema_text, weights, inputs, out_folder, **options):
    """Refreshes the BatchNorm weights from the inputs' statistics and writes all weights to out_folder;
    returns the lines the reference prints while doing so."""
    lib = load()
    keep = []
    w = _weights_array(weights, keep)
    ins, entry_count = _inputs_array(inputs, keep)
    report = ctypes.create_string_buffer(1 << 20)
    opt = _options(**options)
    rc = lib.nnf_backend_update_bn_weights(schema_text.encode(), w, len(weights), ins, len(inputs), entry_count or 0, ctypes.byref(opt),
                                           out_folder.encode(), report, 1 << 20)
    if rc != 0:
        raise BackendError(rc, report.value.decode(errors="replace"))
    return report.value.decode()


def plan_schema(schema_text, input_configs, output_names, memory_bytes=288 << 30, **options):
    lib = load()
    keep = []
    ins, _ = _inputs_array(input_configs, keep, with_data=False)
    names = (ctypes.c_char_p * len(output_names))(*[n.encode() for n in output_names])
    report = ctypes.create_string_buffer(REPORT_CAPACITY)
    opt = _options(**options)
    rc = lib.nnf_backend_plan_schema(schema_text.encode(), ins, len(input_configs), names, len(output_names), ctypes.byref(opt),
                                     memory_bytes, report, REPORT_CAPACITY)
    if rc != 0:
        raise BackendError(rc, report.value.decode(errors="replace"))
    return parse_report(report.value.decode())


def time_kernels(schema_text, weights, inputs, output_names, warmup=2, passes=5, shared_input_pool=None, entry_count=None, **options):
    """Device time of the schema's launch plan on one resident packet (forward_propagation_hip::time_kernels).
    inputs: {data layer: array [entries][feature maps][...]} or, with shared_input_pool (a flat float32 array at least as
    long as the largest input), {data layer: (feature_map_count, [dimension sizes, x first])} - every data layer then reads
    its entries from the start of the pool (the values do not matter for the time). Returns the parsed report."""
    lib = load()
    keep = []
    w = _weights_array(weights, keep)
    if shared_input_pool is None:
        ins, entry_count = _inputs_array(inputs, keep)
    else:
        pool = np.ascontiguousarray(shared_input_pool, dtype=np.float32)
        keep.append(pool)
        ins, _ = _inputs_array(inputs, keep, with_data=False)
        for i, (name, (fm, dims)) in enumerate(sorted(inputs.items())):
            assert entry_count * fm * int(np.prod(dims, dtype=np.int64)) <= pool.size, name
            ins[i].data = pool.ctypes.data_as(_FP)
    names = (ctypes.c_char_p * len(output_names))(*[n.encode() for n in output_names])
    report = ctypes.create_string_buffer(REPORT_CAPACITY)
    opt = _options(**options)
    rc = lib.nnf_backend_time_kernels(schema_text.encode(), w, len(weights), ins, len(inputs), entry_count or 0, names, len(output_names),
                                      ctypes.byref(opt), warmup, passes, report, REPORT_CAPACITY)
    if rc != 0:
        raise BackendError(rc, report.value.decode(errors="replace"))
    return parse_report(report.value.decode())


def rewrite_schema(schema_text, keep_unregistered_layers=False):
    lib = load()
    out = ctypes.create_string_buffer(REPORT_CAPACITY)
    rc = lib.nnf_backend_rewrite_schema(schema_text.encode(), int(keep_unregistered_layers), out, REPORT_CAPACITY)
    if rc != 0:
        raise BackendError(rc, out.value.decode(errors="replace"))
    return out.value.decode()


def list_layers(schema_text, keep_unregistered_layers=False):
    """-> [{"type", "name", "inputs", "parameters", "external"}] in forward propagation order"""
    lib = load()
    out = ctypes.create_string_buffer(REPORT_CAPACITY)
    rc = lib.nnf_backend_list_layers(schema_text.encode(), int(keep_unregistered_layers), out, REPORT_CAPACITY)
    if rc != 0:
        raise BackendError(rc, out.value.decode(errors="replace"))
    res = []
    for line in out.value.decode().splitlines():
        kind, name, inputs, params, origin = line[len("layer: "):].split("\t")
        res.append({"type": kind, "name": name, "inputs": inputs.split(",") if inputs else [], "parameters": params, "external": origin == "external"})
    return res


def write_weights(folder, weights):
    lib = load()
    keep = []
    w = _weights_array(weights, keep)
    report = ctypes.create_string_buffer(4096)
    rc = lib.nnf_backend_write_weights(folder.encode(), w, len(weights), report, 4096)
    if rc != 0:
        raise BackendError(rc, report.value.decode(errors="replace"))


def read_weights(folder, layer_name, chunk_sizes):
    lib = load()
    chunks = [np.empty(s, dtype=np.float32) for s in chunk_sizes]
    sizes = (ctypes.c_uint32 * len(chunks))(*chunk_sizes)
    ptrs = (_FP * len(chunks))(*[c.ctypes.data_as(_FP) for c in chunks])
    report = ctypes.create_string_buffer(4096)
    rc = lib.nnf_backend_read_weights(folder.encode(), layer_name.encode(), len(chunks), sizes, ptrs, report, 4096)
    if rc != 0:
        raise BackendError(rc, report.value.decode(errors="replace"))
    return chunks


# ---- data set files (".dt") -------------------------------------------------------------------------

DATASET_GUID = bytes([0x2c, 0x62, 0xe0, 0x5a, 0xc6, 0x21, 0x43, 0xb2, 0xa8, 0x2c, 0x85, 0xcd, 0x58, 0x58, 0x15, 0xd9])


def write_dataset(path, array):
    """array [entries][feature maps][...spatial, x last] -> nnForge's data set file: GUID, u32 feature maps, u32 dimension
    count, u32 sizes (x first), u32 entry count, fp32 entries (nnforge/structured_data_stream_writer.cpp:26-66)."""
    a = np.ascontiguousarray(array, dtype="<f4")
    dims = list(a.shape[2:])[::-1]
    with open(path, "wb") as f:
        f.write(DATASET_GUID)
        f.write(np.array([a.shape[1], len(dims)] + dims + [a.shape[0]], dtype="<u4").tobytes())
        f.write(a.tobytes())


def read_dataset(path):
    """-> array [entries][feature maps][...spatial, x last] of a data set file."""
    with open(path, "rb") as f:
        raw = f.read()
    if raw[:16] != DATASET_GUID:
        raise ValueError("%s is not a structured data file" % path)
    fm, dim_count = np.frombuffer(raw, dtype="<u4", count=2, offset=16)
    dims = [int(d) for d in np.frombuffer(raw, dtype="<u4", count=int(dim_count), offset=24)]
    offset = 24 + 4 * int(dim_count)
    entries = int(np.frombuffer(raw, dtype="<u4", count=1, offset=offset)[0])
    per_entry = int(fm) * int(np.prod(dims, dtype=np.int64))
    data = np.frombuffer(raw, dtype="<f4", count=entries * per_entry, offset=offset + 4)
    return data.reshape([entries, int(fm)] + dims[::-1]).copy()


def _dataset_files(files, keep):
    arr = (DatasetFile * max(1, len(files)))()
    for i, (name, path) in enumerate(sorted(files.items())):
        keep.extend([name.encode(), str(path).encode()])
        arr[i].layer_name, arr[i].path = keep[-2], keep[-1]
    return arr


def run_dataset(schema_text, weights, input_files, output_files, compact_samples=1, **options):
    """input_files / output_files: {layer name: path of a data set file}. Returns the parsed report."""
    lib = load()
    keep = []
    w = _weights_array(weights, keep)
    ins, outs = _dataset_files(input_files, keep), _dataset_files(output_files, keep)
    report = ctypes.create_string_buffer(REPORT_CAPACITY)
    opt = _options(**options)
    rc = lib.nnf_backend_run_dataset(schema_text.encode(), w, len(weights), ins, len(input_files), outs, len(output_files), compact_samples,
                                     ctypes.byref(opt), report, REPORT_CAPACITY)
    if rc != 0:
        raise BackendError(rc, report.value.decode(errors="replace"))
    return parse_report(report.value.decode())


def rewrite_dataset(in_path, out_path, compact_samples=1, part_count=1, part=0):
    """Host only. Returns the report text (configuration, entry counts, per-neuron average of what was read)."""
    lib = load()
    report = ctypes.create_string_buffer(1 << 20)
    rc = lib.nnf_backend_rewrite_dataset(str(in_path).encode(), str(out_path).encode(), compact_samples, part_count, part, report, 1 << 20)
    if rc != 0:
        raise BackendError(rc, report.value.decode(errors="replace"))
    return report.value.decode()
