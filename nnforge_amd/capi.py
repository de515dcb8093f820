"""ctypes binding of the C ABI in include/nnforge_hip.h (plain pointers and sizes, no torch types).

Callers pass device addresses as integers (e.g. ``tensor.data_ptr()``) and a HIP stream handle as
an integer (e.g. ``torch.cuda.current_stream().cuda_stream``). There is no fallback: if the
library has not been built, loading raises.
"""

import ctypes
import os

from . import build as _build

MAX_OPS = 8
MAX_INPUTS = 4

OP_BATCH_NORM = 1
OP_RELU = 2
OP_PRELU = 3
OP_ELU = 4
OP_SIGMOID = 5
OP_TANH = 6
OP_ABSOLUTE = 7
OP_DROPOUT = 8

E_INVAL = -1
E_UNSUPPORTED = -2
E_ALIGN = -3
E_OVERLAP = -4
E_TOOBIG = -5
E_SCRATCH = -6


class Op(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("chunk", ctypes.c_int32), ("f0", ctypes.c_float), ("f1", ctypes.c_float)]


class ChainDesc(ctypes.Structure):
    _fields_ = [
        ("entry_count", ctypes.c_uint32),
        ("feature_map_count", ctypes.c_uint32),
        ("neuron_count_per_feature_map", ctypes.c_uint32),
        ("input_count", ctypes.c_uint32),
        ("has_add", ctypes.c_uint32),
        ("add_alpha", ctypes.c_float),
        ("arm_op_count", ctypes.c_uint32 * MAX_INPUTS),
        ("tail_op_count", ctypes.c_uint32),
        ("ops", Op * MAX_OPS),
    ]


_VP = ctypes.c_void_p
_U32 = ctypes.c_uint32
_U64 = ctypes.c_uint64
_F = ctypes.c_float
_PP = ctypes.POINTER(ctypes.c_void_p)
_UP = ctypes.POINTER(ctypes.c_uint32)

# name -> argtypes, exactly the declarations of include/nnforge_hip.h (all return int unless noted)
SIGNATURES = {
    "nnf_hip_chain_forward": [_VP, ctypes.POINTER(ChainDesc), _VP, _PP, _PP],
    "nnf_hip_chain_forward_batch": [_VP, _U32, ctypes.POINTER(ChainDesc), ctypes.POINTER(_VP), ctypes.POINTER(ctypes.POINTER(_VP)), ctypes.POINTER(ctypes.POINTER(_VP))],
    "nnf_hip_batch_norm_forward": [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _U32, _U32, _U32],
    "nnf_hip_rectified_linear_forward": [_VP, _VP, _VP, _F, _U64],
    "nnf_hip_parametric_rectified_linear_forward": [_VP, _VP, _VP, _VP, _U32, _U32, _U32],
    "nnf_hip_exponential_linear_forward": [_VP, _VP, _VP, _U64],
    "nnf_hip_sigmoid_forward": [_VP, _VP, _VP, _U64],
    "nnf_hip_hyperbolic_tangent_forward": [_VP, _VP, _VP, _F, _F, _U64],
    "nnf_hip_add_forward": [_VP, _VP, _PP, _U32, _F, _U64],
    "nnf_hip_absolute_forward": [_VP, _VP, _VP, _U64],
    "nnf_hip_dropout_forward": [_VP, _VP, _VP, _U64],
    "nnf_hip_concat_forward": [_VP, _VP, _PP, ctypes.POINTER(_U32), _U32, _U32],
    "nnf_hip_concat_forward_partial": [_VP, _VP, _PP, ctypes.POINTER(_U32), ctypes.POINTER(ctypes.c_uint8), _U32, _U32],
    "nnf_hip_maxout_forward": [_VP, _VP, _VP, _U32, _U32, _U32, _U32],
    "nnf_hip_max_subsampling_forward": [_VP, _VP, _VP, _U32, _U32, _U32, ctypes.POINTER(_U32), ctypes.POINTER(_U32),
                                        ctypes.POINTER(_U32), ctypes.POINTER(_U32), _U32, _U32, ctypes.c_int32],
    "nnf_hip_feature_map_stat_init": [_VP, _VP, _U32],
    "nnf_hip_feature_map_stat_workspace_bytes": [_U32, _U32, _U32, ctypes.POINTER(ctypes.c_size_t)],
    "nnf_hip_feature_map_stat_partial_count": [_U32, _U32, _U32, ctypes.c_size_t, ctypes.POINTER(_U32)],
    "nnf_hip_feature_map_stat_accumulate_static": [_VP, _VP, _VP, _U32, _U32, _U32],
    "nnf_hip_feature_map_stat_accumulate": [_VP, _VP, _VP, ctypes.c_size_t, _VP, _U32, _U32, _U32],
    "nnf_hip_softmax_forward": [_VP, _VP, _VP, _U32, _U32, _U32],
    "nnf_hip_average_subsampling_forward": [_VP, _VP, _VP, _U32, _U32, _U32, _U32, _U32, _U32, _F],
    "nnf_hip_device_count": [ctypes.POINTER(ctypes.c_int)],
    "nnf_hip_set_device": [ctypes.c_int],
    "nnf_hip_device_info": [ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(_U64),
                            ctypes.POINTER(_U32), ctypes.POINTER(_U32), ctypes.POINTER(_U32)],
    "nnf_hip_malloc": [_PP, ctypes.c_size_t],
    "nnf_hip_free": [_VP],
    "nnf_hip_memcpy_h2d": [_VP, _VP, ctypes.c_size_t, _VP],
    "nnf_hip_memcpy_d2h": [_VP, _VP, ctypes.c_size_t, _VP],
    "nnf_hip_memcpy_d2d": [_VP, _VP, ctypes.c_size_t, _VP],
    "nnf_hip_host_malloc": [_PP, ctypes.c_size_t],
    "nnf_hip_host_free": [_VP],
    "nnf_hip_stream_create": [_PP],
    "nnf_hip_stream_destroy": [_VP],
    "nnf_hip_stream_synchronize": [_VP],
    "nnf_hip_device_synchronize": [],
    "nnf_hip_event_create": [_PP],
    "nnf_hip_event_destroy": [_VP],
    "nnf_hip_event_record": [_VP, _VP],
    "nnf_hip_event_synchronize": [_VP],
    "nnf_hip_event_elapsed_ms": [ctypes.POINTER(_F), _VP, _VP],
    "nnf_hip_stream_wait_event": [_VP, _VP],
    "nnf_hip_copy_kernel": [_VP, _VP, _VP, ctypes.c_size_t],
    "nnf_hip_check_division_sequences": [_VP, _VP],
    "nnf_hip_average_subsampling_nd_forward": [_VP, _VP, _VP, _U32, _U32, _U32, _UP, _UP, _U32, _U32, _F],
    "nnf_hip_max_subsampling_tiling_forward": [_VP, _VP, _VP, _U32, _U32, _U32, _UP, _UP, ctypes.c_int32],
    "nnf_hip_max_subsampling_fused_forward": [_VP, _VP, _VP, ctypes.POINTER(ChainDesc), _PP, _U32, _U32, _U32, _UP, _UP, _UP, _UP, _U32, _U32, ctypes.c_int32],
    "nnf_hip_average_subsampling_fused_forward": [_VP, _VP, _VP, ctypes.POINTER(ChainDesc), _PP, _U32, _U32, _U32, _U32, _U32, _U32, _F],
    "nnf_hip_max_subsampling_fusable": [_U32, _U32, _U32, _UP, _UP, _UP, _UP, _U32, _U32],
    "nnf_hip_average_subsampling_fusable": [_U32, _U32, _U32, _U32, _U32, _U32],
    "nnf_hip_average_subsampling_joined_forward": [_VP, _VP, _PP, ctypes.POINTER(ChainDesc), _PP, _U32, _U32, _U32, _U32, _U32, _U32, _F],
    "nnf_hip_average_subsampling_joinable": [_U32, _U32, _U32, _U32, _U32, _U32],
    "nnf_hip_launch_count": [ctypes.POINTER(_U64)],
    "nnf_hip_chain_forward_strided": [_VP, ctypes.POINTER(ChainDesc), _VP, _U32, _PP, _PP],
    "nnf_hip_chain_forward_strided_status": [ctypes.POINTER(ChainDesc), _U32],
    "nnf_hip_chain_forward_strided_batch": [_VP, _U32, ctypes.POINTER(ChainDesc), ctypes.POINTER(_VP), ctypes.POINTER(_U32), ctypes.POINTER(ctypes.POINTER(_VP)), ctypes.POINTER(ctypes.POINTER(_VP))],
    "nnf_hip_stream_begin_capture": [_VP],
    "nnf_hip_stream_end_capture": [_VP, _PP],
    "nnf_hip_graph_launch": [_VP, _VP],
    "nnf_hip_graph_destroy": [_VP],
}
STRING_FUNCTIONS = {"nnf_hip_error_string": [ctypes.c_int], "nnf_hip_version": []}

_lib = None


class NnfHipError(RuntimeError):
    def __init__(self, code, message):
        RuntimeError.__init__(self, "%s (code %d)" % (message, code))
        self.code = code


def _share_hip_runtime_with_torch():
    """PyTorch wheels bundle their own HIP runtime. A process must not end up with two of them
    (the one loaded second does not see the GPU), so when torch is installed it is imported before
    this library is loaded: the library's libamdhip64 dependency then resolves to the runtime torch
    already mapped. Without torch the system's ROCm runtime is used."""
    try:
        import torch  # noqa: F401
    except ImportError:
        pass


def library_path():
    return _build.HIP_LIBRARY


def load():
    """Loads libnnforge_hip.so built in-tree; raises if it is missing (there is no fallback path)."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(
            "%s is missing: build it first (python -c 'import __graft_entry__ as g; g.build()')" % path)
    _share_hip_runtime_with_torch()
    lib = ctypes.CDLL(path)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
    for name, argtypes in STRING_FUNCTIONS.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_char_p
    _lib = lib
    return lib


def error_string(code):
    return load().nnf_hip_error_string(code).decode()


def check(code):
    if code != 0:
        raise NnfHipError(code, error_string(code))


def pointer_array(addresses):
    arr = (ctypes.c_void_p * max(1, len(addresses)))()
    for i, a in enumerate(addresses):
        arr[i] = a
    return arr


def make_desc(entry_count, feature_map_count, plane, arms, tail=(), has_add=None, add_alpha=1.0):
    """arms: one list of ops per input tensor; tail: ops after the join. An op is a tuple
    (kind, chunk, f0, f1) with trailing fields optional."""
    d = ChainDesc()
    d.entry_count = entry_count
    d.feature_map_count = feature_map_count
    d.neuron_count_per_feature_map = plane
    d.input_count = len(arms)
    d.has_add = int(has_add if has_add is not None else len(arms) > 1)
    d.add_alpha = add_alpha
    k = 0
    for j, arm in enumerate(arms):
        d.arm_op_count[j] = len(arm)
        for op in arm:
            _fill_op(d.ops[k], op)
            k += 1
    d.tail_op_count = len(tail)
    for op in tail:
        _fill_op(d.ops[k], op)
        k += 1
    return d


def _fill_op(dst, op):
    op = tuple(op) + (0, 0.0, 0.0)
    dst.kind = op[0]
    dst.chunk = int(op[1])
    dst.f0 = float(op[2])
    dst.f1 = float(op[3])


def chain_forward(desc, output, inputs, chunks=(), stream=0):
    """output / inputs / chunks: device addresses (ints). Raises NnfHipError on a non-zero return."""
    lib = load()
    ins = pointer_array(list(inputs))
    chk = pointer_array(list(chunks))
    check(lib.nnf_hip_chain_forward(stream, ctypes.byref(desc), output, ins, chk if len(chunks) else None))
