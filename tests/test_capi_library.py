"""The C-ABI library: it loads, exports every symbol include/nnforge_hip.h declares, and its
argument checks (which run before any GPU work) return the documented codes."""

import ctypes
import os
import re

from nnforge_amd import build, capi

HEADER = os.path.join(build.REPO_ROOT, "include", "nnforge_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"NNF_HIP_API\s+[\w\s\*]+?\b(nnf_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    names = declared_symbols()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), name
    # and the binding covers the header exactly
    bound = set(capi.SIGNATURES) | set(capi.STRING_FUNCTIONS)
    assert bound == set(names)


def test_backend_library_exports_every_declared_symbol():
    from nnforge_amd import backend

    text = open(os.path.join(build.REPO_ROOT, "include", "nnforge_hip_backend.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"NNF_BACKEND_API\s+[\w\s\*]+?\b(nnf_backend_\w+)\s*\(", text)))
    assert len(names) >= 9, names
    lib = backend.load()
    for name in names:
        assert hasattr(lib, name), name
        assert getattr(lib, name).argtypes is not None, "no ctypes signature for " + name


def test_struct_layout_matches_the_header():
    # nnf_hip_op: 4 x 4 bytes; nnf_hip_chain_desc: 6 + 4 + 1 words, then 8 ops
    assert ctypes.sizeof(capi.Op) == 16
    assert ctypes.sizeof(capi.ChainDesc) == 4 * 11 + 16 * capi.MAX_OPS
    text = open(HEADER).read()
    assert "#define NNF_HIP_MAX_OPS %d" % capi.MAX_OPS in text
    assert "#define NNF_HIP_MAX_INPUTS %d" % capi.MAX_INPUTS in text
    for name, value in (("NNF_HIP_OP_BATCH_NORM", capi.OP_BATCH_NORM), ("NNF_HIP_OP_RELU", capi.OP_RELU), ("NNF_HIP_OP_PRELU", capi.OP_PRELU),
                        ("NNF_HIP_OP_ELU", capi.OP_ELU), ("NNF_HIP_OP_SIGMOID", capi.OP_SIGMOID), ("NNF_HIP_OP_TANH", capi.OP_TANH)):
        assert re.search(r"%s\s*=\s*%d\b" % (name, value), text), name


def test_argument_checks_need_no_gpu():
    lib = capi.load()
    fake = 0x10000  # never dereferenced: the checks below fail before any launch
    assert lib.nnf_hip_rectified_linear_forward(None, None, fake, 0.0, 8) == capi.E_INVAL
    assert lib.nnf_hip_rectified_linear_forward(None, fake + 4, fake + 4096, 0.0, 8) == capi.E_ALIGN
    assert lib.nnf_hip_rectified_linear_forward(None, fake + 16, fake, 0.0, 8) == capi.E_OVERLAP
    assert lib.nnf_hip_rectified_linear_forward(None, fake, fake + (1 << 40), 0.0, 1 << 33) == capi.E_TOOBIG
    assert lib.nnf_hip_softmax_forward(None, fake, fake + 4096, 4, 0, 1) == capi.E_INVAL
    assert lib.nnf_hip_average_subsampling_forward(None, fake, fake + 4096, 1, 1, 4, 4, 5, 1, 1.0) == capi.E_INVAL
    assert lib.nnf_hip_copy_kernel(None, fake, fake + 4096, 24) == capi.E_INVAL
    desc = capi.make_desc(1, 4, 4, [[], []], has_add=False)
    ins = capi.pointer_array([fake, fake + 4096])
    assert lib.nnf_hip_chain_forward(None, ctypes.byref(desc), fake + 8192, ins, None) == capi.E_INVAL
    desc = capi.make_desc(0, 4, 4, [[(capi.OP_RELU, 0, 0.0)]])
    assert lib.nnf_hip_chain_forward(None, ctypes.byref(desc), fake, capi.pointer_array([fake]), None) == 0  # zero entries: no work
    for code in (0, capi.E_INVAL, capi.E_UNSUPPORTED, capi.E_ALIGN, capi.E_OVERLAP, capi.E_TOOBIG, 1, 98):
        assert lib.nnf_hip_error_string(code)
    assert b"gfx950" in lib.nnf_hip_version()


def test_statistics_workspace_of_a_packet_serves_every_shorter_packet():
    """The driver sizes the statistics workspace once, for a full packet, and the last packet of a run is
    shorter. The reduction is cut into runs of entries so that the grid fills whole rounds of resident
    workgroups, and fewer entries can mean MORE runs (256 feature maps of 7x7: 29 entries -> 15 runs, 16
    entries -> 16 runs): the plan therefore has to be made inside the workspace that is there."""
    lib = capi.load()
    need, count = ctypes.c_size_t(), ctypes.c_uint32()
    grew = 0
    for fm, plane, packet in ((64, 49, 29), (256, 49, 12), (256, 49, 64), (2048, 49, 64), (64, 3136, 40), (3, 224 * 224, 8),
                              (1000, 1, 300), (7, 100003, 5), (512, 196, 33)):
        assert lib.nnf_hip_feature_map_stat_workspace_bytes(packet, fm, plane, ctypes.byref(need)) == 0
        assert need.value % 32 == 0 and need.value >= 32 * fm
        for entries in range(1, packet + 1):
            assert lib.nnf_hip_feature_map_stat_partial_count(entries, fm, plane, need.value, ctypes.byref(count)) == 0, (fm, plane, packet, entries)
            assert fm <= count.value <= need.value // 32 and count.value % fm == 0
            own = ctypes.c_size_t()
            assert lib.nnf_hip_feature_map_stat_workspace_bytes(entries, fm, plane, ctypes.byref(own)) == 0
            grew += own.value > need.value
    assert grew > 0, "no case where a shorter packet prefers more partial states: the test lost its point"
    # a workspace below one state per feature map holds no plan; zero entries need none
    assert lib.nnf_hip_feature_map_stat_partial_count(4, 64, 49, 32 * 63, ctypes.byref(count)) == capi.E_INVAL
    assert lib.nnf_hip_feature_map_stat_partial_count(0, 64, 49, 0, ctypes.byref(count)) == 0 and count.value == 0
