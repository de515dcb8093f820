"""The benchmark configurations as data: shapes, fused groups and their algorithmic bytes.

Each fused group is what the backend's fusion pass makes of a run of element-wise layers in an
nnForge schema; the ResNet-50 list follows the schema generator of the reference
(examples/imagenet/imagenet_toolset.cpp:476-550, 729-831): per bottleneck block
reduce_fm -> BN -> ReLU, bottleneck(3x3, carries the stride) -> BN -> ReLU, restore_fm -> BN,
Add([shortcut_bn or previous block output, restore_fm_bn]) -> ReLU. Convolution outputs are
replaced by synthetic tensors, so every group reads its inputs from memory and writes one output.

No arithmetic lives here; bench.py and the tests turn these descriptions into C-ABI calls.
"""

from collections import namedtuple

from . import capi

TANH_SCALE = 1.7159
TANH_STEEPNESS = 0.6666
BN_EPSILON = 1e-5

# arms: per input tensor the list of ops applied before the join (Add); tail: ops after it.
# chunks: layout of chunk_ptrs, a list of ("bn", C) / ("prelu", C) entries in pointer order.
Group = namedtuple("Group", "name entry_count feature_map_count plane arms tail chunks")


def group_elements(g):
    return g.entry_count * g.feature_map_count * g.plane


def group_algorithmic_bytes(g):
    """Compulsory traffic of the fused group: every input tensor read once, the output written
    once, plus the per-feature-map weights."""
    tensors = len(g.arms) + 1
    weights = sum(4 * c if kind == "bn" else c for kind, c in g.chunks)
    return 4 * (tensors * group_elements(g) + weights)


def unfused_passes(g):
    """Tensor passes (reads + writes) the plain backend makes for the same layers, one tester
    call per layer (nnforge/plain/forward_propagation_plain.cpp:137-186)."""
    passes = 0
    for arm in g.arms:
        passes += 2 * len(arm)
    if len(g.arms) > 1:
        passes += len(g.arms) + 1
    passes += 2 * len(g.tail)
    return passes


def bn_relu(name, n, c, plane):
    return Group(name, n, c, plane, [[(capi.OP_BATCH_NORM, 0)]], [(capi.OP_RELU, 0, 0.0)], [("bn", c)])


def bn_add_relu(name, n, c, plane):
    # Add inputs in schema order: [residual, BN(main path)]
    return Group(name, n, c, plane, [[], [(capi.OP_BATCH_NORM, 0)]], [(capi.OP_RELU, 0, 0.0)], [("bn", c)])


def bn_bn_add_relu(name, n, c, plane):
    # Add inputs: [BN(shortcut), BN(main path)]
    return Group(name, n, c, plane, [[(capi.OP_BATCH_NORM, 0)], [(capi.OP_BATCH_NORM, 4)]], [(capi.OP_RELU, 0, 0.0)],
                 [("bn", c), ("bn", c)])


def config0(n=32, c=64, hw=56):
    return bn_relu("bn_relu", n, c, hw * hw)


def config2(n=128, c=256, hw=56):
    return Group("bn_add_prelu", n, c, hw * hw, [[], [(capi.OP_BATCH_NORM, 0)]], [(capi.OP_PRELU, 4)], [("bn", c), ("prelu", c)])


def config3(n=64, c=512, hw=28):
    return Group("bn_elu_sigmoid_tanh", n, c, hw * hw,
                 [[(capi.OP_BATCH_NORM, 0), (capi.OP_ELU,), (capi.OP_SIGMOID,), (capi.OP_TANH, 0, TANH_SCALE, TANH_STEEPNESS)]],
                 [], [("bn", c)])


CONFIG1_SHAPE = (256, 1000, 1)  # softmax: entries, feature maps, neurons per feature map

RESNET50_BLOCKS = (3, 4, 6, 3)


def resnet50_groups(n=64):
    """The 49 fused groups of the ResNet-50 post-convolution stack, in execution order."""
    groups = [bn_relu("conv1_bn+relu1", n, 64, 112 * 112)]
    resolution = 56
    restored = 256
    for stage, block_count in enumerate(RESNET50_BLOCKS):
        for block in range(block_count):
            reduction = (block == 0) and (stage != 0)
            if reduction:
                restored *= 2
            bottleneck = restored // 4
            name = "res%d%s" % (stage + 2, chr(ord("a") + block))
            # the stride-2 sits on the 3x3 convolution: reduce_fm still runs at the previous resolution
            groups.append(bn_relu(name + "_reduce_fm", n, bottleneck, resolution * resolution))
            if reduction:
                resolution //= 2
            groups.append(bn_relu(name + "_bottleneck", n, bottleneck, resolution * resolution))
            if block == 0:
                groups.append(bn_bn_add_relu(name + "_shortcut+restore+add", n, restored, resolution * resolution))
            else:
                groups.append(bn_add_relu(name + "_restore+add", n, restored, resolution * resolution))
    return groups


def resnet50_tail(n=64):
    """(pool input shape, softmax shape): 7x7 global average over 2048 feature maps, 1000-way softmax."""
    return (n, 2048, 7, 7), (n, 1000, 1)


def resnet50_algorithmic_bytes(n=64):
    pool_in, softmax_shape = resnet50_tail(n)
    groups = sum(group_algorithmic_bytes(g) for g in resnet50_groups(n))
    pool = 4 * (pool_in[0] * pool_in[1] * pool_in[2] * pool_in[3] + pool_in[0] * pool_in[1])
    softmax = 4 * 2 * softmax_shape[0] * softmax_shape[1]
    return groups, pool, softmax
