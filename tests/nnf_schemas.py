"""Small networks for the backend tests: described once as Python data, rendered to nnForge's
text-format schema for the backend, and evaluated layer by layer with the CPU oracle the way
nnForge's plain backend would run them."""

import numpy as np

import nnf_testing as T
import oracle


from nnforge_amd.schemas import L, PARAM_BLOCK, schema_text  # noqa: F401 (re-exported: the tests build their networks with these)


def parse_schema_text(text):
    """A reader of nnForge's text-format schema written for the tests alone (the backend's C++ reader is what is under
    test): -> (name, [{"type", "name", "inputs", "blocks": {message name: [fields]}}]) with fields = {field: value or
    [values]}; repeated nested messages keep their order."""
    import re

    tokens = re.findall(r'"[^"]*"|[{}]|[^\s{}:"]+:?', text)
    pos = 0

    def message(top):
        nonlocal pos
        fields = []
        while pos < len(tokens):
            tok = tokens[pos]
            pos += 1
            if tok == "}":
                assert not top
                return fields
            key = tok.rstrip(":")
            if tokens[pos] == "{":
                pos += 1
                fields.append((key, message(False)))
            else:
                fields.append((key, tokens[pos].strip('"')))
                pos += 1
        assert top
        return fields

    root = message(True)
    layers = []
    for key, value in root:
        if key != "layer":
            continue
        layer = {"type": None, "name": None, "inputs": [], "blocks": {}}
        for k, v in value:
            if k == "type":
                layer["type"] = v
            elif k == "name":
                layer["name"] = v
            elif k == "input_layer_name":
                layer["inputs"].append(v)
            else:
                layer["blocks"].setdefault(k, []).append(v)
        layers.append(layer)
    return dict((k, v) for k, v in root if k == "name").get("name"), layers


def layers_for_the_oracle(parsed_layers):
    """The layers of parse_schema_text as the L(...) records evaluate() takes; layers of other types become Data layers
    (their values are supplied, as for the backend)."""
    out = []
    for l in parsed_layers:
        t, blocks = l["type"], l["blocks"]
        first = lambda name: dict((k, v) for k, v in blocks[name][0] if not isinstance(v, list)) if name in blocks else {}
        if t == "TanH":
            f = first("tanh_param")
            out.append(L(t, l["name"], l["inputs"], scale=float(f.get("scale", 1.0)), steepness=float(f.get("steepness", 1.0))))
        elif t == "AverageSubsampling":
            dims = [dict(v) for k, v in blocks["average_subsampling_param"][0] if k == "dimension_param"]
            out.append(L(t, l["name"], l["inputs"], windows=[int(d["subsampling_size"]) for d in dims]))
        elif t == "Dropout":
            out.append(L(t, l["name"], l["inputs"], dropout_rate=float(first("dropout_param").get("dropout_rate", 0.5))))
        elif t in ("Absolute", "ReLU", "Sigmoid", "ELU", "Softmax"):
            out.append(L(t, l["name"], l["inputs"]))
        else:
            out.append(L("Data", l["name"]))
    return out


def make_weights(layers, gen):
    weights = {}
    for l in layers:
        if l["type"] == "BatchNorm":
            weights[l["name"]] = list(T.bn_params(gen, l["params"]["feature_map_count"]))
        elif l["type"] == "PReLU":
            weights[l["name"]] = [T.uniform(gen, l["params"]["feature_map_count"], -0.1, 0.3)]
    return weights


def evaluate(layers, weights, inputs):
    """Reference evaluation, one oracle call per layer. inputs: {data layer: array}. Returns all values."""
    values = dict(inputs)
    for l in layers:
        t, name, p = l["type"], l["name"], l["params"]
        if t == "Data":
            continue
        ins = [values[i] for i in l["inputs"]]
        if t == "BatchNorm":
            v = oracle.batch_norm(ins[0], *weights[name])
        elif t == "ReLU":
            v = oracle.rectified_linear(ins[0], p.get("negative_slope", 0.0))
        elif t == "PReLU":
            v = oracle.parametric_rectified_linear(ins[0], weights[name][0])
        elif t == "ELU":
            v = oracle.exponential_linear(ins[0])
        elif t == "Sigmoid":
            v = oracle.sigmoid(ins[0])
        elif t == "TanH":
            v = oracle.hyperbolic_tangent(ins[0], p.get("scale", 1.0), p.get("steepness", 1.0))
        elif t == "Add":
            v = oracle.add(ins, p.get("alpha", 1.0)).reshape(ins[0].shape)
        elif t == "Softmax":
            v = oracle.softmax(ins[0])
        elif t == "AverageSubsampling":
            # the plain tester's multiplier: window sum unless alpha is given
            x = ins[0]
            dims = list(x.shape[2:])[::-1]
            windows = p["windows"] if "windows" in p else [d // o for d, o in zip(dims, p["subsampled"])]
            fm_window = p.get("fm_window", 1) if "fm_subsampled" not in p else x.shape[1] // p["fm_subsampled"]
            v = oracle.average_subsampling(x, windows, feature_map_window=fm_window, entry_window=p.get("entry_window", 1),
                                           alpha=p.get("alpha"))
        elif t == "Absolute":
            v = oracle.absolute(ins[0])
        elif t == "Dropout":
            v = oracle.dropout(ins[0])
        elif t == "Concat":
            v = oracle.concat(ins)
        elif t == "Maxout":
            v = oracle.maxout(ins[0], p["feature_map_subsampling_size"])
        elif t == "MaxSubsampling":
            v = oracle.max_subsampling(ins[0], p["windows"], strides=p.get("strides"), round_ups=p.get("round_ups"),
                                       feature_map_window=p.get("fm_window", 1), entry_window=p.get("entry_window", 1),
                                       is_min=p.get("function") == "MIN", tiling=p.get("tiling", False))
        else:
            raise ValueError(t)
        values[name] = v
    return values


def resnet_block(c=8, with_shortcut_bn=True):
    layers = [L("Data", "conv_main"), L("Data", "conv_shortcut"),
              L("BatchNorm", "main_bn", ["conv_main"], feature_map_count=c)]
    shortcut = "conv_shortcut"
    if with_shortcut_bn:
        layers.append(L("BatchNorm", "shortcut_bn", ["conv_shortcut"], feature_map_count=c))
        shortcut = "shortcut_bn"
    layers += [L("Add", "res", [shortcut, "main_bn"]), L("ReLU", "res_relu", ["res"])]
    return layers


def classifier_tail(c=8, with_shortcut_bn=True):
    """ResNet-like tail: block -> 7x7 global pooling -> softmax."""
    return resnet_block(c, with_shortcut_bn) + [L("AverageSubsampling", "pool", ["res_relu"], windows=[7, 7], alpha=1.0 / 49.0),
                              L("Softmax", "prob", ["pool"])]


def activation_chain(c=6):
    return [L("Data", "x"), L("BatchNorm", "bn", ["x"], feature_map_count=c), L("ELU", "elu", ["bn"]), L("Sigmoid", "sig", ["elu"]),
            L("TanH", "tanh", ["sig"], scale=1.7159, steepness=0.6666)]


def inception_like(c=8):
    """A stem pooled 3x3 every 2 (rounded up), three branches (BatchNorm+ReLU, Absolute behind a
    Dropout, a min pooling with stride 1 cut back by a second branch input), joined by Concat, halved by
    Maxout, then Dropout in front of the output activation."""
    return [
        L("Data", "stem"),
        L("MaxSubsampling", "pool1", ["stem"], windows=[3, 3], strides=[2, 2], round_ups=[True, True]),
        L("BatchNorm", "b1_bn", ["pool1"], feature_map_count=c),
        L("ReLU", "b1_relu", ["b1_bn"]),
        L("Dropout", "b2_drop", ["pool1"], dropout_rate=0.25),
        L("Absolute", "b2_abs", ["b2_drop"]),
        L("PReLU", "b3_prelu", ["pool1"], feature_map_count=c),
        L("Concat", "join", ["b1_relu", "b2_abs", "b3_prelu", "pool1"]),
        L("Maxout", "mo", ["join"], feature_map_subsampling_size=2),
        L("Dropout", "drop", ["mo"]),
        L("MaxSubsampling", "pool2", ["drop"], windows=[2, 2], function="MIN"),
        L("TanH", "out", ["pool2"]),
    ]


def inception_block(c=16):
    """Four branches behind one input, each ending in a fused group that only the Concat reads - BatchNorm -> ReLU twice
    (different widths), a PReLU on its own, and BatchNorm + a second input joined by an Add -> ReLU - then Concat, Maxout
    and an activation: the block whose Concat has nothing to copy."""
    return [
        L("Data", "conv_a"), L("Data", "conv_b"), L("Data", "conv_c"), L("Data", "conv_d"), L("Data", "conv_e"),
        L("BatchNorm", "a_bn", ["conv_a"], feature_map_count=c), L("ReLU", "a_relu", ["a_bn"]),
        L("BatchNorm", "b_bn", ["conv_b"], feature_map_count=2 * c), L("ReLU", "b_relu", ["b_bn"], negative_slope=0.125),
        L("PReLU", "c_prelu", ["conv_c"], feature_map_count=c),
        L("BatchNorm", "d_bn", ["conv_d"], feature_map_count=c), L("Add", "d_sum", ["conv_e", "d_bn"]), L("ReLU", "d_relu", ["d_sum"]),
        L("Concat", "join", ["a_relu", "b_relu", "c_prelu", "d_relu"]),
        L("Maxout", "mo", ["join"], feature_map_subsampling_size=5),
        L("TanH", "out", ["mo"], scale=1.7159, steepness=0.6666),
    ]


def random_network(gen, layer_count=14, c=6, size=12, with_entry_factors=False):
    """A random DAG of the layer types the backend runs: chains of element-wise layers, Adds and Concats of values of
    equal shape, Maxout, max / min / average pooling, with some values consumed more than once. with_entry_factors:
    also max subsampling with tiling and windows over entries, so that values hold different numbers of entries per
    entry read (layers with several inputs then only join values that agree on it, and so do the outputs).
    -> (layers, {value name: (feature maps, [w, h])}, output names)."""
    layers = [L("Data", "in0"), L("Data", "in1")]
    shapes = {"in0": (c, [size, size]), "in1": (c, [size, size])}
    factors = {"in0": 1, "in1": 1}   # entries per entry read
    names = ["in0", "in1"]
    unary = ["BatchNorm", "ReLU", "PReLU", "ELU", "Sigmoid", "TanH", "Absolute", "Dropout"]
    for i in range(layer_count):
        name = "l%d" % i
        # mostly continue from the newest value (chains), sometimes branch off an older one
        src = names[-1] if gen.random() < 0.65 else names[int(gen.integers(0, len(names)))]
        fm, dims = shapes[src]
        roll = gen.random()
        same_shape = [n for n in names if shapes[n] == shapes[src] and factors[n] == factors[src] and n != src]
        same_plane = [n for n in names if shapes[n][1] == dims and factors[n] == factors[src] and n != src]
        factors[name] = factors[src]
        if with_entry_factors and roll < 0.22 and min(dims) >= 5 and factors[src] == 1:
            layers.append(L("MaxSubsampling", name, [src], windows=[2, 2], tiling=True, **({"function": "MIN"} if gen.random() < 0.3 else {})))
            shapes[name] = (fm, [(d - 1) // 2 for d in dims])
            factors[name] = 4
        elif with_entry_factors and roll < 0.30 and factors[src] > 1:
            window = 2 if (factors[src] == 4 and gen.random() < 0.5) else factors[src]
            kind = "AverageSubsampling" if gen.random() < 0.5 else "MaxSubsampling"
            layers.append(L(kind, name, [src], windows=[1, 1], entry_window=window))
            shapes[name] = (fm, dims)
            factors[name] = factors[src] // window
        elif roll < 0.50:
            t = unary[int(gen.integers(0, len(unary)))]
            params = {}
            if t in ("BatchNorm", "PReLU"):
                params["feature_map_count"] = fm
            elif t == "ReLU" and gen.random() < 0.5:
                params["negative_slope"] = 0.125
            elif t == "TanH":
                params = {"scale": 1.7159, "steepness": 0.6666}
            elif t == "Dropout":
                params = {"dropout_rate": 0.25}
            layers.append(L(t, name, [src], **params))
            shapes[name] = (fm, dims)
        elif roll < 0.65 and same_shape:
            others = [same_shape[int(j)] for j in gen.permutation(len(same_shape))[:int(gen.integers(1, 3))]]
            params = {"alpha": 0.5} if gen.random() < 0.3 else {}
            layers.append(L("Add", name, [src] + others, **params))
            shapes[name] = (fm, dims)
        elif roll < 0.75 and same_plane:
            others = [same_plane[int(j)] for j in gen.permutation(len(same_plane))[:int(gen.integers(1, 3))]]
            layers.append(L("Concat", name, [src] + others))
            shapes[name] = (fm + sum(shapes[o][0] for o in others), dims)
        elif roll < 0.82 and fm % 2 == 0 and fm >= 4:
            layers.append(L("Maxout", name, [src], feature_map_subsampling_size=2))
            shapes[name] = (fm // 2, dims)
        elif roll < 0.92 and min(dims) >= 6:
            if gen.random() < 0.5:
                layers.append(L("MaxSubsampling", name, [src], windows=[3, 3], strides=[2, 2], round_ups=[True, True],
                                **({"function": "MIN"} if gen.random() < 0.3 else {})))
                shapes[name] = (fm, [(d + 2 - 3 + 2) // 2 for d in dims])
            else:
                layers.append(L("MaxSubsampling", name, [src], windows=[2, 2]))
                shapes[name] = (fm, [d // 2 for d in dims])
        elif min(dims) >= 4 and gen.random() < 0.6:
            layers.append(L("AverageSubsampling", name, [src], windows=[2, 2]))
            shapes[name] = (fm, [d // 2 for d in dims])
        elif min(dims) >= 2:
            # the average over whole planes (behind an Add and its layers: one launch with them)
            layers.append(L("AverageSubsampling", name, [src], windows=list(dims)))
            shapes[name] = (fm, [1, 1])
        else:
            layers.append(L("Absolute", name, [src]))
            shapes[name] = (fm, dims)
        names.append(name)
    consumed = {i for l in layers for i in l["inputs"]}
    outputs = [n for n in names[2:] if n not in consumed]          # every value nobody reads
    extra = [n for n in names[2:] if n in consumed]
    if extra:
        outputs.append(extra[int(gen.integers(0, len(extra)))])    # and one that is read as well
    if with_entry_factors:
        # the outputs must agree on the number of entries: those of the last one's kind
        outputs = [n for n in outputs if factors[n] == factors[outputs[-1]]]
    return layers, shapes, outputs

