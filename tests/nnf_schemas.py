"""Small networks for the backend tests: described once as Python data, rendered to nnForge's
text-format schema for the backend, and evaluated layer by layer with the CPU oracle the way
nnForge's plain backend would run them."""

import numpy as np

import nnf_testing as T
import oracle


def L(type_name, name, inputs=(), **params):
    return {"type": type_name, "name": name, "inputs": list(inputs), "params": params}


PARAM_BLOCK = {"BatchNorm": "batch_norm_param", "ReLU": "relu_param", "PReLU": "prelu_param", "TanH": "tanh_param",
               "Add": "add_param", "AverageSubsampling": "average_subsampling_param", "Dropout": "dropout_param",
               "Maxout": "maxout_param", "MaxSubsampling": "max_subsampling_param"}


def schema_text(layers, name="test_net"):
    out = ['name: "%s"' % name]
    for l in layers:
        out.append("layer {")
        out.append('\ttype: "%s"' % l["type"])
        out.append('\tname: "%s"' % l["name"])
        for i in l["inputs"]:
            out.append('\tinput_layer_name: "%s"' % i)
        p = l["params"]
        if p and l["type"] in PARAM_BLOCK:
            out.append("\t%s {" % PARAM_BLOCK[l["type"]])
            for k, v in p.items():
                if k == "windows":
                    for d, w in enumerate(v):
                        extra = ""
                        if p.get("round_ups") and p["round_ups"][d]:
                            extra += " round_up: true"
                        if p.get("strides"):
                            extra += " stride: %d" % p["strides"][d]
                        out.append("\t\tdimension_param { subsampling_size: %d%s }" % (w, extra))
                elif k in ("strides", "round_ups"):
                    continue
                elif k == "fm_window":
                    out.append("\t\tfeature_map_param { subsampling_size: %d }" % v)
                elif k == "function":
                    out.append("\t\tfunction: %s" % v)
                elif isinstance(v, bool):
                    out.append("\t\t%s: %s" % (k, "true" if v else "false"))
                else:
                    out.append("\t\t%s: %r" % (k, v))
            out.append("\t}")
        out.append("}")
    return "\n".join(out) + "\n"


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
            v = oracle.average_subsampling(ins[0], p["windows"], alpha=p.get("alpha"))
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
                                       feature_map_window=p.get("fm_window", 1), is_min=p.get("function") == "MIN")
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


def classifier_tail(c=8):
    """ResNet-like tail: block -> 7x7 global pooling -> softmax."""
    return resnet_block(c) + [L("AverageSubsampling", "pool", ["res_relu"], windows=[7, 7], alpha=1.0 / 49.0),
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
