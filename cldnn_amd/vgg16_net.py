"""VGG-16 as a quantized clDNN topology: 13 3x3 convolutions with ReLU in five groups, a 2x2 / stride-2 max pooling
behind each group, and three fully_connected layers (25088 -> 4096 -> 4096 -> classes), the first of which reads the
7x7 plane of 512 features.  Synthetic parameters only.

layer_plan() lists what the network consists of; topology() turns a parameter dictionary into primitives.  The parameter
dictionary maps a layer's name ("conv1" .. "conv13", "fc6", "fc7", "fc8") to dict(w, bias, wqf, calib).
"""
import numpy as np

from . import workloads

GROUP_ENDS = ("conv2", "conv4", "conv7", "conv10", "conv13")


def layer_plan(classes=1000, fc_width=4096):
    """-> list of steps ("conv", spec, input id) / ("pool", id, input id) / ("fc", id, input id, ifm, plane, ofm, relu)"""
    steps, cur = [], "input"
    for l in workloads.vgg16():
        steps.append(("conv", l, cur))
        cur = l["name"]
        if cur in GROUP_ENDS:
            steps.append(("pool", "pool%d" % (GROUP_ENDS.index(cur) + 1), cur))
            cur = steps[-1][1]
    steps.append(("fc", "fc6", cur, 512, 7, fc_width, True))
    steps.append(("fc", "fc7", "fc6", fc_width, 1, fc_width, True))
    steps.append(("fc", "fc8", "fc7", fc_width, 1, classes, False))
    return steps


def random_weights(seed=1337, classes=1000, fc_width=4096):
    r = np.random.default_rng(seed)
    p = {}
    for l in workloads.vgg16():
        p[l["name"]] = dict(w=r.integers(-127, 128, (l["ofm"], l["ifm"], 3, 3)).astype(np.int8), bias=r.integers(-1000, 1001, l["ofm"]).astype(np.int32),
                            wqf=np.ones(l["ofm"], np.float32))
    for step in layer_plan(classes, fc_width):
        if step[0] == "fc":
            _, n, _, ifm, plane, ofm, _ = step
            p[n] = dict(w=r.integers(-127, 128, (ofm, ifm, plane, plane)).astype(np.int8), bias=(r.standard_normal(ofm) * 10).astype(np.float32),
                        wqf=np.ones(ofm, np.float32))
    return p


def topology(cl, eng, params, batch, image_hw=224, classes=1000, fc_width=4096):
    """Input: "input", u8 bfyx [batch, 3, hw, hw]; output: "fc8" (s8)."""
    DT, F = cl.data_types, cl.format

    def vec(v):
        return cl.make_memory(eng, np.ascontiguousarray(np.asarray(v).reshape(1, 1, 1, -1)))

    prims = [cl.input_layout("input", cl.layout(DT.u8, F.bfyx, cl.tensor(batch, 3, image_hw, image_hw)))]
    for step in layer_plan(classes, fc_width):
        if step[0] == "conv":
            _, l, src = step
            n, q = l["name"], params[l["name"]]
            prims += [cl.data(n + "_w", cl.make_memory(eng, q["w"])), cl.data(n + "_b", vec(q["bias"])), cl.data(n + "_q", vec(q["wqf"])),
                      cl.data(n + "_c", vec(q["calib"])),
                      cl.convolution(n, src, [n + "_w"], [n + "_b"], [n + "_q"], [n + "_c"], input_offset=cl.tensor(0, 0, -1, -1, 0),
                                     with_activation=True, output_data_type=DT.i8)]
        elif step[0] == "pool":
            _, n, src = step
            prims.append(cl.pooling(n, src, cl.pooling_mode.max, cl.tensor(1, 1, 2, 2), cl.tensor(1, 1, 2, 2)))
        else:
            _, n, src, _, _, _, relu = step
            q = params[n]
            prims += [cl.data(n + "_w", cl.make_memory(eng, q["w"])), cl.data(n + "_b", vec(q["bias"])), cl.data(n + "_q", vec(q["wqf"])),
                      cl.data(n + "_c", vec(q["calib"])),
                      cl.fully_connected(n, src, n + "_w", n + "_b", n + "_q", n + "_c", 1.0, with_activation=relu)]
    return cl.topology(*prims)
