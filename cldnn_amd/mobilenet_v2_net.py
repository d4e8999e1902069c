"""MobileNet-v2 (width 1.0, 224x224) as a quantized clDNN topology, the way an int8 deployment writes it: 3x3 stem,
17 inverted-residual blocks (1x1 expansion, 3x3 depthwise convolution with groups = features, 1x1 linear projection),
ReLU6 as a clamp{0, 6} activation primitive behind the convolution (folded into it by optimize_data), residual sums
without activation (so they stay stand-alone eltwise primitives, as in the reference, whose fusing needs an
activation), 1x1 to 1280 features, global average pooling, fully_connected.  Synthetic parameters only.

layer_plan() lists what the network consists of; topology() turns a parameter dictionary into primitives.  The
parameter dictionary maps a convolution's name to dict(w, bias, wqf, calib), a block name ("b3", ...) that has a
residual sum to dict(ecal), and "fc1000" to dict(w, bias, wqf, calib).
"""
import numpy as np

from . import workloads


def layer_plan():
    """-> list of steps ("conv", spec, input id) / ("sum", block, shortcut id, branch id) / ("pool",) / ("fc",) in execution
    order; a convolution whose spec says act == "relu6" is followed by the clamp primitive <name>_relu6, which is then
    the id later steps read."""
    convs = {l["name"]: l for l in workloads.mobilenet_v2()}

    def out_id(l):
        return l["name"] + ("_relu6" if l["act"] == "relu6" else "")
    steps = [("conv", convs["conv1"], "input")]
    cur, cin, idx = out_id(convs["conv1"]), 32, 0
    for t, c, n, s in ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)):
        for i in range(n):
            idx += 1
            block_in, src = cur, cur
            if t != 1:
                l = convs["b%d_expand" % idx]
                steps.append(("conv", l, src))
                src = out_id(l)
            l = convs["b%d_dw" % idx]
            steps.append(("conv", l, src))
            l2 = convs["b%d_project" % idx]
            steps.append(("conv", l2, out_id(l)))
            cur = l2["name"]
            if i > 0 and s in (1, 2) and cin == c:  # stride 1, same width: the block is residual
                steps.append(("sum", "b%d" % idx, block_in, cur))
                cur = "b%d" % idx
            cin = c
    steps.append(("conv", convs["conv_last"], cur))
    steps += [("pool",), ("fc",)]
    return steps


def random_weights(seed=1337, classes=1000):
    """int8 weights and int32 / f32 biases for every layer (no factors yet)."""
    r = np.random.default_rng(seed)
    p = {}
    for l in workloads.mobilenet_v2():
        p[l["name"]] = dict(w=r.integers(-127, 128, (l["ofm"], l["ifm"] // l["groups"], l["k"], l["k"])).astype(np.int8),
                            bias=r.integers(-300, 301, l["ofm"]).astype(np.int32))
    p["fc1000"] = dict(w=r.integers(-127, 128, (classes, 1280, 1, 1)).astype(np.int8), bias=(r.standard_normal(classes) * 10).astype(np.float32),
                       wqf=np.ones(classes, np.float32))
    return p


def topology(cl, eng, params, batch, image_hw=224):
    """cl = the cldnn_amd.api module, eng = its engine.  Input: "input", u8 bfyx [batch, 3, hw, hw]; output: "fc1000" (s8)."""
    DT, F = cl.data_types, cl.format

    def vec(v):
        return cl.make_memory(eng, np.ascontiguousarray(np.asarray(v).reshape(1, 1, 1, -1)))

    prims = [cl.input_layout("input", cl.layout(DT.u8, F.bfyx, cl.tensor(batch, 3, image_hw, image_hw)))]
    last = None
    for step in layer_plan():
        if step[0] == "conv":
            _, l, src = step
            n, q = l["name"], params[l["name"]]
            prims += [cl.data(n + "_w", cl.make_memory(eng, q["w"])), cl.data(n + "_b", vec(q["bias"])), cl.data(n + "_q", vec(q["wqf"])),
                      cl.data(n + "_c", vec(q["calib"])),
                      cl.convolution(n, src, [n + "_w"], [n + "_b"], [n + "_q"], [n + "_c"], stride=cl.tensor(1, 1, l["stride"], l["stride"]),
                                     input_offset=cl.tensor(0, 0, -l["pad"], -l["pad"], 0), groups=l["groups"], output_data_type=DT.i8)]
            last = n
            if l["act"] == "relu6":
                prims.append(cl.activation(n + "_relu6", n, cl.activation_func.clamp, (0.0, 6.0)))
                last = n + "_relu6"
        elif step[0] == "sum":
            _, n, shortcut, branch = step
            prims += [cl.data(n + "_ecal", vec(params[n]["ecal"])),
                      cl.eltwise(n, shortcut, branch, cl.eltwise_mode.sum, output_calibration_factors=n + "_ecal")]
            last = n
        elif step[0] == "pool":
            prims.append(cl.pooling("pool", last, cl.pooling_mode.average))
        else:
            q = params["fc1000"]
            prims += [cl.data("fc1000_w", cl.make_memory(eng, q["w"])), cl.data("fc1000_b", vec(q["bias"])), cl.data("fc1000_q", vec(q["wqf"])),
                      cl.data("fc1000_c", vec(q["calib"])),
                      cl.fully_connected("fc1000", "pool", "fc1000_w", "fc1000_b", "fc1000_q", "fc1000_c", 1.0)]
    return cl.topology(*prims)
