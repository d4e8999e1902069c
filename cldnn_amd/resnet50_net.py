"""ResNet-50 (Caffe form: stride on the first 1x1 of a down-sampling block) as a quantized clDNN topology, the way an
int8 deployment writes it: convolution / pooling / eltwise / fully_connected primitives with int8 weights, int32 bias,
per-feature quantization and calibration factors.  Synthetic parameters only.

layer_plan() lists what the network consists of; topology() turns a parameter dictionary into primitives.  The
parameter dictionary maps a convolution's name to dict(w, bias, wqf, calib), a block name ("res2a", ...) to
dict(ecal) for the calibration of its residual sum, and "fc1000" to dict(w, bias, wqf, calib).
"""
import numpy as np

from . import workloads


def layer_plan():
    """-> list of steps: ("conv", spec, input id, relu) / ("pool1",) / ("sum", block, shortcut id, branch id) /
    ("pool5",) / ("fc",) in execution order; ids are the primitive ids topology() uses."""
    convs = {l["name"]: l for l in workloads.resnet50()}
    steps = [("conv", convs["conv1"], "input", True), ("pool1",)]
    cur = "pool1"
    for stage, blocks in ((2, 3), (3, 4), (4, 6), (5, 3)):
        for b in range(blocks):
            n = "res%d%s" % (stage, chr(ord("a") + b))
            shortcut = cur
            if b == 0:
                steps.append(("conv", convs[n + "_branch1"], cur, False))
                shortcut = n + "_branch1"
            steps.append(("conv", convs[n + "_branch2a"], cur, True))
            steps.append(("conv", convs[n + "_branch2b"], n + "_branch2a", True))
            steps.append(("conv", convs[n + "_branch2c"], n + "_branch2b", False))
            steps.append(("sum", n, shortcut, n + "_branch2c"))
            cur = n
    steps += [("pool5",), ("fc",)]
    return steps


def random_weights(seed=1337, classes=1000):
    """int8 weights and int32 / f32 biases for every layer (no factors yet)."""
    r = np.random.default_rng(seed)
    p = {}
    for l in workloads.resnet50():
        p[l["name"]] = dict(w=r.integers(-127, 128, (l["ofm"], l["ifm"], l["k"], l["k"])).astype(np.int8),
                            bias=r.integers(-1000, 1001, l["ofm"]).astype(np.int32), wqf=np.ones(l["ofm"], np.float32))
    p["fc1000"] = dict(w=r.integers(-127, 128, (classes, 2048, 1, 1)).astype(np.int8), bias=(r.standard_normal(classes) * 10).astype(np.float32),
                       wqf=np.ones(classes, np.float32))
    return p


def topology(cl, eng, params, batch, image_hw=224):
    """cl = the cldnn_amd.api module, eng = its engine.  Input: "input", u8 bfyx [batch, 3, hw, hw]; output: "fc1000" (s8)."""
    DT, F = cl.data_types, cl.format

    def vec(v):
        return cl.make_memory(eng, np.ascontiguousarray(np.asarray(v).reshape(1, 1, 1, -1)))

    prims = [cl.input_layout("input", cl.layout(DT.u8, F.bfyx, cl.tensor(batch, 3, image_hw, image_hw)))]
    for step in layer_plan():
        if step[0] == "conv":
            _, l, src, relu = step
            n, q = l["name"], params[l["name"]]
            prims += [cl.data(n + "_w", cl.make_memory(eng, q["w"])), cl.data(n + "_b", vec(q["bias"])), cl.data(n + "_q", vec(q["wqf"])),
                      cl.data(n + "_c", vec(q["calib"])),
                      cl.convolution(n, src, [n + "_w"], [n + "_b"], [n + "_q"], [n + "_c"], stride=cl.tensor(1, 1, l["stride"], l["stride"]),
                                     input_offset=cl.tensor(0, 0, -l["pad"], -l["pad"], 0), with_activation=relu, output_data_type=DT.i8)]
        elif step[0] == "pool1":
            prims.append(cl.pooling("pool1", "conv1", cl.pooling_mode.max, cl.tensor(1, 1, 3, 3), cl.tensor(1, 1, 2, 2)))
        elif step[0] == "sum":
            _, n, shortcut, branch = step
            prims += [cl.data(n + "_ecal", vec(params[n]["ecal"])),
                      cl.eltwise(n, shortcut, branch, cl.eltwise_mode.sum, with_activation=True, output_calibration_factors=n + "_ecal")]
        elif step[0] == "pool5":
            prims.append(cl.pooling("pool5", "res5c", cl.pooling_mode.average))
        else:
            q = params["fc1000"]
            prims += [cl.data("fc1000_w", cl.make_memory(eng, q["w"])), cl.data("fc1000_b", vec(q["bias"])), cl.data("fc1000_q", vec(q["wqf"])),
                      cl.data("fc1000_c", vec(q["calib"])),
                      cl.fully_connected("fc1000", "pool5", "fc1000_w", "fc1000_b", "fc1000_q", "fc1000_c", 1.0)]
    return cl.topology(*prims)
