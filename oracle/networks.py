"""Whole networks through the CPU oracle, layer by layer: ResNet-50, VGG-16 and MobileNet-v2 as the benchmark builds them.

TEST INFRASTRUCTURE ONLY: imported by tests/ and by bench.py's cpu_baseline leg, never by the product package.  The
layer lists come from the network definitions of the package (plain Python lists of layer shapes); every tensor is
computed by oracle/refconv (convolution, pooling, eltwise, fully_connected), so what pins those pins these walks.
"""
import numpy as np

from cldnn_amd import mobilenet_v2_net as mn
from cldnn_amd import resnet50_net as rn
from cldnn_amd import vgg16_net as vg
from oracle import refconv as rc


def resnet50(x, params, fused=(), calibrate=False):
    """Oracle forward pass, layer by layer.  `fused` names the blocks whose residual sum runs inside the closing
    convolution (fused_conv_eltwise: the convolution's result is not saturated before the sum); the others use the
    stand-alone eltwise on the saturated int8 tensor.  With calibrate=True the pass also chooses every layer's factors:
    the root mean square of its outputs lands at about a quarter of the int8 range (what a calibration tool does), so
    that few values saturate and no layer dies.  Returns the tensors by primitive id."""
    t = {"input": x}
    for step in rn.layer_plan():
        if step[0] == "conv":
            _, l, src, relu = step
            q = params[l["name"]]
            kw = dict(stride=(l["stride"],) * 2, pad=(l["pad"],) * 2)
            if calibrate:
                _, acc = rc.conv(t[src], q["w"], q["bias"], wqf=q["wqf"], calib=np.ones(l["ofm"], np.float32), out_dt="s8", want_acc=True, **kw)
                full = acc.astype(np.float64) + q["bias"].reshape(1, -1, 1, 1)
                q["calib"] = (32.0 / (np.sqrt((full * full).mean(axis=(0, 2, 3))) + 1.0)).astype(np.float32)
            if l["closes_block"] and l["name"][:-9] in fused:
                continue  # computed together with the residual sum
            t[l["name"]] = rc.conv(t[src], q["w"], q["bias"], wqf=q["wqf"], calib=q["calib"], out_dt="s8", act="relu" if relu else "none", **kw)
        elif step[0] == "pool1":
            t["pool1"] = rc.pool(t["conv1"], "max", (3, 3), (2, 2))
        elif step[0] == "sum":
            _, n, shortcut, branch = step
            if calibrate:
                params[n] = dict(ecal=np.full(params[branch]["w"].shape[0], 0.6, np.float32))
            if n in fused:
                q = params[branch]
                t[n] = rc.conv(t[n + "_branch2b"], q["w"], q["bias"], wqf=q["wqf"], calib=q["calib"], out_dt="s8", eltw=t[shortcut],
                               eltw_act="relu", eltw_calib=params[n]["ecal"])
            else:
                t[n] = rc.eltwise_sum(t[shortcut], t[branch], calib=params[n]["ecal"], relu=True)
        elif step[0] == "pool5":
            t["pool5"] = rc.pool(t["res5c"], "average", None, global_pooling=True)
        else:
            q = params["fc1000"]
            if calibrate:
                acc = np.einsum("bfyx,ofyx->bo", t["pool5"].astype(np.int64), q["w"].astype(np.int64)).astype(np.float64)
                q["calib"] = np.full(q["w"].shape[0], 40.0 / (np.sqrt((acc * acc).mean()) + 1.0), np.float32)
            t["fc1000"] = rc.fully_connected(t["pool5"], q["w"], q["bias"], wqf=q["wqf"], calib=q["calib"])
    return t


def vgg16(x, params, calibrate=False):
    """Oracle forward pass; calibrate=True also chooses every layer's factors (root mean square of the outputs at about a
    quarter of the int8 range)."""
    t = {"input": x}
    for step in vg.layer_plan():
        if step[0] == "conv":
            _, l, src = step
            q = params[l["name"]]
            if calibrate:
                _, acc = rc.conv(t[src], q["w"], q["bias"], wqf=q["wqf"], calib=np.ones(l["ofm"], np.float32), pad=(1, 1), out_dt="s8", want_acc=True)
                full = acc.astype(np.float64) + q["bias"].reshape(1, -1, 1, 1)
                q["calib"] = (32.0 / (np.sqrt((full * full).mean(axis=(0, 2, 3))) + 1.0)).astype(np.float32)
            t[l["name"]] = rc.conv(t[src], q["w"], q["bias"], wqf=q["wqf"], calib=q["calib"], pad=(1, 1), out_dt="s8", act="relu")
        elif step[0] == "pool":
            _, n, src = step
            t[n] = rc.pool(t[src], "max", (2, 2), (2, 2))
        else:
            _, n, src, ifm, plane, ofm, relu = step
            q = params[n]
            xin = t[src].reshape(x.shape[0], ifm, plane, plane)
            if calibrate:
                acc = np.einsum("bfyx,ofyx->bo", xin.astype(np.int64), q["w"].astype(np.int64)).astype(np.float64)
                q["calib"] = np.full(ofm, 40.0 / (np.sqrt((acc * acc).mean()) + 1.0), np.float32)
            t[n] = rc.fully_connected(xin, q["w"], q["bias"], wqf=q["wqf"], calib=q["calib"], act="relu" if relu else "none")
    return t


def mobilenet_v2(x, params, folded=True, calibrate=False):
    """Oracle forward pass.  folded: the clamp{0, 6} behind a convolution acts inside it on the dequantised value, before
    the calibration (what optimize_data makes of the pair, as the reference's prepare_primitive_fusing does); otherwise
    it is a primitive of its own and clamps the convolution's int8 output.  calibrate=True also chooses the factors:
    the dequantised values of a ReLU6 layer get a root mean square of 3 and are requantised with 127 / 6; a linear
    layer's outputs a root mean square of 30."""
    t = {"input": x}
    last = None
    for step in mn.layer_plan():
        if step[0] == "conv":
            _, l, src = step
            q, n = params[l["name"]], l["name"]
            relu6 = l["act"] == "relu6"
            kw = dict(stride=(l["stride"],) * 2, pad=(l["pad"],) * 2, groups=l["groups"], out_dt="s8")
            if calibrate:
                one = np.ones(l["ofm"], np.float32)
                _, acc = rc.conv(t[src], q["w"], q["bias"], wqf=one, calib=one, want_acc=True, **kw)
                full = acc.astype(np.float64) + q["bias"].reshape(1, -1, 1, 1)
                rms = np.sqrt((full * full).mean(axis=(0, 2, 3))) + 1.0
                q["wqf"] = ((3.0 if relu6 else 30.0) / rms).astype(np.float32)
                q["calib"] = np.full(l["ofm"], 127.0 / 6.0 if relu6 else 1.0, np.float32)
            if relu6 and folded:
                t[n + "_relu6"] = rc.conv(t[src], q["w"], q["bias"], wqf=q["wqf"], calib=q["calib"], act="clamp", act_m=0.0, act_n=6.0, **kw)
            else:
                t[n] = rc.conv(t[src], q["w"], q["bias"], wqf=q["wqf"], calib=q["calib"], **kw)
                if relu6:
                    t[n + "_relu6"] = np.clip(t[n], 0, 6)  # the stand-alone activation clamps the int8 values themselves
            last = n + ("_relu6" if relu6 else "")
        elif step[0] == "sum":
            _, n, shortcut, branch = step
            if calibrate:
                params[n] = dict(ecal=np.full(t[branch].shape[1], 0.75, np.float32))
            t[n] = rc.eltwise([t[shortcut], t[branch]], "sum", calib=params[n]["ecal"])
            last = n
        elif step[0] == "pool":
            t["pool"] = rc.pool(t[last], "average", None, global_pooling=True)
        else:
            q = params["fc1000"]
            if calibrate:
                acc = np.einsum("bfyx,ofyx->bo", t["pool"].astype(np.int64), q["w"].astype(np.int64)).astype(np.float64)
                q["calib"] = np.full(q["w"].shape[0], 40.0 / (np.sqrt((acc * acc).mean()) + 1.0), np.float32)
            t["fc1000"] = rc.fully_connected(t["pool"], q["w"], q["bias"], wqf=q["wqf"], calib=q["calib"])
    return t
