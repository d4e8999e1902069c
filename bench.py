#!/usr/bin/env python3
"""Benchmark of the quantized convolution hot path on one MI355X.

A "step" is one pass of a whole int8 convolution stack over one batch of synthetic input through
the C-ABI, inputs already resident in HBM: one launch per layer, or one launch per convolution
chain where neighbouring layers feed each other (a 3x3 and the 1x1 convolutions behind it).
Default workload: the 53 convolutions of ResNet-50 at batch 32 with the residual add fused into the
16 block-closing 1x1 convolutions (fused_conv_eltwise).  The default run also times the other four
configurations (VGG-16 b16, MobileNet-v2 b32, ResNet-50 b1, the single convolution) more briefly.

Prints ONE JSON line (metric, value, roofline with the dominant kernel, cpu_baseline, other_workloads ...).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from cldnn_amd import hip, workloads  # noqa: E402

PEAK_INT8_OPS = 5.0e15   # MI355X dense int8 MFMA peak, op/s
PEAK_HBM = 8.0e12        # bytes/s


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class Layer:
    pass


def chain_groups(layers, fuse_residual):
    """The launches a stack is cut into: a spatial layer (a dense convolution on multiples of 64 features, or a
    depthwise 3x3) together with the one or two 1x1 / stride-1 layers that read its result in the network
    (follows_prev), else the layer alone.  Whether the library accepts a group as a chain is decided when it is built."""
    out, i = [], 0
    while i < len(layers):
        n = 1
        h = layers[i]
        dense_head = h["groups"] == 1 and h["ifm"] % 64 == 0
        dw_head = h["k"] == 3 and h["groups"] == h["ifm"] == h["ofm"]
        if h["k"] > 1 and (dense_head or dw_head):
            while n < 3 and i + n < len(layers):
                l, q = layers[i + n], layers[i + n - 1]
                ok = l["follows_prev"] and l["k"] == 1 and l["stride"] == 1 and l["groups"] == 1 and l["ifm"] == q["ofm"] \
                    and l["in_hw"] == q["out_hw"] and (not q["closes_block"] or fuse_residual)
                if not ok:
                    break
                n += 1
        out.append(layers[i:i + n])
        i += n
    return out


def build_stack(eng, layers, batch, fuse_residual, seed=1337, tile=0, in_dt=np.uint8, chains=True, siblings=None, calibration="benchmark"):
    """Create device tensors and convolution objects for every layer (seeded synthetic data).

    chains: neighbouring layers that feed each other in the network (follows_prev) run as ONE launch of the
    convolution chain kernel where the library accepts them (a spatial convolution followed by one or two 1x1
    convolutions); a chained layer reads what the layer before it produced instead of a fresh random tensor, and the
    result of a chain's first stage, which only the second stage reads, is never written.
    siblings (default: as chains): a layer that reads the same tensor as the one before it (shares_input: a block's
    opening 1x1 beside the shortcut projection) runs in that layer's launch; its result is the tail of the launch's
    output buffer.  Such a layer reads the same input data as its neighbour either way.
    calibration: "benchmark" = the baseline's factors, log-uniform in [1e-4, 1e-2] (most outputs end at 0 or 127);
    "spread" = 40 / sigma(accumulator) * U(0.5, 2) per feature, which spreads the outputs over the int8 range so that a
    wrong accumulator shows in the output (parity tests)."""
    siblings = chains if siblings is None else siblings
    out = []
    follows = set()  # indices of layers that run as stage 1 / 2 of a chain
    if chains and not tile:
        i = 0
        for group in chain_groups(layers, fuse_residual):
            if len(group) > 1:
                layers[i] = dict(layers[i], chain_len=len(group))
                follows.update(range(i + 1, i + len(group)))
            i += len(group)
    for i, l in enumerate(layers):
        r = np.random.default_rng(seed + i)
        L = Layer()
        L.spec = l
        ifm, ofm, k, g = l["ifm"], l["ofm"], l["k"], l["groups"]
        hw, ohw = l["in_hw"], l["out_hw"]
        lo, hi = (0, 256) if in_dt == np.uint8 else (-128, 128)
        L.follows = i in follows
        L.chain = None
        L.shares = bool(l.get("shares_input")) and i > 0 and not out[-1].follows
        L.sibling = None
        if L.follows:
            L.x = None
        elif L.shares:
            L.x = out[-1].x
        else:
            L.x = r.integers(lo, hi, (batch, ifm, hw, hw), dtype=np.int16).astype(in_dt)
        L.w = r.integers(-127, 128, (ofm, ifm // g, k, k), dtype=np.int16).astype(np.int8)
        L.bias = r.integers(-1000, 1001, ofm).astype(np.int32)
        L.wqf = np.ones(ofm, np.float32)
        L.calib = np.exp(r.uniform(np.log(1e-4), np.log(1e-2), ofm)).astype(np.float32)
        if calibration == "spread":
            L.calib = (40.0 / (np.sqrt((ifm // g) * k * k) * 147.4 * 73.3) * r.uniform(0.5, 2.0, ofm)).astype(np.float32)
        L.fused = bool(fuse_residual and l["closes_block"])
        L.eltw = L.ecal = None
        act = l["act"]
        kw = dict(stride=(l["stride"],) * 2, pad=(l["pad"],) * 2, groups=g, bias_dt=hip.I32, has_wqf=True, has_calib=True)
        if act == "relu6":
            kw.update(act="clamp", act_m=0.0, act_n=6.0)
            # the clamp acts on the dequantised value: scale it into range, requantise with 127/6
            sig = np.sqrt((ifm // g) * k * k) * 147.4 * 73.3
            L.wqf = (3.0 / sig * r.uniform(0.5, 2.0, ofm)).astype(np.float32)
            L.calib = np.full(ofm, 127.0 / 6.0, np.float32)
        else:
            kw.update(act=act)
        # zero border as wide as the padding; a first layer (3 input features) takes b_fs_yx_fsv4
        first = ifm <= 4 and g == 1
        if L.follows:  # reads the int8 tensor of the stage before it, which stays in registers
            L.xin = None
            in_tensor = hip.Tensor.make(hip.S8, hip.FS_B_YX_FSV16, batch, ifm, hw, hw)
        elif L.shares:
            L.xin = out[-1].xin
            in_tensor = L.xin.tensor
        else:
            L.xin = hip.upload(eng, L.x, "b_fs_yx_fsv4" if first else "fs_b_yx_fsv16", (l["pad"], l["pad"]))
            in_tensor = L.xin.tensor
        L.ein = None
        if L.fused:
            L.eltw = r.integers(-128, 128, (batch, ofm, ohw, ohw), dtype=np.int16).astype(np.int8)
            L.ecal = r.uniform(0.25, 1.0, ofm).astype(np.float32)
            L.ein = hip.upload(eng, L.eltw, "fs_b_yx_fsv16")
            kw.update(act="none", eltw_t=L.ein.tensor, eltw_act="relu", has_eltw_calib=True)
        L.kw = kw
        if first:
            kw["out_fmt"] = hip.FS_B_YX_FSV16
        L.desc = hip.conv_desc(in_tensor, L.w.shape, "s8", tile=0 if first else tile, **kw)
        try:
            L.conv = hip.Conv(eng, L.desc, L.w, L.bias, L.wqf, L.calib, L.ecal)
        except hip.HipError:
            if not tile:
                raise
            L.desc = hip.conv_desc(in_tensor, L.w.shape, "s8", tile=0, **kw)  # forced row not applicable here
            L.conv = hip.Conv(eng, L.desc, L.w, L.bias, L.wqf, L.calib, L.ecal)
        L.out = hip.Buffer(eng, L.desc.output)
        L.info = L.conv.info()
        L.kept = True
        out.append(L)
    # the chains: as many stages as the library takes (three, else two); where it refuses a head, that layer runs
    # alone and the layers behind it are tried as a chain of their own (a block's closing 1x1 with the next block's
    # opening 1x1)
    i = 0
    while i < len(out):
        L = out[i]
        want = L.spec.get("chain_len", 1)
        n = want
        while n > 1:
            members = out[i:i + n]
            # the first stage's result is read by the next stage only, unless it closes a block (then the next
            # block's sum reads it too)
            keep = [bool(L.spec["closes_block"])] + [True] * (n - 1)
            try:
                L.chain = hip.ConvChain(eng, [(M.desc, M.w, M.bias, M.wqf, M.calib, M.ecal) for M in members], keep)
            except hip.HipError as e:
                if e.status != -6:
                    raise
                n -= 1
                continue
            L.members = members
            L.chain_args = L.chain.pointers([M.out if k else None for M, k in zip(members, keep)], [M.ein for M in members])
            L.info = L.chain.info()
            L.kept = keep[0]
            for M in members[1:]:
                M.info = None  # counted in the chain head
            break
        if n < want:
            # the first layer left out needs a real input tensor: the layer before it writes it
            M = out[i + n]
            M.follows, M.xin_from = False, out[i + n - 1]
            if want - n > 1:
                M.spec = dict(M.spec, chain_len=want - n)
        i += n
    # two convolutions of one input in one launch, where the library has a short epilogue for the pair
    for H, M in zip(out, out[1:]):
        if not (siblings and not tile and M.shares and H.chain is None and M.chain is None and not H.fused and not M.fused
                and H.spec["ofm"] % 16 == 0):
            continue
        cat = lambda a, b: np.concatenate([a, b])
        w = cat(H.w, M.w)
        kw = dict(H.kw, sibling_split=H.spec["ofm"], sibling_act=M.kw["act"], sibling_act_m=M.kw.get("act_m", 0.0),
                  sibling_act_n=M.kw.get("act_n", 0.0))
        desc = hip.conv_desc(H.xin.tensor, w.shape, "s8", **kw)
        try:
            both = hip.Conv(eng, desc, w, cat(H.bias, M.bias), cat(H.wqf, M.wqf), cat(H.calib, M.calib), None)
        except hip.HipError as e:
            if e.status != -6:
                raise
            continue
        if b"generic" in both.info().kernel_name:  # no short epilogue for this pair: two launches are faster
            both.close()
            continue
        H.conv.close(), M.conv.close(), H.out.close(), M.out.close()
        H.conv, H.desc, H.info, H.sibling = both, desc, both.info(), M
        H.whole = hip.Buffer(eng, desc.output)
        H.out, M.out = hip.Window(H.whole, 0, H.spec["ofm"]), hip.Window(H.whole, H.spec["ofm"], M.spec["ofm"])
        M.conv, M.info, M.follows = None, None, True  # written by the launch of H
    return out


def launches(stack):
    """what one step enqueues: (library function, arguments) per launch"""
    lib = hip.lib()
    seq = []
    for L in stack:
        if L.follows:
            continue
        src = L.xin.ptr if L.xin is not None else L.xin_from.out.ptr
        if L.chain is not None:
            seq.append((lib.cldnn_hip_conv_chain_enqueue, (L.chain.h, src, L.chain_args[0], L.chain_args[1])))
        else:
            seq.append((lib.cldnn_hip_conv_enqueue, (L.conv.h, src, L.out.ptr, L.ein.ptr if L.ein is not None else None)))
    return seq


def run_step(seq):
    for fn, args in seq:
        st = fn(*args)
        if st:
            hip.check(st)


class GpuTimer:
    """HIP events on the engine's own stream (the stream the kernels are launched on)."""

    def __init__(self, eng):
        self.eng, self.ev = eng, None

    def __enter__(self):
        self.ev = C.c_void_p()
        hip.check(hip.lib().cldnn_hip_event_record_begin(self.eng.h, C.byref(self.ev)))
        return self

    def __exit__(self, *a):
        hip.check(hip.lib().cldnn_hip_event_record_end(self.ev))

    def seconds(self):
        if self.ev is not None:  # read once, then give the event back
            ns = C.c_uint64()
            hip.check(hip.lib().cldnn_hip_event_elapsed_ns(self.ev, C.byref(ns)))
            hip.check(hip.lib().cldnn_hip_event_release(self.ev))
            self.ev, self.value = None, ns.value * 1e-9
        return self.value


def cpu_pass(eng, stack, images, verify):
    """Run the CPU oracle on the first `images` image(s) of every layer; optionally compare with the
    GPU results of the same images (a convolution is independent per image).  A layer that runs as a later stage of
    a chain (or behind a layer whose chain was refused) reads what the oracle computed for the layer before it."""
    from oracle import refconv as rc
    threads = rc.lib().rc_threads_available()
    t_total, checked, mism = 0.0, 0, 0
    prev = None
    for L in stack:
        l = L.spec
        kw = dict(stride=(l["stride"],) * 2, pad=(l["pad"],) * 2, groups=l["groups"], out_dt="s8",
                  act=L.kw.get("act", "none"), act_m=L.kw.get("act_m", 0.0), act_n=L.kw.get("act_n", 0.0))
        if L.fused:
            kw.update(eltw=L.eltw[:images], eltw_act="relu", eltw_calib=L.ecal)
        x = L.x[:images] if L.x is not None else prev
        t0 = time.perf_counter()
        ref = rc.conv(x, L.w, L.bias, wqf=L.wqf, calib=L.calib, nthreads=threads, **kw)
        t_total += time.perf_counter() - t0
        prev = ref
        if verify and L.kept:
            got = hip.download(eng, L.out)[:images]
            checked += ref.size
            mism += int(np.count_nonzero(ref != got))
    return t_total, threads, checked, mism


def cpu_baseline_and_check(eng, stack, batch, budget_seconds):
    """Bounded CPU sample: probe with one image, then as many images as fit the time budget."""
    t1, threads, checked, mism = cpu_pass(eng, stack, 1, verify=True)
    n = max(1, min(batch, int(budget_seconds / max(t1, 1e-3))))
    tn = t1
    if n > 1:
        tn, threads, checked, mism = cpu_pass(eng, stack, n, verify=True)
    return dict(images=n, seconds=tn, threads=threads, checked=checked, mismatches=mism)


def copy_calibration(args):
    """A plain device copy of known size (256 MiB read + 256 MiB written per step): the yardstick that the
    FETCH_SIZE / WRITE_SIZE counter readings of the convolution kernels are scaled by."""
    eng = hip.Engine(0, profiling=True)
    t = hip.Tensor.make(hip.F32, hip.BFYX, 1, 64, 1024, 1024)
    src, dst = hip.Buffer(eng, t), hip.Buffer(eng, t)
    for _ in range(args.warmup):
        hip.reorder(eng, src, dst)
    eng.finish()
    with GpuTimer(eng) as tm:
        for _ in range(args.steps):
            hip.reorder(eng, src, dst)
    eng.finish()
    nbytes = 2 * src.nbytes
    print(json.dumps({"metric": "device copy", "value": nbytes * args.steps / tm.seconds() / 1e9, "unit": "GB/s", "n_gpus": 1,
                      "steps": args.steps, "warmup": args.warmup, "ms_per_step": tm.seconds() / args.steps * 1e3,
                      "higher_is_better": True, "config": {"workload": "copy_256m", "read_bytes": src.nbytes,
                                                           "written_bytes": src.nbytes}}), flush=True)


def network_workload(args):
    """A whole quantized network built and run through the clDNN API with optimize_data: what an application sees per
    network.execute(), input already on the device.  resnet50_b32_network: 53 convolutions, 2 poolings, 16 residual sums,
    fully_connected; mobilenet_v2_b32_network: 52 convolutions (17 depthwise), 35 clamps, 10 residual sums, pooling,
    fully_connected; vgg16_b16_network: 13 convolutions, 5 poolings, 3 fully_connected (the first over a 7x7 plane)."""
    from cldnn_amd import api as cl
    batch = 32
    eng = cl.engine(enable_parallelisation=args.second_stream)
    r = np.random.default_rng(1337)
    resnet, vgg = args.workload.startswith("resnet50"), args.workload.startswith("vgg16")
    out_id, fcs = "fc1000", []
    if resnet:
        from cldnn_amd import resnet50_net as net_def
        layers, fcs = workloads.resnet50(), [("fc1000", 2048, 1000)]
        primitives = "53 convolution, 2 pooling, 16 eltwise (fused), 1 fully_connected"
    elif vgg:
        from cldnn_amd import vgg16_net as net_def
        batch, out_id = 16, "fc8"
        layers, fcs = workloads.vgg16(), [("fc6", 25088, 4096), ("fc7", 4096, 4096), ("fc8", 4096, 1000)]
        primitives = "13 convolution, 5 pooling, 3 fully_connected"
    else:
        from cldnn_amd import mobilenet_v2_net as net_def
        layers, fcs = workloads.mobilenet_v2(), [("fc1000", 1280, 1000)]
        primitives = "52 convolution (17 depthwise), 35 activation clamp (folded), 10 eltwise, 1 pooling, 1 fully_connected"
    params = net_def.random_weights()
    IN_RMS, ECAL = 35.0, 1.0  # keep the signal alive through the blocks without a calibration pass
    for l in layers:  # factors by rule (no calibration pass: timing does not depend on the values)
        k = (l["ifm"] // l["groups"]) * l["k"] ** 2
        q = params[l["name"]]
        if l["act"] == "relu6":  # the clamp acts on the dequantised value: scale it into range, requantise with 127 / 6
            q["wqf"] = (3.0 / (np.sqrt(k) * IN_RMS * 73.3) * r.uniform(0.7, 1.4, l["ofm"])).astype(np.float32)
            q["calib"] = np.full(l["ofm"], 127.0 / 6.0, np.float32)
        else:
            q.setdefault("wqf", np.ones(l["ofm"], np.float32))
            q["calib"] = (32.0 / (np.sqrt(k) * IN_RMS * 73.3) * r.uniform(0.7, 1.4, l["ofm"])).astype(np.float32)
    for step in net_def.layer_plan():
        if step[0] == "sum":
            params[step[1]] = dict(ecal=np.full(params[step[3]]["w"].shape[0], ECAL if resnet else 0.75, np.float32))
    for name, k, ofm in fcs:
        params[name]["calib"] = np.full(ofm, 40.0 / (np.sqrt(k) * 30.0 * 73.3), np.float32)
    t0 = time.perf_counter()
    topo, opts = net_def.topology(cl, eng, params, batch), cl.build_options(optimize_data=True)
    if args.tuning_cache:
        # measure what the cache file does not hold yet (needs an engine with profiling), then run from the file
        tuner = cl.engine(enable_profiling=True)
        t0 = time.perf_counter()
        cl.network(tuner, net_def.topology(cl, tuner, params, batch),
                   cl.build_options(optimize_data=True, tuning_config=(cl.tuning_mode.tuning_tune_and_cache, args.tuning_cache)))
        log("tuning pass over %s: %.1f s" % (args.tuning_cache, time.perf_counter() - t0))
        opts = cl.build_options(optimize_data=True, tuning_config=(cl.tuning_mode.tuning_use_cache, args.tuning_cache))
    net = cl.network(eng, topo, opts)
    x = r.integers(0, 256, (batch, 3, 224, 224)).astype(np.uint8)
    net.set_input_data("input", cl.make_memory(eng, x))
    log("built the network in %.1f s" % (time.perf_counter() - t0))

    def run():
        outs = net.execute()
        outs[out_id].get_event().wait()
        return outs

    t0 = time.perf_counter()
    while time.perf_counter() - t0 < args.clock_warmup:  # see clock_warmup()
        run()
    for _ in range(args.warmup):
        run()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        outs = run()
    dt = time.perf_counter() - t0
    logits = outs[out_id].get_memory().read()
    in_flight = None
    if args.in_flight > 1:
        # several requests kept going the way the reference's users do it: one network, engine (= stream) and host thread
        # per request; kernels of different requests overlap on the device
        import threading
        nets = [net]
        for k in range(args.in_flight - 1):
            e2 = cl.engine(enable_parallelisation=args.second_stream)
            n2 = cl.network(e2, net_def.topology(cl, e2, params, batch), opts)
            n2.set_input_data("input", cl.make_memory(e2, np.roll(x, k + 1, axis=0)))
            nets.append(n2)

        def request_loop(n, count):
            for _ in range(count):
                n.execute()[out_id].get_event().wait()
        for n in nets:
            request_loop(n, 5)
        threads = [threading.Thread(target=request_loop, args=(n, args.steps)) for n in nets]
        t1 = time.perf_counter()
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        dt2 = time.perf_counter() - t1
        in_flight = {"requests": len(nets), "steps_per_request": args.steps, "images_per_s": len(nets) * batch * args.steps / dt2,
                     "ms_per_request_step": dt2 / args.steps * 1e3,
                     "what": "independent requests: one network, engine (HIP stream at default priority) and host thread each"}
    cpu, verified = None, None
    if not args.no_cpu and args.cpu_seconds > 0:
        # the same network through the CPU oracle, layer by layer, on the first images of the batch: a bounded sample
        # (one image as a probe, then as many as the time budget holds) and a bit-exact check of the logits
        from oracle import networks as oracle_networks
        from oracle import refconv as rc
        fused = [n["id"].split("_fused_")[1] for n in cl.plan(topo, opts) if "_fused_" in n["id"]]

        def oracle_logits(xs):
            if resnet:
                return oracle_networks.resnet50(xs, params, fused=fused)[out_id]
            if vgg:
                return oracle_networks.vgg16(xs, params)[out_id]
            return oracle_networks.mobilenet_v2(xs, params, folded=True)[out_id]
        t1 = time.perf_counter()
        ref = oracle_logits(x[:1])
        seconds, images = time.perf_counter() - t1, 1
        more = max(1, min(batch, int(args.cpu_seconds / max(seconds, 1e-3))))
        if more > 1:
            t1 = time.perf_counter()
            ref = oracle_logits(x[:more])
            seconds, images = time.perf_counter() - t1, more
        threads = rc.lib().rc_threads_available()
        mismatches = int((logits[:images] != ref).sum())
        cpu = {"value": images / seconds, "unit": "images/s", "cores": threads, "kind": "port",
               "sample": "first %d image(s) of the batch through every layer of the network in oracle/refconv.c (OpenMP over "
                         "batch x ofm), %.1f s on %d threads = %.0f s of CPU work" % (images, seconds, threads, seconds * threads)}
        verified = {"outputs_compared": int(ref.size), "mismatches": mismatches,
                    "what": "logits of the first %d image(s) of the batch-%d execute() (they depend on every layer) vs the CPU "
                            "oracle run layer by layer (bit-exact)" % (images, batch)}
        if mismatches:
            log("PARITY FAILURE in %s: %d mismatching logits" % (args.workload, mismatches))
    # multiply-adds the kernels execute: the graph passes let the layers in front of a stride-2 block compute only what
    # that block reads, so this can be less than the model's nominal count
    nominal = 2.0 * batch * (workloads.macs(layers) + sum(k * ofm for _, k, ofm in fcs))
    plan = {n["id"]: n for n in cl.plan(topo, opts)}
    ops = 0.0
    for n in plan.values():
        if n["type"] in ("convolution", "fused_conv_eltwise"):
            ofm, ifm, fx, fy = plan[n["deps"][1 if n["type"] == "convolution" else 2]]["size"]
            ops += 2.0 * np.prod(n["size"]) * ifm * fx * fy
    name = "ResNet-50" if resnet else ("VGG-16" if vgg else "MobileNet-v2")
    # what the built network launches: members of a convolution chain are written by the launch of the chain's head
    infos = {i: net.get_primitive_info(i) for i in net.get_all_primitive_ids()}
    followers = [i for i, inf in infos.items() if str(inf.get("kernel", "")).startswith("in the chain of")]
    paired = [i for i, inf in infos.items() if "launched_by" in inf]  # written by the launch of a convolution of the same input
    executed = [i for i, inf in infos.items() if inf.get("type") not in ("data", "input_layout")]
    if args.per_layer:
        for i in executed:
            log("%-40s %s" % (i, "in the launch of " + infos[i]["launched_by"] if i in paired else infos[i].get("kernel", infos[i].get("type"))))
    print(json.dumps({
        "metric": "%s int8 network images/sec @b%d (whole topology through the clDNN API)" % (name, batch), "value": batch * args.steps / dt,
        "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "i8xi8->i32 (f32 requantisation)", "data": "synthetic",
        "config": {"workload": args.workload, "batch": batch, "primitives": primitives,
                   "clock_warmup_s": args.clock_warmup,
                   "build": "optimize_data" + (", tuning cache" if args.tuning_cache else "") + (", second stream" if args.second_stream else ""), "primitives_per_execute": len(executed), "launches_per_execute": len(executed) - len(followers) - len(paired),
                   "convolutions_in_a_neighbours_launch": len(paired),
                   "chained_convolutions": len(followers) + len({str(infos[i]["kernel"]) for i in followers}),
                   "executed_ops_per_step": ops, "nominal_ops_per_step": nominal},
        "roofline": {"bound": "mfma", "achieved": ops * args.steps / dt / 1e12, "peak": PEAK_INT8_OPS / 1e12, "unit": "TOP/s",
                     "frac": ops * args.steps / dt / PEAK_INT8_OPS, "traffic": None, "kernel": "all kernels of one network.execute()"},
        "requests_in_flight": in_flight, "cpu_baseline": cpu, "verified": verified,
        "distinct_logit_values": int(len(np.unique(logits)))}), flush=True)
    if verified and verified["mismatches"]:
        sys.exit(1)


def kernel_sources_digest():
    """sha256 over the library's sources (cldnn_amd/csrc: *.hip, *.h, *.cpp, Makefile) in name order: what a counter
    summary under profiles/ is stamped with."""
    import hashlib
    d = os.path.join(ROOT, "cldnn_amd", "csrc")
    h = hashlib.sha256()
    for name in sorted(os.listdir(d)):
        if name.endswith((".hip", ".h", ".cpp")) or name == "Makefile":
            h.update(name.encode() + b"\0")
            with open(os.path.join(d, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def measured_traffic(workload):
    """HBM bytes per launch from the committed counter summary of this workload.  None when there is none, or when
    the summary is older than the kernels: it carries the digest of the library sources it was taken with (and the
    commit, for the reader), and any change to cldnn_amd/csrc/ since makes it stale."""
    path = os.path.join(ROOT, "profiles", "conv_stack_%s_hbm_traffic.txt" % workload)
    if not os.path.exists(path):
        return None
    value = digest = None
    with open(path) as f:
        for line in f:
            if line.startswith("traffic_bytes_per_launch:"):
                value = int(line.split(":")[1])
            if line.startswith("kernel_sources_sha256:"):
                digest = line.split(":")[1].strip()
    if value is None or not digest or digest != kernel_sources_digest():
        return None
    return value


def stack_of(wl):
    if wl.startswith("resnet50"):
        return workloads.resnet50(), (1 if wl.endswith("b1") else 32), wl.endswith("fused")
    if wl == "vgg16_b16":
        return workloads.vgg16(), 16, False
    if wl == "mobilenet_v2_b32":
        return workloads.mobilenet_v2(), 32, False
    return [workloads._layer("c1", 64, 64, 3, 1, 1, 56)], 1, False


def release_stack(stack):
    for L in stack:
        if L.chain is not None:
            L.chain.close()
        if L.conv is not None:
            L.conv.close()
        L.out.close()
        if L.sibling is not None:
            L.whole.close()
        if L.xin is not None:
            L.xin.close()
        if L.ein is not None:
            L.ein.close()


def time_launches(eng, stack, seq, steps):
    """GPU time of every launch inside whole steps (so every kernel starts with cold caches, as in the real run):
    one event pair per launch on the engine's stream.  -> seconds per launch, in launch order"""
    acc = [0.0] * len(seq)
    for _ in range(steps):
        timers = []
        for fn, a in seq:
            tmr = GpuTimer(eng)
            with tmr:
                st = fn(*a)
                if st:
                    hip.check(st)
            timers.append(tmr)
        eng.finish()
        for i, tmr in enumerate(timers):
            acc[i] += tmr.seconds()
    return [v / steps for v in acc]


def kernel_rooflines(heads, times):
    """Per kernel instance: launches per step, average duration, algorithmic ops and bytes per launch, and the
    fraction of the roofline that bounds it (int8 MFMA peak or HBM peak, whichever the layer's work is closer to)."""
    groups = {}
    for L, dt in zip(heads, times):
        g = groups.setdefault(L.info.kernel_name.decode(), dict(n=0, t=0.0, ops=0, bytes=0))
        g["n"] += 1
        g["t"] += dt
        g["ops"] += L.info.ops
        g["bytes"] += L.info.bytes
    rows = []
    for name, g in groups.items():
        t_m, t_h = g["ops"] / PEAK_INT8_OPS, g["bytes"] / PEAK_HBM
        bound = "mfma" if t_m > t_h else "hbm"
        rows.append({"name": name, "launches_per_step": g["n"], "avg_us": g["t"] / g["n"] * 1e6, "share_of_step": 0.0,
                     "ops_per_launch": g["ops"] / g["n"], "bytes_per_launch": g["bytes"] / g["n"], "bound": bound,
                     "achieved": g["ops"] / g["t"] / 1e12 if bound == "mfma" else g["bytes"] / g["t"] / 1e9,
                     "unit": "TOP/s" if bound == "mfma" else "GB/s", "frac": max(t_m, t_h) / g["t"], "_t": g["t"]})
    total = sum(r["_t"] for r in rows)
    for r in rows:
        r["share_of_step"] = r.pop("_t") / total
    rows.sort(key=lambda r: -r["share_of_step"])
    return rows


CLOCK_WARMUP_SECONDS = 0.3


def clock_warmup(eng, step, seconds=None):
    """The clocks of an idle device rise over tens of milliseconds of load (a layer timed right after idling runs
    10 % and more slower than in a steady stream of work), and a short run (--steps 20 --warmup 5 is 15 ms) would be
    timed on that ramp.  Untimed steps for CLOCK_WARMUP_SECONDS of wall time come first, then the W warm-up steps, then
    exactly K timed steps; the JSON line names this under config.clock_warmup_s."""
    seconds = CLOCK_WARMUP_SECONDS if seconds is None else seconds
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(5):
            step()
        eng.finish()


def measure_stack(args, wl, steps, warmup, in_flight_n, cpu_seconds, extras):
    """Build one workload's stack, time `steps` whole steps, per-kernel times, optionally requests in flight and the
    CPU oracle leg (bounded sample + bit-exact check).  -> result dict, parity ok"""
    layers, batch, fuse = stack_of(wl)
    if args.only and extras:
        keep = set(args.only.split(","))
        layers = [l for l in layers if l["name"] in keep]
        if not layers:
            log("bench.py: no layer of %s is named in --only" % wl)
            sys.exit(2)
    eng = hip.Engine(0, profiling=True)
    t0 = time.perf_counter()
    stack = build_stack(eng, layers, batch, fuse, tile=args.tile, chains=not args.no_chains)
    seq = launches(stack)
    heads = [L for L in stack if not L.follows]
    eng.finish()
    log("%s: built %d layers (%d launches per step) in %.1f s" % (wl, len(stack), len(seq), time.perf_counter() - t0))

    ops = sum(L.info.ops for L in heads)
    nbytes = sum(L.info.bytes for L in heads)
    clock_warmup(eng, lambda: run_step(seq), args.clock_warmup)
    for _ in range(warmup):
        run_step(seq)
    eng.finish()
    t_wall0 = time.perf_counter()
    with GpuTimer(eng) as tm:
        for _ in range(steps):
            run_step(seq)
    eng.finish()
    t_wall = time.perf_counter() - t_wall0
    t_gpu = tm.seconds()
    n_launch = len(seq) * steps

    per_launch = time_launches(eng, stack, seq, max(3, min(10, steps // 4)))
    kernels = kernel_rooflines(heads, per_launch)

    in_flight = None
    if in_flight_n > 1 and not args.only:
        # What an application gets that keeps several requests going (the reference's users run one network per request
        # and thread): every request has an engine = stream of its own; kernels of different requests overlap on the
        # device and fill what one request's kernels leave idle.
        import threading
        engines = [eng] + [hip.Engine(0, profiling=False) for _ in range(in_flight_n - 1)]
        stacks = [stack] + [build_stack(e, layers, batch, fuse, seed=1337 + 1000 * (k + 1), tile=args.tile, chains=not args.no_chains)
                            for k, e in enumerate(engines[1:])]
        seqs = [seq] + [launches(st) for st in stacks[1:]]

        def request_loop(k, count):
            for _ in range(count):
                run_step(seqs[k])
            engines[k].finish()
        for k in range(len(engines)):
            request_loop(k, 5)
        threads = [threading.Thread(target=request_loop, args=(k, steps)) for k in range(len(engines))]
        t0 = time.perf_counter()
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        dt = time.perf_counter() - t0
        in_flight = {"requests": len(engines), "steps_per_request": steps, "images_per_s": len(engines) * batch * steps / dt,
                     "ms_per_request_step": dt / steps * 1e3, "tops": len(engines) * ops * steps / dt / 1e12,
                     "frac_of_int8_peak": len(engines) * ops * steps / dt / PEAK_INT8_OPS,
                     "what": "independent requests of this workload, one engine (HIP stream at default priority) and one host thread each"}
        for st in stacks[1:]:
            release_stack(st)
        del stacks, seqs
        for e in engines[1:]:
            e.close()
    host_io = None
    if args.host_io and extras:
        # what a caller holding host tensors pays: bfyx input host -> device, device reorder into the blocked layout
        # with its border, the stack, blocked output device -> host
        first, last_l = stack[0], stack[-1]
        plain = hip.Buffer(eng, hip.Tensor.make(first.xin.tensor.dtype, hip.BFYX, *first.x.shape))
        for _ in range(2):
            plain.write_raw(first.x); hip.reorder(eng, plain, first.xin); run_step(seq); last_l.out.read_raw()
        t0 = time.perf_counter()
        for _ in range(steps):
            plain.write_raw(first.x)
            hip.reorder(eng, plain, first.xin)
            run_step(seq)
            last_l.out.read_raw()
        dt = time.perf_counter() - t0
        host_io = {"images_per_s": batch * steps / dt, "ms_per_step": dt / steps * 1e3,
                   "host_to_device_bytes": int(first.x.nbytes), "device_to_host_bytes": int(last_l.out.nbytes)}
        plain.close()

    def table(stk, times):
        log("%-18s %-52s %6s %9s %8s %8s %7s" % ("layer", "kernel", "grid", "us", "TOP/s", "GB/s", "bound"))
        for L, dt in zip(stk, times):
            tops, gbs = L.info.ops / dt / 1e12, L.info.bytes / dt / 1e9
            t_m, t_h = L.info.ops / PEAK_INT8_OPS, L.info.bytes / PEAK_HBM
            name = L.spec["name"] + ("+%d" % (len(L.members) - 1) if L.chain is not None else "") + ("|1" if L.sibling is not None else "")
            log("%-18s %-52s %6d %9.1f %8.1f %8.0f %7s %5.1f%%" % (
                name, L.info.kernel_name.decode(), L.info.grid, dt * 1e6, tops, gbs,
                "mfma" if t_m > t_h else "hbm", 100 * max(t_m, t_h) / dt))
        log("sum of per-launch times: %.1f us" % (sum(times) * 1e6))

    if (args.per_layer or args.tune) and extras:
        table(heads, per_launch)
        if args.tune:
            # every row of the tile table forced on every layer where it applies (no chains); report the best row per layer
            names = [hip.lib().cldnn_hip_tile_config_name(i).decode() for i in range(hip.lib().cldnn_hip_tile_config_count())]
            base = build_stack(eng, layers, batch, fuse, chains=False)
            bseq = launches(base)
            run_step(bseq)
            base_t = time_launches(eng, base, bseq, max(3, steps // 3))
            best = [(t, "table:" + L.info.kernel_name.decode()) for t, L in zip(base_t, base)]
            for row in range(1, len(names) + 1):
                alt = build_stack(eng, layers, batch, fuse, tile=row, chains=False)
                aseq = launches(alt)
                for _ in range(2):
                    run_step(aseq)
                times = time_launches(eng, alt, aseq, max(3, steps // 3))
                for i, (t, L) in enumerate(zip(times, alt)):
                    if L.info.tile_index == row - 1 and t < best[i][0]:
                        best[i] = (t, names[row - 1])
                release_stack(alt)
            log("%-18s %6s %6s %5s %3s %9s %9s  %s" % ("layer", "M", "OFM", "K", "k", "table us", "best us", "best row"))
            for L, t0, (t1, nm) in zip(base, base_t, best):
                l = L.spec
                log("%-18s %6d %6d %5d %3d %9.1f %9.1f  %s" % (l["name"], batch * l["out_hw"] ** 2, l["ofm"],
                                                             l["ifm"] * l["k"] ** 2, l["k"], t0 * 1e6, t1 * 1e6, nm))
            log("sum with the table: %.1f us; sum of per-layer bests: %.1f us" % (sum(base_t) * 1e6, sum(t for t, _ in best) * 1e6))
            release_stack(base)

    dom = kernels[0]
    # the roofline the workload is priced against: the dense stacks against the int8 matrix peak (the baseline's
    # metric), the depthwise / 1x1 network and the batch-1 stack (weights dominate) against HBM
    hbm_bound = wl in ("mobilenet_v2_b32", "resnet50_b1")
    res = {
        "value": batch * steps / t_wall,
        "unit": "images/s",
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": t_wall / steps * 1e3,
        "config": {"workload": wl, "batch": batch, "layers": len(stack), "launches_per_step": len(seq),
                   "chained_layers": sum(len(L.members) for L in stack if L.chain is not None),
                   "layers_in_a_neighbours_launch": sum(1 for L in stack if L.sibling is not None),
                   "layout": "fs_b_yx_fsv16",
                   "variant": "stride on the first 1x1 (Caffe form)" if wl.startswith("resnet50") else wl,
                   "fused_residual_layers": sum(1 for L in stack if L.fused),
                   "clock_warmup_s": args.clock_warmup},
        "achieved_tops": ops * steps / t_gpu / 1e12,
        "roofline": {
            "bound": "hbm" if hbm_bound else "mfma",
            "achieved": nbytes * steps / t_gpu / 1e9 if hbm_bound else ops * steps / t_gpu / 1e12,
            "peak": PEAK_HBM / 1e9 if hbm_bound else PEAK_INT8_OPS / 1e12,
            "unit": "GB/s" if hbm_bound else "TOP/s",
            "frac": nbytes * steps / t_gpu / PEAK_HBM if hbm_bound else ops * steps / t_gpu / PEAK_INT8_OPS,
            "traffic": measured_traffic(wl),
            "kernel": "all convolution kernels of the step",
            "launches": n_launch,
            "avg_launch_us": t_gpu / n_launch * 1e6,
            "ops_per_launch": ops / len(seq),
            "bytes_per_launch": nbytes / len(seq),
            "dominant_kernel": dom,
            "kernels": kernels[1:6],
        },
        "roofline_hbm": {
            "bound": "hbm",
            "achieved": nbytes * steps / t_gpu / 1e9,
            "peak": PEAK_HBM / 1e9,
            "unit": "GB/s",
            "frac": nbytes * steps / t_gpu / PEAK_HBM,
            "bytes_per_launch": nbytes / len(seq),
        },
        "gpu_seconds_events": t_gpu,
        "wall_seconds": t_wall,
    }
    if host_io:
        res["pcie_inclusive"] = host_io
    if in_flight:
        res["requests_in_flight"] = in_flight
    ok = True
    if cpu_seconds > 0:
        cb = cpu_baseline_and_check(eng, stack, batch, cpu_seconds)
        res["cpu_baseline"] = {
            "value": cb["images"] / cb["seconds"],
            "unit": "images/s",
            "cores": cb["threads"],
            "kind": "port",
            "sample": "first %d image(s) of every layer of the same stack through oracle/refconv.c "
                      "(OpenMP over batch x ofm), %.1f s on %d threads = %.0f s of CPU work" % (cb["images"], cb["seconds"], cb["threads"], cb["seconds"] * cb["threads"]),
        }
        res["verified"] = {"outputs_compared": cb["checked"], "mismatches": cb["mismatches"],
                           "what": "GPU batch-%d results of the first %d image(s), every tensor the step writes, vs the CPU "
                                   "oracle run layer by layer (bit-exact)" % (batch, cb["images"])}
        if cb["mismatches"]:
            log("PARITY FAILURE in %s: %d mismatching outputs" % (wl, cb["mismatches"]))
            ok = False
    release_stack(stack)
    eng.close()
    return res, ok


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="resnet50_b32_fused",
                    choices=["resnet50_b32_fused", "resnet50_b32", "resnet50_b1", "vgg16_b16", "mobilenet_v2_b32", "c1",
                             "copy_256m", "resnet50_b32_network", "mobilenet_v2_b32_network", "vgg16_b16_network"])
    ap.add_argument("--tile", type=int, default=0, help="force one row (index+1) of the tile table on every layer (no chains)")
    ap.add_argument("--no-chains", action="store_true", help="every layer is a launch of its own (no convolution chains, no two convolutions of one input in one launch)")
    ap.add_argument("--per-layer", action="store_true", help="print the per-launch table to stderr")
    ap.add_argument("--tune", action="store_true", help="try every row of the tile table on every layer, print the best")
    ap.add_argument("--only", default="", help="comma-separated layer names: run just these layers of the workload "
                                               "(same buffers every step, so their tensors stay cache-resident)")
    ap.add_argument("--tuning-cache", default="", help="network workloads only: tune what this cache file lacks "
                                                       "(build option tuning_config, tune_and_cache), then run from it")
    ap.add_argument("--second-stream", action="store_true", help="network workloads only: engine option enable_parallelisation "
                    "(shortcut convolutions run on a second stream beside the branch)")
    ap.add_argument("--in-flight", type=int, default=2,
                    help="after the headline measurement also time this many independent requests of the same workload in "
                         "flight at once, one engine (HIP stream) and one host thread each; reported under "
                         "requests_in_flight, never as the headline value (0 or 1 = skip)")
    ap.add_argument("--clock-warmup", type=float, default=CLOCK_WARMUP_SECONDS,
                    help="seconds of untimed steps before the warm-up steps (0 for counter runs under rocprofv3 --pmc, where "
                         "every dispatch is serialised and recorded)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / full-size check")
    ap.add_argument("--no-others", action="store_true", help="default workload only: do not time the other four configurations")
    ap.add_argument("--host-io", action="store_true",
                    help="also report the rate with the first layer's input crossing PCIe into the device and the last "
                         "layer's output crossing back, every step (never the headline value)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on one GPU; --gpus %d is not supported (the path shards by batch, no "
            "figure at several GPUs is produced)" % args.gpus)
        sys.exit(2)

    wl = args.workload
    if wl == "copy_256m":
        return copy_calibration(args)
    if wl.endswith("_network"):
        return network_workload(args)

    res, ok = measure_stack(args, wl, args.steps, args.warmup, args.in_flight, 0.0 if args.no_cpu else args.cpu_seconds, True)
    line = {
        "metric": "ResNet-50 int8 conv stack images/sec @b32; achieved TOPS vs INT8 MFMA peak"
        if wl.startswith("resnet50_b32") else "int8 conv stack images/sec",
        "value": res.pop("value"), "unit": res.pop("unit"), "n_gpus": 1, "steps": res.pop("steps"), "warmup": res.pop("warmup"),
        "ms_per_step": res.pop("ms_per_step"), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "i8xi8->i32 (f32 requantisation)", "data": "synthetic",
    }
    line.update(res)
    if wl == "resnet50_b32_fused" and not args.no_others and not args.only and not args.tune:
        # the other four configurations of the baseline, shorter runs, same measurement (a CPU sample of a few seconds each)
        others = {}
        for other in ("vgg16_b16", "mobilenet_v2_b32", "resnet50_b1", "c1"):
            r, ok2 = measure_stack(args, other, max(20, args.steps // 4), max(5, args.warmup // 4), 0,
                                   0.0 if args.no_cpu else min(args.cpu_seconds, 4.0), False)
            ok = ok and ok2
            keep = {k: r[k] for k in ("ms_per_step", "achieved_tops", "config")}
            keep["images_per_s"] = r["value"]
            keep["roofline"] = {k: r["roofline"][k] for k in ("bound", "achieved", "peak", "unit", "frac", "dominant_kernel")}
            for k in ("cpu_baseline", "verified"):
                if k in r:
                    keep[k] = r[k]
            others[other] = keep
        line["other_workloads"] = others
    print(json.dumps(line), flush=True)
    if not ok:
        sys.exit(1)


if __name__ == "__main__":
    main()
