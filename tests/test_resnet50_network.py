"""A whole quantized ResNet-50 (53 convolutions, 2 poolings, 16 residual sums, 1 fully_connected) through the clDNN
API against the CPU oracle run layer by layer, bit for bit, as written and with optimize_data."""
import numpy as np
import pytest

from cldnn_amd import resnet50_net as rn
from oracle import refconv as rc
from oracle.networks import resnet50 as run_oracle


BLOCKS = [s[1] for s in rn.layer_plan() if s[0] == "sum"]


def test_layer_plan_shape():
    steps = rn.layer_plan()
    assert sum(s[0] == "conv" for s in steps) == 53 and sum(s[0] == "sum" for s in steps) == 16
    assert steps[0][1]["name"] == "conv1" and steps[-1] == ("fc",)


def test_fused_and_stand_alone_sum_differ_only_where_the_convolution_saturates():
    """the property the two oracle forms rest on: (closing convolution, saturated to int8) + stand-alone sum equals the
    fused primitive wherever the convolution's result fits into int8"""
    r = np.random.default_rng(1)
    x = r.integers(0, 128, (1, 64, 6, 6)).astype(np.int8)
    w = r.integers(-127, 128, (256, 64, 1, 1)).astype(np.int8)
    bias, one = r.integers(-1000, 1001, 256).astype(np.int32), np.ones(256, np.float32)
    cal, ecal = np.full(256, 0.003, np.float32), r.uniform(0.4, 0.9, 256).astype(np.float32)
    sc = r.integers(-128, 128, (1, 256, 6, 6)).astype(np.int8)
    c = rc.conv(x, w, bias, wqf=one, calib=cal, out_dt="s8")
    fused = rc.conv(x, w, bias, wqf=one, calib=cal, out_dt="s8", eltw=sc, eltw_act="relu", eltw_calib=ecal)
    alone = rc.eltwise_sum(sc, c, calib=ecal, relu=True)
    inside = (c > -128) & (c < 127)
    assert 0.5 < inside.mean() < 0.999                      # both regions occur
    np.testing.assert_array_equal(fused[inside], alone[inside])
    assert (fused[~inside] != alone[~inside]).any()


@pytest.mark.gpu
def test_resnet50_int8_network_matches_the_oracle():
    from cldnn_amd import api as cl
    eng = cl.engine()
    B = 2
    x = np.random.default_rng(7).integers(0, 256, (B, 3, 224, 224)).astype(np.uint8)
    params = rn.random_weights(seed=11)
    run_oracle(x, params, fused=BLOCKS, calibrate=True)
    topo = rn.topology(cl, eng, params, B)
    # a watched sum is an output: it is neither fused nor shrunk.  The first list leaves the junction behind res2c to the
    # eltwise_shrinking / eltwise_remove_stride passes, the second one those behind res3d and res4f.
    for optimize, watch in ((True, ["pool1", "res2a", "res3d", "res4f", "res5c", "pool5", "fc1000"]),
                            (True, ["res2c", "res3a", "res4b", "res5a", "fc1000"]),
                            (False, ["pool1", "res2a", "res3d", "res4f", "res5c", "pool5", "fc1000"])):
        # optimize_data fuses a residual sum into its closing convolution unless the sum is itself an output; the plan says
        # which ones (node ids <convolution>_fused_<sum>), and the oracle follows it: the two forms differ where the
        # convolution's own result leaves the int8 range
        opts = cl.build_options(optimize_data=optimize, outputs=watch)
        plan = {n["id"]: n for n in cl.plan(topo, opts)}
        fused = [i.split("_fused_")[1] for i in plan if "_fused_" in i]
        assert sorted(fused) == (sorted(b for b in BLOCKS if b not in watch) if optimize else [])
        for junction, size in (("res2c", 28), ("res3d", 14), ("res4f", 7)):
            name = "%s_branch2c_fused_%s" % (junction, junction)
            if name in plan:  # the sum and the 3x3 convolution before it produce only what the stride-2 block behind them reads
                assert plan[name]["size"][2:] == [size, size] and plan[name]["eltw_stride"][2:] == [2, 2]
                assert plan[junction + "_branch2b"]["stride"][2:] == [2, 2]
        ref = run_oracle(x, params, fused=fused)
        assert 5 < np.abs(ref["res5c"].astype(np.int32)).mean() < 100 and len(np.unique(ref["fc1000"])) > 50  # alive to the end
        net = cl.network(eng, topo, opts)
        net.set_input_data("input", cl.make_memory(eng, x))
        outs = net.execute()
        for name in watch:
            got = outs[name].get_memory().read()
            assert got.shape == ref[name].shape, name
            bad = int((got != ref[name]).sum())
            assert bad == 0, "%s (optimize_data=%s): %d of %d values differ" % (name, optimize, bad, got.size)


@pytest.mark.gpu
def test_memory_pool_shares_buffers_without_changing_results():
    """engine option enable_memory_pool (reference src/memory_pool.cpp): intermediate tensors of identical layout share
    buffers once their consumers are done; same results, less device memory"""
    from cldnn_amd import api as cl
    B = 2
    x = np.random.default_rng(3).integers(0, 256, (B, 3, 224, 224)).astype(np.uint8)
    params = rn.random_weights(seed=5)
    run_oracle(x, params, fused=BLOCKS, calibrate=True)
    used, logits = {}, {}
    for pool in (True, False):
        eng = cl.engine(enable_memory_pool=pool)
        base = eng.get_temp_used_device_memory_size()
        net = cl.network(eng, rn.topology(cl, eng, params, B), cl.build_options(optimize_data=True))
        # without a pool the read / write pass (reference prepare_primitive_fusing.cpp:468-534) lets a fused closer write
        # over its shortcut when the two have one layout and nothing reads the shortcut later: every block but the
        # three whose sum was shrunk to the stride of the block behind it
        in_place = sorted(i.split("_fused_")[1] for i in net.get_all_primitive_ids()
                          if "_fused_" in i and net.get_primitive_info(i).get("second_input_in_output"))
        assert in_place == ([] if pool else sorted(b for b in BLOCKS if b not in ("res2c", "res3d", "res4f"))), in_place
        # convolution chains: the 3x3, the closer with its sum and the next block's opener of stage 2 are one launch
        # (not where the closer writes over its shortcut, i.e. not without a pool)
        kernels = {i: net.get_primitive_info(i).get("kernel", "") for i in net.get_all_primitive_ids()}
        followers = sorted(i for i, k in kernels.items() if k.startswith("in the chain of"))
        if pool:
            # (the third chain's closer reads its shortcut with the stride of the block behind it)
            assert followers == ["res2a_branch2c_fused_res2a", "res2b_branch2a", "res2b_branch2c_fused_res2b", "res2c_branch2a",
                                 "res2c_branch2c_fused_res2c"], followers
            assert kernels["res2a_branch2b"].startswith("conv_chain<3 stages") and kernels["res2b_branch2a"] == "in the chain of res2a_branch2b"
        # a projection block's shortcut convolution and its opening 1x1 read the same tensor: one launch for the two
        # (not where the closer writes over the shortcut, which then needs a buffer of its own)
        paired = sorted(i for i in net.get_all_primitive_ids() if "launched_by" in net.get_primitive_info(i))
        assert paired == (["res%da_branch2a" % s for s in (2, 3, 4, 5)] if pool else []), paired
        net.set_input_data("input", cl.make_memory(eng, x))
        for _ in range(2):  # a second run reuses the same buffers
            logits[pool] = net.execute()["fc1000"].get_memory().read()
        used[pool] = eng.get_temp_used_device_memory_size() - base
        del net
    np.testing.assert_array_equal(logits[True], logits[False])
    np.testing.assert_array_equal(logits[True], run_oracle(x, params, fused=BLOCKS)["fc1000"])
    # 26 MB of either figure are weights; without a pool the 13 closers that write over their shortcuts save nearly as
    # much as the pool does.  With the pool the two convolution chains of stage 2 (pooled engines only: a closer that
    # writes over its shortcut is not chained) cost one 64-feature tensor each, because a chain's last member is written
    # by the launch that still reads the head's input and cannot take that buffer over; and the four buffers that hold a
    # projection together with the block's opening 1x1 have layouts nothing else in the network has, so they are never
    # taken over (4 MB at this batch)
    assert max(used.values()) < 43e6 and used[True] < 1.12 * used[False], used


@pytest.mark.gpu
def test_shortcut_convolutions_on_the_second_stream():
    """engine option enable_parallelisation: a convolution whose only user comes later in the order (the projection
    shortcut of res2a / res3a / res4a / res5a) runs on the engine's second stream beside the branch; same results, with
    and without the memory pool, run after run"""
    from cldnn_amd import api as cl
    B = 2
    params = rn.random_weights(seed=13)
    run_oracle(np.random.default_rng(1).integers(0, 256, (B, 3, 224, 224)).astype(np.uint8), params, fused=BLOCKS, calibrate=True)
    watch = ["res2a", "res3b", "res5a", "fc1000"]
    xs = [np.random.default_rng(seed).integers(0, 256, (B, 3, 224, 224)).astype(np.uint8) for seed in (2, 3)]
    refs = None
    for pool in (True, False):
        eng = cl.engine(enable_parallelisation=True, enable_memory_pool=pool)
        topo = rn.topology(cl, eng, params, B)
        opts = cl.build_options(optimize_data=True, outputs=watch)
        if refs is None:
            fused = [n["id"].split("_fused_")[1] for n in cl.plan(topo, opts) if "_fused_" in n["id"]]
            refs = [run_oracle(x, params, fused=fused) for x in xs]
        net = cl.network(eng, topo, opts)
        side = [i for i in net.get_all_primitive_ids() if "_branch" in i and net.get_primitive_info(i).get("stream") == 1]
        assert side == ["res2a_branch1", "res3a_branch1", "res4a_branch1", "res5a_branch1"]
        # whatever launch does the work of a shortcut's reader waits for the shortcut: the reader itself, or the head of
        # the chain the reader is a member of (res2a_branch2b launches res2a_branch2c + sum as well)
        for s in side:
            waiting = []
            for i in net.get_all_primitive_ids():
                info = net.get_primitive_info(i)
                if s in info.get("waits_for", []):
                    waiting.append((i, info.get("kernel", "")))
            assert waiting, "nothing waits for %s" % s
            assert all(not k.startswith("in the chain of") for _, k in waiting), waiting
        chained = [i for i in net.get_all_primitive_ids() if net.get_primitive_info(i).get("kernel", "").startswith("in the chain of")]
        if any(i.startswith("res2a_branch2c") for i in chained):
            assert "res2a_branch1" in net.get_primitive_info("res2a_branch2b").get("waits_for", [])
        for k in (0, 1, 0):
            net.set_input_data("input", cl.make_memory(eng, xs[k]))
            outs = net.execute()
            for name in watch:
                np.testing.assert_array_equal(outs[name].get_memory().read(), refs[k][name], err_msg="%s pool=%s input %d" % (name, pool, k))


@pytest.mark.gpu
def test_resnet50_network_at_the_benchmark_batch_matches_the_oracle():
    """Batch 32 is where the tile table, the paired launches, the chains and the memory pool take the rows and sizes the
    benchmark runs (at batch 2 they take others).  The production plan has one output, the logits, which depend on every
    layer; a second build watches the block ends to say where a difference starts.  The oracle runs the first images."""
    from cldnn_amd import api as cl
    eng = cl.engine()
    B, checked = 32, 2
    x = np.random.default_rng(57).integers(0, 256, (B, 3, 224, 224)).astype(np.uint8)
    params = rn.random_weights(seed=59)
    run_oracle(x[:2], params, fused=BLOCKS, calibrate=True)
    topo = rn.topology(cl, eng, params, B)
    for watch in (["fc1000"], ["res2c", "res3d", "res4f", "res5c", "fc1000"]):
        opts = cl.build_options(optimize_data=True, outputs=watch)
        fused = [n["id"].split("_fused_")[1] for n in cl.plan(topo, opts) if "_fused_" in n["id"]]
        ref = run_oracle(x[:checked], params, fused=fused)
        net = cl.network(eng, topo, opts)
        kernels = {i: net.get_primitive_info(i).get("kernel", "") for i in net.get_all_primitive_ids()}
        assert sum(k.startswith("in the chain of") for k in kernels.values()) >= 2, "no chains at the benchmark batch"
        assert not any(k.startswith("conv_ref") for k in kernels.values()), kernels
        net.set_input_data("input", cl.make_memory(eng, x))
        outs = net.execute()
        for name in watch:
            got = outs[name].get_memory().read()[:checked]
            bad = int((got != ref[name]).sum())
            assert bad == 0, "%s (outputs %s): %d of %d values differ" % (name, watch, bad, got.size)
