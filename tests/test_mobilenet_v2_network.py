"""A whole quantized MobileNet-v2 (52 convolutions of which 17 depthwise, ReLU6 as clamp activations, 10 residual sums
without activation, global average pooling, fully_connected) through the clDNN API against the CPU
oracle run layer by layer, bit for bit."""
import numpy as np
import pytest

from cldnn_amd import mobilenet_v2_net as mn
from oracle.networks import mobilenet_v2 as run_oracle


def test_layer_plan_shape():
    steps = mn.layer_plan()
    assert [s[0] for s in steps].count("conv") == 52 and [s[0] for s in steps].count("sum") == 10
    assert steps[-2:] == [("pool",), ("fc",)]
    sums = [s for s in steps if s[0] == "sum"]
    assert sums[0][1:] == ("b3", "b2_project", "b3_project") and sums[1][1:] == ("b5", "b4_project", "b5_project")
    assert sums[2][1:] == ("b6", "b5", "b6_project")  # the second sum of a group reads the first one


@pytest.mark.gpu
def test_mobilenet_v2_int8_network_matches_the_oracle():
    from cldnn_amd import api as cl
    eng = cl.engine()
    B = 2
    x = np.random.default_rng(17).integers(0, 256, (B, 3, 224, 224)).astype(np.uint8)
    params = mn.random_weights(seed=23)
    run_oracle(x, params, calibrate=True)
    topo = mn.topology(cl, eng, params, B)
    # linear points only: a watched clamp would stay a primitive of its own also in the optimised build
    watch = ["b1_project", "b3", "b7_project", "b10", "b14_project", "b17_project", "pool", "fc1000"]
    for optimize in (True, False):
        opts = cl.build_options(optimize_data=optimize, outputs=watch)
        plan = {n["id"]: n for n in cl.plan(topo, opts)}
        folded = [i for i, n in plan.items() if n["type"] == "convolution" and n.get("fused_activation") == cl.activation_func.clamp]
        if optimize:
            # every clamp is folded into the convolution before it; the residual sums have no activation: the reference
            # would leave them stand-alone, here they run inside their projection convolution with the int8 saturation of
            # the convolution's result kept (conv_saturate), except the two that are watched; every convolution up to
            # the classifier runs in the blocked layout
            assert len(folded) == 35 and not any(n["type"] == "activation" for n in plan.values())
            assert sorted(i for i, n in plan.items() if n["type"] == "eltwise") == ["b10_fsv16", "b3_fsv16"]
            fused = [n for i, n in plan.items() if "_fused_" in i]
            assert len(fused) == 8 and all(n["conv_saturate"] == 1 for n in fused)
            assert all(n["format"] == cl.format.fs_b_yx_fsv16 for n in plan.values() if n["type"] == "convolution" and not n.get("fully_connected"))
        else:
            assert folded == [] and sum(n["type"] == "activation" for n in plan.values()) == 35
        ref = run_oracle(x, params, folded=optimize)
        if optimize:
            assert 3 < np.abs(ref["b17_project"].astype(np.int32)).mean() < 100 and len(np.unique(ref["fc1000"])) > 50  # alive to the end
        net = cl.network(eng, topo, opts)
        net.set_input_data("input", cl.make_memory(eng, x))
        outs = net.execute()
        for name in watch:
            got = outs[name].get_memory().read()
            assert got.shape == ref[name].shape, name
            bad = int((got != ref[name]).sum())
            assert bad == 0, "%s (optimize_data=%s): %d of %d values differ" % (name, optimize, bad, got.size)
    # an engine without a memory pool also lets the fused sums write over their shortcuts (read / write pass): both
    # options on one node, same logits
    eng2 = cl.engine(enable_memory_pool=False)
    net = cl.network(eng2, mn.topology(cl, eng2, params, B), cl.build_options(optimize_data=True))
    both = [i for i in net.get_all_primitive_ids() if "_fused_" in i and net.get_primitive_info(i).get("second_input_in_output")
            and net.get_primitive_info(i).get("conv_saturate") == 1]
    assert len(both) == 10, both
    net.set_input_data("input", cl.make_memory(eng2, x))
    np.testing.assert_array_equal(net.execute()["fc1000"].get_memory().read(), run_oracle(x, params, folded=True)["fc1000"])


@pytest.mark.gpu
def test_mobilenet_v2_network_at_the_benchmark_batch_matches_the_oracle():
    """Batch 32: the rows of the tile table, the depthwise chains and the memory pool as the benchmark runs them; the
    oracle runs the first images.  One build with the logits as the only output (the production plan), one that also
    watches linear points along the way."""
    from cldnn_amd import api as cl
    eng = cl.engine()
    B, checked = 32, 2
    x = np.random.default_rng(61).integers(0, 256, (B, 3, 224, 224)).astype(np.uint8)
    params = mn.random_weights(seed=67)
    run_oracle(x[:2], params, calibrate=True)
    topo = mn.topology(cl, eng, params, B)
    ref = run_oracle(x[:checked], params, folded=True)
    for watch in (["fc1000"], ["b1_project", "b7_project", "b14_project", "b17_project", "fc1000"]):
        net = cl.network(eng, topo, cl.build_options(optimize_data=True, outputs=watch))
        kernels = {i: net.get_primitive_info(i).get("kernel", "") for i in net.get_all_primitive_ids()}
        assert sum(k.startswith("in the chain of") for k in kernels.values()) >= 10, "no depthwise chains at the benchmark batch"
        net.set_input_data("input", cl.make_memory(eng, x))
        outs = net.execute()
        for name in watch:
            got = outs[name].get_memory().read()[:checked]
            bad = int((got != ref[name]).sum())
            assert bad == 0, "%s (outputs %s): %d of %d values differ" % (name, watch, bad, got.size)
