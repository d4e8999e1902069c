"""A whole quantized VGG-16 (13 convolutions, 5 max poolings, 3 fully_connected layers of which the first reads a 7x7
plane: K = 25088) through the clDNN API against the CPU oracle run layer by layer, bit for bit."""
import numpy as np
import pytest

from cldnn_amd import vgg16_net as vg
from oracle.networks import vgg16 as run_oracle


def test_layer_plan_shape():
    steps = vg.layer_plan()
    assert [s[0] for s in steps].count("conv") == 13 and [s[0] for s in steps].count("pool") == 5
    assert [s[1] for s in steps if s[0] == "fc"] == ["fc6", "fc7", "fc8"] and steps[-3][3:6] == (512, 7, 4096)


@pytest.mark.gpu
def test_vgg16_int8_network_matches_the_oracle():
    from cldnn_amd import api as cl
    eng = cl.engine()
    B = 2
    x = np.random.default_rng(41).integers(0, 256, (B, 3, 224, 224)).astype(np.uint8)
    params = vg.random_weights(seed=43)
    ref = run_oracle(x, params, calibrate=True)
    assert 5 < np.abs(ref["pool5"].astype(np.int32)).mean() < 100 and len(np.unique(ref["fc8"])) > 50  # alive to the end
    topo = vg.topology(cl, eng, params, B)
    watch = ["pool1", "conv5", "pool3", "pool5", "fc6", "fc7", "fc8"]
    for optimize in (True, False):
        opts = cl.build_options(optimize_data=optimize, outputs=watch)
        if optimize:
            plan = {n["id"]: n for n in cl.plan(topo, opts)}
            # the pooling layers stay in the blocked layout between the convolutions
            assert all(plan[i]["format"] == cl.format.fs_b_yx_fsv16 for i in ("pool2", "pool4", "conv6", "conv12"))
        net = cl.network(eng, topo, opts)
        net.set_input_data("input", cl.make_memory(eng, x))
        outs = net.execute()
        for name in watch:
            got = outs[name].get_memory().read()
            assert got.reshape(ref[name].shape).shape == ref[name].shape, name
            bad = int((got.reshape(ref[name].shape) != ref[name]).sum())
            assert bad == 0, "%s (optimize_data=%s): %d of %d values differ" % (name, optimize, bad, got.size)


@pytest.mark.gpu
def test_vgg16_network_at_the_benchmark_batch_matches_the_oracle():
    """Batch 16: the rows of the tile table the benchmark runs (the large-tile rows only apply from 50 000 pixels on); the
    oracle runs the first image."""
    from cldnn_amd import api as cl
    eng = cl.engine()
    B, checked = 16, 1
    x = np.random.default_rng(71).integers(0, 256, (B, 3, 224, 224)).astype(np.uint8)
    params = vg.random_weights(seed=73)
    run_oracle(x[:1], params, calibrate=True)
    ref = run_oracle(x[:checked], params)
    topo = vg.topology(cl, eng, params, B)
    for watch in (["fc8"], ["conv5", "pool3", "conv10", "pool5", "fc8"]):
        net = cl.network(eng, topo, cl.build_options(optimize_data=True, outputs=watch))
        net.set_input_data("input", cl.make_memory(eng, x))
        outs = net.execute()
        for name in watch:
            got = outs[name].get_memory().read()
            got = got.reshape((B,) + ref[name].shape[1:])[:checked]
            bad = int((got != ref[name]).sum())
            assert bad == 0, "%s (outputs %s): %d of %d values differ" % (name, watch, bad, got.size)
