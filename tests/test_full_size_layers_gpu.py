"""Every distinct layer of the five benchmark configurations at its REAL batch size against the oracle.

The row of the tile-config table depends on the pixel count, so the kernels production uses at batch 32 / 16 / 1 are
not the ones the small-shape tests reach.  Here each distinct layer signature is built exactly as bench.py builds it
(same seeded data, same descriptors, same chain grouping), run once at full size, and the first image(s) of its
output are compared with the oracle bit for bit (a convolution is independent per image).  The kernels the committed
profiles name as dominant are asserted by name.

The benchmark's calibration factors saturate most outputs (about half are ReLU zeros, most of the rest 127), so a second
test runs every signature with factors that spread the outputs over the int8 range, and compares the raw int32
accumulators of the first image as well."""
import numpy as np
import pytest

import bench
from cldnn_amd import hip, workloads

pytestmark = pytest.mark.gpu

CONFIGS = {  # workload -> (layers, batch, residual fused, images compared)
    "resnet50_b32_fused": (workloads.resnet50(), 32, True, 2),
    "resnet50_b1": (workloads.resnet50(), 1, False, 1),
    "vgg16_b16": (workloads.vgg16(), 16, False, 1),
    "mobilenet_v2_b32": (workloads.mobilenet_v2(), 32, False, 2),
    "c1": ([workloads._layer("c1", 64, 64, 3, 1, 1, 56)], 1, False, 1),
}

# kernels the per-layer tables under profiles/ show for these layers (kernel family and row of the tile table)
EXPECTED = {
    ("resnet50_b32_fused", "conv1"): "conv_stream<stem_p64",
    ("resnet50_b32_fused", "res2a_branch2b"): "conv_chain<3 stages",
    ("resnet50_b32_fused", "res2c_branch2b"): "conv_chain<2 stages",
    ("resnet50_b32_fused", "res3a_branch2b"): "conv_bdir<bdir_p128_f64",
    ("resnet50_b32_fused", "res4a_branch2b"): "conv_bdir<bdir_p64_f64",
    ("resnet50_b32_fused", "res4a_branch2c"): "conv_wsl<wsl_p64",
    ("resnet50_b32_fused", "res5a_branch2b"): "conv_bdir<bdir_k2_p64_f64",
    ("resnet50_b32_fused", "res2a_branch1|1"): "conv_stream<stream_p32",
    ("resnet50_b32_fused", "res4a_branch1|1"): "conv_mfma<p64_f128",
    ("resnet50_b32_fused", "res5a_branch1|1"): "conv_mfma<p64_f128",
    ("resnet50_b32_fused", "res3a_branch2c"): "conv_stream<stream_p32",
    ("resnet50_b32_fused", "res3b_branch2a"): "conv_wsl<wsl_p64",
    ("vgg16_b16", "conv1"): "conv_stream<stem_p32",
    ("vgg16_b16", "conv2"): "conv_wsl<wsl_p128",
    ("vgg16_b16", "conv4"): "conv_wsl<wsl_p128",
    ("vgg16_b16", "conv8"): "conv_bdir<bdir_p256_f64",
    ("vgg16_b16", "conv11"): "conv_bdir<bdir_k2_p128_f64",
    ("vgg16_b16", "conv6"): "conv_bdir<bdir_p256_f128",
    ("vgg16_b16", "conv9"): "conv_bdir<bdir_p128_f128",
    ("mobilenet_v2_b32", "b2_dw"): "conv_dwchain<3 stages",
    ("mobilenet_v2_b32", "b17_dw"): "conv_dw3x3_kernel",
    ("c1", "c1"): "conv_bdir<bdir_p64_f64",
}


def signature(group, fuse):
    return tuple((l["ifm"], l["ofm"], l["k"], l["stride"], l["pad"], l["in_hw"], l["groups"], l["act"], bool(l["closes_block"] and fuse))
                 for l in group)


def cases():
    out = []
    for wl, (layers, batch, fuse, images) in CONFIGS.items():
        seen = set()
        for g in bench.chain_groups(layers, fuse):
            s = signature(g, fuse)
            if s in seen and (wl, g[0]["name"]) not in EXPECTED:
                continue
            seen.add(s)
            out.append(pytest.param(wl, [dict(l) for l in g], id="%s-%s" % (wl, g[0]["name"] + ("+%d" % (len(g) - 1) if len(g) > 1 else ""))))
        # two convolutions of one input in one launch (a projection and the block's opening 1x1)
        for a, b in zip(layers, layers[1:]):
            if b.get("shares_input") and not (fuse and (a["closes_block"] or b["closes_block"])):
                out.append(pytest.param(wl, [dict(a), dict(b)], id="%s-%s|1" % (wl, a["name"])))
    return out


@pytest.fixture(scope="module")
def eng():
    e = hip.Engine()
    yield e
    e.close()


@pytest.mark.parametrize("wl,group", cases())
def test_layer_at_its_real_batch_matches_the_oracle(eng, wl, group):
    _, batch, fuse, images = CONFIGS[wl]
    stack = bench.build_stack(eng, group, batch, fuse)
    head = stack[0]
    name = head.info.kernel_name.decode()
    assert not name.startswith("conv_ref"), name  # every layer of the configurations runs on a fast kernel
    pair = len(group) == 2 and bool(group[1].get("shares_input"))
    if pair and batch > 1:
        assert head.sibling is stack[1], "the two convolutions of one input run as two launches"
    for L in stack:
        # a member of a group that the library did not take as a chain is a launch of its own, on its own row
        if L is not head and (L.follows or pair):
            continue
        want = EXPECTED.get((wl, L.spec["name"] + ("|1" if pair else "")))
        if want:
            got = L.info.kernel_name.decode()
            assert got.startswith(want), "%s runs on %s, the profile shows %s" % (L.spec["name"], got, want)
    bench.run_step(bench.launches(stack))
    eng.finish()
    _, _, checked, mismatches = bench.cpu_pass(eng, stack, min(images, batch), verify=True)
    kept = [L for L in stack if L.kept]
    assert checked == sum(min(images, batch) * L.spec["ofm"] * L.spec["out_hw"] ** 2 for L in kept)
    assert mismatches == 0, "%d of %d outputs differ from the oracle (%s)" % (mismatches, checked, name)
    bench.release_stack(stack)


@pytest.mark.parametrize("wl,group", cases())
def test_layer_at_its_real_batch_with_spread_outputs_and_accumulators(eng, wl, group):
    from oracle import refconv as rc
    _, batch, fuse, images = CONFIGS[wl]
    # outputs, launched as production launches them (chains, pairs), with factors under which a wrong sum shows
    stack = bench.build_stack(eng, group, batch, fuse, calibration="spread")
    bench.run_step(bench.launches(stack))
    eng.finish()
    _, _, checked, mismatches = bench.cpu_pass(eng, stack, 1, verify=True)
    assert checked > 0 and mismatches == 0, "%d of %d outputs differ from the oracle" % (mismatches, checked)
    for L in stack:
        if L.kept and L.spec["act"] == "relu" and not L.fused:
            got = hip.download(eng, L.out)[:1]
            inside = np.count_nonzero((got > 0) & (got < 127))
            assert inside > 0.2 * got.size, "the outputs of %s do not spread over the int8 range" % L.spec["name"]
    bench.release_stack(stack)
    # int32 accumulators of the first image, every layer a launch of its own on the row production picks at this batch
    stack = bench.build_stack(eng, group, batch, fuse, chains=False, calibration="spread")
    for L in stack:
        l = L.spec
        acc = L.conv.accumulators(L.xin)[:1]
        _, ref_acc = rc.conv(L.x[:1], L.w, None, wqf=L.wqf, calib=L.calib, stride=(l["stride"],) * 2, pad=(l["pad"],) * 2,
                             groups=l["groups"], out_dt="s8", want_acc=True)
        assert acc.shape == ref_acc.shape
        bad = int(np.count_nonzero(acc != ref_acc))
        assert bad == 0, "%d of %d accumulators of %s differ (%s)" % (bad, acc.size, l["name"], L.info.kernel_name.decode())
    bench.release_stack(stack)


def vgg_layer(name):
    return [dict(l) for l in workloads.vgg16() if l["name"] == name]


@pytest.mark.parametrize("row", ["halo_p256_f128", "halo_p512_f128"])
@pytest.mark.parametrize("name", ["conv4", "conv6", "conv9"])
def test_staged_patch_rows_at_full_size(eng, name, row):
    """The two rows that only a tuning cache or tile_override selects, on VGG-16's layers at the benchmark batch: one
    patch request per step and two, 128 to 512 features, several feature tiles per position tile."""
    L_ = hip.lib()
    names = [L_.cldnn_hip_tile_config_name(i).decode() for i in range(L_.cldnn_hip_tile_config_count())]
    stack = bench.build_stack(eng, vgg_layer(name), 16, False, tile=names.index(row) + 1, calibration="spread")
    kernel = stack[0].info.kernel_name.decode()
    if not kernel.startswith("conv_halo<" + row):
        bench.release_stack(stack)
        pytest.skip("%s does not take %s (%s runs it)" % (row, name, kernel))
    bench.run_step(bench.launches(stack))
    eng.finish()
    _, _, checked, mismatches = bench.cpu_pass(eng, stack, 1, verify=True)
    assert checked > 0 and mismatches == 0, "%d of %d outputs differ from the oracle (%s)" % (mismatches, checked, kernel)
    bench.release_stack(stack)
