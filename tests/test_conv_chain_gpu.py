"""cldnn_hip_conv_chain_*: two or three convolutions in one launch against the oracle run layer by layer.

A chain must give the bits the separate convolutions give: the oracle computes stage after stage, each on the int8
tensor the stage before it produced.  Covered: the tail of a ResNet bottleneck (3x3 -> 1x1 expansion with fused
residual -> next 1x1 reduction), its two-stage form, the unfused form, results kept and not kept, u8 and s8 inputs,
pixel counts that do not fill the last granule, padded output buffers, and the refusals."""
import numpy as np
import pytest

from cldnn_amd import hip
from oracle import refconv as rc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def eng():
    e = hip.Engine()
    yield e
    e.close()


def layer(r, ifm, ofm, k, in_dt):
    w = r.integers(-127, 128, (ofm, ifm, k, k)).astype(np.int8)
    bias = r.integers(-1000, 1001, ofm).astype(np.int32)
    wqf = np.ones(ofm, np.float32)
    rms = 147.4 if in_dt == np.uint8 else 40.0
    calib = (40.0 / (np.sqrt(ifm * k * k) * rms * 73.3) * r.uniform(0.5, 2.0, ofm)).astype(np.float32)
    return w, bias, wqf, calib


def bottleneck_tail(eng, seed, B, H, W, mid, stages, fused, in_dt=np.uint8, keep=None, out_pad=(0, 0)):
    """builds descriptors + data of 3x3(mid->mid) -> 1x1(mid->4mid)[+residual] [-> 1x1(4mid->mid)], returns what both
    the chain and the oracle need"""
    r = np.random.default_rng(seed)
    lo, hi = (0, 256) if in_dt == np.uint8 else (-128, 128)
    x = r.integers(lo, hi, (B, mid, H, W)).astype(in_dt)
    shapes = [(mid, mid, 3), (mid, 4 * mid, 1), (4 * mid, mid, 1)][:stages]
    xin = hip.upload(eng, x, "fs_b_yx_fsv16", (1, 1))
    spec, prev_t = [], xin.tensor
    ref_in, refs = x, []
    bufs = []
    for k, (ifm, ofm, fk) in enumerate(shapes):
        w, bias, wqf, calib = layer(r, ifm, ofm, fk, in_dt if k == 0 else np.int8)
        is_fused = fused and k == 1
        eltw = ecal = ebuf = None
        kw = dict(stride=(1, 1), pad=(fk // 2,) * 2, bias_dt=hip.I32, has_wqf=True, has_calib=True, out_pad=out_pad if k == 1 else (0, 0))
        okw = dict(stride=(1, 1), pad=(fk // 2,) * 2, out_dt="s8")
        if is_fused:
            eltw = r.integers(-128, 128, (B, ofm, H, W)).astype(np.int8)
            ecal = r.uniform(0.25, 1.0, ofm).astype(np.float32)
            ebuf = hip.upload(eng, eltw, "fs_b_yx_fsv16")
            kw.update(act="none", eltw_t=ebuf.tensor, eltw_act="relu", has_eltw_calib=True)
            okw.update(act="none", eltw=eltw, eltw_act="relu", eltw_calib=ecal)
        else:
            kw.update(act="relu")
            okw.update(act="relu")
        d = hip.conv_desc(prev_t, w.shape, "s8", **kw)
        spec.append((d, w, bias, wqf, calib, ecal))
        bufs.append((hip.Buffer(eng, d.output), ebuf))
        ref = rc.conv(ref_in, w, bias, wqf=wqf, calib=calib, **okw)
        refs.append(ref)
        ref_in, prev_t = ref, hip.Tensor.make(hip.S8, hip.FS_B_YX_FSV16, B, ofm, H, W)  # the next stage reads a dense tensor
    return xin, spec, bufs, refs


@pytest.mark.parametrize("in_dt", [np.uint8, np.int8], ids=["u8", "s8"])
@pytest.mark.parametrize("stages,fused", [(3, True), (2, True), (3, False), (2, False)], ids=["3fused", "2fused", "3plain", "2plain"])
def test_bottleneck_tail_chain_matches_the_oracle(eng, stages, fused, in_dt):
    mid = 64
    B, H, W = 3, 13, 11  # 429 pixels: the last granule of 32 is partly filled, granules span rows and images
    keep = [False] + [True] * (stages - 1)
    xin, spec, bufs, refs = bottleneck_tail(eng, 21, B, H, W, mid, stages, fused, in_dt)
    ch = hip.ConvChain(eng, spec, keep)
    info = ch.info()
    assert b"conv_chain" in info.kernel_name
    assert info.ops == sum(2 * r.size * s[1].shape[1] * s[1].shape[2] * s[1].shape[3] for r, s in zip(refs, spec))
    outs = [b if k else None for (b, _), k in zip(bufs, keep)]
    ch.enqueue(xin, outs, [e for _, e in bufs])
    eng.finish()
    for k in range(stages):
        if keep[k]:
            got = hip.download(eng, bufs[k][0])
            bad = np.argwhere(got != refs[k])
            assert bad.size == 0, "stage %d: %d of %d differ, first at %s" % (k, len(bad), got.size, bad[0])
    # the same chain with every result written, into buffers that were dirty
    ch2 = hip.ConvChain(eng, spec, None)
    for b, _ in bufs:
        b.write_raw(np.full(b.nbytes, 0x55, np.uint8))
    ch2.enqueue(xin, [b for b, _ in bufs], [e for _, e in bufs])
    eng.finish()
    for k in range(stages):
        assert np.array_equal(hip.download(eng, bufs[k][0]), refs[k]), "stage %d (all kept)" % k
    ch.close(), ch2.close(), xin.close()
    for b, e in bufs:
        b.close()
        if e is not None:
            e.close()


def test_chain_equals_separate_convolutions_on_a_full_size_slice(eng):
    """56x56 like the first ResNet stage, two images: the chain against the three convolution objects run one by one"""
    B, H, W, mid = 2, 56, 56, 64
    xin, spec, bufs, refs = bottleneck_tail(eng, 5, B, H, W, mid, 3, True)
    ch = hip.ConvChain(eng, spec, [False, True, True])
    ch.enqueue(xin, [None, bufs[1][0], bufs[2][0]], [e for _, e in bufs])
    eng.finish()
    assert np.array_equal(hip.download(eng, bufs[1][0]), refs[1])
    assert np.array_equal(hip.download(eng, bufs[2][0]), refs[2])
    # one by one through cldnn_hip_conv_enqueue
    src = xin
    for k, (d, w, bias, wqf, calib, ecal) in enumerate(spec):
        c = hip.Conv(eng, d, w, bias, wqf, calib, ecal)
        out = hip.Buffer(eng, d.output)
        c.enqueue(src, out, bufs[k][1])
        eng.finish()
        assert np.array_equal(hip.download(eng, out), refs[k])
        c.close()
        src = out
    ch.close()


@pytest.mark.parametrize("B,H,W", [(3, 14, 14), (2, 56, 56)], ids=["14x14", "56x56"])
def test_chain_with_a_strided_head_and_a_sub_sampled_shortcut(eng, B, H, W):
    """the last block of a ResNet stage after eltwise_remove_stride: the 3x3 takes the stride of the block behind it, the
    closing 1x1 adds a shortcut that it reads with that stride (fused_conv_eltwise eltw_stride)"""
    r = np.random.default_rng(77)
    mid = 64
    x = r.integers(0, 256, (B, mid, H, W)).astype(np.uint8)
    xin = hip.upload(eng, x, "fs_b_yx_fsv16", (1, 1))
    w0, b0, q0, c0 = layer(r, mid, mid, 3, np.uint8)
    w1, b1, q1, c1 = layer(r, mid, 4 * mid, 1, np.int8)
    OH, OW = (H + 1) // 2, (W + 1) // 2
    shortcut = r.integers(-128, 128, (B, 4 * mid, H, W)).astype(np.int8)   # full resolution, read at every second pixel
    ecal = r.uniform(0.25, 1.0, 4 * mid).astype(np.float32)
    ebuf = hip.upload(eng, shortcut, "fs_b_yx_fsv16")
    d0 = hip.conv_desc(xin.tensor, w0.shape, "s8", stride=(2, 2), pad=(1, 1), bias_dt=hip.I32, has_wqf=True, has_calib=True, act="relu")
    mid_t = hip.Tensor.make(hip.S8, hip.FS_B_YX_FSV16, B, mid, OH, OW)
    d1 = hip.conv_desc(mid_t, w1.shape, "s8", bias_dt=hip.I32, has_wqf=True, has_calib=True, act="none", eltw_t=ebuf.tensor, eltw_act="relu",
                       has_eltw_calib=True, eltw_stride=(2, 2))
    ref0 = rc.conv(x, w0, b0, wqf=q0, calib=c0, stride=(2, 2), pad=(1, 1), out_dt="s8", act="relu")
    ref1 = rc.conv(ref0, w1, b1, wqf=q1, calib=c1, out_dt="s8", act="none", eltw=shortcut, eltw_act="relu", eltw_calib=ecal, eltw_stride=(2, 2))
    assert ref1.shape == (B, 4 * mid, OH, OW)
    ch = hip.ConvChain(eng, [(d0, w0, b0, q0, c0, None), (d1, w1, b1, q1, c1, ecal)], [False, True])
    out = hip.Buffer(eng, d1.output)
    ch.enqueue(xin, [None, out], [None, ebuf])
    eng.finish()
    got = hip.download(eng, out)
    bad = np.argwhere(got != ref1)
    assert bad.size == 0, "%d of %d differ, first at %s" % (len(bad), got.size, bad[0])
    ch.close(), xin.close(), out.close(), ebuf.close()


def test_chain_refusals(eng):
    xin, spec, bufs, refs = bottleneck_tail(eng, 9, 1, 8, 8, 64, 3, True)
    # a second stage that is not 1x1
    d3 = hip.conv_desc(hip.Tensor.make(hip.S8, hip.FS_B_YX_FSV16, 1, 64, 8, 8, 1, 1), (64, 64, 3, 3), "s8", pad=(1, 1), bias_dt=hip.I32,
                       has_wqf=True, has_calib=True, act="relu")
    bad = [spec[0], (d3,) + spec[0][1:]]
    with pytest.raises(hip.HipError) as err:
        hip.ConvChain(eng, bad)
    assert err.value.status == -6 and "chain" in str(err.value)
    # the last stage must be kept; a kept stage needs a buffer
    with pytest.raises(hip.HipError):
        hip.ConvChain(eng, spec, [False, True, False])
    ch = hip.ConvChain(eng, spec, [False, True, True])
    with pytest.raises(hip.HipError):
        ch.enqueue(xin, [None, None, bufs[2][0]], [e for _, e in bufs])
    with pytest.raises(hip.HipError):
        ch.enqueue(xin, [None, bufs[1][0], bufs[2][0]], None)  # the fused stage has no second input
    ch.close()
    # a chain of one
    with pytest.raises(hip.HipError):
        hip.ConvChain(eng, spec[:1])
    # 128 mid features: the weights of the three stages (275 KB) do not fit into LDS
    xin, spec, bufs, refs = bottleneck_tail(eng, 9, 1, 8, 8, 128, 3, True)
    with pytest.raises(hip.HipError) as err:
        hip.ConvChain(eng, spec, [False, True, True])
    assert err.value.status == -6 and "LDS" in str(err.value)


# ------------------------------------------------------------------ depthwise chains (MobileNet blocks)
def relu6_layer(r, ofm, ifm_g, k, act):
    """factors as the benchmark's MobileNet stack has them: a clamp{0, 6} acts on the dequantised value"""
    w = r.integers(-127, 128, (ofm, ifm_g, k, k)).astype(np.int8)
    bias = r.integers(-1000, 1001, ofm).astype(np.int32)
    if act == "relu6":
        sig = np.sqrt(ifm_g * k * k) * 100.0 * 73.3
        wqf = (3.0 / sig * r.uniform(0.5, 2.0, ofm)).astype(np.float32)
        calib = np.full(ofm, 127.0 / 6.0, np.float32)
        kw = dict(act="clamp", act_m=0.0, act_n=6.0)
    else:
        wqf = np.ones(ofm, np.float32)
        calib = (40.0 / (np.sqrt(ifm_g * k * k) * 60.0 * 73.3) * r.uniform(0.5, 2.0, ofm)).astype(np.float32)
        kw = dict(act="none")
    return w, bias, wqf, calib, kw


@pytest.mark.parametrize("in_dt", [np.uint8, np.int8], ids=["u8", "s8"])
@pytest.mark.parametrize("mid,proj,stride,stages", [(32, 16, 1, 3), (96, 24, 2, 3), (144, 32, 1, 3), (192, 64, 2, 3), (384, 64, 1, 3),
                                                    (144, 24, 1, 2)],
                         ids=["b1", "b2_s2", "b4", "b7_s2", "b8", "two_stages"])
def test_depthwise_chain_matches_the_oracle(eng, mid, proj, stride, stages, in_dt):
    """depthwise 3x3 -> 1x1 projection -> 1x1 expansion of the next block in one launch, against the three
    convolutions of the oracle; feature counts that do not fill slices of 64 (or, for the projection, of 16), stride 2,
    pixel counts that do not fill a 64-pixel granule, every result kept and only the needed ones"""
    r = np.random.default_rng(33)
    B, H, W = 3, 13, 10
    OH, OW = (H + 2 - 3) // stride + 1, (W + 2 - 3) // stride + 1
    lo, hi = (0, 256) if in_dt == np.uint8 else (-128, 128)
    x = r.integers(lo, hi, (B, mid, H, W)).astype(in_dt)
    shapes = [(mid, 1, 3, "relu6", mid), (proj, mid, 1, "none", 1), (6 * proj, proj, 1, "relu6", 1)][:stages]
    xin = hip.upload(eng, x, "fs_b_yx_fsv16", (1, 1))
    spec, refs, bufs = [], [], []
    prev_t, ref_in = xin.tensor, x
    for k, (ofm, ifm_g, fk, act, groups) in enumerate(shapes):
        w, bias, wqf, calib, akw = relu6_layer(r, ofm, ifm_g, fk, act)
        s = stride if k == 0 else 1
        d = hip.conv_desc(prev_t, w.shape, "s8", stride=(s, s), pad=(fk // 2,) * 2, groups=groups, bias_dt=hip.I32, has_wqf=True,
                          has_calib=True, **akw)
        spec.append((d, w, bias, wqf, calib, None))
        bufs.append(hip.Buffer(eng, d.output))
        ref = rc.conv(ref_in, w, bias, wqf=wqf, calib=calib, stride=(s, s), pad=(fk // 2,) * 2, groups=groups, out_dt="s8", **akw)
        refs.append(ref)
        ref_in, prev_t = ref, hip.Tensor.make(hip.S8, hip.FS_B_YX_FSV16, B, ofm, OH, OW)
    for keep in ([False] + [True] * (stages - 1), None):
        ch = hip.ConvChain(eng, spec, keep)
        assert b"conv_dwchain" in ch.info().kernel_name
        for b in bufs:
            b.write_raw(np.full(b.nbytes, 0x55, np.uint8))
        ch.enqueue(xin, [b if (keep is None or keep[k]) else None for k, b in enumerate(bufs)])
        eng.finish()
        for k in range(stages):
            if keep is None or keep[k]:
                got = hip.download(eng, bufs[k])
                bad = np.argwhere(got != refs[k])
                assert bad.size == 0, "stage %d: %d of %d differ, first at %s" % (k, len(bad), got.size, bad[0])
        ch.close()
    assert len(np.unique(refs[-1])) > 8  # the data does exercise the requantisation
    xin.close()
    for b in bufs:
        b.close()


@pytest.mark.parametrize("saturate,eltw_dt", [(0, np.int8), (1, np.int8), (0, np.uint8)], ids=["sum", "sum_saturated", "sum_u8"])
def test_depthwise_chain_with_the_blocks_sum_on_the_projection(eng, saturate, eltw_dt):
    """MobileNet block with a shortcut: depthwise 3x3 -> 1x1 projection + residual sum (no activation; with the
    convolution's own int8 saturation kept or not) -> next expansion; the projection's compile-time form of the sum"""
    r = np.random.default_rng(57)
    B, H, W, mid, proj = 2, 14, 9, 192, 32
    x = r.integers(0, 256, (B, mid, H, W)).astype(np.uint8)
    xin = hip.upload(eng, x, "fs_b_yx_fsv16", (1, 1))
    lo, hi = (0, 256) if eltw_dt == np.uint8 else (-128, 128)
    e = r.integers(lo, hi, (B, proj, H, W)).astype(eltw_dt)
    ecal = r.uniform(0.5, 1.0, proj).astype(np.float32)
    ebuf = hip.upload(eng, e, "fs_b_yx_fsv16")
    shapes = [(mid, 1, 3, "relu6", mid), (proj, mid, 1, "none", 1), (6 * proj, proj, 1, "relu6", 1)]
    spec, refs, bufs = [], [], []
    prev_t, ref_in = xin.tensor, x
    for k, (ofm, ifm_g, fk, act, groups) in enumerate(shapes):
        w, bias, wqf, calib, akw = relu6_layer(r, ofm, ifm_g, fk, act)
        kw = dict(stride=(1, 1), pad=(fk // 2,) * 2, groups=groups, bias_dt=hip.I32, has_wqf=True, has_calib=True, **akw)
        okw = dict(stride=(1, 1), pad=(fk // 2,) * 2, groups=groups, out_dt="s8", **akw)
        if k == 1:
            kw.update(eltw_t=ebuf.tensor, eltw_act="none", has_eltw_calib=True, conv_saturate=saturate)
            okw.update(eltw=e, eltw_act="none", eltw_calib=ecal)
        d = hip.conv_desc(prev_t, w.shape, "s8", **kw)
        spec.append((d, w, bias, wqf, calib, ecal if k == 1 else None))
        bufs.append(hip.Buffer(eng, d.output))
        if k == 1:
            calib = calib * 3  # a share of the convolution results beyond +-127
            spec[-1] = (d, w, bias, wqf, calib, ecal)
        if k == 1 and saturate:
            # the kept saturation equals a convolution writing s8 followed by the stand-alone quantized sum
            plain = {key: val for key, val in okw.items() if not key.startswith("eltw")}
            refs.append(rc.eltwise([e, rc.conv(ref_in, w, bias, wqf=wqf, calib=calib, **plain)], "sum", calib=ecal))
        else:
            refs.append(rc.conv(ref_in, w, bias, wqf=wqf, calib=calib, **okw))
        ref_in, prev_t = refs[-1], hip.Tensor.make(hip.S8, hip.FS_B_YX_FSV16, B, ofm, H, W)
    ch = hip.ConvChain(eng, spec, [False, True, True])
    assert b"conv_dwchain" in ch.info().kernel_name
    ch.enqueue(xin, [None, bufs[1], bufs[2]], [None, ebuf, None])
    eng.finish()
    for k in (1, 2):
        got = hip.download(eng, bufs[k])
        bad = np.argwhere(got != refs[k])
        assert bad.size == 0, "stage %d: %d of %d differ, first at %s" % (k, len(bad), got.size, bad[0])
    if saturate:  # the data does reach the saturation
        unsat = rc.conv(refs[0], spec[1][1], spec[1][2], wqf=spec[1][3], calib=spec[1][4], out_dt="s8", act="none", eltw=e, eltw_act="none",
                        eltw_calib=ecal)
        assert (unsat != refs[1]).any()
    ch.close()
    xin.close(), ebuf.close()
    for b in bufs:
        b.close()
