"""Parity of the HIP convolution (through the C-ABI) with the CPU oracle and with the
reference's known-answer tables.  Integer results must be bit-exact; float outputs are
compared at 1e-5 relative (they are the same sequence of float operations)."""
import numpy as np
import pytest

import kat
from cldnn_amd import hip
from oracle import refconv as rc

pytestmark = pytest.mark.gpu
K = kat.load()


@pytest.fixture(scope="module")
def eng():
    e = hip.Engine()
    yield e
    e.close()


def both(eng, x, w, bias=None, wqf=None, calib=None, fmt="bfyx", impl=hip.IMPL_AUTO, tile=0, in_pad=(0, 0),
         out_pad=(0, 0), acc=True, **kw):
    ref = rc.conv(x, w, bias, wqf=wqf, calib=calib, want_acc=acc, **kw)
    got = hip.conv_forward(eng, x, w, bias, wqf, calib, fmt=fmt, impl=impl, tile=tile, in_pad=in_pad, out_pad=out_pad,
                           want_acc=acc, want_info=True, **kw)
    return ref, got


def assert_same(ref_out, got_out):
    assert ref_out.shape == got_out.shape and ref_out.dtype == got_out.dtype
    if ref_out.dtype == np.float32:
        np.testing.assert_allclose(got_out, ref_out, rtol=1e-5, atol=0)
    else:
        bad = np.argwhere(ref_out != got_out)
        assert bad.size == 0, "first mismatch at %s: ref %s got %s (%d of %d differ)" % (
            bad[0], ref_out[tuple(bad[0])], got_out[tuple(bad[0])], len(bad), ref_out.size)


# ------------------------------------------------------------------ the reference's own tables
@pytest.mark.parametrize("fmt", ["bfyx", "fs_b_yx_fsv16"])
@pytest.mark.parametrize("case", K["conv_quantized"], ids=lambda c: c["name"])
def test_kat_conv_quantized(eng, case, fmt):
    p = kat.diag_problem(case)
    out = hip.conv_forward(eng, p["x"], p["w"], p["bias"], p["wqf"], out_dt=case["out_dt"], act="relu", fmt=fmt)
    if case["out_dt"] == "f32":
        np.testing.assert_allclose(out, p["expected"], atol=case["tol"], rtol=0)
    else:
        np.testing.assert_array_equal(out.astype(np.int64), p["expected"].astype(np.int64))


@pytest.mark.parametrize("fmt", ["bfyx", "fs_b_yx_fsv16"])
@pytest.mark.parametrize("case", K["fused"], ids=lambda c: c["name"])
def test_kat_fused(eng, case, fmt):
    if fmt != "bfyx" and case["in_dt"] == "f32":
        pytest.skip("the blocked int8 layout carries int8 data")
    p = kat.diag_problem(case, fused=True)
    out = hip.conv_forward(eng, p["x"], p["w"], p["bias"],
                           p["wqf"] if case["pass_wqf"] else None,
                           p["conv_calib"] if case["pass_conv_calib"] else None,
                           out_dt=case["out_dt"], act="none", eltw=p["nci"],
                           non_conv_scale=float(p["non_conv_scale"]), eltw_act="relu",
                           eltw_calib=p["eltw_calib"] if case["pass_eltw_calib"] else None, fmt=fmt)
    if case["out_dt"] == "f32":
        np.testing.assert_allclose(out, p["expected"], atol=case["tol"], rtol=0)
    else:
        np.testing.assert_array_equal(out.astype(np.int64), p["expected"].astype(np.int64))


@pytest.mark.parametrize("case", K["indexing"], ids=lambda c: c["name"])
def test_kat_indexing(eng, case):
    p = kat.indexing_problem(case, K["indexing"])
    out = hip.conv_forward(eng, p["x"], p["w"], p["bias"], stride=p["stride"], pad=p["pad"], groups=p["groups"],
                           act=p["act"])
    assert out.shape == p["expected"].shape
    np.testing.assert_allclose(out.astype(np.float64), p["expected"], atol=max(p["tol"], 1e-5), rtol=0)


@pytest.mark.parametrize("case", K["api"], ids=lambda c: c["name"])
def test_kat_api_tables(eng, case):
    """further tables of the reference's convolution tests: padding above / below, output padding, split as groups"""
    p = kat.api_problem(case, K["indexing"])
    lo = (p["pad"][0] + p["pad_above"][0], p["pad"][1] + p["pad_above"][1])
    hi = (p["pad"][0] + p["pad_below"][0], p["pad"][1] + p["pad_below"][1])
    assert p["out_pad_lower"] == p["out_pad_upper"]
    out = hip.conv_forward(eng, p["x"], p["w"], p["bias"], stride=p["stride"], pad=lo, pad_end=hi,
                           groups=max(p["groups"], p["split"]), act="relu_slope" if p["act_slope"] else p["act"],
                           act_m=p["act_slope"], out_pad=p["out_pad_lower"])
    kat.assert_close_where_given(out, p["expected"], p["tol"])


@pytest.mark.parametrize("case", [c for c in K["quantized_recipe"] if c["scale"] != "two_layers"], ids=lambda c: c["name"])
@pytest.mark.parametrize("fmt", ["bfyx", "fs_b_yx_fsv16"])
def test_kat_quantized_recipe(eng, case, fmt):
    """float-vs-int8 tolerance tests of the reference (convolution_gpu_test.cpp:3741-3969): int8 result / factor within 3 of
    the float table, and identical to the oracle"""
    x = np.array(case["input"], np.float32).reshape(case["in_shape"])
    wf = np.array(case["weights_f"], np.float32).reshape(case["w_shape"])
    bias = np.array(case["bias"], np.float32)
    exp = np.array(case["float_output"], np.float64).reshape(case["out_shape"])
    wq, wqf = kat.quantize_weights(wf)
    kw = dict(stride=tuple(case["stride"]), out_dt="s8")
    if case["scale"] == "single":
        scale = np.float32(127.0) / np.float32(np.abs(exp).max())
        kw.update(oqf=float(scale))
        calib = None
    else:
        calib = scale = kat.calibrate(exp.astype(np.float32))
    out = hip.conv_forward(eng, x.astype(np.int8), wq.astype(np.int8), bias, wqf, calib, fmt=fmt, **kw)
    ref = rc.conv(x.astype(np.int8), wq.astype(np.int8), bias, wqf=wqf, calib=calib, **kw)
    np.testing.assert_array_equal(out, ref)
    assert np.abs(out.astype(np.float64) / np.reshape(scale, (1, -1, 1, 1)) - exp).max() <= case["tol"]


ASYM = [
    # IFM OFM  H   W  k groups stride pad(lo)  pad_end  in_pad  fmt
    (64, 64, 14, 14, 3, 1, (1, 1), (1, 1), (2, 3), (0, 0), "fs_b_yx_fsv16"),   # bounds-checked taps
    (64, 64, 14, 14, 3, 1, (1, 1), (1, 1), (2, 3), (2, 3), "fs_b_yx_fsv16"),   # zero border wide enough for the high side
    (64, 128, 15, 13, 3, 1, (2, 2), (0, 1), (2, 1), (2, 2), "fs_b_yx_fsv16"),
    (32, 32, 12, 12, 3, 32, (1, 1), (1, 0), (0, 2), (0, 0), "fs_b_yx_fsv16"),  # depthwise
    (32, 32, 12, 12, 3, 32, (2, 2), (0, 1), (1, 1), (1, 2), "fs_b_yx_fsv16"),
    (3, 64, 20, 20, 7, 1, (2, 2), (3, 3), (2, 4), (4, 4), "b_fs_yx_fsv4"),     # first layer
    (16, 24, 9, 11, 3, 1, (1, 1), (2, 0), (0, 2), (0, 0), "bfyx"),             # layout-agnostic kernel
]


@pytest.mark.parametrize("shape", ASYM, ids=lambda s: "x".join(str(v) for v in s[:6]) + "_" + s[-1])
def test_asymmetric_padding(eng, shape):
    """different zero padding in front of and behind the input (padding_above / padding_below of the primitive)"""
    IFM, OFM, H, W, k, groups, stride, lo, hi, in_pad, fmt = shape
    x, w, bias, wqf, calib = problem(77, 2, IFM, H, W, OFM, k, k, groups=groups)
    kw = dict(stride=stride, pad=lo, pad_end=hi, groups=groups, out_dt="u8", act="relu")
    out = hip.conv_forward(eng, x, w, bias, wqf, calib, fmt=fmt, in_pad=in_pad, **kw)
    ref = rc.conv(x, w, bias, wqf=wqf, calib=calib, **kw)
    assert out.shape == ref.shape
    np.testing.assert_array_equal(out, ref)


# ------------------------------------------------------------------ seeded random problems vs the oracle
def problem(seed, B, IFM, H, W, OFM, FY, FX, in_dt=np.uint8, groups=1, spread=True):
    r = np.random.default_rng(seed)
    lo, hi = (0, 256) if in_dt == np.uint8 else (-128, 128)
    x = r.integers(lo, hi, (B, IFM, H, W)).astype(in_dt)
    w = r.integers(-127, 128, (OFM, IFM // groups, FY, FX)).astype(np.int8)
    bias = r.integers(-1000, 1001, OFM).astype(np.int32)
    k = (IFM // groups) * FY * FX
    sigma = np.sqrt(k) * 147.4 * 73.3 if in_dt == np.uint8 else np.sqrt(k) * 73.9 * 73.3
    if spread:  # outputs spread over the int8 range so rounding and both saturation ends are hit
        calib = (40.0 / sigma * r.uniform(0.5, 2.0, OFM)).astype(np.float32)
    else:       # the benchmark's data: log-uniform in [1e-4, 1e-2]
        calib = np.exp(r.uniform(np.log(1e-4), np.log(1e-2), OFM)).astype(np.float32)
    wqf = np.ones(OFM, np.float32)
    return x, w, bias, wqf, calib


SHAPES = [
    # B IFM H  W  OFM FY FX stride pad
    (1, 64, 56, 56, 64, 3, 3, (1, 1), (1, 1)),     # BASELINE config 1
    (2, 64, 14, 14, 256, 1, 1, (1, 1), (0, 0)),
    (3, 256, 14, 14, 128, 1, 1, (2, 2), (0, 0)),   # strided 1x1
    (2, 32, 9, 11, 48, 3, 3, (1, 1), (1, 1)),      # ragged: ofm 48, odd sizes
    (1, 3, 32, 32, 64, 7, 7, (2, 2), (3, 3)),      # stem shape, IFM = 3
    (2, 128, 7, 7, 128, 3, 3, (1, 1), (1, 1)),
    (1, 40, 10, 6, 24, 5, 3, (2, 1), (2, 1)),      # ifm 40 -> 3 slices, asymmetric filter
    (1, 16, 5, 5, 16, 1, 1, (1, 1), (0, 0)),       # one k-chunk: padded K-step
]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s[:7])))
@pytest.mark.parametrize("in_dt", [np.uint8, np.int8], ids=["u8", "s8"])
def test_ref_kernel_bfyx(eng, shape, in_dt):
    B, IFM, H, W, OFM, FY, FX, stride, pad = shape
    x, w, bias, wqf, calib = problem(11, B, IFM, H, W, OFM, FY, FX, in_dt)
    (ro, ra), (go, ga, info) = both(eng, x, w, bias, wqf, calib, stride=stride, pad=pad, out_dt="s8", act="relu")
    assert info.impl == hip.IMPL_REF
    np.testing.assert_array_equal(ga, ra)
    assert_same(ro, go)


def tiles():
    return list(range(1, hip.lib().cldnn_hip_tile_config_count() + 1))


def tile_names():
    L = hip.lib()
    return [L.cldnn_hip_tile_config_name(i).decode() for i in range(L.cldnn_hip_tile_config_count())]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s[:7])))
@pytest.mark.parametrize("in_dt", [np.uint8, np.int8], ids=["u8", "s8"])
def test_mfma_kernel_all_tiles(eng, shape, in_dt):
    """every row of the tile table (LDS-staged and streaming kernels) x both addressing modes"""
    B, IFM, H, W, OFM, FY, FX, stride, pad = shape
    x, w, bias, wqf, calib = problem(12, B, IFM, H, W, OFM, FY, FX, in_dt)
    ref_o, ref_a = rc.conv(x, w, bias, wqf=wqf, calib=calib, stride=stride, pad=pad, out_dt="s8", act="relu",
                           want_acc=True)
    names = tile_names()
    seen = set()
    for border in (True, False):
        in_pad = (pad[0] + (1 if FY > 1 else 0), pad[1]) if border else (0, 0)
        for tile in [0] + tiles():
            kw = dict(stride=stride, pad=pad, out_dt="s8", act="relu", fmt="fs_b_yx_fsv16", in_pad=in_pad, tile=tile,
                      want_acc=True, want_info=True)
            ksteps = -(-(FY * FX * -(-IFM // 16)) // 4)
            no_border = not border and pad != (0, 0)
            if tile and names[tile - 1].startswith("stream") and (no_border or ksteps > 8):
                with pytest.raises(hip.HipError):  # needs constant tap offsets (zero border) and K <= 512
                    hip.conv_forward(eng, x, w, bias, wqf, calib, **kw)
                continue
            if tile and names[tile - 1].startswith("stem"):
                with pytest.raises(hip.HipError):  # the first-layer row goes with b_fs_yx_fsv4 input
                    hip.conv_forward(eng, x, w, bias, wqf, calib, **kw)
                continue
            if tile and names[tile - 1].startswith("halo") and (no_border or -(-IFM // 16) % 4 != 0 or (FY, FX) != (3, 3) or stride != (1, 1)):
                with pytest.raises(hip.HipError):  # nine taps, stride 1, constant tap offsets, feature slices in fours
                    hip.conv_forward(eng, x, w, bias, wqf, calib, **kw)
                continue
            if tile and names[tile - 1].startswith(("bdir", "wsl", "gemv")) and (no_border or -(-IFM // 16) % 4 != 0):
                with pytest.raises(hip.HipError):  # needs constant tap offsets and feature slices in fours
                    hip.conv_forward(eng, x, w, bias, wqf, calib, **kw)
                continue
            go, ga, info = hip.conv_forward(eng, x, w, bias, wqf, calib, **kw)
            name = info.kernel_name.decode()
            assert info.impl == hip.IMPL_MFMA and ("fast" in name or "gemv" in name), name  # the small-batch kernel has one epilogue
            seen.add(name)
            np.testing.assert_array_equal(ga, ref_a, err_msg=name)
            assert_same(ref_o, go)
    assert any("conv_mfma" in n and "border" in n for n in seen)
    assert any("stream" in n for n in seen) == (-(-(FY * FX * -(-IFM // 16)) // 4) <= 8)
    assert any("bdir" in n for n in seen) == (-(-IFM // 16) % 4 == 0)
    assert any("wsl" in n for n in seen) == (-(-IFM // 16) % 4 == 0)
    assert any("halo" in n for n in seen) == (-(-IFM // 16) % 4 == 0 and (FY, FX) == (3, 3) and stride == (1, 1))
    if pad != (0, 0):
        assert any("checked" in n for n in seen)


HALO_SHAPES = [
    # B IFM H  W  OFM pad dilation border(y, x)
    (2, 128, 56, 56, 256, (1, 1), (1, 1), (1, 1)),   # several position tiles per image, two feature blocks, two feature tiles
    (40, 64, 9, 11, 128, (1, 1), (1, 1), (1, 1)),    # tiles that span several images; one feature block
    (1, 64, 6, 150, 128, (1, 1), (1, 1), (1, 1)),    # long rows: the halo exceeds the tile, two patch requests per wave and step
    (1, 64, 5, 200, 128, (1, 1), (1, 1), (1, 1)),    # rows too long for the 256-position row's request slots
    (3, 192, 20, 20, 200, (1, 1), (1, 1), (2, 3)),   # border wider than the padding; partly filled last feature tile
    (2, 64, 17, 15, 64, (2, 2), (2, 2), (2, 2)),     # dilated filter
    (1, 64, 12, 12, 96, (0, 0), (1, 1), (0, 0)),     # no padding: the output is smaller than the input
    (17, 256, 14, 14, 128, (1, 1), (1, 1), (1, 1)),  # four feature blocks; more tiles than one round of workgroups per feature tile needs
]


@pytest.mark.parametrize("row", ["halo_p256_f128", "halo_p512_f128"])
@pytest.mark.parametrize("shape", HALO_SHAPES, ids=lambda s: "x".join(map(str, s[:5])))
@pytest.mark.parametrize("in_dt", [np.uint8, np.int8], ids=["u8", "s8"])
def test_staged_patch_kernel(eng, shape, in_dt, row):
    """the nine-tap stride-1 kernel with both operands in LDS: accumulators and every epilogue form against the oracle"""
    B, IFM, H, W, OFM, pad, dil, border = shape
    tile = tile_names().index(row) + 1
    x, w, bias, wqf, calib = problem(61, B, IFM, H, W, OFM, 3, 3, in_dt)
    base = dict(pad=pad, dilation=dil, fmt="fs_b_yx_fsv16", in_pad=border, tile=tile, want_info=True)
    plain = dict(pad=pad, dilation=dil)
    if W == 200 and row == "halo_p256_f128":
        with pytest.raises(hip.HipError, match="rows too long"):
            hip.conv_forward(eng, x, w, bias, wqf, calib, out_dt="s8", act="relu", **base)
        return
    # requantised with relu (the short branch-free form) + raw accumulators
    ref_o, ref_a = rc.conv(x, w, bias, wqf=wqf, calib=calib, out_dt="s8", act="relu", want_acc=True, **plain)
    go, ga, info = hip.conv_forward(eng, x, w, bias, wqf, calib, out_dt="s8", act="relu", want_acc=True, **base)
    assert info.impl == hip.IMPL_MFMA and info.kernel_name.decode().startswith("conv_halo<" + row), info.kernel_name
    np.testing.assert_array_equal(ga, ref_a)
    assert_same(ref_o, go)
    # no activation, unsigned output, into a buffer with a border of its own
    ref = rc.conv(x, w, bias, wqf=wqf, calib=calib, out_dt="u8", **plain)
    assert_same(ref, hip.conv_forward(eng, x, w, bias, wqf, calib, out_dt="u8", out_pad=(1, 2), **base)[0])
    # the run-time form (weight factors other than one) and the element-wise one (float output)
    wq2 = (wqf * np.random.default_rng(5).uniform(0.5, 2.0, OFM)).astype(np.float32)
    ref = rc.conv(x, w, bias, wqf=wq2, calib=calib, out_dt="s8", act="clamp", act_m=-1000.0, act_n=3000.0, **plain)
    assert_same(ref, hip.conv_forward(eng, x, w, bias, wq2, calib, out_dt="s8", act="clamp", act_m=-1000.0, act_n=3000.0, **base)[0])
    ref = rc.conv(x, w, bias, wqf=wq2, calib=calib, out_dt="f32", act="relu", **plain)
    assert_same(ref, hip.conv_forward(eng, x, w, bias, wq2, calib, out_dt="f32", act="relu", **base)[0])
    # fused residual sum with relu
    OH, OW = ref.shape[2:]
    e = np.random.default_rng(6).integers(-128, 128, (B, OFM, OH, OW)).astype(np.int8)
    ecal = np.random.default_rng(7).uniform(0.3, 1.2, OFM).astype(np.float32)
    kw = dict(out_dt="s8", act="none", eltw=e, eltw_act="relu", eltw_calib=ecal)
    ref = rc.conv(x, w, bias, wqf=wqf, calib=calib, **kw, **plain)
    got, info = hip.conv_forward(eng, x, w, bias, wqf, calib, **kw, **base)
    assert "fast" in info.kernel_name.decode()
    assert_same(ref, got)


def test_staged_patch_kernel_refuses_what_it_cannot_run(eng):
    tile = tile_names().index("halo_p256_f128") + 1
    x, w, bias, wqf, calib = problem(62, 1, 64, 12, 12, 64, 3, 3)
    kw = dict(out_dt="s8", fmt="fs_b_yx_fsv16", tile=tile)
    for bad in (dict(pad=(1, 1), in_pad=(0, 0)),                      # no border: tap offsets are not constant
                dict(pad=(1, 1), in_pad=(1, 1), stride=(2, 2))):      # stride
        with pytest.raises(hip.HipError):
            hip.conv_forward(eng, x, w, bias, wqf, calib, **kw, **bad)
    x1, w1, b1, q1, c1 = problem(63, 1, 64, 12, 12, 64, 1, 1)
    with pytest.raises(hip.HipError):                                 # one tap
        hip.conv_forward(eng, x1, w1, b1, q1, c1, **kw)
    x2, w2, b2, q2, c2 = problem(64, 1, 32, 12, 12, 64, 3, 3)
    with pytest.raises(hip.HipError):                                 # 32 input features: not a whole block of 64
        hip.conv_forward(eng, x2, w2, b2, q2, c2, pad=(1, 1), in_pad=(1, 1), **kw)


@pytest.mark.parametrize("out_dt", ["s8", "u8", "f32"])
@pytest.mark.parametrize("act", [("none", 0, 0), ("relu", 0, 0), ("relu_slope", 0.1, 0), ("clamp", 0.0, 6.0)],
                         ids=lambda a: a[0])
def test_mfma_epilogue_variants(eng, out_dt, act):
    x, w, bias, wqf, calib = problem(13, 2, 64, 12, 12, 96, 3, 3)
    r = np.random.default_rng(3)
    wqf = (3.0 / (np.sqrt(576) * 147.4 * 73.3) * r.uniform(0.5, 2, 96)).astype(np.float32)
    calib = np.full(96, 127 / 6, np.float32) * r.uniform(0.9, 1.1, 96).astype(np.float32)
    calib[::7] *= -1  # negative scales: relu cannot be folded into the final clamp
    kw = dict(stride=(1, 1), pad=(1, 1), out_dt=out_dt, act=act[0], act_m=act[1], act_n=act[2], iqf=0.75)
    for tile, in_pad in ((0, (0, 0)), (0, (1, 1)), (10, (1, 1)), (13, (1, 1)), (15, (1, 1)), (16, (1, 1)), (18, (1, 1)), (19, (1, 1)), (20, (1, 1))):  # table's choice, direct-activation, weights-stationary and split-K rows
        (ro, ra), (go, ga, info) = both(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", tile=tile, in_pad=in_pad, **kw)
        # the short epilogue covers int8 outputs with none / relu / clamp; everything else takes the long form
        assert (b"generic" in info.kernel_name) == (out_dt == "f32" or act[0] == "relu_slope")
        assert tile == 0 or b"bdir" in info.kernel_name or b"wsl" in info.kernel_name
        np.testing.assert_array_equal(ga, ra)
        assert_same(ro, go)


@pytest.mark.parametrize("in_dt", [np.uint8, np.int8], ids=["u8", "s8"])
@pytest.mark.parametrize("shape", [(5, 64, 7, 7, 70, 7, 7, 0), (20, 256, 1, 1, 200, 1, 1, 0), (3, 64, 4, 4, 96, 3, 3, 0), (2, 128, 3, 3, 64, 3, 3, 1),
                                   (16, 512, 7, 7, 128, 7, 7, 0)],
                         ids=["plane7x7_b5", "1x1_b20", "3x3_out2x2", "3x3_padded", "vgg_fc6_slice"])
def test_small_batch_kernel(eng, shape, in_dt):
    """few output pixels, long K: 16-feature fragments, the waves of a workgroup split K; a filter wider than one tap
    gathers the activations into fragment order first.  Every output type and activation, the residual sum, the raw
    accumulators; pixel counts and feature counts that do not fill the fragments."""
    B, IFM, H, W, OFM, FY, FX, pad = shape
    x, w, bias, wqf, calib = problem(31, B, IFM, H, W, OFM, FY, FX, in_dt)
    gemv = tile_names().index("gemv_p16_f16") + 1
    OH, OW = H + 2 * pad - FY + 1, W + 2 * pad - FX + 1
    r = np.random.default_rng(8)
    for out_dt, act in (("s8", ("relu", 0, 0)), ("u8", ("none", 0, 0)), ("f32", ("relu_slope", 0.1, 0)), ("s8", ("clamp", -20.0, 90.0))):
        kw = dict(stride=(1, 1), pad=(pad, pad), out_dt=out_dt, act=act[0], act_m=act[1], act_n=act[2], iqf=0.75)
        (ro, ra), (go, ga, info) = both(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", tile=gemv, in_pad=(pad, pad), **kw)
        assert b"conv_gemv" in info.kernel_name and info.grid == -(-B * OH * OW // 16) * -(-OFM // 64) * 4
        np.testing.assert_array_equal(ga, ra)
        assert_same(ro, go)
    e = r.integers(-128, 128, (B, OFM, OH, OW)).astype(np.int8)
    ecal = r.uniform(0.3, 1.2, OFM).astype(np.float32)
    kw = dict(stride=(1, 1), pad=(pad, pad), out_dt="s8", act="none", eltw=e, eltw_act="relu", eltw_calib=ecal)
    (ro, ra), (go, ga, info) = both(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", tile=gemv, in_pad=(pad, pad), **kw)
    assert b"conv_gemv" in info.kernel_name
    assert_same(ro, go)
    if shape == (20, 256, 1, 1, 200, 1, 1, 0):  # every 16 pixels stream the weights again: the row refuses more than 4096 pixels
        xb, wb, bb, qb, cb = problem(32, 2, 64, 56, 56, 64, 1, 1, in_dt)
        with pytest.raises(hip.HipError):
            hip.conv_forward(eng, xb, wb, bb, qb, cb, fmt="fs_b_yx_fsv16", tile=gemv, out_dt="s8")
    # the table picks it by itself from 16 K-steps (K = 1024) on when at most 32 pixels come out
    _, _, info = hip.conv_forward(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", in_pad=(pad, pad), pad=(pad, pad), out_dt="s8", want_acc=True, want_info=True)
    assert (b"conv_gemv" in info.kernel_name) == (B * OH * OW <= 32 and IFM * FY * FX >= 1024), info.kernel_name


@pytest.mark.parametrize("out_dt,e_dt", [("s8", np.int8), ("u8", np.uint8), ("f32", np.float32)], ids=["s8", "u8", "f32"])
def test_residual_read_from_the_output_buffer(eng, out_dt, e_dt):
    """second_input_in_output (reference fused_conv_eltwise_gpu.cpp:92-121): the residual operand already sits in the
    output buffer and every result replaces the value it was summed with; same numbers as with a separate operand,
    on every kernel family and on the plain-layout and depthwise kernels"""
    r = np.random.default_rng(12)
    def residual(shape):
        if e_dt == np.float32:
            return r.integers(-128, 128, shape).astype(np.float32)
        lo, hi = (-128, 128) if e_dt == np.int8 else (0, 256)
        return r.integers(lo, hi, shape).astype(e_dt)
    x, w, bias, wqf, calib = problem(41, 2, 64, 14, 14, 128, 1, 1)
    e = residual((2, 128, 14, 14))
    ecal = r.uniform(0.3, 1.2, 128).astype(np.float32)
    kw = dict(out_dt=out_dt, act="none", eltw=e, eltw_act="relu", eltw_calib=ecal)
    ref = rc.conv(x, w, bias, wqf=wqf, calib=calib, **kw)
    seen = set()
    for tile in [0] + [t for t in tiles() if not tile_names()[t - 1].startswith(("stem", "halo"))]:
        out, info = hip.conv_forward(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", tile=tile, in_place=True, want_info=True, **kw)
        seen.add(info.kernel_name.decode().split("<")[0])
        assert_same(ref, out)
    assert {"conv_mfma", "conv_stream", "conv_bdir", "conv_wsl", "conv_gemv"} <= seen, seen
    out = hip.conv_forward(eng, x, w, bias, wqf, calib, fmt="bfyx", in_place=True, **kw)  # layout-agnostic kernel
    assert_same(ref, out)
    # 3x3 with padding (a second input as large as the output, not as the input), and depthwise
    x, w, bias, wqf, calib = problem(42, 2, 64, 9, 9, 64, 3, 3)
    e = residual((2, 64, 9, 9))
    kw = dict(out_dt=out_dt, pad=(1, 1), act="none", eltw=e, eltw_act="relu", eltw_calib=ecal[:64])
    assert_same(rc.conv(x, w, bias, wqf=wqf, calib=calib, **kw), hip.conv_forward(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", in_pad=(1, 1), in_place=True, **kw))
    x, w, bias, wqf, calib = problem(43, 2, 32, 9, 9, 32, 3, 3, groups=32)
    e = residual((2, 32, 9, 9))
    kw = dict(out_dt=out_dt, pad=(1, 1), groups=32, act="none", eltw=e, eltw_act="relu", eltw_calib=ecal[:32])
    out, info = hip.conv_forward(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", in_pad=(1, 1), in_place=True, want_info=True, **kw)
    assert b"conv_dw" in info.kernel_name
    assert_same(rc.conv(x, w, bias, wqf=wqf, calib=calib, **kw), out)


@pytest.mark.parametrize("in_dt", [np.uint8, np.int8], ids=["u8", "s8"])
def test_fused_sum_that_keeps_the_convolution_saturation(eng, in_dt):
    """conv_saturate: the fused kernel limits the convolution's rounded result to the s8 range before it adds the second
    input, which makes it equal to a convolution writing s8 followed by the reference's stand-alone quantized sum
    (generic_eltwise_ref.cl:318-330) -- not to fused_conv_eltwise, which adds to the unsaturated value"""
    x, w, bias, wqf, calib = problem(51, 2, 64, 14, 14, 128, 1, 1, in_dt)
    calib = calib * 3  # a good share of the convolution results beyond +-127
    r = np.random.default_rng(9)
    e = r.integers(-128, 128, (2, 128, 14, 14)).astype(np.int8)
    ecal = r.uniform(0.3, 1.2, 128).astype(np.float32)
    conv_s8 = rc.conv(x, w, bias, wqf=wqf, calib=calib, out_dt="s8")
    ref = rc.eltwise([e, conv_s8], "sum", calib=ecal)
    unsaturated = rc.conv(x, w, bias, wqf=wqf, calib=calib, out_dt="s8", act="none", eltw=e, eltw_act="none", eltw_calib=ecal)
    assert 0.02 < (ref != unsaturated).mean() < 0.9  # the two forms do differ on this data
    kw = dict(out_dt="s8", act="none", eltw=e, eltw_act="none", eltw_calib=ecal, conv_saturate=1)
    seen = set()
    for tile in [0] + [t for t in tiles() if not tile_names()[t - 1].startswith(("stem", "halo"))]:
        out, info = hip.conv_forward(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", tile=tile, want_info=True, **kw)
        seen.add(info.kernel_name.decode().split("<")[0])
        assert_same(ref, out)
    assert {"conv_mfma", "conv_stream", "conv_bdir", "conv_wsl", "conv_gemv"} <= seen, seen
    assert_same(ref, hip.conv_forward(eng, x, w, bias, wqf, calib, fmt="bfyx", **kw))                # layout-agnostic kernel
    assert_same(ref, hip.conv_forward(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", round_even=False, non_conv_scale=1.0, in_place=False, **kw))
    with pytest.raises(hip.HipError):  # goes with the quantized fused form only
        hip.conv_forward(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", out_dt="s8", conv_saturate=1)
    # depthwise
    x, w, bias, wqf, calib = problem(52, 2, 32, 9, 9, 32, 3, 3, in_dt, groups=32)
    calib = calib * 3
    e = r.integers(-128, 128, (2, 32, 9, 9)).astype(np.int8)
    ref = rc.eltwise([e, rc.conv(x, w, bias, wqf=wqf, calib=calib, out_dt="s8", pad=(1, 1), groups=32)], "sum", calib=ecal[:32])
    out, info = hip.conv_forward(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", in_pad=(1, 1), pad=(1, 1), groups=32, out_dt="s8", act="none",
                                 eltw=e, eltw_act="none", eltw_calib=ecal[:32], conv_saturate=1, want_info=True)
    assert b"conv_dw" in info.kernel_name
    assert_same(ref, out)


def test_mfma_f32_bias_added_after_dequantisation(eng):
    x, w, _, wqf, calib = problem(14, 1, 32, 8, 8, 32, 3, 3, np.int8)
    bias = np.random.default_rng(1).uniform(-50, 50, 32).astype(np.float32)
    wqf = np.full(32, 1e-3, np.float32)
    (ro, ra), (go, ga, info) = both(eng, x, w, bias, wqf, None, fmt="fs_b_yx_fsv16", pad=(1, 1), out_dt="f32")
    np.testing.assert_array_equal(ga, ra)
    assert_same(ro, go)


def test_mfma_round_to_even_variant(eng):
    case = next(c for c in K["conv_quantized"] if c["name"] == "i8_to_u8")
    p = kat.diag_problem(case)
    got = hip.conv_forward(eng, p["x"], p["w"], p["bias"], p["wqf"], out_dt="u8", act="relu", fmt="fs_b_yx_fsv16",
                           round_even=True)
    ref = rc.conv(p["x"], p["w"], p["bias"], wqf=p["wqf"], out_dt="u8", act="relu", round_even=True)
    np.testing.assert_array_equal(got, ref)
    assert got[0, 5, 0, 1] == 126  # 126.5 -> 126 under round-to-even, 127 in the reference


@pytest.mark.parametrize("fast", [True, False], ids=["fast", "generic"])
@pytest.mark.parametrize("eltw_dt", [np.int8, np.uint8], ids=["s8", "u8"])
def test_mfma_fused_eltwise(eng, fast, eltw_dt):
    x, w, bias, wqf, calib = problem(15, 2, 64, 14, 14, 256, 1, 1)
    r = np.random.default_rng(5)
    lo, hi = (-128, 128) if eltw_dt == np.int8 else (0, 256)
    e = r.integers(lo, hi, (2, 256, 14, 14)).astype(eltw_dt)
    ecal = r.uniform(0.3, 1.2, 256).astype(np.float32)
    kw = dict(out_dt="s8", act="none", eltw=e, eltw_act="relu", eltw_calib=ecal,
              non_conv_scale=1.0 if fast else 0.5)
    for tile in [0] + [t for t in tiles() if not tile_names()[t - 1].startswith(("stem", "halo"))]:
        (ro, ra), (go, ga, info) = both(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", tile=tile, **kw)
        assert (b"fast" in info.kernel_name) == (fast and b"gemv" not in info.kernel_name)  # the small-batch kernel has one epilogue
        np.testing.assert_array_equal(ga, ra)
        assert_same(ro, go)
    np.testing.assert_array_equal(ga, ra)
    assert_same(ro, go)


@pytest.mark.parametrize("shape", [(2, 64, 14, 14, 256, 1, 1, 1), (2, 128, 7, 7, 512, 1, 1, 1), (1, 64, 15, 15, 64, 3, 3, 2),
                                   (3, 64, 28, 28, 64, 1, 1, 1)],
                         ids=["closer", "closer_small", "3x3_s2", "narrow"])
@pytest.mark.parametrize("es", [(2, 2), (1, 3)], ids=["es2x2", "es1x3"])
def test_fused_eltwise_read_with_stride(eng, shape, es):
    """the residual operand is a larger tensor read at (y * esy, x * esx): what a shrunk residual sum hands to the
    convolution it is fused into (reference fused_conv_eltwise_gpu_ref.cl:180-196)"""
    B, IFM, H, W, OFM, FY, FX, st = shape
    x, w, bias, wqf, calib = problem(41, B, IFM, H, W, OFM, FY, FX)
    pad = (FY // 2, FX // 2)
    OH, OW = (H + 2 * pad[0] - FY) // st + 1, (W + 2 * pad[1] - FX) // st + 1
    r = np.random.default_rng(6)
    e = r.integers(-128, 128, (B, OFM, OH * es[0] + 1, OW * es[1])).astype(np.int8)
    ecal = r.uniform(0.3, 1.2, OFM).astype(np.float32)
    kw = dict(stride=(st, st), pad=pad, out_dt="s8", act="none", eltw=e, eltw_act="relu", eltw_calib=ecal, eltw_stride=es)
    ref = rc.conv(x, w, bias, wqf=wqf, calib=calib, **kw)
    # the operand really is sub-sampled
    plain = rc.conv(x, w, bias, wqf=wqf, calib=calib, **dict(kw, eltw=np.ascontiguousarray(e[:, :, ::es[0], ::es[1]][:, :, :OH, :OW]),
                                                             eltw_stride=(1, 1)))
    np.testing.assert_array_equal(ref, plain)
    for fmt, impl in (("bfyx", hip.IMPL_REF), ("fs_b_yx_fsv16", hip.IMPL_AUTO)):
        assert_same(ref, hip.conv_forward(eng, x, w, bias, wqf, calib, fmt=fmt, impl=impl, **kw))
    seen = set()
    for tile in [t for t in tiles() if not tile_names()[t - 1].startswith(("stem", "halo"))]:
        try:
            got, info = hip.conv_forward(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", tile=tile, want_info=True,
                                         in_pad=(pad[0] + (1 if FY > 1 else 0), pad[1]), **kw)
        except hip.HipError:  # a kernel family that does not take this shape refuses it
            continue
        seen.add(info.kernel_name.decode().split("<")[0])
        assert_same(ref, got)
    assert len(seen) >= 3, seen


def test_mfma_padded_buffers(eng):
    # physical zero borders on input and output (what a following 3x3 layer asks of its producer)
    x, w, bias, wqf, calib = problem(16, 2, 64, 14, 14, 64, 3, 3)
    kw = dict(stride=(1, 1), pad=(1, 1), out_dt="s8", act="relu")
    (ro, ra), (go, ga, info) = both(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", in_pad=(1, 1), out_pad=(1, 2), **kw)
    np.testing.assert_array_equal(ga, ra)
    assert_same(ro, go)


def test_output_border_stays_zero(eng):
    x, w, bias, wqf, calib = problem(17, 1, 32, 6, 6, 32, 1, 1)
    xin = hip.upload(eng, x, "fs_b_yx_fsv16")
    d = hip.conv_desc(xin.tensor, w.shape, "s8", out_pad=(1, 1), bias_dt=hip.I32, has_wqf=True, has_calib=True, act="relu")
    c = hip.Conv(eng, d, w, bias, wqf, calib)
    out = hip.Buffer(eng, d.output)
    c.enqueue(xin, out)
    eng.finish()
    raw = out.read_raw().reshape(2, 1, 8, 8, 16)
    assert raw[:, :, 0].any() == 0 and raw[:, :, -1].any() == 0 and raw[:, :, :, 0].any() == 0 and raw[:, :, :, -1].any() == 0
    assert raw[:, :, 1:-1, 1:-1].any()


@pytest.mark.parametrize("shape", [(2, 32, 20, 20, 3, 1, 1), (1, 96, 15, 17, 3, 2, 1), (2, 144, 9, 9, 5, 1, 2),
                                   (1, 960, 7, 7, 3, 1, 1)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("in_dt", [np.uint8, np.int8], ids=["u8", "s8"])
def test_depthwise_kernel(eng, shape, in_dt):
    B, C, H, W, F, s, p = shape
    x, w, bias, wqf, calib = problem(18, B, C, H, W, C, F, F, in_dt, groups=C)
    r = np.random.default_rng(2)
    sig = np.sqrt(F * F) * 147.4 * 73.3
    wqf = (3.0 / sig * r.uniform(0.5, 2, C)).astype(np.float32)
    calib = np.full(C, 127 / 6, np.float32)
    kw = dict(stride=(s, s), pad=(p, p), groups=C, out_dt="s8", act="clamp", act_m=0.0, act_n=6.0)
    (ro, ra), (go, ga, info) = both(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", **kw)
    assert info.impl == hip.IMPL_DEPTHWISE and b"conv_dw_kernel" in info.kernel_name
    np.testing.assert_array_equal(ga, ra)
    assert_same(ro, go)
    # with a physical zero border the 3x3 layers take the dot-product kernel; relu6, relu, no activation, u8 output
    variants = [kw, dict(kw, act="relu", act_m=0.0, act_n=0.0), dict(kw, act="none", out_dt="u8"), dict(kw, out_dt="u8")]
    for i, v in enumerate(variants):
        wq = wqf if i != 1 else np.ones(C, np.float32)
        cal = calib if i != 1 else (40.0 / (F * 147.4 * 73.3) * r.uniform(0.5, 2, C)).astype(np.float32)
        (ro, ra), (go, ga, info) = both(eng, x, w, bias, wq, cal, fmt="fs_b_yx_fsv16", in_pad=(p, p + 1), out_pad=(0, 1), **v)
        assert (b"conv_dw3x3_kernel" in info.kernel_name) == (F == 3), info.kernel_name
        np.testing.assert_array_equal(ga, ra)
        assert_same(ro, go)
    # the layout-agnostic kernel must agree as well (grouped path, one launch)
    (ro2, _), (go2, _, info2) = both(eng, x, w, bias, wqf, calib, fmt="bfyx", acc=True, **kw)
    assert info2.impl == hip.IMPL_REF
    assert_same(ro2, go2)


@pytest.mark.parametrize("shape", [(2, 3, 32, 32, 64, 7, 7, 2, 3), (1, 3, 20, 20, 32, 3, 3, 1, 1), (2, 3, 19, 21, 32, 3, 3, 2, 1),
                                   (1, 4, 9, 9, 16, 5, 5, 1, 2), (1, 1, 12, 12, 80, 3, 1, 1, 0)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("in_dt", [np.uint8, np.int8], ids=["u8", "s8"])
def test_first_layer_fsv4(eng, shape, in_dt):
    """First layers (at most 4 input features) read b_fs_yx_fsv4 and write fs_b_yx_fsv16: a matrix-core fragment is
    4 horizontal taps x 4 features (the role b_fs_yx_fsv4 has in the reference, convolution_gpu_test.cpp:4931-5115)."""
    B, IFM, H, W, OFM, FY, FX, s, p = shape
    x, w, bias, wqf, calib = problem(21, B, IFM, H, W, OFM, FY, FX, in_dt)
    kw = dict(stride=(s, s), pad=(p, p), out_dt="s8", act="relu")
    (ro, ra), (go, ga, info) = both(eng, x, w, bias, wqf, calib, fmt="b_fs_yx_fsv4", in_pad=(p, p), **kw)
    assert info.impl == hip.IMPL_MFMA and b"stem_p" in info.kernel_name, info.kernel_name
    np.testing.assert_array_equal(ga, ra)
    assert_same(ro, go)
    # without the zero border the layout-agnostic kernel takes over
    (ro, ra), (go, ga, info) = both(eng, x, w, bias, wqf, calib, fmt="b_fs_yx_fsv4", **kw)
    assert info.impl == (hip.IMPL_MFMA if p == 0 else hip.IMPL_REF)
    assert_same(ro, go)


def test_benchmark_calibration_data(eng):
    # the benchmark's own factor distribution (mostly saturated outputs) on config 1
    x, w, bias, wqf, calib = problem(19, 1, 64, 56, 56, 64, 3, 3, spread=False)
    (ro, ra), (go, ga, info) = both(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", pad=(1, 1), out_dt="s8", act="relu")
    np.testing.assert_array_equal(ga, ra)
    assert_same(ro, go)


@pytest.mark.parametrize("fmt", ["yxfb", "byxf", "fs_b_yx_fsv16", "b_fs_yx_fsv4"])
def test_reorder_round_trip_and_layout_independence(eng, fmt):
    r = np.random.default_rng(20)
    x = r.integers(0, 256, (2, 21, 5, 7)).astype(np.uint8)
    buf = hip.upload(eng, x, fmt, (1, 2))
    np.testing.assert_array_equal(hip.download(eng, buf), x)
    # raw bytes sit where the layout formula says
    raw = buf.read_raw()
    import ctypes as C
    L = hip.lib()
    for (b, f, y, xx) in [(0, 0, 0, 0), (1, 20, 4, 6), (1, 16, 2, 3), (0, 5, 1, 1)]:
        assert raw[L.cldnn_hip_tensor_offset(C.byref(buf.tensor), b, f, y, xx)] == x[b, f, y, xx]
    # result of a convolution does not depend on the storage layout
    w = r.integers(-127, 128, (8, 21, 3, 3)).astype(np.int8)
    one = np.ones(8, np.float32)
    a = hip.conv_forward(eng, x, w, None, one, pad=(1, 1), out_dt="f32", fmt="bfyx")
    b_ = hip.conv_forward(eng, x, w, None, one, pad=(1, 1), out_dt="f32", fmt=fmt)
    np.testing.assert_array_equal(a, b_)


@pytest.mark.parametrize("shape", [(2, 3, 6, 8), (1, 4, 5, 12), (2, 7, 3, 16), (1, 3, 4, 6)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("pad", [(0, 0), (3, 3), (1, 4)], ids=lambda p: "pad%dx%d" % p)
@pytest.mark.parametrize("fmt", ["b_fs_yx_fsv4", "fs_b_yx_fsv16"])
def test_reorder_into_blocked_layouts(eng, shape, pad, fmt):
    """the byte paths of the reorder (row widths that are and are not whole dwords, borders that do and do not keep the
    16-byte alignment): every element where the layout formula says, feature padding zero, borders untouched"""
    import ctypes as C
    r = np.random.default_rng(21)
    x = r.integers(1, 256, shape).astype(np.uint8)
    buf = hip.upload(eng, x, fmt, pad)
    np.testing.assert_array_equal(hip.download(eng, buf), x)
    raw = buf.read_raw()
    L = hip.lib()
    expect = np.zeros_like(raw)
    for idx in np.ndindex(*shape):
        expect[L.cldnn_hip_tensor_offset(C.byref(buf.tensor), *[int(i) for i in idx])] = x[idx]
    np.testing.assert_array_equal(raw, expect)
    buf.close()


def test_two_engines_from_two_threads():
    """one engine (= stream) and one host thread per request: the C-ABI keeps no state that two requests could share
    (the last error message is per thread)"""
    import threading
    results, errors = {}, []
    probs = {k: problem(50 + k, 2, 64, 14, 14, 128, 3, 3) for k in range(2)}
    refs = {k: rc.conv(p[0], p[1], p[2], wqf=p[3], calib=p[4], pad=(1, 1), out_dt="s8", act="relu") for k, p in probs.items()}

    def request(k):
        try:
            e = hip.Engine(0)
            x, w, bias, wqf, calib = probs[k]
            for _ in range(20):
                results[k] = hip.conv_forward(e, x, w, bias, wqf, calib, pad=(1, 1), out_dt="s8", act="relu", fmt="fs_b_yx_fsv16")
            with pytest.raises(hip.HipError, match="tile_override out of range"):
                hip.conv_forward(e, x, w, bias, wqf, calib, pad=(1, 1), out_dt="s8", fmt="fs_b_yx_fsv16", tile=10 ** 6)
            e.close()
        except Exception as err:  # noqa: BLE001 - reported by the main thread
            errors.append(err)
    threads = [threading.Thread(target=request, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for k in range(2):
        assert_same(refs[k], results[k])


def test_reorder_f32_to_int8_goes_towards_zero_and_saturates(eng):
    """the reference's reorder converts with convert_char (jitter.cpp:483): towards zero; its pooling test relies on
    9.5 -> 9 (pooling_gpu_test.cpp:264-309).  Out-of-range values saturate here."""
    v = np.array([0.5, 1.5, -0.5, -1.5, 2.4, 300.0, -300.0, 127.5, 9.5, -6.99], np.float32).reshape(1, 10, 1, 1)
    src = hip.upload(eng, v)
    dst = hip.Buffer(eng, hip.Tensor.make("s8", "bfyx", 1, 10, 1, 1))
    hip.reorder(eng, src, dst)
    np.testing.assert_array_equal(hip.download(eng, dst).ravel(), [0, 1, 0, -1, 2, 127, -128, 127, 9, -6])


def test_lock_unlock_and_events(eng):
    import ctypes as C
    L = hip.lib()
    t = hip.Tensor.make("u8", "bfyx", 1, 1, 4, 4)
    b = hip.Buffer(eng, t)
    p = L.cldnn_hip_buffer_lock(b.h)
    assert p
    host = (C.c_uint8 * 16).from_address(p)
    assert list(host) == [0] * 16  # zero-initialised at allocation
    for i in range(16):
        host[i] = i
    hip.check(L.cldnn_hip_buffer_unlock(b.h))
    np.testing.assert_array_equal(b.read_raw(), np.arange(16, dtype=np.uint8))
    ev = C.c_void_p()
    hip.check(L.cldnn_hip_event_record(eng.h, C.byref(ev)))
    hip.check(L.cldnn_hip_event_wait(ev))
    assert L.cldnn_hip_event_is_set(ev) == 1
    hip.check(L.cldnn_hip_event_release(ev))
    uev = C.c_void_p()
    hip.check(L.cldnn_hip_event_create_user(eng.h, 0, C.byref(uev)))
    assert L.cldnn_hip_event_is_set(uev) == 0 and L.cldnn_hip_event_is_user(uev) == 1
    fired = []
    cb = hip.EVENT_HANDLER(lambda _: fired.append(1))
    hip.check(L.cldnn_hip_event_add_handler(uev, cb, None))
    hip.check(L.cldnn_hip_event_set(uev))
    assert fired == [1] and L.cldnn_hip_event_is_set(uev) == 1
    hip.check(L.cldnn_hip_event_release(uev))


def test_error_paths(eng):
    x = np.zeros((1, 16, 4, 4), np.uint8)
    w = np.zeros((16, 16, 3, 3), np.int8)
    xin = hip.upload(eng, x, "fs_b_yx_fsv16")
    d = hip.conv_desc(xin.tensor, w.shape, "s8", pad=(1, 1), has_wqf=True)
    d.output.y += 1
    with pytest.raises(hip.HipError) as ei:
        hip.Conv(eng, d, w, None, np.ones(16, np.float32))
    assert ei.value.status == -7
    d = hip.conv_desc(xin.tensor, w.shape, "s8", pad=(1, 1), has_wqf=False)  # u8 without quantisation
    with pytest.raises(hip.HipError) as ei:
        hip.Conv(eng, d, w)
    assert ei.value.status == -2
    plain = hip.upload(eng, x, "bfyx")  # the matrix-core kernels read the blocked layout only
    d = hip.conv_desc(plain.tensor, w.shape, "s8", pad=(1, 1), has_wqf=True, impl=hip.IMPL_MFMA)
    with pytest.raises(hip.HipError) as ei:
        hip.Conv(eng, d, w, None, np.ones(16, np.float32))
    assert ei.value.status == -6
    d = hip.conv_desc(xin.tensor, (16, 1, 3, 3), "s8", pad=(1, 1), has_wqf=True, groups=16, impl=hip.IMPL_MFMA)  # depthwise has its own kernel
    with pytest.raises(hip.HipError) as ei:
        hip.Conv(eng, d, np.zeros((16, 1, 3, 3), np.int8), None, np.ones(16, np.float32))
    assert ei.value.status == -6


@pytest.mark.parametrize("in_dt", [np.uint8, np.int8], ids=["u8", "s8"])
@pytest.mark.parametrize("shape", [(2, 64, 10, 9, 64, 3, 2), (3, 128, 7, 7, 128, 3, 32), (2, 48, 6, 6, 96, 1, 3), (1, 256, 14, 14, 256, 3, 4)],
                         ids=["g2_3x3", "g32_3x3_resnext", "g3_1x1_ifm16", "g4_3x3"])
def test_grouped_convolution_on_the_matrix_core_kernels(eng, shape, in_dt):
    """2 <= groups < features: one launch of the dense kernels on a block-diagonal weight matrix.  Accumulators and
    requantised outputs equal the oracle's grouped convolution, and the oracle's grouped result equals its dense result
    on the block-diagonal expansion (the identity the kernel relies on)."""
    B, IFM, H, W, OFM, FK, G = shape
    r = np.random.default_rng(41)
    lo, hi = (0, 256) if in_dt == np.uint8 else (-128, 128)
    x = r.integers(lo, hi, (B, IFM, H, W)).astype(in_dt)
    w = r.integers(-127, 128, (OFM, IFM // G, FK, FK)).astype(np.int8)
    bias = r.integers(-1000, 1001, OFM).astype(np.int32)
    wqf = np.ones(OFM, np.float32)
    calib = (40.0 / (np.sqrt(IFM // G * FK * FK) * 147.4 * 73.3) * r.uniform(0.5, 2.0, OFM)).astype(np.float32)
    pad = FK // 2
    kw = dict(stride=(1, 1), pad=(pad, pad), groups=G, out_dt="s8", act="relu")
    (ro, ra), (go, ga, info) = both(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", in_pad=(pad, pad), **kw)
    name = info.kernel_name.decode()
    assert info.impl == hip.IMPL_MFMA and not name.startswith("conv_ref"), name
    assert info.ops == 2 * ro.size * (IFM // G) * FK * FK  # algorithmic work counts the real weights
    np.testing.assert_array_equal(ga, ra)
    assert_same(ro, go)
    dense = np.zeros((OFM, IFM, FK, FK), np.int8)
    for f in range(OFM):
        g = f // (OFM // G)
        dense[f, g * (IFM // G):(g + 1) * (IFM // G)] = w[f]
    assert np.array_equal(rc.conv(x, dense, bias, wqf=wqf, calib=calib, stride=(1, 1), pad=(pad, pad), out_dt="s8", act="relu"), ro)
    # the fused residual form
    e = r.integers(-128, 128, (B, OFM, H, W)).astype(np.int8)
    ecal = r.uniform(0.3, 1.2, OFM).astype(np.float32)
    kw = dict(stride=(1, 1), pad=(pad, pad), groups=G, out_dt="s8", act="none", eltw=e, eltw_act="relu", eltw_calib=ecal)
    (ro, ra), (go, ga, info) = both(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", in_pad=(pad, pad), **kw)
    assert info.impl == hip.IMPL_MFMA
    assert_same(ro, go)
    # plain layouts keep the one-thread-per-output kernel
    _, (go, ga, info) = both(eng, x, w, bias, wqf, calib, fmt="bfyx", stride=(1, 1), pad=(pad, pad), groups=G, out_dt="s8", act="relu")
    assert info.impl == hip.IMPL_REF


# two convolutions of the same input in one launch (a block's shortcut projection and its opening 1x1): every output
# feature must equal what its own convolution gives alone
SIBLINGS = [
    # B, IFM, H, W, OFM of the first, OFM of the second, filter, stride, padding
    (2, 64, 14, 14, 256, 64, 1, 1, 0),
    (2, 256, 14, 14, 128, 64, 1, 2, 0),
    (1, 128, 9, 9, 64, 48, 3, 1, 1),
    (3, 64, 7, 7, 80, 24, 1, 1, 0),    # a last feature slice that is partly filled
]


@pytest.mark.parametrize("acts", [("none", "relu"), ("relu", "none"), ("relu", "relu"), ("none", "none"), ("relu_slope", "relu"),
                                  ("none", "clamp")], ids=lambda a: "-".join(a))
@pytest.mark.parametrize("shape", SIBLINGS, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("in_dt", [np.uint8, np.int8], ids=["u8", "s8"])
def test_two_convolutions_of_one_input_in_one_launch(eng, shape, acts, in_dt):
    B, IFM, H, W, F1, F2, FK, stride, pad = shape
    x, w, bias, wqf, calib = problem(77, B, IFM, H, W, F1 + F2, FK, FK, in_dt)
    par = {"none": (0.0, 0.0), "relu": (0.0, 0.0), "relu_slope": (0.25, 0.0), "clamp": (-3000.0, 2500.0)}
    kw = dict(stride=(stride, stride), pad=(pad, pad), out_dt="s8")
    halves = []
    for (lo, hi), act in zip(((0, F1), (F1, F1 + F2)), acts):
        halves.append(rc.conv(x, w[lo:hi], bias[lo:hi], wqf=wqf[lo:hi], calib=calib[lo:hi], act=act, act_m=par[act][0],
                              act_n=par[act][1], **kw))
    ref = np.concatenate(halves, axis=1)
    short = all(a in ("none", "relu") for a in acts)
    names = tile_names()
    rows = [0] + [i + 1 for i, n in enumerate(names) if n in ("p64_f64", "bdir_p64_f64", "wsl_p64", "stream_p32", "bdir_k2_p64_f64")]
    seen = set()
    for tile in rows:
        args = dict(fmt="fs_b_yx_fsv16", in_pad=(pad, pad), tile=tile, want_info=True, act=acts[0], act_m=par[acts[0]][0],
                    act_n=par[acts[0]][1], sibling_split=F1, sibling_act=acts[1], **kw)
        d_extra = dict(sibling_act_m=par[acts[1]][0], sibling_act_n=par[acts[1]][1])
        try:
            got, info = hip.conv_forward(eng, x, w, bias, wqf, calib, **args, **d_extra)
        except hip.HipError:
            assert tile != 0  # a forced row that does not fit the shape
            continue
        name = info.kernel_name.decode()
        seen.add(name)
        assert ("generic" in name) == (not short), name
        assert_same(ref, got)
    assert seen
    # negative output factors under a relu: the clamp form does not apply, the element-wise epilogue takes over
    if acts == ("none", "relu"):
        calib2 = calib.copy()
        calib2[F1 + 3] *= -1
        ref2 = ref.copy()
        ref2[:, F1 + 3] = rc.conv(x, w[F1 + 3:F1 + 4], bias[F1 + 3:F1 + 4], wqf=wqf[:1], calib=calib2[F1 + 3:F1 + 4], act="relu", **kw)[:, 0]
        got, info = hip.conv_forward(eng, x, w, bias, wqf, calib2, fmt="fs_b_yx_fsv16", in_pad=(pad, pad), want_info=True, act="none",
                                     sibling_split=F1, sibling_act="relu", **kw)
        assert b"generic" in info.kernel_name
        assert_same(ref2, got)


def test_sibling_split_is_validated(eng):
    x, w, bias, wqf, calib = problem(5, 1, 64, 6, 6, 96, 1, 1)
    for bad in (8, 96, 100, -16):
        with pytest.raises(hip.HipError):
            hip.conv_forward(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", out_dt="s8", sibling_split=bad, sibling_act="relu")
    e = np.zeros((1, 96, 6, 6), np.int8)
    with pytest.raises(hip.HipError):  # not together with a fused second input
        hip.conv_forward(eng, x, w, bias, wqf, calib, fmt="fs_b_yx_fsv16", out_dt="s8", sibling_split=32, sibling_act="relu", eltw=e)


# ------------------------------------------------------------------ the reference's differential recipe, as written
# reference tests/test_cases/convolution_gpu_test.cpp:4931-5115 (TEST_P(convolution_gpu, b_fs_yx_fsv4)): iota-filled char
# data 2 x F x 56 x 56 and iota-filled char weights 32 x F x k x k, offset -(k / 2), stride and output padding from the
# parameter list; with "bias" also float bias / weight-quantization / calibration ramps (0.1 / 0.3 / 0.2, step 0.01,
# wrapping at 0.9).  The reference compares its semantic kernel with its b_fs_yx_fsv4 kernel; here the oracle stands for
# the semantic kernel and every layout the library computes in is compared with it byte for byte.
B4_PARAMS = [(1, 32, 1, 0, False), (3, 32, 1, 0, False), (7, 3, 1, 0, False), (1, 32, 1, 0, True), (3, 32, 1, 0, True),
             (7, 3, 1, 0, True), (1, 32, 1, 1, False), (3, 32, 1, 1, False), (7, 3, 1, 1, False), (1, 32, 2, 0, False),
             (3, 32, 2, 0, False), (7, 3, 2, 0, False), (3, 64, 2, 1, True)]  # convolution_gpu_test.cpp:5091-5106


def b4_ramp(start, n):
    out, x = [], np.float32(start)
    for _ in range(n):
        x = np.float32(x + np.float32(0.01))
        if x >= np.float32(0.9):
            x = np.float32(start)
        out.append(x)
    return np.array(out, np.float32)


@pytest.mark.parametrize("fmt", ["bfyx", "fs_b_yx_fsv16", "b_fs_yx_fsv4"])
@pytest.mark.parametrize("k,F,stride,out_pad,with_bias", B4_PARAMS,
                         ids=["k%d_f%d_s%d_op%d%s" % (p[0], p[1], p[2], p[3], "_bias" if p[4] else "") for p in B4_PARAMS])
def test_reference_differential_recipe_with_iota_data(eng, fmt, k, F, stride, out_pad, with_bias):
    if fmt == "b_fs_yx_fsv4" and F > 4:
        pytest.skip("b_fs_yx_fsv4 feeds first layers (at most 4 input features) here")
    B, H, W, OFM = 2, 56, 56, 32
    x = (np.arange(B * F * H * W, dtype=np.int64) % 256).astype(np.uint8).view(np.int8).reshape(B, F, H, W)
    w = (np.arange(OFM * F * k * k, dtype=np.int64) % 256).astype(np.uint8).view(np.int8).reshape(OFM, F, k, k)
    bias = wqf = calib = None
    if with_bias:
        bias, calib, wqf = b4_ramp(0.1, OFM), b4_ramp(0.2, OFM), b4_ramp(0.3, OFM)
    kw = dict(stride=(stride, stride), pad=(k // 2, k // 2), out_dt="s8")
    border = (k // 2, k // 2) if fmt != "bfyx" else (0, 0)
    # (the unquantized form wraps around in 8 bits: it has no int32 accumulators to compare)
    ro, (go, info) = both(eng, x, w, bias, wqf, calib, fmt=fmt, in_pad=border, out_pad=(out_pad, out_pad), acc=False, **kw)
    assert ro.shape == (B, OFM, (H + stride - 1) // stride, (W + stride - 1) // stride)
    if with_bias and fmt != "bfyx":
        assert info.impl == hip.IMPL_MFMA, info.kernel_name  # the quantized form runs on the matrix-core kernels
    assert_same(ro, go)
