"""fully_connected (the layer that closes an int8 classification network): oracle against the reference's tables
(tests/test_cases/fully_connected_gpu_test.cpp), then the HIP path through the C-ABI and the clDNN API."""
import json
import os

import numpy as np
import pytest

from oracle import refconv as rc

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "fc_kat.json")) as f:
    CASES = json.load(f)["cases"]
NP = {"s8": np.int8, "f32": np.float32}


def _to_bfyx(flat, shape, layout):
    b, f, h, w = shape
    if layout == "yxfb":
        return np.ascontiguousarray(np.array(flat).reshape(h, w, f, b).transpose(3, 2, 0, 1))
    return np.array(flat).reshape(shape)


def problem(case):
    dt = NP[case["dt"]]
    x = _to_bfyx(case["input"], case["in_shape"], case.get("in_layout")).astype(dt)
    w = np.array(case["weights"]).reshape(case["w_shape"]).astype(dt)
    bias = None if case["bias"] is None else np.array(case["bias"], np.float32)
    B, OFM = x.shape[0], w.shape[0]
    exp = _to_bfyx(case["expected"], [B, OFM, 1, 1], case.get("out_layout")).astype(np.float64)
    return x, w, bias, exp


def act_of(case):
    return ("relu_slope" if case["slope"] else case["act"]), case["slope"]


@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_oracle_known_answers(case):
    x, w, bias, exp = problem(case)
    act, m = act_of(case)
    out = rc.fully_connected(x, w, bias, act=act, act_m=m)
    assert out.shape == exp.shape and out.dtype == x.dtype
    np.testing.assert_allclose(out.astype(np.float64), exp, atol=1e-6, rtol=0)


def quantized_problem(seed, B=3, F=70, H=2, W=3, OFM=37, bias=True, calib=True):
    r = np.random.default_rng(seed)
    x = r.integers(-128, 128, (B, F, H, W)).astype(np.int8)
    w = r.integers(-127, 128, (OFM, F, H, W)).astype(np.int8)
    k = F * H * W
    q = (r.uniform(0.5, 2.0, OFM) * 60.0 / (np.sqrt(k) * 73.9 * 73.3)).astype(np.float32)  # results spread over, and beyond, int8
    b = (r.standard_normal(OFM) * 20).astype(np.float32) if bias else None
    c = r.uniform(0.5, 1.5, OFM).astype(np.float32) if calib else None
    return x, w, b, q, c


def test_quantized_epilogue_against_a_plain_restatement():
    """(char)round(((float)acc * q * iqf + bias) * calib): low byte kept, relu on the char (reference
    fully_connected_gpu_bfyx_ref.cl:63-84).  Restated here with numpy integer / float32 arithmetic step by step."""
    x, w, b, q, c = quantized_problem(5)
    out = rc.fully_connected(x, w, b, wqf=q, calib=c, iqf=0.5, act="relu")
    acc = np.einsum("bfyx,ofyx->bo", x.astype(np.int64), w.astype(np.int64))
    v = acc.astype(np.float32) * q
    v = v * np.float32(0.5)
    v = v + b
    v = v * c
    r = np.sign(v) * np.floor(np.abs(v) + np.float32(0.5))
    ch = r.astype(np.int64).astype(np.int8)          # keeps the low byte
    exp = np.maximum(ch, 0).reshape(out.shape)
    np.testing.assert_array_equal(out, exp)
    assert (np.abs(r) > 127).any()                   # the data does leave the int8 range somewhere: wrapping is exercised
    # without a bias the reference's kernel does not scale at all: the low byte of the accumulator
    raw = rc.fully_connected(x, w, None, wqf=q, calib=c)
    np.testing.assert_array_equal(raw, acc.astype(np.int8).reshape(raw.shape))
    # one output factor instead of per-feature calibration
    o = rc.fully_connected(x, w, b, wqf=q, oqf=0.75)
    v2 = (acc.astype(np.float32) * q * np.float32(1.0) + b) * np.float32(0.75)
    np.testing.assert_array_equal(o.ravel(), (np.sign(v2) * np.floor(np.abs(v2) + np.float32(0.5))).astype(np.int64).astype(np.int8).ravel())


def test_unquantized_int8_wraps_like_the_convolution():
    x, w, _, _, _ = quantized_problem(6, bias=False)
    out = rc.fully_connected(x, w)
    acc = np.einsum("bfyx,ofyx->bo", x.astype(np.int64), w.astype(np.int64))
    np.testing.assert_array_equal(out.ravel(), acc.astype(np.int8).ravel())


# ------------------------------------------------------------------------------------------ plan (no GPU)
def test_plan_fully_connected_layouts():
    from cldnn_amd import api as cl
    keep = []

    def attach(a):
        a = np.ascontiguousarray(a)
        keep.append(a)
        b, f, h, w = a.shape
        return cl.memory.attach(cl.layout(cl.DT_OF[a.dtype], cl.format.bfyx, cl.tensor(b, f, w, h)), a)

    def topo(batch, fmt):
        return cl.topology(cl.input_layout("in", cl.layout(cl.data_types.f32, fmt, cl.tensor(batch, 8, 2, 3))),
                           cl.data("w", attach(np.ones((5, 8, 3, 2), np.float32))), cl.fully_connected("fc", "in", "w"))

    by = lambda t: {n["id"]: n for n in cl.plan(t)}
    # reference src/fully_connected.cpp:58-80: bfyx batch 1 -> bfyx, bfyx batch > 1 and yxfb -> yxfb; size [b, ofm, 1, 1]
    n = by(topo(1, cl.format.bfyx))["fc"]
    assert n["format"] == cl.format.bfyx and n["size"] == [1, 5, 1, 1] and n["fully_connected"] is True
    assert by(topo(4, cl.format.bfyx))["fc"]["format"] == cl.format.yxfb
    assert by(topo(1, cl.format.yxfb))["fc"]["format"] == cl.format.yxfb
    bad = cl.topology(cl.input_layout("in", cl.layout(cl.data_types.f32, cl.format.bfyx, cl.tensor(1, 8, 2, 3))),
                      cl.data("w", attach(np.ones((5, 8, 3, 3), np.float32))), cl.fully_connected("fc", "in", "w"))
    with pytest.raises(cl.error) as e:
        cl.plan(bad)
    assert "spatial size" in str(e.value)


# ------------------------------------------------------------------------------------------ GPU
@pytest.fixture(scope="module")
def eng():
    from cldnn_amd import hip
    e = hip.Engine(0)
    yield e
    e.close()


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_gpu_known_answers(eng, case):
    from cldnn_amd import hip
    x, w, bias, exp = problem(case)
    act, m = act_of(case)
    out = hip.conv_forward(eng, x, w, bias, act=act, act_m=m, fc=True)
    np.testing.assert_allclose(out.astype(np.float64), exp, atol=1e-6, rtol=0)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["bfyx", "fs_b_yx_fsv16"])
@pytest.mark.parametrize("kw", [dict(), dict(bias=False), dict(calib=False), dict(F=2048, H=1, W=1, OFM=1000, B=4)],
                         ids=["bias_calib", "no_bias", "output_factor", "resnet_fc1000"])
def test_gpu_quantized_matches_oracle(eng, fmt, kw):
    from cldnn_amd import hip
    x, w, b, q, c = quantized_problem(9, **kw)
    args = dict(iqf=0.5, oqf=1.0 if c is not None else 0.75, act="relu")
    ref = rc.fully_connected(x, w, b, wqf=q, calib=c, **args)
    out = hip.conv_forward(eng, x, w, b, q, c, fmt=fmt, fc=True, **args)
    np.testing.assert_array_equal(out, ref)


@pytest.mark.gpu
@pytest.mark.parametrize("act", ["relu", "none"])
@pytest.mark.parametrize("bias_dt", [np.float32, np.int32], ids=["f32_bias", "i32_bias"])
@pytest.mark.parametrize("shape", [dict(F=2048, H=1, W=1, OFM=1000, B=32), dict(F=64, H=3, W=3, OFM=70, B=5), dict(F=128, H=1, W=1, OFM=64, B=2)],
                         ids=["resnet_fc1000_b32", "3x3_plane", "small"])
def test_gpu_quantized_blocked_kernels(eng, shape, bias_dt, act):
    """every matrix-core kernel family that takes the shape, short and long epilogue (a float bias takes the short
    form, an int32 bias the long one; both add the bias as a float after the dequantisation)"""
    from cldnn_amd import hip
    x, w, b, q, c = quantized_problem(10, **shape)
    b = (b * 3).astype(bias_dt)
    ref = rc.fully_connected(x, w, b, wqf=q, calib=c, iqf=0.5, act=act)
    assert len(np.unique(ref)) > 30 and (act == "none") == bool((ref < 0).any())
    L = hip.lib()
    seen = set()
    for tile in range(0, L.cldnn_hip_tile_config_count() + 1):
        try:
            out, info = hip.conv_forward(eng, x, w, b, q, c, fmt="fs_b_yx_fsv16", fc=True, iqf=0.5, act=act, tile=tile, want_info=True)
        except hip.HipError:
            continue  # a row that does not take this shape refuses it
        name = info.kernel_name.decode()
        assert ("fast" in name) == (bias_dt == np.float32 and "gemv" not in name), name  # the small-batch kernel has one epilogue
        seen.add(name.split("<")[0])
        np.testing.assert_array_equal(out, ref, err_msg=name)
    assert len(seen) >= 2 and "conv_gemv" in seen, seen
    # what the table picks by itself for a batch of at most 32 and K >= 1024: the small-batch kernel
    _, info = hip.conv_forward(eng, x, w, b, q, c, fmt="fs_b_yx_fsv16", fc=True, iqf=0.5, act=act, want_info=True)
    assert ("gemv" in info.kernel_name.decode()) == (x.shape[0] <= 32 and x[0].size >= 1024), info.kernel_name


@pytest.mark.gpu
def test_api_known_answers_and_quantized_network():
    from cldnn_amd import api as cl
    e = cl.engine()
    vm = lambda v: cl.make_memory(e, np.ascontiguousarray(np.asarray(v).reshape(1, 1, 1, -1)))
    for case in CASES:
        x, w, bias, exp = problem(case)
        act, m = act_of(case)
        b, f, h, wd = x.shape
        int8 = case["dt"] == "s8"
        xin = np.array(case["input_f32"], np.float32).reshape(x.shape) if int8 else x
        fmt = cl.format.yxfb if case.get("in_layout") == "yxfb" else cl.format.bfyx
        prims = [cl.input_layout("input", cl.layout(cl.data_types.f32, fmt, cl.tensor(b, f, wd, h))), cl.data("weights", cl.make_memory(e, w))]
        src = "input"
        if int8:
            prims.append(cl.reorder("reorder_to_int", "input", cl.layout(cl.data_types.i8, cl.format.bfyx, cl.tensor(b, f, wd, h))))
            src = "reorder_to_int"
        if bias is not None:
            prims.append(cl.data("bias", vm(bias)))
        prims.append(cl.fully_connected("full_con_prim", src, "weights", "bias" if bias is not None else "", with_activation=case["act"] == "relu",
                                        activation_slp=case["slope"]))
        out_id = "full_con_prim"
        if int8:
            prims.append(cl.reorder("reorder_to_float", out_id, cl.layout(cl.data_types.f32, cl.format.bfyx, cl.tensor(b, w.shape[0], 1, 1))))
            out_id = "reorder_to_float"
        net = cl.network(e, cl.topology(*prims))
        net.set_input_data("input", cl.make_memory(e, xin, fmt))
        outs = net.execute()
        assert list(outs) == [out_id]
        np.testing.assert_allclose(outs[out_id].get_memory().read().astype(np.float64), exp, atol=1e-6, rtol=0, err_msg=case["name"])
    # quantized, behind a blocked convolution and a global pooling, optimised build: conv -> pool -> fc
    r = np.random.default_rng(2)
    x = r.integers(0, 256, (2, 64, 7, 7)).astype(np.uint8)
    w1 = r.integers(-127, 128, (128, 64, 1, 1)).astype(np.int8)
    c1 = (40.0 / (np.sqrt(64) * 147.4 * 73.3) * r.uniform(0.5, 2.0, 128)).astype(np.float32)
    one = np.ones(128, np.float32)
    _, w2, b2, q2, c2 = quantized_problem(4, B=2, F=128, H=1, W=1, OFM=10)
    t = cl.topology(cl.input_layout("input", cl.layout(cl.data_types.u8, cl.format.bfyx, cl.tensor(2, 64, 7, 7))),
                    cl.data("w1", cl.make_memory(e, w1)), cl.data("q1", vm(one)), cl.data("c1", vm(c1)),
                    cl.data("w2", cl.make_memory(e, w2)), cl.data("b2", vm(b2)), cl.data("q2", vm(q2)), cl.data("c2", vm(c2)),
                    cl.convolution("conv", "input", ["w1"], None, ["q1"], ["c1"], with_activation=True, output_data_type=cl.data_types.i8),
                    cl.pooling("pool", "conv", cl.pooling_mode.average),
                    cl.fully_connected("fc", "pool", "w2", "b2", "q2", "c2", 1.0))
    for optimize in (False, True):
        net = cl.network(e, t, cl.build_options(optimize_data=optimize))
        net.set_input_data("input", cl.make_memory(e, x))
        out = net.execute()["fc"].get_memory().read()
        a = rc.conv(x, w1, None, wqf=one, calib=c1, act="relu", out_dt="s8")
        p = rc.pool(a, "average", None, global_pooling=True)
        np.testing.assert_array_equal(out, rc.fully_connected(p, w2, b2, wqf=q2, calib=c2))
