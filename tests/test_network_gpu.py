"""The convolution path through the clDNN-compatible API on the GPU: topology -> network -> execute,
checked against the reference's known-answer tables and the CPU oracle.

The tests are shaped like the reference's (tests/test_cases/convolution_gpu_test.cpp:4006-4200,
tests/test_cases/fused_conv_eltwise_gpu_test.cpp:31-236, tests/test_cases/memory_test.cpp,
tests/test_cases/topology_test.cpp): build a topology from input_layout / data / convolution primitives,
run a network, read the output memory.
"""
import ctypes as C

import numpy as np
import pytest

import kat
from cldnn_amd import api as cl
from oracle import refconv as rc

pytestmark = pytest.mark.gpu
K = kat.load()
F = cl.format
DT = cl.data_types
CL_DT = {"s8": DT.i8, "u8": DT.u8, "f32": DT.f32, "i32": DT.i32}
OPT = [False, True]


@pytest.fixture(scope="module")
def eng():
    return cl.engine()


def vec_mem(eng, values):
    a = np.ascontiguousarray(values).reshape(1, 1, 1, -1)
    return cl.make_memory(eng, a)


def run(eng, topo, inputs, optimize):
    net = cl.network(eng, topo, cl.build_options(optimize_data=optimize))
    for k, v in inputs.items():
        net.set_input_data(k, v)
    return net, net.execute()


def check(out, expected, out_dt, tol=0.0):
    if out_dt == "f32":
        np.testing.assert_allclose(out, expected, atol=max(tol, 1e-5), rtol=1e-5)
    else:
        np.testing.assert_array_equal(out.astype(np.int64), np.asarray(expected).astype(np.int64))


# ------------------------------------------------------------------------------------------ known answers
@pytest.mark.parametrize("optimize", OPT, ids=["plain", "optimize_data"])
@pytest.mark.parametrize("case", K["conv_quantized"], ids=lambda c: c["name"])
def test_kat_conv_quantized(eng, case, optimize):
    p = kat.diag_problem(case)
    topo = cl.topology(
        cl.input_layout("input", cl.layout(CL_DT[case["in_dt"]], F.bfyx, cl.tensor(1, len(case["features"]), 4, 1))),
        cl.data("weights", cl.make_memory(eng, p["w"])), cl.data("biases", vec_mem(eng, p["bias"])),
        cl.data("quantizations", vec_mem(eng, p["wqf"])),
        cl.convolution("conv", "input", ["weights"], ["biases"], ["quantizations"], with_activation=True,
                       output_data_type=CL_DT[case["out_dt"]]))
    net, outs = run(eng, topo, {"input": cl.make_memory(eng, p["x"])}, optimize)
    assert list(outs) == ["conv"]
    check(outs["conv"].get_memory().read(), p["expected"], case["out_dt"], case.get("tol", 0.0))


@pytest.mark.parametrize("optimize", OPT, ids=["plain", "optimize_data"])
@pytest.mark.parametrize("case", K["fused"], ids=lambda c: c["name"])
def test_kat_fused_conv_eltwise(eng, case, optimize):
    p = kat.diag_problem(case, fused=True)
    n = len(case["features"])
    topo = cl.topology(
        cl.input_layout("input", cl.layout(CL_DT[case["in_dt"]], F.bfyx, cl.tensor(1, n, 4, 1))),
        cl.input_layout("non_conv_input", cl.layout(CL_DT[case["in_dt"]], F.bfyx, cl.tensor(1, n, 2, 1))),
        cl.data("weights", cl.make_memory(eng, p["w"])), cl.data("biases", vec_mem(eng, p["bias"])),
        cl.data("wqf", vec_mem(eng, p["wqf"])), cl.data("conv_calib", vec_mem(eng, p["conv_calib"])),
        cl.data("eltw_calib", vec_mem(eng, p["eltw_calib"])),
        cl.fused_conv_eltwise("fused_conv", "input", "non_conv_input", cl.eltwise_mode.sum, ["weights"], ["biases"],
                              ["wqf"] if case["pass_wqf"] else None, ["conv_calib"] if case["pass_conv_calib"] else None, 1.0,
                              float(p["non_conv_scale"]), "eltw_calib" if case["pass_eltw_calib"] else "",
                              eltw_with_activation=True,
                              output_data_type=CL_DT[case["out_dt"]] if case.get("out_dt_explicit", True) else None))
    net, outs = run(eng, topo, {"input": cl.make_memory(eng, p["x"]), "non_conv_input": cl.make_memory(eng, p["nci"])}, optimize)
    check(outs["fused_conv"].get_memory().read(), p["expected"], case["out_dt"], case.get("tol", 0.0))


@pytest.mark.parametrize("case", K["indexing"], ids=lambda c: c["name"])
def test_kat_indexing(eng, case):
    p = kat.indexing_problem(case, K["indexing"])
    b, f, h, w = p["x"].shape
    prims = [cl.input_layout("input", cl.layout(cl.DT_OF[p["x"].dtype], F.bfyx, cl.tensor(b, f, w, h))),
             cl.data("weights", cl.make_memory(eng, p["w"]))]
    if p["bias"] is not None:
        prims.append(cl.data("biases", vec_mem(eng, p["bias"])))
    prims.append(cl.convolution("conv", "input", ["weights"], ["biases"] if p["bias"] is not None else None,
                                stride=cl.tensor(1, 1, p["stride"][1], p["stride"][0]),
                                input_offset=cl.tensor(0, 0, -p["pad"][1], -p["pad"][0], 0), groups=p["groups"],
                                with_activation=p["act"] == "relu"))
    net, outs = run(eng, cl.topology(*prims), {"input": cl.make_memory(eng, p["x"])}, False)
    out = outs["conv"].get_memory().read()
    assert out.shape == p["expected"].shape
    np.testing.assert_allclose(out.astype(np.float64), p["expected"], atol=max(p["tol"], 1e-5), rtol=0)


def yx(t):
    """(y, x) -> tensor with batch / feature 0 (offsets, paddings)"""
    return cl.tensor(0, 0, t[1], t[0], 0)


@pytest.mark.parametrize("optimize", OPT, ids=["plain", "optimize_data"])
@pytest.mark.parametrize("case", K["api"], ids=lambda c: c["name"])
def test_kat_api_tables(eng, case, optimize):
    """further tables of the reference's convolution tests through the primitive's own arguments: padding_above / below,
    input offset, output padding, one weights / bias primitive per part of a split, groups, negative slope"""
    p = kat.api_problem(case, K["indexing"])
    b, f, h, w = p["x"].shape
    prims = [cl.input_layout("input", cl.layout(cl.DT_OF[p["x"].dtype], F.bfyx, cl.tensor(b, f, w, h)))]
    wid, bid = [], []
    for i, (wp, bp) in enumerate(zip(p["w_parts"], p["bias_parts"])):
        prims += [cl.data(f"weights{i}", cl.make_memory(eng, np.ascontiguousarray(wp))), cl.data(f"biases{i}", vec_mem(eng, bp))]
        wid.append(f"weights{i}"), bid.append(f"biases{i}")
    lo, up = p["out_pad_lower"], p["out_pad_upper"]
    prims.append(cl.convolution("conv", "input", wid, bid, stride=cl.tensor(1, 1, p["stride"][1], p["stride"][0]),
                                input_offset=yx((-p["pad"][0], -p["pad"][1])), groups=p["groups"],
                                with_activation=p["act"] == "relu", activation_slp=p["act_slope"],
                                padding_above=yx(p["pad_above"]), padding_below=yx(p["pad_below"]),
                                output_padding=cl.padding((0, 0, lo[0], lo[1]), (0, 0, up[0], up[1]))))
    net, outs = run(eng, cl.topology(*prims), {"input": cl.make_memory(eng, p["x"])}, optimize)
    mem = outs["conv"].get_memory()
    l = mem.get_layout()
    assert [l.padding.lower_size.sizes[i] for i in (3, 2)] == list(lo) and [l.padding.upper_size.sizes[i] for i in (3, 2)] == list(up)
    kat.assert_close_where_given(mem.read(), p["expected"], p["tol"])


@pytest.mark.parametrize("optimize", OPT, ids=["plain", "optimize_data"])
@pytest.mark.parametrize("case", [c for c in K["quantized_recipe"] if c["scale"] != "two_layers"], ids=lambda c: c["name"])
def test_kat_quantized_recipe(eng, case, optimize):
    """reference convolution_gpu_test.cpp:3741-3969: a float network gives the scale, the int8 network must come within 3"""
    x = np.array(case["input"], np.float32).reshape(case["in_shape"])
    wf = np.array(case["weights_f"], np.float32).reshape(case["w_shape"])
    bias = np.array(case["bias"], np.float32)
    b, f, h, w = x.shape
    stride = cl.tensor(0, 0, case["stride"][1], case["stride"][0])  # the test passes { 0, 0, 1, 2 }
    tf = cl.topology(cl.input_layout("input_f", cl.layout(DT.f32, F.bfyx, cl.tensor(b, f, w, h))), cl.data("weights_f", cl.make_memory(eng, wf)),
                     cl.data("biases", vec_mem(eng, bias)), cl.convolution("conv_f", "input_f", ["weights_f"], ["biases"], stride=stride))
    net_f, outs_f = run(eng, tf, {"input_f": cl.make_memory(eng, x)}, optimize)
    fl = outs_f["conv_f"].get_memory().read()
    np.testing.assert_allclose(fl, np.array(case["float_output"], np.float32).reshape(case["out_shape"]), atol=1e-4)
    wq, wqf = kat.quantize_weights(wf)
    prims = [cl.input_layout("input", cl.layout(DT.i8, F.bfyx, cl.tensor(b, f, w, h))), cl.data("weights", cl.make_memory(eng, wq.astype(np.int8))),
             cl.data("biases", vec_mem(eng, bias)), cl.data("w_qfs", vec_mem(eng, wqf))]
    if case["scale"] == "single":
        scale = np.float32(127.0) / np.abs(fl).max()
        prims.append(cl.convolution("conv", "input", ["weights"], ["biases"], ["w_qfs"], None, 1.0, float(scale), stride=stride))
    else:
        scale = kat.calibrate(fl)
        prims += [cl.data("out_calibrations", vec_mem(eng, scale)),
                  cl.convolution("conv", "input", ["weights"], ["biases"], ["w_qfs"], ["out_calibrations"], 1.0, stride=stride)]
    net, outs = run(eng, cl.topology(*prims), {"input": cl.make_memory(eng, x.astype(np.int8))}, optimize)
    out = outs["conv"].get_memory().read()
    assert out.dtype == np.int8
    assert np.abs(out.astype(np.float64) / np.reshape(scale, (1, -1, 1, 1)) - fl).max() <= case["tol"]


@pytest.mark.parametrize("optimize", OPT, ids=["plain", "optimize_data"])
def test_kat_calibration_advance(eng, optimize):
    """reference convolution_gpu_test.cpp:4199-4343: two convolutions, calibration of the first divided out of the second's
    weights, both outputs requested; int8 network within 3 of the float network"""
    case = next(c for c in K["quantized_recipe"] if c["scale"] == "two_layers")
    x = np.array(case["input"], np.float32).reshape(case["in_shape"])
    w1 = np.array(case["weights_f"], np.float32).reshape(case["w_shape"])
    w2 = np.array(case["weights_f_2"], np.float32).reshape(case["w2_shape"])
    b1, b2 = np.array(case["bias"], np.float32), np.array(case["bias_2"], np.float32)
    b, f, h, w = x.shape
    s1, s2 = cl.tensor(0, 0, case["stride"][1], case["stride"][0]), cl.tensor(0, 0, case["stride_2"][1], case["stride_2"][0])
    tf = cl.topology(cl.input_layout("input_f", cl.layout(DT.f32, F.bfyx, cl.tensor(b, f, w, h))),
                     cl.data("weights_f", cl.make_memory(eng, w1)), cl.data("biases", vec_mem(eng, b1)),
                     cl.data("weights_f_2", cl.make_memory(eng, w2)), cl.data("biases_2", vec_mem(eng, b2)),
                     cl.convolution("conv_f", "input_f", ["weights_f"], ["biases"], stride=s1),
                     cl.convolution("conv_f_2", "conv_f", ["weights_f_2"], ["biases_2"], stride=s2))
    net_f = cl.network(eng, tf, cl.build_options(optimize_data=optimize, outputs=["conv_f", "conv_f_2"]))
    net_f.set_input_data("input_f", cl.make_memory(eng, x))
    outs_f = net_f.execute()
    assert sorted(outs_f) == ["conv_f", "conv_f_2"]
    f1, f2 = outs_f["conv_f"].get_memory().read(), outs_f["conv_f_2"].get_memory().read()
    np.testing.assert_allclose(f1, rc.conv(x, w1, b1, stride=tuple(case["stride"])), atol=1e-4)
    c1, c2 = kat.calibrate(f1), kat.calibrate(f2)
    w2c = w2 / c1.reshape(1, -1, 1, 1)  # apply_calibration_on_weights (:3618-3632): per INPUT feature
    q1, wqf1 = kat.quantize_weights(w1)
    q2, wqf2 = kat.quantize_weights(w2c)
    t = cl.topology(cl.input_layout("input", cl.layout(DT.i8, F.bfyx, cl.tensor(b, f, w, h))),
                    cl.data("weights", cl.make_memory(eng, q1.astype(np.int8))), cl.data("biases", vec_mem(eng, b1)),
                    cl.data("weights_2", cl.make_memory(eng, q2.astype(np.int8))), cl.data("biases_2", vec_mem(eng, b2)),
                    cl.data("w_qf", vec_mem(eng, wqf1)), cl.data("w_qf_2", vec_mem(eng, wqf2)),
                    cl.data("calib", vec_mem(eng, c1)), cl.data("calib_2", vec_mem(eng, c2)),
                    cl.convolution("conv", "input", ["weights"], ["biases"], ["w_qf"], ["calib"], 1.0, stride=s1),
                    cl.convolution("conv_2", "conv", ["weights_2"], ["biases_2"], ["w_qf_2"], ["calib_2"], 1.0, stride=s2))
    net = cl.network(eng, t, cl.build_options(optimize_data=optimize, outputs=["conv", "conv_2"]))
    net.set_input_data("input", cl.make_memory(eng, x.astype(np.int8)))
    outs = net.execute()
    assert sorted(outs) == ["conv", "conv_2"]
    o2 = outs["conv_2"].get_memory().read()
    assert np.abs(o2.astype(np.float64) / c2.reshape(1, -1, 1, 1) - f2).max() <= case["tol"]
    # and bit-exact against the oracle run layer by layer
    r1 = rc.conv(x.astype(np.int8), q1.astype(np.int8), b1, wqf=wqf1, calib=c1, stride=tuple(case["stride"]), out_dt="s8")
    r2 = rc.conv(r1, q2.astype(np.int8), b2, wqf=wqf2, calib=c2, stride=tuple(case["stride_2"]), out_dt="s8")
    np.testing.assert_array_equal(outs["conv"].get_memory().read(), r1)
    np.testing.assert_array_equal(o2, r2)


FUSE_INPUT = [1.0, 2.0, -15.0, 3.0, 4.0, -15.0, 5.0, 6.0, -15.0, 7.0, -15.0, 0.0, 0.0, -15.0, 0.5, -0.5, -15.0, 8.0, 1.5, 5.2]


@pytest.mark.parametrize("with_reorder", [True, False], ids=["basic_0", "dont_fuse_if_conv_elt_are_outputs"])
def test_conv_eltwise_float_graphs(eng, with_reorder):
    """reference fused_conv_eltwise_gpu_test.cpp:41-118: a float 1x1 convolution summed with its own input, optimised build;
    the reference asserts the output's id and layout, the values here are input + w * input"""
    x = np.array(FUSE_INPUT, np.float32).reshape(1, 1, 5, 4)
    wv = np.array([[[[2.5]]]], np.float32)
    prims = [cl.input_layout("input", cl.layout(DT.f32, F.bfyx, cl.tensor(1, 1, 4, 5))), cl.data("weights", cl.make_memory(eng, wv)),
             cl.convolution("conv", "input", ["weights"])]
    if with_reorder:
        prims += [cl.eltwise("eltwise", "input", "conv", cl.eltwise_mode.sum), cl.reorder("out", "eltwise", F.bfyx, DT.f32)]
    else:
        prims += [cl.eltwise("out", "input", "conv", cl.eltwise_mode.sum)]
    net, outs = run(eng, cl.topology(*prims), {"input": cl.make_memory(eng, x)}, True)
    assert list(outs) == ["out"]
    mem = outs["out"].get_memory()
    l = mem.get_layout()
    assert l.format == F.bfyx and [l.size.sizes[i] for i in range(4)] == [1, 1, 4, 5]
    np.testing.assert_allclose(mem.read(), x + 2.5 * x, rtol=1e-6)


def test_three_convolutions_same_weights(eng):
    """reference convolution_gpu_test.cpp:762-824: one weights primitive feeds three chained 1x1 convolutions"""
    x = np.ones((1, 2, 2, 2), np.float32)
    t = cl.topology(cl.input_layout("input", cl.layout(DT.f32, F.bfyx, cl.tensor(1, 2, 2, 2))),
                    cl.data("weights", cl.make_memory(eng, np.ones((2, 2, 1, 1), np.float32))),
                    cl.convolution("conv1", "input", ["weights"]), cl.convolution("conv2", "conv1", ["weights"]),
                    cl.convolution("conv3", "conv2", ["weights"]))
    net, outs = run(eng, t, {"input": cl.make_memory(eng, x)}, True)
    out = outs["conv3"].get_memory().read()
    assert out.shape == (1, 2, 2, 2) and np.all(out == 8.0)


def test_with_output_size_same_input(eng):
    """reference convolution_gpu_test.cpp:737-760: two convolutions with user-given output sizes read one input; both
    are outputs, in the order of their ids"""
    r = np.random.default_rng(5)
    x = r.standard_normal((1, 4, 320, 320)).astype(np.float32)
    w1, w2 = (r.standard_normal((64, 4, 7, 7)).astype(np.float32) for _ in range(2))
    t = cl.topology(cl.input_layout("input", cl.layout(DT.f32, F.bfyx, cl.tensor(1, 4, 320, 320))),
                    cl.data("weights", cl.make_memory(eng, w1)), cl.data("weights2", cl.make_memory(eng, w2)),
                    cl.convolution("conv1", "input", ["weights"], stride=cl.tensor(1, 1, 2, 2), input_offset=cl.tensor(0, 0, -3, -3, 0),
                                   output_size=cl.tensor(1, 64, 160, 160)),
                    cl.convolution("conv2", "input", ["weights2"], stride=cl.tensor(1, 1, 1, 1), input_offset=cl.tensor(0, 0, -3, -3, 0),
                                   output_size=cl.tensor(1, 64, 320, 320)))
    net, outs = run(eng, t, {"input": cl.make_memory(eng, x)}, False)
    assert sorted(outs) == ["conv1", "conv2"]
    o1 = outs["conv1"].get_memory().read()
    assert o1.shape == (1, 64, 160, 160) and outs["conv2"].get_memory().read().shape == (1, 64, 320, 320)
    np.testing.assert_allclose(o1[:, :4], rc.conv(x, w1[:4], None, stride=(2, 2), pad=(3, 3)), rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("optimize", OPT, ids=["plain", "optimize_data"])
@pytest.mark.parametrize("offset,stride", [((1, 2), 1), ((2, 0), 2), ((1, -1), 1)], ids=["x1y2", "x2_s2", "x1_ypad1"])
def test_positive_input_offset(eng, offset, stride, optimize):
    """a positive input offset moves the origin into the data: the convolution runs on the view that leaves `offset`
    elements out on both sides (reference src/gpu/convolution_gpu.cpp:94-98, sliding_window_utils.h:113-126)"""
    r = np.random.default_rng(31)
    B, Cn, H, W, OFM = 2, 64, 11, 14, 64
    x = r.integers(-128, 128, (B, Cn, H, W)).astype(np.int8)
    w = r.integers(-127, 128, (OFM, Cn, 3, 3)).astype(np.int8)
    cal = r.uniform(2e-4, 8e-4, OFM).astype(np.float32)
    ox, oy = offset
    t = cl.topology(cl.input_layout("input", cl.layout(DT.i8, F.bfyx, cl.tensor(B, Cn, W, H))), cl.data("w", cl.make_memory(eng, w)),
                    cl.data("q", vec_mem(eng, np.ones(OFM, np.float32))), cl.data("c", vec_mem(eng, cal)),
                    cl.convolution("conv", "input", ["w"], None, ["q"], ["c"], stride=cl.tensor(1, 1, stride, stride),
                                   input_offset=cl.tensor(0, 0, ox, oy, 0), with_activation=True))
    net, outs = run(eng, t, {"input": cl.make_memory(eng, x)}, optimize)
    vy, vx = max(oy, 0), max(ox, 0)
    view = x[:, :, vy:H - vy, vx:W - vx]
    ref = rc.conv(view, w, None, wqf=np.ones(OFM, np.float32), calib=cal, stride=(stride, stride), pad=(max(-oy, 0), max(-ox, 0)), act="relu")
    got = outs["conv"].get_memory().read()
    assert got.shape == ref.shape
    np.testing.assert_array_equal(got, ref)
    # the view must not be the whole tensor shifted: the last rows / columns are left out as well
    assert ref.shape[3] == (W - 2 * vx + 2 * max(-ox, 0) - 3) // stride + 1


# ------------------------------------------------------------------------------------------ networks vs the oracle
def rand_layer(r, ofm, ifm, k, in_u8=True):
    w = r.integers(-127, 128, (ofm, ifm, k, k)).astype(np.int8)
    bias = r.integers(-1000, 1001, ofm).astype(np.int32)
    sigma = np.sqrt(ifm * k * k) * (147.4 if in_u8 else 73.9) * 73.3
    calib = (40.0 / sigma * r.uniform(0.5, 2.0, ofm)).astype(np.float32)
    return w, bias, np.ones(ofm, np.float32), calib


def bottleneck(eng, seed, B=2, C=64, M=32, H=14, W=14, unsigned=False):
    """1x1 reduce -> 3x3 -> 1x1 expand + shortcut, relu: one ResNet bottleneck block.

    Signed activations by default: the reference's stand-alone quantized eltwise saturates to the signed range
    (generic_eltwise_ref.cl:318-330, convert_char_sat), so only then do the fused and the two-primitive graph agree."""
    r = np.random.default_rng(seed)
    np_dt, dt, name = (np.uint8, DT.u8, "u8") if unsigned else (np.int8, DT.i8, "s8")
    x = (r.integers(0, 256, (B, C, H, W)) if unsigned else r.integers(-128, 128, (B, C, H, W))).astype(np_dt)
    L = [rand_layer(r, M, C, 1, unsigned), rand_layer(r, M, M, 3, unsigned), rand_layer(r, C, M, 1, unsigned)]
    ecal = r.uniform(0.4, 0.9, C).astype(np.float32)
    prims = [cl.input_layout("input", cl.layout(dt, F.bfyx, cl.tensor(B, C, W, H)))]
    for i, (w, b, q, c) in enumerate(L):
        prims += [cl.data(f"w{i}", cl.make_memory(eng, w)), cl.data(f"b{i}", vec_mem(eng, b)), cl.data(f"q{i}", vec_mem(eng, q)),
                  cl.data(f"c{i}", vec_mem(eng, c))]
    prims += [cl.data("ecal", vec_mem(eng, ecal)),
              cl.convolution("reduce", "input", ["w0"], ["b0"], ["q0"], ["c0"]),
              cl.activation("reduce_relu", "reduce", cl.activation_func.relu),
              cl.convolution("mid", "reduce_relu", ["w1"], ["b1"], ["q1"], ["c1"], input_offset=cl.tensor(0, 0, -1, -1, 0),
                             with_activation=True),
              cl.convolution("expand", "mid", ["w2"], ["b2"], ["q2"], ["c2"], output_data_type=DT.i8),
              cl.eltwise("sum", "input", "expand", cl.eltwise_mode.sum, True, 0.0, output_calibration_factors="ecal"),
              cl.reorder("out", "sum", F.bfyx)]

    def oracle():
        a = rc.conv(x, L[0][0], L[0][1], wqf=L[0][2], calib=L[0][3], out_dt=name, act="relu")
        a = rc.conv(a, L[1][0], L[1][1], wqf=L[1][2], calib=L[1][3], pad=(1, 1), out_dt=name, act="relu")
        return rc.conv(a, L[2][0], L[2][1], wqf=L[2][2], calib=L[2][3], out_dt=name, eltw=x, eltw_act="relu", eltw_calib=ecal)

    return cl.topology(*prims), x, oracle


@pytest.mark.parametrize("optimize", OPT, ids=["plain", "optimize_data"])
def test_bottleneck_block(eng, optimize):
    topo, x, oracle = bottleneck(eng, 7)
    net, outs = run(eng, topo, {"input": cl.make_memory(eng, x)}, optimize)
    out = outs["out"].get_memory().read()
    expected = oracle()
    assert out.dtype == np.int8 and out.shape == expected.shape
    np.testing.assert_array_equal(out, expected)
    executed = net.get_executed_primitive_ids()
    if optimize:
        # the graph the layout rule and the fusing passes produce: blocked int8 matrix-core kernels throughout
        assert "reduce_relu" not in executed and "sum" not in executed and "expand_fused_sum" in executed
        for pid in ("reduce", "mid", "expand_fused_sum"):
            info = net.get_primitive_info(pid)
            assert info["format"] == F.fs_b_yx_fsv16 and info["kernel"].startswith(("conv_mfma", "conv_stream")), info
        assert "border" in net.get_primitive_info("mid")["kernel"]
    else:
        assert {"reduce", "reduce_relu", "mid", "expand", "sum", "out"} <= set(executed)
        assert net.get_primitive_info("mid")["kernel"].startswith("conv_ref")
    assert net.get_all_primitive_org_ids()[0] == "input"


def test_unsigned_bottleneck_block(eng):
    """Unsigned activations with a signed expand convolution: the data types of the benchmark's residual blocks."""
    topo, x, oracle = bottleneck(eng, 8, unsigned=True)
    net, outs = run(eng, topo, {"input": cl.make_memory(eng, x)}, True)
    out = outs["out"].get_memory().read()
    assert out.dtype == np.uint8 and out.max() > 127
    np.testing.assert_array_equal(out, oracle())


def test_fused_and_unfused_graphs_agree(eng):
    """conv + eltwise executed as two primitives equals the fused primitive (the property the reference's fusing pass
    relies on, src/graph_optimizer/prepare_primitive_fusing.cpp:181-337)."""
    topo, x, _ = bottleneck(eng, 11, B=3, C=48, M=16, H=9, W=11)
    outs = []
    for optimize in OPT:
        net, o = run(eng, topo, {"input": cl.make_memory(eng, x)}, optimize)
        outs.append(o["out"].get_memory().read())
    np.testing.assert_array_equal(outs[0], outs[1])


@pytest.mark.parametrize("optimize", OPT, ids=["plain", "optimize_data"])
def test_unquantized_int8_convolution_keeps_its_sum_unfused(eng, optimize):
    """an int8 1x1 convolution without quantization factors stays on the plain-layout kernel (its accumulator is the
    8-bit type, wrap-around included, fused_conv_eltwise_gpu_ref.cl:43-48) and, as in the reference
    (prepare_primitive_fusing.cpp:197-205), its relu sum stays a primitive of its own: the sum adds to the int8 tensor
    the convolution wrote.  The fused primitive would accumulate in int and give other numbers on this data."""
    r = np.random.default_rng(23)
    B, Cn, H, W = 2, 32, 6, 7
    x = r.integers(-128, 128, (B, Cn, H, W)).astype(np.int8)
    w = r.integers(-3, 4, (Cn, Cn, 1, 1)).astype(np.int8)
    ecal = r.uniform(0.4, 0.9, Cn).astype(np.float32)
    t = cl.topology(cl.input_layout("input", cl.layout(DT.i8, F.bfyx, cl.tensor(B, Cn, W, H))), cl.data("w", cl.make_memory(eng, w)),
                    cl.data("e", vec_mem(eng, ecal)),
                    cl.convolution("conv", "input", ["w"]),
                    cl.eltwise("sum", "input", "conv", cl.eltwise_mode.sum, True, 0.0, output_calibration_factors="e"),
                    cl.reorder("out", "sum", F.bfyx))
    net, outs = run(eng, t, {"input": cl.make_memory(eng, x)}, optimize)
    conv = rc.conv(x, w, None)  # 8-bit accumulation
    exact = np.einsum("bchw,fc->bfhw", x.astype(np.int64), w[:, :, 0, 0].astype(np.int64))
    assert np.count_nonzero(conv.astype(np.int64) != exact) > conv.size // 4  # it does wrap around
    expected = rc.eltwise_sum(x, conv, calib=ecal, relu=True)
    np.testing.assert_array_equal(outs["out"].get_memory().read(), expected)
    executed = net.get_executed_primitive_ids()
    assert "conv" in executed and "sum" in executed


@pytest.mark.parametrize("optimize", OPT, ids=["plain", "optimize_data"])
def test_grouped_quantized_convolution_through_network(eng, optimize):
    """groups = 4 with quantization: as written on the plain-layout kernel, with optimize_data blocked on the matrix-core
    kernels (block-diagonal weights); same numbers, those of the oracle's grouped convolution"""
    r = np.random.default_rng(29)
    B, Cn, OFM, H, W, G = 2, 64, 96, 9, 8, 4
    x = r.integers(-128, 128, (B, Cn, H, W)).astype(np.int8)
    w = r.integers(-127, 128, (OFM, Cn // G, 3, 3)).astype(np.int8)
    bias = r.integers(-1000, 1001, OFM).astype(np.int32)
    cal = (40.0 / (np.sqrt(Cn // G * 9) * 73.9 * 73.3) * r.uniform(0.5, 2.0, OFM)).astype(np.float32)
    t = cl.topology(cl.input_layout("input", cl.layout(DT.i8, F.bfyx, cl.tensor(B, Cn, W, H))), cl.data("w", cl.make_memory(eng, w)),
                    cl.data("b", vec_mem(eng, bias)), cl.data("q", vec_mem(eng, np.ones(OFM, np.float32))), cl.data("c", vec_mem(eng, cal)),
                    cl.convolution("conv", "input", ["w"], ["b"], ["q"], ["c"], groups=G, input_offset=cl.tensor(0, 0, -1, -1, 0),
                                   with_activation=True),
                    cl.reorder("out", "conv", F.bfyx))
    net, outs = run(eng, t, {"input": cl.make_memory(eng, x)}, optimize)
    expected = rc.conv(x, w, bias, wqf=np.ones(OFM, np.float32), calib=cal, groups=G, pad=(1, 1), out_dt="s8", act="relu")
    np.testing.assert_array_equal(outs["out"].get_memory().read(), expected)
    kernel = net.get_primitive_info("conv")["kernel"]
    assert kernel.startswith("conv_ref") != bool(optimize), kernel


def test_closer_writes_over_its_shortcut_without_a_memory_pool():
    """prepare_conv_eltw_read_write_opt (reference prepare_primitive_fusing.cpp:468-534): the fused closer of a block whose
    shortcut is an intermediate tensor of the same layout, read by nothing later, takes the shortcut's buffer as its
    output.  Applied on engines without a memory pool; same numbers either way, over repeated runs."""
    r = np.random.default_rng(21)
    B, C, M, H, W = 2, 64, 32, 10, 12
    x = r.integers(-128, 128, (B, C, H, W)).astype(np.int8)
    L = [rand_layer(r, C, C, 1, False), rand_layer(r, M, C, 1, False), rand_layer(r, M, M, 3, False), rand_layer(r, C, M, 1, False)]
    ecal = r.uniform(0.4, 0.9, C).astype(np.float32)
    results = {}
    for pool in (False, True):
        e = cl.engine(enable_memory_pool=pool)
        prims = [cl.input_layout("input", cl.layout(DT.i8, F.bfyx, cl.tensor(B, C, W, H))), cl.data("ecal", vec_mem(e, ecal))]
        for i, (w, b, q, c) in enumerate(L):
            prims += [cl.data(f"w{i}", cl.make_memory(e, w)), cl.data(f"b{i}", vec_mem(e, b)), cl.data(f"q{i}", vec_mem(e, q)), cl.data(f"c{i}", vec_mem(e, c))]
        prims += [cl.convolution("shortcut", "input", ["w0"], ["b0"], ["q0"], ["c0"], with_activation=True),
                  cl.convolution("reduce", "shortcut", ["w1"], ["b1"], ["q1"], ["c1"], with_activation=True),
                  cl.convolution("mid", "reduce", ["w2"], ["b2"], ["q2"], ["c2"], input_offset=cl.tensor(0, 0, -1, -1, 0), with_activation=True),
                  cl.convolution("expand", "mid", ["w3"], ["b3"], ["q3"], ["c3"], output_data_type=DT.i8),
                  cl.eltwise("sum", "shortcut", "expand", cl.eltwise_mode.sum, True, 0.0, output_calibration_factors="ecal"),
                  cl.pooling("pool", "sum", cl.pooling_mode.max, cl.tensor(1, 1, 2, 2), cl.tensor(1, 1, 2, 2))]
        net = cl.network(e, cl.topology(*prims), cl.build_options(optimize_data=True))
        info = net.get_primitive_info("expand_fused_sum")
        assert bool(info.get("second_input_in_output")) == (not pool)
        for k in range(3):
            xk = np.roll(x, k, axis=3)
            net.set_input_data("input", cl.make_memory(e, xk))
            results[pool, k] = net.execute()["pool"].get_memory().read()
    for k in range(3):
        xk = np.roll(x, k, axis=3)
        s = rc.conv(xk, L[0][0], L[0][1], wqf=L[0][2], calib=L[0][3], out_dt="s8", act="relu")
        a = rc.conv(s, L[1][0], L[1][1], wqf=L[1][2], calib=L[1][3], out_dt="s8", act="relu")
        a = rc.conv(a, L[2][0], L[2][1], wqf=L[2][2], calib=L[2][3], pad=(1, 1), out_dt="s8", act="relu")
        a = rc.conv(a, L[3][0], L[3][1], wqf=L[3][2], calib=L[3][3], out_dt="s8", eltw=s, eltw_act="relu", eltw_calib=ecal)
        ref = rc.pool(a, "max", (2, 2), stride=(2, 2))
        np.testing.assert_array_equal(results[False, k], ref)
        np.testing.assert_array_equal(results[True, k], ref)


def test_network_runs_again_with_new_input(eng):
    topo, x, _ = bottleneck(eng, 3)
    net = cl.network(eng, topo, cl.build_options(optimize_data=True))
    net.set_input_data("input", cl.make_memory(eng, x))
    first = net.execute()["out"].get_memory().read()
    net.set_input_data("input", cl.make_memory(eng, np.zeros_like(x)))
    second = net.execute()["out"].get_memory().read()
    net.set_input_data("input", cl.make_memory(eng, x))
    third = net.execute()["out"].get_memory().read()
    assert not np.array_equal(first, second)
    np.testing.assert_array_equal(first, third)


def test_user_blocked_input_and_padded_input(eng):
    """An input the user already holds in fs_b_yx_fsv16 is consumed in place; a bfyx input with physical padding is read
    through its pitches (reference tests: input padding variants of convolution_gpu_test.cpp)."""
    r = np.random.default_rng(5)
    x = r.integers(-128, 128, (2, 32, 6, 7)).astype(np.int8)
    w, b, q, c = rand_layer(r, 32, 32, 3, in_u8=False)
    expected = rc.conv(x, w, b, wqf=q, calib=c, pad=(1, 1), out_dt="s8", act="relu")
    consts = [cl.data("w", cl.make_memory(eng, w)), cl.data("b", vec_mem(eng, b)), cl.data("q", vec_mem(eng, q)),
              cl.data("c", vec_mem(eng, c))]
    conv = cl.convolution("conv", "input", ["w"], ["b"], ["q"], ["c"], input_offset=cl.tensor(0, 0, -1, -1, 0), with_activation=True)
    pad = cl.padding((0, 0, 2, 3), (0, 0, 1, 0))
    lay = cl.layout(DT.i8, F.bfyx, cl.tensor(2, 32, 7, 6), pad)
    m = cl.memory.allocate(eng, lay)
    m.write(x)
    for optimize in OPT:
        net, outs = run(eng, cl.topology(cl.input_layout("input", lay), conv, *consts), {"input": m}, optimize)
        np.testing.assert_array_equal(outs["conv"].get_memory().read(), expected)
    # blocked by the user: stage it with a reorder network first
    stage = cl.topology(cl.input_layout("input", cl.layout(DT.i8, F.bfyx, cl.tensor(2, 32, 7, 6))),
                        cl.reorder("blocked", "input", F.fs_b_yx_fsv16))
    _, so = run(eng, stage, {"input": cl.make_memory(eng, x)}, False)
    xb = so["blocked"].get_memory()
    assert xb.get_layout().format == F.fs_b_yx_fsv16
    topo = cl.topology(cl.input_layout("input", xb.get_layout()), conv, *consts, cl.reorder("plain", "conv", F.bfyx))
    net, outs = run(eng, topo, {"input": xb}, True)
    assert "input_to_fsv16_0" not in net.get_all_primitive_ids()
    np.testing.assert_array_equal(outs["plain"].get_memory().read(), expected)


def test_first_layer_through_network(eng):
    """3-channel image -> 7x7 stride-2 quantized convolution: with optimize_data the input goes through b_fs_yx_fsv4."""
    r = np.random.default_rng(12)
    x = r.integers(0, 256, (2, 3, 30, 30)).astype(np.uint8)
    w = r.integers(-127, 128, (32, 3, 7, 7)).astype(np.int8)
    b = r.integers(-500, 500, 32).astype(np.int32)
    q = np.ones(32, np.float32)
    c = (40.0 / (np.sqrt(147) * 147.4 * 73.3) * r.uniform(0.5, 2, 32)).astype(np.float32)
    expected = rc.conv(x, w, b, wqf=q, calib=c, pad=(3, 3), stride=(2, 2), out_dt="s8", act="relu")
    topo = cl.topology(cl.input_layout("input", cl.layout(DT.u8, F.bfyx, cl.tensor(2, 3, 30, 30))),
                       cl.data("w", cl.make_memory(eng, w)), cl.data("b", vec_mem(eng, b)), cl.data("q", vec_mem(eng, q)),
                       cl.data("c", vec_mem(eng, c)),
                       cl.convolution("stem", "input", ["w"], ["b"], ["q"], ["c"], stride=cl.tensor(1, 1, 2, 2),
                                      input_offset=cl.tensor(0, 0, -3, -3, 0), with_activation=True, output_data_type=DT.i8))
    for optimize in OPT:
        net, outs = run(eng, topo, {"input": cl.make_memory(eng, x)}, optimize)
        np.testing.assert_array_equal(outs["stem"].get_memory().read(), expected)
    assert "stem_p" in net.get_primitive_info("stem_fsv16")["kernel"]
    assert net.get_primitive_info("input_to_fsv4_0")["format"] == F.b_fs_yx_fsv4


def test_depthwise_through_network(eng):
    r = np.random.default_rng(9)
    C = 32
    x = r.integers(0, 256, (2, C, 10, 10)).astype(np.uint8)
    w = r.integers(-127, 128, (C, 1, 3, 3)).astype(np.int8)
    b = r.integers(-500, 500, C).astype(np.int32)
    q = np.ones(C, np.float32)
    c = (40.0 / (3 * 147.4 * 73.3) * r.uniform(0.5, 2, C)).astype(np.float32)
    expected = rc.conv(x, w, b, wqf=q, calib=c, pad=(1, 1), stride=(2, 2), groups=C, out_dt="u8", act="relu")
    topo = cl.topology(cl.input_layout("input", cl.layout(DT.u8, F.bfyx, cl.tensor(2, C, 10, 10))),
                       cl.data("w", cl.make_memory(eng, w)), cl.data("b", vec_mem(eng, b)), cl.data("q", vec_mem(eng, q)),
                       cl.data("c", vec_mem(eng, c)),
                       cl.convolution("dw", "input", ["w"], ["b"], ["q"], ["c"], stride=cl.tensor(1, 1, 2, 2),
                                      input_offset=cl.tensor(0, 0, -1, -1, 0), with_activation=True, groups=C))
    for optimize in OPT:
        net, outs = run(eng, topo, {"input": cl.make_memory(eng, x)}, optimize)
        np.testing.assert_array_equal(outs["dw"].get_memory().read(), expected)
    assert net.get_primitive_info("dw_fsv16")["kernel"].startswith("conv_dw")


def test_attached_constants_and_input(eng):
    """Host memory attached with cldnn_attach_memory serves as constants and as network input."""
    r = np.random.default_rng(2)
    x = r.integers(-128, 128, (1, 16, 5, 5)).astype(np.int8)
    w, b, q, c = rand_layer(r, 16, 16, 1, in_u8=False)

    def att(a, shape):
        a = np.ascontiguousarray(a)
        return cl.memory.attach(cl.layout(cl.DT_OF[a.dtype], F.bfyx, cl.tensor(*shape)), a)

    topo = cl.topology(cl.input_layout("input", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 16, 5, 5))),
                       cl.data("w", att(w, (16, 16, 1, 1))), cl.data("b", att(b, (1, 1, 16, 1))),
                       cl.data("q", att(q, (1, 1, 16, 1))), cl.data("c", att(c, (1, 1, 16, 1))),
                       cl.convolution("conv", "input", ["w"], ["b"], ["q"], ["c"]))
    net, outs = run(eng, topo, {"input": att(x, (1, 16, 5, 5))}, True)
    np.testing.assert_array_equal(outs["conv"].get_memory().read(), rc.conv(x, w, b, wqf=q, calib=c, out_dt="s8"))


def test_cpp_api_program():
    """The same path through the C++ wrappers: tests/cpp/conv_network_test.cpp compares five networks with the oracle."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "cpp", "conv_network_test")
    if not os.path.exists(exe):
        subprocess.run(["make", "-C", os.path.dirname(exe), "conv_network_test"], check=True)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0 and "all cases passed" in r.stdout, r.stdout + r.stderr


# ------------------------------------------------------------------------------------------ runtime objects
def test_memory_lock_roundtrip_and_identity(eng):
    a = np.arange(2 * 3 * 4 * 5, dtype=np.float32).reshape(2, 3, 4, 5)
    for fmt in (F.bfyx, F.yxfb, F.byxf):
        m = cl.make_memory(eng, a, fmt)
        np.testing.assert_array_equal(m.read(), a)
    m2 = cl.memory.allocate(eng, m.get_layout())
    assert m.is_the_same_buffer(m) and not m.is_the_same_buffer(m2)
    assert np.count_nonzero(m2.read()) == 0  # fresh memory is zero-filled
    assert eng.get_temp_used_device_memory_size() > 0
    assert eng.get_max_used_device_memory_size() >= eng.get_temp_used_device_memory_size()
    info = eng.get_info()
    assert info.cores_count >= 64 and info.supports_immad == 1 and info.max_global_mem_size > (1 << 34)


def test_set_input_errors(eng):
    topo, x, _ = bottleneck(eng, 1)
    net = cl.network(eng, topo)
    with pytest.raises(cl.error) as e:
        net.execute()
    assert "has not been set" in str(e.value)
    with pytest.raises(cl.error) as e:
        net.set_input_data("input", cl.make_memory(eng, x[:1]))
    assert "layout" in str(e.value)
    with pytest.raises(cl.error):
        net.set_input_data("mid", cl.make_memory(eng, x))
    with pytest.raises(cl.error):
        cl._call("cldnn_get_network_output_memory", net.h, b"out")  # not executed yet


def test_events_and_profiling():
    eng = cl.engine(enable_profiling=True)
    topo, x, oracle = bottleneck(eng, 4)
    net = cl.network(eng, topo, cl.build_options(optimize_data=True))
    net.set_input_data("input", cl.make_memory(eng, x))
    gate = cl.event.create_user_event(eng)
    assert gate.is_user_event()
    gate.set()
    outs = net.execute([gate])
    ev = outs["out"].get_event()
    ev.wait()
    prof = ev.get_profiling_info()
    assert set(prof) == {"submission", "starting", "executing"}
    assert 0 < prof["executing"] < 50_000_000
    np.testing.assert_array_equal(outs["out"].get_memory().read(), oracle())
    fired = []
    cb = cl.EVENT_HANDLER(lambda p: fired.append(1))
    cl._call("cldnn_add_event_handler", ev.h, cb, None)
    assert fired == [1]  # the event is complete: the handler runs at once


@pytest.mark.parametrize("profiling", [False, True], ids=["plain", "profiling"])
def test_execute_behind_a_user_event_that_is_set_afterwards(profiling):
    """reference network::execute enqueues behind its dependency events and returns; an OpenCL user event among them
    may be set later by the same thread.  Here the run is postponed: execute returns at once, the output's event is
    not complete, and the run is submitted when the last gate is set."""
    eng = cl.engine(enable_profiling=profiling)
    topo, x, oracle = bottleneck(eng, 4)
    net = cl.network(eng, topo, cl.build_options(optimize_data=True))
    net.set_input_data("input", cl.make_memory(eng, x))
    gate_a, gate_b = cl.event.create_user_event(eng), cl.event.create_user_event(eng)
    fired = []
    outs = net.execute([gate_a, gate_b])        # returns although neither gate is set
    ev = outs["out"].get_event()
    cb = cl.EVENT_HANDLER(lambda p: fired.append(1))
    cl._call("cldnn_add_event_handler", ev.h, cb, None)
    assert fired == []                           # nothing has run
    assert "expand_fused_sum" in net.get_executed_primitive_ids()
    gate_a.set()
    assert fired == []                           # one gate is still closed
    gate_b.set()                                 # submits the run from this thread
    ev.wait()
    np.testing.assert_array_equal(outs["out"].get_memory().read(), oracle())
    import time
    for _ in range(200):                         # the handler of a stream event is called from a helper thread
        if fired:
            break
        time.sleep(0.01)
    assert fired == [1]
    # the network runs again the ordinary way, and behind a gate that is already open
    x2 = np.roll(x, 1, axis=0)
    net.set_input_data("input", cl.make_memory(eng, x2))
    outs = net.execute([gate_a])
    outs["out"].get_event().wait()
    assert not np.array_equal(x, x2)
    # a postponed run must be submitted before the input can be replaced: set_input_data waits for the gate, so the
    # gate is opened from another thread
    import threading
    gate_c = cl.event.create_user_event(eng)
    net.set_input_data("input", cl.make_memory(eng, x))
    outs = net.execute([gate_c])
    threading.Timer(0.05, gate_c.set).start()
    net.set_input_data("input", cl.make_memory(eng, x2))   # blocks until the timer opens the gate and the run is over
    np.testing.assert_array_equal(outs["out"].get_memory().read(), oracle())


def test_unsupported_requests_fail_loudly(eng):
    lay = cl.layout(DT.f16, F.bfyx, cl.tensor(1, 16, 4, 4))
    with pytest.raises(cl.error) as e:
        cl.memory.allocate(eng, lay)
    assert e.value.status == cl.UNSUPPORTED_FORMAT
    topo = cl.topology(cl.input_layout("input", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 16, 4, 4))),
                       cl.activation("act", "input", cl.activation_func.logistic))
    net = cl.network(eng, topo)
    net.set_input_data("input", cl.make_memory(eng, np.zeros((1, 16, 4, 4), np.int8)))
    with pytest.raises(cl.error) as e:
        net.execute()
    assert "not supported" in str(e.value)


# ------------------------------------------------------------------------------------------ concatenation
def inception_like(eng, seed, B=2, C=32, H=9, W=7, f=(32, 48, 16)):
    """three quantized branches (1x1, 3x3, 3x3) side by side along the features, a 3x3 convolution behind them: what an
    inception block hands to the next one.  The 3x3 behind the concatenation needs a zero border, which the in-place
    form has to give to every branch."""
    r = np.random.default_rng(seed)
    x = r.integers(0, 256, (B, C, H, W)).astype(np.uint8)
    ks = (1, 3, 3)
    L = [rand_layer(r, f[i], C, ks[i]) for i in range(3)] + [rand_layer(r, 24, sum(f), 3)]
    prims = [cl.input_layout("input", cl.layout(DT.u8, F.bfyx, cl.tensor(B, C, W, H)))]
    for i, (w, b, q, c) in enumerate(L):
        prims += [cl.data(f"w{i}", cl.make_memory(eng, w)), cl.data(f"b{i}", vec_mem(eng, b)), cl.data(f"q{i}", vec_mem(eng, q)),
                  cl.data(f"c{i}", vec_mem(eng, c))]
    for i in range(3):
        prims.append(cl.convolution(f"br{i}", "input", [f"w{i}"], [f"b{i}"], [f"q{i}"], [f"c{i}"], with_activation=True,
                                    input_offset=cl.tensor(0, 0, -(ks[i] // 2), -(ks[i] // 2), 0), output_data_type=DT.u8))
    prims += [cl.concatenation("cat", ["br0", "br1", "br2"], cl.concatenation_axis.along_f),
              cl.convolution("next", "cat", ["w3"], ["b3"], ["q3"], ["c3"], with_activation=True, input_offset=cl.tensor(0, 0, -1, -1, 0),
                             output_data_type=DT.u8)]

    def oracle():
        br = [rc.conv(x, L[i][0], L[i][1], wqf=L[i][2], calib=L[i][3], pad=(ks[i] // 2,) * 2, out_dt="u8", act="relu") for i in range(3)]
        cat = np.concatenate(br, axis=1)
        return cat, rc.conv(cat, L[3][0], L[3][1], wqf=L[3][2], calib=L[3][3], pad=(1, 1), out_dt="u8", act="relu")

    return cl.topology(*prims), x, oracle


@pytest.mark.parametrize("optimize", OPT, ids=["plain", "optimize_data"])
def test_concatenation_of_quantized_branches(eng, optimize):
    topo, x, oracle = inception_like(eng, 11)
    net = cl.network(eng, topo, cl.build_options(optimize_data=optimize, outputs=["cat", "next"]) if not optimize
                     else cl.build_options(optimize_data=True))
    net.set_input_data("input", cl.make_memory(eng, x))
    outs = net.execute()
    cat, nxt = oracle()
    np.testing.assert_array_equal(outs["next"].get_memory().read(), nxt)
    info = net.get_primitive_info("cat")
    if optimize:
        # the branches wrote straight into the concatenation's buffer (reference prepare_buffer_fusing.cpp:38-140), each with
        # the border the convolution behind the concatenation needs
        assert info["in_place"] is True and info["format"] == F.fs_b_yx_fsv16 and info["pad_lower"][2:] == [1, 1]
        offs = [net.get_primitive_info(f"br{i}")["concat_offset"] for i in range(3)]
        plane = 2 * (9 + 2) * (7 + 2) * 16  # batch x padded rows x padded pixels x 16 features
        assert offs == [0, 2 * plane, 5 * plane]
        for _ in range(2):  # again: same buffers
            np.testing.assert_array_equal(net.execute()["next"].get_memory().read(), nxt)
    else:
        assert info["in_place"] is False
        np.testing.assert_array_equal(outs["cat"].get_memory().read(), cat)


def test_concatenation_as_an_output_is_in_place_too(eng):
    """the concatenation's own buffer is what the application reads (through the reorder back to its format)"""
    topo, x, oracle = inception_like(eng, 12, B=1, f=(16, 16, 32))
    net = cl.network(eng, topo, cl.build_options(optimize_data=True, outputs=["cat", "next"]))
    net.set_input_data("input", cl.make_memory(eng, x))
    outs = net.execute()
    cat, nxt = oracle()
    np.testing.assert_array_equal(outs["cat"].get_memory().read(), cat)
    np.testing.assert_array_equal(outs["next"].get_memory().read(), nxt)
    assert net.get_primitive_info("cat_fsv16")["in_place"] is True


@pytest.mark.parametrize("dtype", [np.float32, np.int8], ids=["f32", "i8"])
@pytest.mark.parametrize("axis", ["b", "f", "x", "y"])
def test_concatenation_copies_along_every_axis(eng, axis, dtype):
    """inputs that are user memory: one copy per input at its offset (reference src/gpu/concatenation_gpu.cpp:64-90,
    concatenation_gpu_ref.cl:18-46); three inputs of different extent along the axis"""
    r = np.random.default_rng(5)
    ax = "bfyx".index(axis)
    shapes = []
    for extent in (2, 5, 1):
        s = [3, 4, 6, 5]
        s[ax] = extent
        shapes.append(tuple(s))
    arrs = [(r.standard_normal(s) * 50).astype(dtype) for s in shapes]
    dt = DT.f32 if dtype == np.float32 else DT.i8
    prims = [cl.input_layout(f"i{k}", cl.layout(dt, F.bfyx, cl.tensor(s[0], s[1], s[3], s[2]))) for k, s in enumerate(shapes)]
    prims.append(cl.concatenation("cat", ["i0", "i1", "i2"], getattr(cl.concatenation_axis, "along_" + axis)))
    for optimize in OPT:
        net, outs = run(eng, cl.topology(*prims), {f"i{k}": cl.make_memory(eng, a) for k, a in enumerate(arrs)}, optimize)
        np.testing.assert_array_equal(outs["cat"].get_memory().read(), np.concatenate(arrs, axis=ax))
        assert net.get_primitive_info("cat")["in_place"] is False


def test_copy_region_between_layouts():
    """the C-ABI entry behind the copies: a bfyx block into the middle of a padded blocked tensor and back"""
    from cldnn_amd import hip
    e = hip.Engine()
    r = np.random.default_rng(8)
    big = r.integers(-128, 128, (2, 40, 7, 6)).astype(np.int8)
    part = r.integers(-128, 128, (1, 19, 3, 4)).astype(np.int8)
    dst = hip.upload(e, big, "fs_b_yx_fsv16", (1, 2))
    src = hip.upload(e, part, "bfyx")
    hip.check(hip.lib().cldnn_hip_copy_region(e.h, src.ptr, C.byref(src.tensor), dst.ptr, C.byref(dst.tensor), 1, 17, 2, 1))
    want = big.copy()
    want[1:2, 17:36, 2:5, 1:5] = part
    np.testing.assert_array_equal(hip.download(e, dst), want)
    assert hip.lib().cldnn_hip_copy_region(e.h, src.ptr, C.byref(src.tensor), dst.ptr, C.byref(dst.tensor), 1, 22, 2, 1) == -7  # does not fit
    src.close(), dst.close(), e.close()


def projection_block(eng, seed, B=2, C=64, M=32, H=14, W=14, stride=2):
    """a down-sampling ResNet block: the shortcut projection (1x1, no activation) and the opening 1x1 (relu) read the same
    tensor with the same stride -> 3x3 -> 1x1 expand + projection, relu"""
    r = np.random.default_rng(seed)
    x = r.integers(-128, 128, (B, C, H, W)).astype(np.int8)
    O = 4 * M
    L = [rand_layer(r, O, C, 1, False), rand_layer(r, M, C, 1, False), rand_layer(r, M, M, 3, False), rand_layer(r, O, M, 1, False)]
    ecal = r.uniform(0.4, 0.9, O).astype(np.float32)
    prims = [cl.input_layout("input", cl.layout(DT.i8, F.bfyx, cl.tensor(B, C, W, H)))]
    for i, (w, b, q, c) in enumerate(L):
        prims += [cl.data(f"w{i}", cl.make_memory(eng, w)), cl.data(f"b{i}", vec_mem(eng, b)), cl.data(f"q{i}", vec_mem(eng, q)),
                  cl.data(f"c{i}", vec_mem(eng, c))]
    st = cl.tensor(1, 1, stride, stride)
    prims += [cl.data("ecal", vec_mem(eng, ecal)),
              cl.convolution("shortcut", "input", ["w0"], ["b0"], ["q0"], ["c0"], stride=st),
              cl.convolution("reduce", "input", ["w1"], ["b1"], ["q1"], ["c1"], stride=st, with_activation=True),
              cl.convolution("mid", "reduce", ["w2"], ["b2"], ["q2"], ["c2"], input_offset=cl.tensor(0, 0, -1, -1, 0), with_activation=True),
              cl.convolution("expand", "mid", ["w3"], ["b3"], ["q3"], ["c3"], output_data_type=DT.i8),
              cl.eltwise("sum", "shortcut", "expand", cl.eltwise_mode.sum, True, 0.0, output_calibration_factors="ecal"),
              cl.reorder("out", "sum", F.bfyx)]

    def oracle():
        s = (stride, stride)
        sc = rc.conv(x, L[0][0], L[0][1], wqf=L[0][2], calib=L[0][3], stride=s, out_dt="s8")
        a = rc.conv(x, L[1][0], L[1][1], wqf=L[1][2], calib=L[1][3], stride=s, out_dt="s8", act="relu")
        a = rc.conv(a, L[2][0], L[2][1], wqf=L[2][2], calib=L[2][3], pad=(1, 1), out_dt="s8", act="relu")
        return sc, rc.conv(a, L[3][0], L[3][1], wqf=L[3][2], calib=L[3][3], out_dt="s8", eltw=sc, eltw_act="relu", eltw_calib=ecal)

    return cl.topology(*prims), x, oracle


@pytest.mark.parametrize("optimize", OPT, ids=["plain", "optimize_data"])
@pytest.mark.parametrize("stride", [1, 2])
def test_projection_and_opening_convolution_share_a_launch(eng, optimize, stride):
    topo, x, oracle = projection_block(eng, 21, stride=stride)
    net, outs = run(eng, topo, {"input": cl.make_memory(eng, x)}, optimize)
    sc, expected = oracle()
    np.testing.assert_array_equal(outs["out"].get_memory().read(), expected)
    a, b = net.get_primitive_info("shortcut"), net.get_primitive_info("reduce")
    if optimize:
        # one launch for the two convolutions of `input`; `reduce` is the tail of the pair's buffer and both carry the
        # border the 3x3 behind `reduce` needs
        assert a["launches_also"] == "reduce" and b["launched_by"] == "shortcut" and "kernel" not in b
        assert "generic" not in a["kernel"]
        assert a["pad_lower"][2:] == [1, 1] and b["pad_lower"][2:] == [1, 1]
        for _ in range(2):  # again, same buffers
            np.testing.assert_array_equal(net.execute()["out"].get_memory().read(), expected)
    else:
        assert "launches_also" not in a and "launched_by" not in b


def test_paired_convolution_that_is_an_output(eng):
    """what the application reads is the reorder back to its own format, which takes the convolution's window of the pair's
    buffer like any other reader"""
    topo, x, oracle = projection_block(eng, 22, stride=1)
    net = cl.network(eng, topo, cl.build_options(optimize_data=True, outputs=["shortcut", "reduce", "out"]))
    net.set_input_data("input", cl.make_memory(eng, x))
    outs = net.execute()
    sc, expected = oracle()
    np.testing.assert_array_equal(outs["out"].get_memory().read(), expected)
    np.testing.assert_array_equal(outs["shortcut"].get_memory().read(), sc)
    assert outs["reduce"].get_memory().read().min() == 0  # relu on the second convolution only
    assert sc.min() < 0
