"""Pooling (the layers between the convolutions of an int8 network): oracle against the reference's known-answer tables
(tests/test_cases/pooling_gpu_test.cpp), the HIP kernels through the C-ABI and the clDNN API against the oracle."""
import json
import os

import numpy as np
import pytest

from oracle import refconv as rc

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "pool_kat.json")) as f:
    CASES = json.load(f)["cases"]
NP = {"s8": np.int8, "u8": np.uint8, "f32": np.float32}


def _to_bfyx(flat, shape, layout):
    b, f, h, w = shape
    if layout == "yxfb":
        return np.ascontiguousarray(np.array(flat).reshape(h, w, f, b).transpose(3, 2, 0, 1))
    return np.array(flat).reshape(shape)


def problem(case):
    x = _to_bfyx(case["input"], case["in_shape"], case.get("in_layout")).astype(NP[case["dt"]])
    exp = _to_bfyx(case["expected"], case["out_shape"], case.get("out_layout")).astype(np.float64)
    return x, exp


def oracle_pool(case, x):
    if case["size"] is None:
        return rc.pool(x, case["mode"], None, global_pooling=True)
    return rc.pool(x, case["mode"], tuple(case["size"]), tuple(case["stride"]), tuple(case["pad"]))


# ------------------------------------------------------------------------------------------ CPU: oracle vs the tables
@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_oracle_known_answers(case):
    x, exp = problem(case)
    out = oracle_pool(case, x)
    assert out.shape == exp.shape
    np.testing.assert_allclose(out.astype(np.float64), exp, atol=max(case["tol"], 1e-12), rtol=0)


@pytest.mark.parametrize("n,pad,size,stride,expect", [
    (112, 0, 3, 2, 56),   # ResNet pool1 (ceil mode of the framework the model comes from)
    (112, 1, 3, 2, 57),   # one more window than floor mode, it still starts inside input + leading padding
    (3, 1, 2, 2, 2), (3, 1, 3, 3, 2), (2, 1, 2, 2, 2), (1, 1, 3, 1, 1), (7, 0, 7, 1, 1), (4, 0, 2, 2, 2), (5, 0, 2, 2, 3),
])
def test_output_extent_rule(n, pad, size, stride, expect):
    """closed form of min(exceed_once, any) (reference src/include/sliding_window_utils.h:135-186): the number of window
    positions i with i * stride - pad <= n - 1 (starts inside the data or the leading padding) that are needed to
    cover input + 2 * pad, i.e. ceil((n + 2 * pad - size) / stride) + 1 clipped by the first condition"""
    brute = 1
    while True:
        first = brute * stride - pad  # position of the next window
        covered = (brute - 1) * stride - pad + max(size, stride)  # end of what the windows so far reach
        if first > n - 1 or covered >= n + pad:
            break
        brute += 1
    assert rc.pool_out_extent(n, pad, size, stride) == expect == brute


def test_int8_average_rounds_half_away_and_max_starts_at_char_min():
    x = np.array([[[[1, 2], [3, 4]]]], np.int8)   # mean 2.5 -> 3
    assert rc.pool(x, "average", (2, 2))[0, 0, 0, 0] == 3
    assert rc.pool(-x, "average", (2, 2))[0, 0, 0, 0] == -3
    u = np.array([[[[200, 100], [7, 9]]]], np.uint8)
    assert rc.pool(u, "max", (2, 2))[0, 0, 0, 0] == 200 and rc.pool(u, "average", (2, 2))[0, 0, 0, 0] == 79


def test_average_dividers():
    """3x3 window, stride 2, padding 1 on a 4x4 plane of ones (windows start at -1, 1, 3; the last one overhangs the
    padded plane): the plain average divides by the window clipped to input + padding, average_no_padding by the taps
    inside the input"""
    x = np.ones((1, 1, 4, 4), np.float32)
    a = rc.pool(x, "average", (3, 3), (2, 2), (1, 1))
    n = rc.pool(x, "average_no_padding", (3, 3), (2, 2), (1, 1))
    np.testing.assert_allclose(a[0, 0], np.outer([2, 3, 1], [2, 3, 1]) / np.outer([3, 3, 2], [3, 3, 2]), rtol=1e-6)
    np.testing.assert_array_equal(n, np.ones_like(n))


# ------------------------------------------------------------------------------------------ GPU
def _gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


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
    x, exp = problem(case)
    if case["size"] is None:
        out = hip.pool_forward(eng, x, case["mode"], None, global_pooling=True)
    else:
        out = hip.pool_forward(eng, x, case["mode"], tuple(case["size"]), tuple(case["stride"]), tuple(case["pad"]))
    assert out.shape == exp.shape
    np.testing.assert_allclose(out.astype(np.float64), exp, atol=max(case["tol"], 1e-6), rtol=0)


POOL_SHAPES = [
    # B  F   H   W  mode                  size   stride  pad
    (2, 64, 112, 112, "max", (3, 3), (2, 2), (0, 0)),                 # ResNet-50 pool1
    (2, 64, 112, 112, "max", (3, 3), (2, 2), (1, 1)),
    (3, 2048, 7, 7, "average", (7, 7), (1, 1), (0, 0)),               # ResNet-50 pool5
    (2, 37, 13, 17, "average", (3, 3), (2, 2), (1, 1)),               # ragged sizes, overhanging last window
    (2, 37, 13, 17, "average_no_padding", (3, 2), (2, 3), (1, 1)),
    (1, 16, 9, 9, "max", (2, 2), (2, 2), (0, 0)),
    (2, 100, 5, 5, "average", (5, 5), (5, 5), (2, 2)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [np.uint8, np.int8, np.float32], ids=["u8", "s8", "f32"])
@pytest.mark.parametrize("fmt", ["bfyx", "fs_b_yx_fsv16", "yxfb"])
@pytest.mark.parametrize("shape", POOL_SHAPES, ids=lambda s: "x".join(str(v) for v in s[:4]) + "_" + s[4])
def test_gpu_pooling_matches_oracle(eng, shape, fmt, dt):
    from cldnn_amd import hip
    B, F, H, W, mode, size, stride, pad = shape
    if fmt == "fs_b_yx_fsv16" and dt == np.float32:
        pytest.skip("the blocked layout carries int8 data")
    r = np.random.default_rng(11)
    x = (r.standard_normal((B, F, H, W)) * 40).astype(dt) if dt == np.float32 else r.integers(0 if dt == np.uint8 else -128, 256 if dt == np.uint8 else 128, (B, F, H, W)).astype(dt)
    ref = rc.pool(x, mode, size, stride, pad)
    out = hip.pool_forward(eng, x, mode, size, stride, pad, fmt=fmt, in_pad=(1, 2) if fmt != "yxfb" else (0, 0), out_pad=(0, 1) if fmt != "yxfb" else (0, 0))
    assert out.shape == ref.shape
    if dt == np.float32:
        np.testing.assert_allclose(out, ref, rtol=1e-5, atol=1e-5)  # sums of up to 49 floats in the same order
    else:
        np.testing.assert_array_equal(out, ref)


@pytest.mark.gpu
def test_gpu_pooling_rejects_bad_arguments(eng):
    from cldnn_amd import hip
    x = np.zeros((1, 4, 4, 4), np.int8)
    with pytest.raises(hip.HipError):
        hip.pool_forward(eng, x, "max", (0, 2))
    with pytest.raises(hip.HipError):
        hip.pool_forward(eng, x, "max", (2, 2), (0, 1))


# ------------------------------------------------------------------------------------------ through the clDNN API
def test_plan_keeps_pooling_between_blocked_convolutions_blocked():
    """conv (int8, quantized) -> max pooling -> conv: the pooling node inherits fs_b_yx_fsv16 from its producer, so no
    reorder separates the three"""
    import ctypes as C
    from cldnn_amd import api as cl
    keep = []

    def attach(a):
        a = np.ascontiguousarray(a)
        keep.append(a)
        b, f, h, w = a.shape
        return cl.memory.attach(cl.layout(cl.DT_OF[a.dtype], cl.format.bfyx, cl.tensor(b, f, w, h)), a)

    def vec(n):
        return attach(np.ones((1, 1, 1, n), np.float32))

    t = cl.topology(cl.input_layout("in", cl.layout(cl.data_types.u8, cl.format.bfyx, cl.tensor(2, 64, 16, 16))),
                    cl.data("w1", attach(np.ones((64, 64, 3, 3), np.int8))), cl.data("q1", vec(64)), cl.data("c1", vec(64)),
                    cl.data("w2", attach(np.ones((128, 64, 1, 1), np.int8))), cl.data("q2", vec(128)), cl.data("c2", vec(128)),
                    cl.convolution("conv1", "in", ["w1"], None, ["q1"], ["c1"], input_offset=cl.tensor(0, 0, -1, -1, 0)),
                    cl.pooling("pool", "conv1", cl.pooling_mode.max, cl.tensor(1, 1, 3, 3), cl.tensor(1, 1, 2, 2)),
                    cl.convolution("conv2", "pool", ["w2"], None, ["q2"], ["c2"]))
    nodes = {n["id"]: n for n in cl.plan(t, cl.build_options(optimize_data=True))}
    assert nodes["pool"]["type"] == "pooling" and nodes["pool"]["format"] == cl.format.fs_b_yx_fsv16
    assert nodes["pool"]["size"] == [2, 64, 8, 8]   # (16 - 3 + 1) / 2 + 1 windows, the last one overhanging
    assert nodes["pool"]["deps"] == ["conv1"] and nodes["conv2_fsv16"]["deps"][0] == "pool"
    with pytest.raises(cl.error):
        cl.plan(cl.topology(cl.input_layout("in", cl.layout(cl.data_types.u8, cl.format.bfyx, cl.tensor(1, 4, 8, 8))),
                            cl.pooling("p", "in", cl.pooling_mode.max, cl.tensor(1, 1, 2, 2), cl.tensor(1, 1, 0, 1))))
    with pytest.raises(cl.error):
        cl.plan(cl.topology(cl.input_layout("in", cl.layout(cl.data_types.u8, cl.format.bfyx, cl.tensor(1, 4, 8, 8))),
                            cl.pooling("p", "in", cl.pooling_mode.bilinear, cl.tensor(1, 1, 2, 2))))


@pytest.fixture(scope="module")
def cl_eng():
    from cldnn_amd import api as cl
    return cl.engine()


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_api_known_answers(cl_eng, case):
    """the tables through input_layout -> [reorder f32 -> i8] -> pooling -> [reorder back], as the reference's tests build them"""
    from cldnn_amd import api as cl
    x, exp = problem(case)
    b, f, h, w = x.shape
    yx = lambda p: cl.tensor(0, 0, p[1], p[0], 0)
    mode = getattr(cl.pooling_mode, case["mode"])
    int8 = case["dt"] != "f32"
    xin = np.array(case["input_f32"], np.float32).reshape(x.shape) if int8 else x
    prims = [cl.input_layout("input", cl.layout(cl.data_types.f32, cl.format.bfyx, cl.tensor(b, f, w, h)))]
    src = "input"
    if int8:
        prims.append(cl.reorder("reorder_input", "input", cl.layout(cl.data_types.i8, cl.format.bfyx, cl.tensor(b, f, w, h))))
        src = "reorder_input"
    if case["size"] is None:
        prims.append(cl.pooling("pool1", src, mode))
    else:
        prims.append(cl.pooling("pool1", src, mode, cl.tensor(1, 1, case["size"][1], case["size"][0]),
                                cl.tensor(1, 1, case["stride"][1], case["stride"][0]), yx((-case["pad"][0], -case["pad"][1]))))
    out_id = "pool1"
    if int8:
        prims.append(cl.reorder("reorder2", "pool1", cl.format.byxf, cl.data_types.f32))
        out_id = "reorder2"
    net = cl.network(cl_eng, cl.topology(*prims), cl.build_options(outputs=[out_id]))
    net.set_input_data("input", cl.make_memory(cl_eng, xin))
    out = net.execute()[out_id].get_memory().read()
    assert out.shape == exp.shape
    np.testing.assert_allclose(out.astype(np.float64), exp, atol=max(case["tol"], 1e-6), rtol=0)


@pytest.mark.gpu
@pytest.mark.parametrize("optimize", [False, True], ids=["plain", "optimize_data"])
def test_api_conv_pool_conv_network(cl_eng, optimize):
    """stem-like chain conv 7x7/2 -> max pooling 3x3/2 -> conv 1x1 -> global average pooling against the oracle"""
    from cldnn_amd import api as cl
    r = np.random.default_rng(3)
    x = r.integers(0, 256, (2, 3, 64, 64)).astype(np.uint8)
    w1 = r.integers(-127, 128, (64, 3, 7, 7)).astype(np.int8)
    w2 = r.integers(-127, 128, (96, 64, 1, 1)).astype(np.int8)
    b1, b2 = r.integers(-1000, 1001, 64).astype(np.int32), r.integers(-1000, 1001, 96).astype(np.int32)
    c1 = (40.0 / (np.sqrt(147) * 147.4 * 73.3) * r.uniform(0.5, 2.0, 64)).astype(np.float32)
    c2 = (40.0 / (np.sqrt(64) * 40 * 73.3) * r.uniform(0.5, 2.0, 96)).astype(np.float32)
    one1, one2 = np.ones(64, np.float32), np.ones(96, np.float32)
    vm = lambda v: cl.make_memory(cl_eng, np.ascontiguousarray(np.asarray(v).reshape(1, 1, 1, -1)))
    t = cl.topology(cl.input_layout("input", cl.layout(cl.data_types.u8, cl.format.bfyx, cl.tensor(2, 3, 64, 64))),
                    cl.data("w1", cl.make_memory(cl_eng, w1)), cl.data("b1", vm(b1)), cl.data("q1", vm(one1)), cl.data("c1", vm(c1)),
                    cl.data("w2", cl.make_memory(cl_eng, w2)), cl.data("b2", vm(b2)), cl.data("q2", vm(one2)), cl.data("c2", vm(c2)),
                    cl.convolution("conv1", "input", ["w1"], ["b1"], ["q1"], ["c1"], stride=cl.tensor(1, 1, 2, 2),
                                   input_offset=cl.tensor(0, 0, -3, -3, 0), with_activation=True),
                    cl.pooling("pool1", "conv1", cl.pooling_mode.max, cl.tensor(1, 1, 3, 3), cl.tensor(1, 1, 2, 2)),
                    cl.convolution("conv2", "pool1", ["w2"], ["b2"], ["q2"], ["c2"], with_activation=True),
                    cl.pooling("pool5", "conv2", cl.pooling_mode.average))
    net = cl.network(cl_eng, t, cl.build_options(optimize_data=optimize, outputs=["pool1", "pool5"]))
    net.set_input_data("input", cl.make_memory(cl_eng, x))
    outs = net.execute()
    a = rc.conv(x, w1, b1, wqf=one1, calib=c1, stride=(2, 2), pad=(3, 3), act="relu")
    p1 = rc.pool(a, "max", (3, 3), (2, 2))
    a2 = rc.conv(p1, w2, b2, wqf=one2, calib=c2, act="relu")
    p5 = rc.pool(a2, "average", None, global_pooling=True)
    np.testing.assert_array_equal(outs["pool1"].get_memory().read(), p1)
    np.testing.assert_array_equal(outs["pool5"].get_memory().read(), p5)
    assert p5.shape == (2, 96, 1, 1) and p5.any()
