"""Stand-alone eltwise (modes, more than two inputs, strides, broadcast, int8 with and without calibration): the oracle
against the reference's known-answer tables (tests/test_cases/eltwise_gpu_test.cpp), the HIP kernel through the C-ABI
and the clDNN API against the oracle."""
import json
import os
import zlib

import numpy as np
import pytest

from oracle import refconv as rc

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "eltwise_kat.json")) as f:
    CASES = json.load(f)["cases"]


def _to_bfyx(flat, tensor, fmt, dtype):
    """tensor = cldnn (batch, feature, x, y); values in the memory order of fmt -> [B, F, Y, X]; null -> 0"""
    b, f, x, y = tensor
    v = np.array([0 if e is None else e for e in flat], np.float64)
    v = v.reshape(y, x, f, b).transpose(3, 2, 0, 1) if fmt == "yxfb" else v.reshape(b, f, y, x)
    return np.ascontiguousarray(v).astype(dtype)


def problem(case):
    dt = np.int8 if case.get("dtype") == "i8" else np.float32
    ins = [_to_bfyx(v, s, case["format"], dt) for v, s in zip(case["inputs"], case["shapes"])]
    strides = [tuple(s) for s in case["strides"]] if "strides" in case else None
    # the expected tensor: input 0's shape, divided by its stride (the only strided table has stride 1 there)
    exp_shape = case["shapes"][0]
    exp = _to_bfyx(case["expected"], exp_shape, case["format"], np.float64)
    given = _to_bfyx([e is not None for e in case["expected"]], exp_shape, case["format"], bool)
    kw = dict(mode=case["mode"], strides=strides, calib=case.get("calib"), coefficients=case.get("coefficients"))
    return ins, kw, exp, given


def check(out, exp, given):
    assert out.shape == exp.shape
    np.testing.assert_allclose(out.astype(np.float64)[given], exp[given], rtol=1e-5, atol=1e-6)


# ------------------------------------------------------------------------------------------ CPU: oracle vs the tables
@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_oracle_known_answers(case):
    ins, kw, exp, given = problem(case)
    check(rc.eltwise(ins, **kw), exp, given)


def test_oracle_closed_forms():
    a = np.array([100, -100, 127, -128, 7, -7, 7, -7], np.int8).reshape(1, 1, 1, 8)
    b = np.array([100, -100, 1, -1, 2, 2, -2, -2], np.int8).reshape(1, 1, 1, 8)
    # int8 arithmetic outside the quantized form wraps like the C type
    assert rc.eltwise([a, b], "sum").ravel().tolist() == [-56, 56, -128, 127, 9, -5, 5, -9]
    assert rc.eltwise([a, b], "prod").ravel().tolist() == [16, 16, 127, -128, 14, -14, -14, 14]
    # C division truncates toward zero and the remainder takes the dividend's sign
    assert rc.eltwise([a, b], "div").ravel().tolist()[4:] == [3, -3, -3, 3]
    assert rc.eltwise([a, b], "mod").ravel().tolist()[4:] == [1, -1, 1, -1]
    # the quantized form adds in int, scales, rounds half away from zero and saturates
    assert rc.eltwise([a, b], "sum", oqf=0.5).ravel().tolist() == [100, -100, 64, -65, 5, -3, 3, -5]
    assert rc.eltwise([a, b], "sum", oqf=2.0).ravel().tolist() == [127, -128, 127, -128, 18, -10, 10, -18]
    assert rc.eltwise([a, b], "sum", oqf=0.5, relu=True).ravel().tolist() == [100, 0, 64, 0, 5, 0, 3, 0]
    # three inputs, left to right, every intermediate wrapped: (100 + 100 -> -56) + 100 = 44
    c = np.full((1, 1, 1, 8), 100, np.int8)
    assert rc.eltwise([a, b, c], "sum").ravel().tolist()[0] == 44
    assert rc.eltwise([a, b, c], "sum", oqf=0.25).ravel().tolist()[0] == 75
    # the two-input quantized sum is the function the network tests use
    r = np.random.default_rng(5)
    x, y = (r.integers(-128, 128, (2, 6, 3, 4)).astype(np.int8) for _ in range(2))
    cal = r.uniform(0.2, 1.2, 6).astype(np.float32)
    assert np.array_equal(rc.eltwise([x, y], "sum", calib=cal, relu=True), rc.eltwise_sum(x, y, calib=cal, relu=True))


def test_oracle_strides_and_broadcast():
    r = np.random.default_rng(6)
    a = r.standard_normal((2, 3, 4, 6)).astype(np.float32)
    b = r.standard_normal((2, 3, 8, 12)).astype(np.float32)
    out = rc.eltwise([a, b], "sum", strides=[(2, 2), (4, 4)])
    assert np.array_equal(out, a[:, :, ::2, ::2] + b[:, :, ::4, ::4])
    per_feature = r.standard_normal((1, 3, 1, 1)).astype(np.float32)
    assert np.array_equal(rc.eltwise([a, per_feature], "prod"), a * per_feature)
    assert np.array_equal(rc.eltwise([per_feature, a], "sub"), per_feature - a)


# ------------------------------------------------------------------------------------------ GPU: the C-ABI
@pytest.fixture(scope="module")
def eng():
    from cldnn_amd import hip
    e = hip.Engine()
    yield e
    e.close()


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["bfyx", "yxfb", "byxf", "fs_b_yx_fsv16", "b_fs_yx_fsv4"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_hip_known_answers(eng, case, fmt):
    from cldnn_amd import hip
    ins, kw, exp, given = problem(case)
    if fmt in ("fs_b_yx_fsv16", "b_fs_yx_fsv4") and ins[0].dtype == np.float32:
        pytest.skip("the blocked layouts hold 8-bit data")
    pad = tuple(case.get("input_padding", (0, 0)))
    check(hip.eltwise_forward(eng, ins, fmt=fmt, in_pad=pad, **kw), exp, given)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["sum", "sub", "max", "prod", "div", "min", "mod"])
@pytest.mark.parametrize("dtype,fmt,quant", [
    (np.int8, "bfyx", False), (np.int8, "fs_b_yx_fsv16", True), (np.uint8, "b_fs_yx_fsv4", False),
    (np.uint8, "fs_b_yx_fsv16", True), (np.float32, "yxfb", False)])
def test_hip_random(eng, mode, dtype, fmt, quant):
    from cldnn_amd import hip
    r = np.random.default_rng(zlib.crc32(repr((mode, fmt, quant)).encode()))
    shape = (2, 21, 5, 7)

    def rnd(s):
        if dtype == np.float32:
            return (r.standard_normal(s) * 4).astype(np.float32)
        info = np.iinfo(dtype)
        return r.integers(info.min, info.max + 1, s).astype(dtype)
    for n, strides, shapes in ((2, None, [shape, shape]), (3, None, [shape, (1, 21, 1, 1), shape]),
                               (2, [(2, 3), (1, 1)], [(2, 21, 10, 21), shape]), (4, None, [shape] * 4)):
        ins = [rnd(s) for s in shapes]
        kw = dict(mode=mode, strides=strides)
        if quant:
            kw.update(calib=r.uniform(0.05, 1.5, 21).astype(np.float32), relu=True)
        exp = rc.eltwise(ins, **kw)
        out = hip.eltwise_forward(eng, ins, fmt=fmt, in_pad=(1, 2), out_pad=(2, 1), **kw)
        if dtype == np.float32:
            ok = np.isfinite(exp)
            np.testing.assert_allclose(out[ok], exp[ok], rtol=1e-5, atol=1e-6)
        else:
            assert np.array_equal(out, exp), (mode, n, strides)


@pytest.mark.gpu
def test_hip_mixed_types_and_errors(eng):
    from cldnn_amd import hip
    r = np.random.default_rng(8)
    a = r.integers(-100, 100, (1, 4, 3, 3)).astype(np.int8)
    b = (r.standard_normal((1, 4, 3, 3)) * 20).astype(np.float32)
    for ins in ([a, b], [b, a]):
        exp = rc.eltwise(ins, "max")
        out = hip.eltwise_forward(eng, ins, "max")
        assert out.dtype == exp.dtype
        np.testing.assert_allclose(out, exp, rtol=1e-6)
    with pytest.raises(hip.HipError, match="not supported for integer types"):
        hip.eltwise_forward(eng, [a, a], "pow")
    with pytest.raises(hip.HipError, match="between 2 and 4"):
        hip.eltwise_forward(eng, [a] * 5, "sum")
    with pytest.raises(hip.HipError, match="coefficients"):
        hip.eltwise_forward(eng, [a, a], "sum", coefficients=[0.5, 0.5])
    with pytest.raises(hip.HipError, match="does not cover"):
        hip.eltwise_forward(eng, [a, r.integers(0, 9, (1, 4, 7, 7)).astype(np.int8)], "sum", strides=[(1, 1), (3, 3)])


# ------------------------------------------------------------------------------------------ GPU: the clDNN API
@pytest.mark.gpu
@pytest.mark.parametrize("optimize", [False, True], ids=["plain", "optimize_data"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_api_known_answers(case, optimize):
    """the reference's tests as they are written: input_layout (+ a reorder that adds padding) -> eltwise -> output"""
    from cldnn_amd import api as cl
    eng = cl.engine()
    ins, kw, exp, given = problem(case)
    fmt = getattr(cl.format, case["format"])
    prims, names, feed = [], [], {}
    for i, a in enumerate(ins):
        name = "input%d" % i
        m = cl.make_memory(eng, a, fmt)
        prims.append(cl.input_layout(name, m.get_layout()))
        feed[name] = m
        if "input_padding" in case:
            py, px = case["input_padding"]
            prims.append(cl.reorder("reorder%d" % i, name, fmt, cl.DT_OF[a.dtype],
                                    output_padding=cl.padding([0, 0, py, px])))
            name = "reorder%d" % i
        names.append(name)
    mode = getattr(cl.eltwise_mode, case["mode"])
    strides = [cl.tensor(1, 1, s[1], s[0]) for s in case["strides"]] if "strides" in case else None
    calib = ""
    if "calib" in case:
        prims.append(cl.data("calib", cl.make_memory(eng, np.array(case["calib"], np.float32).reshape(1, 1, 1, -1))))
        calib = "calib"
    prims.append(cl.eltwise("eltwise", names, mode, stride=strides, coefficients=case.get("coefficients"),
                            output_calibration_factors=calib))
    net = cl.network(eng, cl.topology(*prims), cl.build_options(optimize_data=optimize))
    for k, v in feed.items():
        net.set_input_data(k, v)
    outs = net.execute()
    assert list(outs) == ["eltwise"]
    check(outs["eltwise"].get_memory().read(), exp, given)


@pytest.mark.gpu
def test_api_argument_checks():
    """reference api/CPP/eltwise.hpp:303-310 (coefficients), src/eltwise.cpp:38-46 (integer modes), 57-66 (strides)"""
    from cldnn_amd import api as cl
    eng = cl.engine()
    a = cl.make_memory(eng, np.zeros((1, 2, 4, 4), np.int8))
    f = cl.make_memory(eng, np.zeros((1, 2, 4, 4), np.float32))
    for bad in (dict(coefficients=[0.5]), dict(coefficients=[0.5, 0.5, 0.5])):
        with pytest.raises(ValueError, match="coefficients count"):
            cl.eltwise("e", ["a", "b"], cl.eltwise_mode.sum, **bad)
    with pytest.raises(ValueError, match="Only eltwise sum"):
        cl.eltwise("e", ["a", "b"], cl.eltwise_mode.max, coefficients=[0.5, 0.5])

    def build(mem, *args, **kw):
        t = cl.topology(cl.input_layout("a", mem.get_layout()), cl.input_layout("b", mem.get_layout()), cl.eltwise("e", *args, **kw))
        return cl.network(eng, t, cl.build_options())
    with pytest.raises(cl.error, match="not supported for integer types"):
        build(a, ["a", "b"], cl.eltwise_mode.pow)
    with pytest.raises(cl.error, match="one stride per input"):
        build(f, ["a", "b"], cl.eltwise_mode.sum, stride=[cl.tensor(1, 1, 2, 2)])
    with pytest.raises(cl.error, match="differ in size after striding"):
        build(f, ["a", "b"], cl.eltwise_mode.sum, stride=[cl.tensor(1, 1, 2, 2), cl.tensor(1, 1, 1, 1)])
    with pytest.raises(cl.error, match="at most 4 inputs"):
        build(f, ["a", "b", "a", "b", "a"], cl.eltwise_mode.sum)
    assert build(f, ["a", "b", "a", "b"], cl.eltwise_mode.sum) is not None


def _ramp(shape, add=0):
    """the reference's test data: element i of the bfyx buffer is (char)(i + add)"""
    n = int(np.prod(shape))
    return ((np.arange(n, dtype=np.int64) + add) & 255).astype(np.uint8).view(np.int8).reshape(shape)


@pytest.mark.gpu
@pytest.mark.parametrize("b,f,size", [(1, 256, 56), (4, 512, 28), (16, 1024, 14), (32, 2048, 14)])
def test_api_b_fs_yx_fsv4_with_calibration(b, f, size):
    """reference tests/test_cases/eltwise_gpu_test.cpp:1833-1971: the quantized sum with per-feature calibration (every
    seventh factor negative) in bfyx and through b_fs_yx_fsv4 reorders; both must equal the oracle"""
    from cldnn_amd import api as cl
    eng = cl.engine()
    x = _ramp((b, f, size, size))
    cal, sign = np.empty(f, np.float32), np.float32(1)
    for i in range(f):
        cal[i] = sign if (i + 1) % 7 else -sign
        sign = np.float32(sign * np.float32(1.0123))
    exp = rc.eltwise([x, x], "sum", calib=cal, relu=True)
    assert 0.2 < (exp > 0).mean() < 0.6 and (exp == 127).any()
    lay = cl.layout(cl.data_types.i8, cl.format.bfyx, cl.tensor(b, f, size, size))
    blocked = cl.layout(cl.data_types.i8, cl.format.b_fs_yx_fsv4, cl.tensor(b, f, size, size))
    common = [cl.input_layout("input1", lay), cl.input_layout("input2", lay),
              cl.data("callib", cl.make_memory(eng, cal.reshape(1, 1, 1, -1)))]
    gold = cl.topology(*common, cl.eltwise("eltw_GOLD", "input1", "input2", cl.eltwise_mode.sum, True, output_calibration_factors="callib"))
    imad = cl.topology(*common, cl.reorder("reorder1_Swizzelled", "input1", blocked), cl.reorder("reorder2_Swizzelled", "input2", blocked),
                       cl.eltwise("eltw_IMAD", "reorder1_Swizzelled", "reorder2_Swizzelled", cl.eltwise_mode.sum, True,
                                  output_calibration_factors="callib"),
                       cl.reorder("reorder_UnSwizzelled", "eltw_IMAD", lay))
    m = cl.make_memory(eng, x)
    for topo, out in ((gold, "eltw_GOLD"), (imad, "reorder_UnSwizzelled")):
        net = cl.network(eng, topo, cl.build_options())
        net.set_input_data("input1", m)
        net.set_input_data("input2", m)
        got = net.execute()[out].get_memory().read()
        assert np.array_equal(got, exp), out


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["min", "max", "sum"])
def test_api_b_fs_yx_fsv4_three_inputs(mode):
    """reference tests/test_cases/eltwise_gpu_test.cpp:1973-2119: three int8 inputs, no calibration (8-bit wrap-around)"""
    from cldnn_amd import api as cl
    eng = cl.engine()
    shape = (1, 256, 56, 56)
    ins = [_ramp(shape, k) for k in (1, 2, 3)]
    exp = rc.eltwise(ins, mode, relu=True)
    lay = cl.layout(cl.data_types.i8, cl.format.bfyx, cl.tensor(1, 256, 56, 56))
    blocked = cl.layout(cl.data_types.i8, cl.format.b_fs_yx_fsv4, cl.tensor(1, 256, 56, 56))
    names = ["input1", "input2", "input3"]
    common = [cl.input_layout(n, lay) for n in names]
    gold = cl.topology(*common, cl.eltwise("eltw_GOLD", names, getattr(cl.eltwise_mode, mode), True))
    imad = cl.topology(*common, *[cl.reorder("r" + n, n, blocked) for n in names],
                       cl.eltwise("eltw_IMAD", ["r" + n for n in names], getattr(cl.eltwise_mode, mode), True),
                       cl.reorder("reorder_UnSwizzelled", "eltw_IMAD", lay))
    for topo, out in ((gold, "eltw_GOLD"), (imad, "reorder_UnSwizzelled")):
        net = cl.network(eng, topo, cl.build_options())
        for n, a in zip(names, ins):
            net.set_input_data(n, cl.make_memory(eng, a))
        got = net.execute()[out].get_memory().read()
        assert np.array_equal(got, exp), out
