"""Pins the CPU oracle (oracle/refconv.c) before anything is compared with it:
 * the reference's own known-answer tables (tests/golden/conv_kat.json),
 * closed forms / invariants a plausible mistake would break
   (brute force on tiny inputs, 1x1 == integer GEMM, box sums, zero padding,
    linearity, rounding ties, saturation, grouped == block-diagonal dense).
"""
import itertools

import numpy as np
import pytest

import kat
from oracle import refconv as rc

K = kat.load()


# ------------------------------------------------------------------ KATs from the reference's tests
@pytest.mark.parametrize("case", K["conv_quantized"], ids=lambda c: c["name"])
def test_kat_conv_quantized(case):
    p = kat.diag_problem(case)
    out = rc.conv(p["x"], p["w"], p["bias"], wqf=p["wqf"], out_dt=case["out_dt"], act="relu")
    if case["out_dt"] == "f32":
        np.testing.assert_allclose(out, p["expected"], atol=case["tol"], rtol=0)
    else:
        np.testing.assert_array_equal(out.astype(np.int64), p["expected"].astype(np.int64))


@pytest.mark.parametrize("case", K["fused"], ids=lambda c: c["name"])
def test_kat_fused(case):
    p = kat.diag_problem(case, fused=True)
    out = rc.conv(p["x"], p["w"], p["bias"],
                  wqf=p["wqf"] if case["pass_wqf"] else None,
                  calib=p["conv_calib"] if case["pass_conv_calib"] else None,
                  out_dt=case["out_dt"], act="none",
                  eltw=p["nci"], non_conv_scale=float(p["non_conv_scale"]), eltw_act="relu",
                  eltw_calib=p["eltw_calib"] if case["pass_eltw_calib"] else None)
    if case["out_dt"] == "f32":
        np.testing.assert_allclose(out, p["expected"], atol=case["tol"], rtol=0)
    else:
        np.testing.assert_array_equal(out.astype(np.int64), p["expected"].astype(np.int64))


@pytest.mark.parametrize("case", K["indexing"], ids=lambda c: c["name"])
def test_kat_indexing(case):
    p = kat.indexing_problem(case, K["indexing"])
    out = rc.conv(p["x"], p["w"], p["bias"], stride=p["stride"], pad=p["pad"], groups=p["groups"], act=p["act"])
    assert out.shape == p["expected"].shape
    np.testing.assert_allclose(out.astype(np.float64), p["expected"], atol=max(p["tol"], 1e-12), rtol=0)


def _api_pads(p):
    """padding above / below add to the padding the input offset asks for (low side, high side)"""
    lo = (p["pad"][0] + p["pad_above"][0], p["pad"][1] + p["pad_above"][1])
    hi = (p["pad"][0] + p["pad_below"][0], p["pad"][1] + p["pad_below"][1])
    return lo, hi


@pytest.mark.parametrize("case", K["api"], ids=lambda c: c["name"])
def test_kat_api_tables(case):
    p = kat.api_problem(case, K["indexing"])
    lo, hi = _api_pads(p)
    out = rc.conv(p["x"], p["w"], p["bias"], stride=p["stride"], pad=lo, pad_end=hi, groups=max(p["groups"], p["split"]),
                  act="relu_slope" if p["act_slope"] else p["act"], act_m=p["act_slope"])
    kat.assert_close_where_given(out, p["expected"], p["tol"])


def quantized_recipe(case):
    """the reference's recipe (convolution_gpu_test.cpp:3741-3969): float network first, then weights requantised per
    feature and the output scaled by 127 / max|float output| (one factor, or one per feature)"""
    x = np.array(case["input"], np.float32).reshape(case["in_shape"])
    wf = np.array(case["weights_f"], np.float32).reshape(case["w_shape"])
    bias = np.array(case["bias"], np.float32)
    fl = rc.conv(x, wf, bias, stride=tuple(case["stride"]))
    wq, wqf = kat.quantize_weights(wf)
    return x, wf, bias, fl, wq.astype(np.int8), wqf


@pytest.mark.parametrize("case", [c for c in K["quantized_recipe"] if c["scale"] != "two_layers"], ids=lambda c: c["name"])
def test_kat_quantized_recipe(case):
    x, wf, bias, fl, wq, wqf = quantized_recipe(case)
    exp = np.array(case["float_output"], np.float64).reshape(case["out_shape"])
    np.testing.assert_allclose(fl, exp, atol=1e-4, rtol=0)  # the table in the test's source is the float network's output
    if case["scale"] == "single":
        oqf = np.float32(127.0) / np.abs(fl).max()
        out = rc.conv(x.astype(np.int8), wq, bias, wqf=wqf, oqf=float(oqf), stride=tuple(case["stride"]), out_dt="s8")
        back = out.astype(np.float64) / oqf
    else:
        calib = kat.calibrate(fl)
        out = rc.conv(x.astype(np.int8), wq, bias, wqf=wqf, calib=calib, stride=tuple(case["stride"]), out_dt="s8")
        back = out.astype(np.float64) / calib.reshape(1, -1, 1, 1)
    assert np.abs(back - exp).max() <= case["tol"]


def test_round_to_even_variant_differs_only_on_ties():
    case = next(c for c in K["conv_quantized"] if c["name"] == "i8_to_u8")
    p = kat.diag_problem(case)
    away = rc.conv(p["x"], p["w"], p["bias"], wqf=p["wqf"], out_dt="u8", act="relu")
    even = rc.conv(p["x"], p["w"], p["bias"], wqf=p["wqf"], out_dt="u8", act="relu", round_even=True)
    diff = np.argwhere(away != even)
    # ties in the table: 125.5 and 135.5 (even neighbour is also the away neighbour) and 126.5 (it is not)
    assert {tuple(int(v) for v in d[[1, 3]]) for d in diff} == {(5, 1)}
    assert away[0, 5, 0, 1] == 127 and even[0, 5, 0, 1] == 126


# ------------------------------------------------------------------ closed forms
def brute(x, w, stride, pad, dil, groups):
    """7-deep python loop, int64, straight from the definition."""
    B, IFM, IH, IW = x.shape
    OFM, IFMg, FY, FX = w.shape
    OH = (IH + 2 * pad[0] - ((FY - 1) * dil[0] + 1)) // stride[0] + 1
    OW = (IW + 2 * pad[1] - ((FX - 1) * dil[1] + 1)) // stride[1] + 1
    out = np.zeros((B, OFM, OH, OW), np.int64)
    ofg = OFM // groups
    for b, f, y, xx in itertools.product(range(B), range(OFM), range(OH), range(OW)):
        g = f // ofg
        s = 0
        for k, j, i in itertools.product(range(IFMg), range(FY), range(FX)):
            iy = y * stride[0] - pad[0] + j * dil[0]
            ix = xx * stride[1] - pad[1] + i * dil[1]
            if 0 <= iy < IH and 0 <= ix < IW:
                s += int(x[b, g * IFMg + k, iy, ix]) * int(w[f, k, j, i])
        out[b, f, y, xx] = s
    return out


CASES = [
    # B IFM IH IW OFM FY FX stride pad dil groups in_dt
    (2, 3, 7, 6, 4, 3, 3, (1, 1), (1, 1), (1, 1), 1, np.uint8),
    (1, 4, 9, 8, 6, 3, 2, (2, 1), (0, 1), (1, 1), 2, np.int8),
    (1, 2, 11, 11, 3, 7, 7, (2, 2), (3, 3), (1, 1), 1, np.uint8),
    (2, 6, 6, 5, 6, 3, 3, (1, 2), (2, 0), (2, 1), 6, np.int8),
    (1, 5, 4, 4, 2, 1, 1, (1, 1), (0, 0), (1, 1), 1, np.uint8),
    (1, 1, 2, 2, 1, 3, 3, (2, 2), (0, 0), (1, 1), 1, np.int8),  # degenerate window -> 1x1 output
]


@pytest.mark.parametrize("c", CASES, ids=lambda c: "x".join(str(v) for v in c[:7]))
def test_accumulators_match_bruteforce(c):
    B, IFM, IH, IW, OFM, FY, FX, stride, pad, dil, groups, dt = c
    r = np.random.default_rng(hash(c[:7]) & 0xFFFF)
    lo, hi = (0, 256) if dt == np.uint8 else (-128, 128)
    x = r.integers(lo, hi, (B, IFM, IH, IW)).astype(dt)
    w = r.integers(-127, 128, (OFM, IFM // groups, FY, FX)).astype(np.int8)
    wqf = np.ones(OFM, np.float32)
    out, acc = rc.conv(x, w, None, wqf=wqf, stride=stride, pad=pad, dilation=dil, groups=groups,
                       out_dt="f32", want_acc=True)
    if FY > IH + 2 * pad[0]:
        # window larger than the padded input: extent 1, overhang reads zero
        assert acc.shape[2:] == (1, 1)
        ref = sum(int(x[0, 0, j, i]) * int(w[0, 0, j, i]) for j in range(IH) for i in range(IW))
        assert acc[0, 0, 0, 0] == ref
        return
    np.testing.assert_array_equal(acc.astype(np.int64), brute(x, w, stride, pad, dil, groups))
    # with wqf = 1 and f32 output the stored value is (float)acc
    np.testing.assert_array_equal(out, acc.astype(np.float32))


def test_1x1_is_integer_gemm():
    r = np.random.default_rng(1)
    x = r.integers(0, 256, (3, 64, 5, 7)).astype(np.uint8)
    w = r.integers(-127, 128, (48, 64, 1, 1)).astype(np.int8)
    _, acc = rc.conv(x, w, None, wqf=np.ones(48, np.float32), out_dt="f32", want_acc=True)
    a = x.astype(np.int64).transpose(0, 2, 3, 1).reshape(-1, 64)
    ref = (a @ w.astype(np.int64).reshape(48, 64).T).reshape(3, 5, 7, 48).transpose(0, 3, 1, 2)
    np.testing.assert_array_equal(acc, ref)


def test_all_ones_is_box_sum_and_border_taps_drop_out():
    r = np.random.default_rng(2)
    x = r.integers(0, 256, (1, 1, 6, 6)).astype(np.uint8)
    w = np.ones((1, 1, 3, 3), np.int8)
    _, acc = rc.conv(x, w, None, wqf=np.ones(1, np.float32), pad=(1, 1), out_dt="f32", want_acc=True)
    xp = np.pad(x[0, 0].astype(np.int64), 1)
    ref = sum(xp[j:j + 6, i:i + 6] for j in range(3) for i in range(3))
    np.testing.assert_array_equal(acc[0, 0], ref)


def test_linearity_in_weights():
    r = np.random.default_rng(3)
    x = r.integers(-128, 128, (1, 8, 6, 6)).astype(np.int8)
    w1 = r.integers(-60, 60, (4, 8, 3, 3)).astype(np.int8)
    w2 = r.integers(-60, 60, (4, 8, 3, 3)).astype(np.int8)
    one = np.ones(4, np.float32)
    a1 = rc.conv(x, w1, None, wqf=one, pad=(1, 1), out_dt="f32", want_acc=True)[1]
    a2 = rc.conv(x, w2, None, wqf=one, pad=(1, 1), out_dt="f32", want_acc=True)[1]
    a12 = rc.conv(x, (w1 + w2).astype(np.int8), None, wqf=one, pad=(1, 1), out_dt="f32", want_acc=True)[1]
    np.testing.assert_array_equal(a12, a1 + a2)


def test_grouped_equals_block_diagonal_dense():
    r = np.random.default_rng(4)
    g, ifg, ofg = 4, 3, 2
    x = r.integers(0, 256, (2, g * ifg, 5, 5)).astype(np.uint8)
    w = r.integers(-127, 128, (g * ofg, ifg, 3, 3)).astype(np.int8)
    wd = np.zeros((g * ofg, g * ifg, 3, 3), np.int8)
    for f in range(g * ofg):
        gi = f // ofg
        wd[f, gi * ifg:(gi + 1) * ifg] = w[f]
    bias = r.integers(-1000, 1000, g * ofg).astype(np.int32)
    cal = np.exp(r.uniform(np.log(1e-4), np.log(1e-2), g * ofg)).astype(np.float32)
    one = np.ones(g * ofg, np.float32)
    a = rc.conv(x, w, bias, wqf=one, calib=cal, pad=(1, 1), groups=g, out_dt="s8", act="relu")
    b = rc.conv(x, wd, bias, wqf=one, calib=cal, pad=(1, 1), groups=1, out_dt="s8", act="relu")
    np.testing.assert_array_equal(a, b)


# ------------------------------------------------------------------ epilogue, element by element
def epi_py(acc, bias, wqf, iqf, calib, act, out_dt, m=0.0, n=0.0):
    """Independent restatement in numpy float32 scalars; rounding via exact rational arithmetic."""
    from fractions import Fraction
    a = np.int32(np.int64(acc) + np.int64(bias))
    v = np.float32(a)
    v = np.float32(v * np.float32(wqf))
    v = np.float32(v * np.float32(iqf))
    if act == "relu":
        v = np.float32(max(np.float32(0), v))
    elif act == "clamp":
        v = np.float32(max(np.float32(m), min(np.float32(n), v)))
    v = np.float32(v * np.float32(calib))
    fr = Fraction(float(v))
    q = (abs(fr) + Fraction(1, 2)).__floor__()  # half away from zero
    q = q if fr >= 0 else -q
    lo, hi = (-128, 127) if out_dt == "s8" else (0, 255)
    return min(hi, max(lo, q))


def test_epilogue_matches_independent_restatement():
    r = np.random.default_rng(5)
    # exact .5 ties, saturation at both ends, tiny values, then random accumulators
    forced = [(a, 0, 1.0, 0.5) for a in (251, 253, -251, -253, 1_000_000_000, -1_000_000_000, 1, -1, 0)]
    rand = [(int(r.integers(-3_000_000, 3_000_000)), int(r.integers(-1000, 1000)),
             float(r.choice([1.0, 0.5, 0.37, 3e-4])), float(r.choice([0.5, 1.0, 1e-3, 21.1666])))
            for _ in range(600)]
    for out_dt in ("s8", "u8"):
        for act, m, nn in (("relu", 0.0, 0.0), ("none", 0.0, 0.0), ("clamp", 0.0, 6.0)):
            for acc, bias, wqf, calib in forced + rand:
                got = rc_epilogue(acc, bias, wqf, 1.0, calib, act, out_dt, m, nn)
                ref = epi_py(acc, bias, wqf, 1.0, calib, act, out_dt, m, nn)
                assert got == ref, (acc, bias, wqf, calib, act, out_dt, got, ref)


def rc_epilogue(acc, bias, wqf, iqf, calib, act, out_dt, m, n):
    import ctypes as C
    L = rc.lib()
    d = rc.Desc()
    d.in_dt, d.w_dt, d.bias_dt, d.out_dt, d.eltw_dt = rc.U8, rc.S8, rc.I32, rc.NAME_OF[out_dt], rc.NONE
    d.has_wqf, d.has_calib, d.iqf, d.oqf = 1, 1, iqf, 1.0
    d.act, d.act_m, d.act_n = rc.ACT_OF[act], m, n
    d.fused, d.non_conv_scale = 0, 1.0
    b = np.array([bias], np.int32)
    q = np.array([wqf], np.float32)
    c = np.array([calib], np.float32)
    return int(L.rc_epilogue(C.byref(d), int(acc), 0, b.ctypes.data, q.ctypes.data, c.ctypes.data, 0.0, None))


def test_round_half_away():
    L = rc.lib()
    for v, e in ((0.5, 1), (-0.5, -1), (1.5, 2), (2.5, 3), (-2.5, -3), (0.49999997, 0), (-0.49999997, 0),
                 (126.5, 127), (8388609.0, 8388609)):
        assert L.rc_round_half_away(v) == e


def test_truncation_rounding_identity_holds_for_every_float():
    # the HIP epilogue computes round-half-away as trunc(x + copysign(pred(0.5), x)); exhaustive over 2^32 patterns
    L = rc.lib()
    L.rc_count_round_trick_mismatches.restype = __import__("ctypes").c_long
    assert L.rc_count_round_trick_mismatches() == 0


def test_output_extent_formula():
    # closed form vs the reference test helper get_expected_output_tensor
    # (tests/test_cases/convolution_gpu_test.cpp:5524-5542)
    for n, pad, k, d, s in itertools.product((1, 5, 7, 56, 224), (0, 1, 3), (1, 3, 7), (1, 2), (1, 2)):
        wnd = (k - 1) * d + 1
        if wnd > n + 2 * pad:
            assert rc.out_extent(n, pad, k, d, s) == 1
        else:
            assert rc.out_extent(n, pad, k, d, s) == (n + 2 * pad - wnd) // s + 1


def test_fused_double_rounding_order():
    # conv result is rounded BEFORE the residual is added: round(2.4)=2, +0.4 -> round(2.4)=2; a single
    # rounding of 2.8 would give 3
    x = np.array([[[[12]]]], np.int8)
    w = np.array([[[[1]]]], np.int8)
    e = np.array([[[[2]]]], np.int8)
    out = rc.conv(x, w, np.zeros(1, np.int32), wqf=np.array([0.2], np.float32), out_dt="s8",
                  eltw=e, non_conv_scale=0.2, eltw_act="relu")
    assert out.item() == 2
