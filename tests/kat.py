"""Builders that turn the committed known-answer tables (tests/golden/conv_kat.json)
into dense bfyx problems, the way the reference's test harnesses lay them out
(tests/test_cases/convolution_gpu_test.cpp:4006-4063,
 tests/test_cases/fused_conv_eltwise_gpu_test.cpp:169-236)."""
import json
import os

import numpy as np

_G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "conv_kat.json")
NP = {"s8": np.int8, "u8": np.uint8, "f32": np.float32, "i32": np.int32}


def load():
    with open(_G) as f:
        return json.load(f)


def _num(v):
    if isinstance(v, str):
        a, b = v.split("/")
        return np.float32(float(a) / float(b))
    return v


def diag_problem(case, fused=False):
    """N independent 1-D features -> (x, w, bias, factors..., expected stored values)."""
    feats = case["features"]
    n = len(feats)
    in_np = NP[case["in_dt"]]
    is_float = case["in_dt"] == "f32"
    x = np.zeros((1, n, 1, 4), in_np)
    w = np.zeros((n, n, 1, 3), np.float32 if is_float else np.int8)
    bias = np.zeros(n, np.float32 if is_float else np.int32)
    for i, ft in enumerate(feats):
        x[0, i, 0, :] = ft["input"]
        w[i, i, 0, :] = ft["weights"]
        bias[i] = ft["bias"]
    out = {"x": x, "w": w, "bias": bias}
    out["wqf"] = np.array([_num(ft["wqf"]) if ft.get("wqf") is not None else 1.0 for ft in feats], np.float32)
    pre = np.array([ft["pre_relu"] for ft in feats], np.float64)  # [n, 2]
    odt = case["out_dt"]
    relu = np.maximum(pre, 0)
    if odt == "u8":
        exp = np.clip(relu, 0, 255)
    elif odt == "s8":
        exp = np.clip(relu, -128, 127)
    else:
        exp = relu
    out["expected"] = exp.reshape(1, n, 1, 2)
    if fused:
        out["conv_calib"] = np.array([ft["conv_calib"] if ft.get("conv_calib") is not None else 1.0 for ft in feats], np.float32)
        out["eltw_calib"] = np.array([ft["eltw_calib"] if ft.get("eltw_calib") is not None else 1.0 for ft in feats], np.float32)
        nci = np.zeros((1, n, 1, 2), in_np)
        for i, ft in enumerate(feats):
            nci[0, i, 0, :] = ft["nci"]
        out["nci"] = nci
        out["non_conv_scale"] = np.float32(_num(case["non_conv_scale"]))
    return out


def _yxfb_to_bfyx(flat, shape):
    b, f, h, w = shape
    return np.ascontiguousarray(np.array(flat).reshape(h, w, f, b).transpose(3, 2, 0, 1))


def indexing_problem(case, all_cases):
    """-> dict(x, w, bias, stride, pad, groups, act, expected[bfyx], tol, dt)"""
    dt = NP[case["dt"]]
    groups = case.get("groups", 1)
    if "replicate_from" in case:
        base = next(c for c in all_cases if c["name"] == case["replicate_from"])
        bp = indexing_problem(base, all_cases)
        pairs, batch = case["feature_pairs"], case["batch"]
        x = np.tile(bp["x"], (batch, pairs, 1, 1))
        w = np.tile(bp["w"], (pairs, 1, 1, 1))
        bias = np.tile(bp["bias"], pairs)
        exp = np.tile(bp["expected"], (batch, pairs, 1, 1))
        return dict(x=x, w=w, bias=bias, stride=tuple(case["stride"]), pad=tuple(case["pad"]), groups=groups,
                    act=case["act"], expected=exp, tol=case["tol"], dt=case["dt"])
    if case.get("in_layout") == "yxfb":
        x = _yxfb_to_bfyx(case["input"], case["in_shape"]).astype(dt)
    else:
        x = np.array(case["input"]).reshape(case["in_shape"]).astype(dt)
    w = np.array(case["weights"]).reshape(case["w_shape"]).astype(dt)
    bias = None
    if case["bias"] is not None:
        bdt = NP[case.get("bias_dt", "f32" if case["dt"] == "f32" else "i32")]
        bias = np.array(case["bias"], bdt)
    if case.get("out_layout") == "yxfb":
        exp = _yxfb_to_bfyx(case["expected"], case["out_shape"]).astype(np.float64)
    else:
        exp = np.array(case["expected"], np.float64).reshape(case["out_shape"])
    return dict(x=x, w=w, bias=bias, stride=tuple(case["stride"]), pad=tuple(case["pad"]), groups=groups,
                act=case["act"], expected=exp, tol=case["tol"], dt=case["dt"])


def api_problem(case, all_indexing):
    """A case of the "api" section -> dict(x, w_parts, bias_parts, w, bias, stride, pad, pad_above, pad_below, out_pad_lower,
    out_pad_upper, groups, split, act, act_slope, expected [bfyx, NaN where the reference asserts nothing], tol, dt).
    w / bias are the parts concatenated along the output features (what `groups = split` takes)."""
    dt = NP[case["dt"]]
    split, groups = case.get("split", 1), case.get("groups", 1)
    if "replicate_from" in case:
        base = next(c for c in all_indexing if c["name"] == case["replicate_from"])
        bp = indexing_problem(base, all_indexing)
        pairs, batch = case["feature_pairs"], case["batch"]
        x = np.tile(bp["x"], (batch, pairs, 1, 1))
        w = np.tile(bp["w"], (pairs, 1, 1, 1))
        bias = np.tile(bp["bias"], pairs)
        exp = np.tile(bp["expected"], (batch, pairs, 1, 1))
    else:
        if case.get("in_layout") == "yxfb":
            x = _yxfb_to_bfyx(case["input"], case["in_shape"]).astype(dt)
        else:
            x = np.array(case["input"]).reshape(case["in_shape"]).astype(dt)
        if "weights_parts" in case:
            w = np.concatenate([np.array(p).reshape(case["w_shape"]) for p in case["weights_parts"]]).astype(dt)
            bias = np.concatenate([np.array(p) for p in case["bias_parts"]]).astype(np.float32)
        else:
            w = np.array(case["weights"]).reshape(case["w_shape"]).astype(dt)
            bias = np.array(case["bias"], np.float32)
        e = np.array([np.nan if v is None else v for v in case["expected"]], np.float64)
        exp = _yxfb_to_bfyx(e, case["out_shape"]) if case.get("out_layout") == "yxfb" else e.reshape(case["out_shape"])
    n = max(split, 1)
    return dict(x=x, w=w, bias=bias, w_parts=np.split(w, n), bias_parts=np.split(bias, n), stride=tuple(case["stride"]),
                pad=tuple(case["pad"]), pad_above=tuple(case.get("pad_above", (0, 0))), pad_below=tuple(case.get("pad_below", (0, 0))),
                out_pad_lower=tuple(case.get("out_pad_lower", (0, 0))), out_pad_upper=tuple(case.get("out_pad_upper", (0, 0))),
                groups=groups, split=split, act=case["act"], act_slope=case.get("act_slope", 0.0), expected=exp, tol=case["tol"],
                dt=case["dt"])


def assert_close_where_given(out, expected, tol):
    mask = ~np.isnan(expected)
    assert out.shape == expected.shape
    np.testing.assert_allclose(out.astype(np.float64)[mask], expected[mask], atol=max(tol, 1e-5), rtol=0)


def quantize_weights(w):
    """per output feature: w -> round(w * 127 / max|w|), factor max|w| / 127
    (reference tests/test_cases/convolution_gpu_test.cpp:3561-3584; C round() = half away from zero)"""
    w = np.asarray(w, np.float32)
    q = np.empty_like(w)
    f = np.empty(w.shape[0], np.float32)
    for o in range(w.shape[0]):
        m = np.float32(np.abs(w[o]).max()) or np.float32(1.0)
        v = w[o] * np.float32(127.0) / m
        q[o] = np.sign(v) * np.floor(np.abs(v) + np.float32(0.5))
        f[o] = m / np.float32(127.0)
    return q, f


def calibrate(out):
    """per feature 127 / max|out| (reference :3585-3602); out [1, F, H, W]"""
    return (np.float32(127.0) / np.abs(out[0]).reshape(out.shape[1], -1).max(axis=1)).astype(np.float32)
