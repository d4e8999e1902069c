"""ctypes front-end of the CPU oracle (oracle/refconv.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg, never by the product package.

Pinned by the reference's own known-answer tables (tests/golden/*.json): conv / fused conv / pooling /
fully_connected in refconv.c, eltwise() here.  Parity unpinned (no table of the reference covers them): float pow and
mod of eltwise(); integer division and modulo by zero (0 here, undefined in the reference).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

S8, U8, I32, F32, NONE = 0, 1, 2, 3, -1
ACT_NONE, ACT_RELU, ACT_RELU_SLOPE, ACT_CLAMP = 0, 1, 2, 3

DT_OF = {np.dtype(np.int8): S8, np.dtype(np.uint8): U8, np.dtype(np.int32): I32, np.dtype(np.float32): F32}
NP_OF = {S8: np.int8, U8: np.uint8, I32: np.int32, F32: np.float32}
NAME_OF = {"s8": S8, "i8": S8, "u8": U8, "i32": I32, "f32": F32}
ACT_OF = {"none": ACT_NONE, "relu": ACT_RELU, "relu_slope": ACT_RELU_SLOPE, "clamp": ACT_CLAMP}


class Pitch(C.Structure):
    _fields_ = [(n, C.c_int64) for n in ("off", "pb", "pf", "py", "px")]


class Desc(C.Structure):
    _fields_ = (
        [(n, C.c_int) for n in ("in_dt", "w_dt", "bias_dt", "out_dt", "eltw_dt")]
        + [(n, C.c_int) for n in ("B", "IFM", "IH", "IW", "OFM", "OH", "OW", "FY", "FX")]
        + [(n, C.c_int) for n in ("sy", "sx", "dy", "dx", "pad_y", "pad_x", "groups")]
        + [("has_wqf", C.c_int), ("has_calib", C.c_int), ("iqf", C.c_float), ("oqf", C.c_float)]
        + [("act", C.c_int), ("act_m", C.c_float), ("act_n", C.c_float)]
        + [("fused", C.c_int), ("non_conv_scale", C.c_float)]
        + [("eltw_act", C.c_int), ("eltw_m", C.c_float), ("eltw_n", C.c_float)]
        + [("has_eltw_calib", C.c_int), ("esy", C.c_int), ("esx", C.c_int)]
        + [("in_p", Pitch), ("out_p", Pitch), ("eltw_p", Pitch)]
        + [("round_even", C.c_int), ("fc", C.c_int)]
    )


class PoolDesc(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("dt", "B", "F", "IH", "IW", "OH", "OW", "ky", "kx", "sy", "sx", "pad_y", "pad_x", "mode",
                                       "divider")]


def build(force=False):
    """Compile oracle/librefconv.so with the Makefile beside it."""
    so = os.path.join(_HERE, "librefconv.so")
    if force and os.path.exists(so):
        os.remove(so)
    subprocess.check_call(["make", "-s", "-C", _HERE, "librefconv.so"])
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "librefconv.so")
        if not os.path.exists(so):
            build()
        L = C.CDLL(so)
        L.rc_out_extent.restype = C.c_int
        L.rc_out_extent.argtypes = [C.c_int] * 5
        L.rc_conv.restype = C.c_int
        L.rc_conv.argtypes = [C.POINTER(Desc)] + [C.c_void_p] * 9 + [C.c_int]
        L.rc_epilogue.restype = C.c_double
        L.rc_epilogue.argtypes = [C.POINTER(Desc), C.c_int32, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                  C.c_double, C.c_void_p]
        L.rc_round_half_away.restype = C.c_float
        L.rc_round_half_away.argtypes = [C.c_float]
        L.rc_threads_available.restype = C.c_int
        L.rc_pool.restype = C.c_int
        L.rc_pool.argtypes = [C.POINTER(PoolDesc), C.c_void_p, C.c_void_p]
        L.rc_pool_out_extent.restype = C.c_int
        L.rc_pool_out_extent.argtypes = [C.c_int] * 4
        _LIB = L
    return _LIB


def out_extent(n, pad, filt, dil, stride):
    return lib().rc_out_extent(n, pad, filt, dil, stride)


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _dense(F, H, W):
    return Pitch(0, F * H * W, H * W, W, 1)


def conv(x, w, bias=None, wqf=None, calib=None, *, stride=(1, 1), pad=(0, 0), dilation=(1, 1), groups=1,
         out_dt=None, iqf=1.0, oqf=1.0, act="none", act_m=0.0, act_n=0.0,
         eltw=None, non_conv_scale=1.0, eltw_act="none", eltw_m=0.0, eltw_n=0.0, eltw_calib=None,
         eltw_stride=(1, 1), round_even=False, want_acc=False, nthreads=0, pad_end=None, fc=False):
    """Reference convolution on dense bfyx numpy arrays.

    x [B,IFM,IH,IW]; w [OFM,IFM/groups,FY,FX]; bias/wqf/calib/eltw_calib [OFM];
    eltw [B,OFM,>=OH*esy..,>=OW*esx..].  stride/pad/dilation are (y, x); pad is the zero padding on the
    low side, pad_end on the high side (default: the same; the reference reaches the asymmetric case with a
    zero border in front of the convolution, src/graph_optimizer/handle_input_padding.cpp:43-77).
    Returns out (and the int32 accumulators when want_acc).
    """
    L = lib()
    x = np.ascontiguousarray(x)
    w = np.ascontiguousarray(w)
    B, IFM, IH, IW = x.shape
    OFM, IFMg, FY, FX = w.shape
    assert IFMg * groups == IFM, (IFMg, groups, IFM)
    if pad_end is None:
        OH = out_extent(IH, pad[0], FY, dilation[0], stride[0])
        OW = out_extent(IW, pad[1], FX, dilation[1], stride[1])
    else:  # the border primitive enlarges the input; the window then slides over the enlarged tensor
        def ext(n, lo, hi, k, dil, st):
            wnd, span = (k - 1) * dil + 1, n + lo + hi
            return 1 if wnd > span else (span - wnd) // st + 1
        OH = ext(IH, pad[0], pad_end[0], FY, dilation[0], stride[0])
        OW = ext(IW, pad[1], pad_end[1], FX, dilation[1], stride[1])
    d = Desc()
    d.in_dt, d.w_dt = DT_OF[x.dtype], DT_OF[w.dtype]
    d.bias_dt = NONE if bias is None else DT_OF[np.asarray(bias).dtype]
    if out_dt is None:
        out_dt = d.in_dt
    elif isinstance(out_dt, str):
        out_dt = NAME_OF[out_dt]
    d.out_dt = out_dt
    d.B, d.IFM, d.IH, d.IW, d.OFM, d.OH, d.OW, d.FY, d.FX = B, IFM, IH, IW, OFM, OH, OW, FY, FX
    d.sy, d.sx, d.dy, d.dx, d.pad_y, d.pad_x, d.groups = stride[0], stride[1], dilation[0], dilation[1], pad[0], pad[1], groups
    d.has_wqf, d.has_calib = int(wqf is not None), int(calib is not None)
    d.iqf, d.oqf = iqf, oqf
    d.act, d.act_m, d.act_n = ACT_OF[act] if isinstance(act, str) else act, act_m, act_n
    d.fused = int(eltw is not None)
    d.non_conv_scale = non_conv_scale
    d.eltw_act = ACT_OF[eltw_act] if isinstance(eltw_act, str) else eltw_act
    d.eltw_m, d.eltw_n = eltw_m, eltw_n
    d.has_eltw_calib = int(eltw_calib is not None)
    d.esy, d.esx = eltw_stride
    d.in_p = _dense(IFM, IH, IW)
    d.out_p = _dense(OFM, OH, OW)
    d.round_even = int(round_even)
    d.fc = int(fc)
    if eltw is not None:
        eltw = np.ascontiguousarray(eltw)
        d.eltw_dt = DT_OF[eltw.dtype]
        d.eltw_p = _dense(eltw.shape[1], eltw.shape[2], eltw.shape[3])
    else:
        d.eltw_dt = NONE
    keep = []

    def f32(a):
        if a is None:
            return None
        a = np.ascontiguousarray(a, dtype=np.float32)
        keep.append(a)
        return a

    if bias is not None:
        bias = np.ascontiguousarray(bias)
    wqf, calib, eltw_calib = f32(wqf), f32(calib), f32(eltw_calib)
    out = np.zeros((B, OFM, OH, OW), dtype=NP_OF[out_dt])
    acc = np.zeros((B, OFM, OH, OW), dtype=np.int32) if want_acc else None
    if nthreads <= 0:
        nthreads = L.rc_threads_available()
    rc = L.rc_conv(C.byref(d), _ptr(x), _ptr(w), _ptr(bias), _ptr(wqf), _ptr(calib), _ptr(eltw), _ptr(eltw_calib),
                   _ptr(out), _ptr(acc), nthreads)
    if rc != 0:
        raise ValueError("refconv: unsupported combination")
    return (out, acc) if want_acc else out


POOL_MODE = {"max": 0, "average": 1, "average_no_padding": 1}


def pool_out_extent(n, pad, size, stride):
    return lib().rc_pool_out_extent(n, pad, size, stride)


def pool(x, mode, size, stride=(1, 1), pad=(0, 0), out_size=None, global_pooling=False):
    """Reference pooling on a dense bfyx array; mode "max" / "average" / "average_no_padding"; size/stride/pad are (y, x);
    pad = -input_offset.  The divider of an average follows src/gpu/pooling_gpu.cpp:36-52,100-108: the window size, unless
    the last window reaches past input + 2 * padding (then the window clipped to input + padding); average_no_padding
    counts the taps inside the input."""
    x = np.ascontiguousarray(x)
    B, F, IH, IW = x.shape
    if global_pooling:
        size = (IH, IW)
    if out_size is None:
        OH, OW = pool_out_extent(IH, pad[0], size[0], stride[0]), pool_out_extent(IW, pad[1], size[1], stride[1])
    else:
        OH, OW = out_size
    d = PoolDesc()
    d.dt = DT_OF[x.dtype]
    d.B, d.F, d.IH, d.IW, d.OH, d.OW = B, F, IH, IW, OH, OW
    d.ky, d.kx, d.sy, d.sx, d.pad_y, d.pad_x = size[0], size[1], stride[0], stride[1], pad[0], pad[1]
    d.mode = POOL_MODE[mode]
    overhang = (OH - 1) * stride[0] + size[0] > IH + 2 * pad[0] or (OW - 1) * stride[1] + size[1] > IW + 2 * pad[1]
    d.divider = 1 if mode == "average_no_padding" else (2 if mode == "average" and overhang else 0)
    out = np.zeros((B, F, OH, OW), x.dtype)
    if lib().rc_pool(C.byref(d), _ptr(x), _ptr(out)) != 0:
        raise ValueError("unsupported pooling")
    return out


def fully_connected(x, w, bias=None, wqf=None, calib=None, *, iqf=1.0, oqf=1.0, act="none", act_m=0.0):
    """Reference fully_connected: x [B, F, Y, X], w [OFM, F, Y, X] -> [B, OFM, 1, 1] in the input's data type.  Quantized
    (wqf given) it has its own epilogue, see rc_desc.fc; otherwise it is the convolution whose filter covers the input."""
    return conv(x, w, bias, wqf=wqf, calib=calib, iqf=iqf, oqf=oqf, act=act, act_m=act_m, fc=wqf is not None)


def _round_half_away(v):
    """OpenCL round() of float32 values (exact: the half is added in double)."""
    v = np.asarray(v, np.float32).astype(np.float64)
    return np.sign(v) * np.floor(np.abs(v) + 0.5)


def eltwise(inputs, mode="sum", strides=None, calib=None, oqf=1.0, relu=False, slope=0.0, coefficients=None):
    """The reference's stand-alone eltwise on logical [B, F, Y, X] arrays.
    - output size: input 0 divided by its stride when strides are given, else the per-axis maximum of the inputs
      (src/eltwise.cpp:57-73);
    - input i is read at (b % B_i, f % F_i, (y * sy_i) % Y_i, (x * sx_i) % X_i)
      (kernel_selector/core/cl_kernels/generic_eltwise_ref.cl:106-135);
    - the inputs are combined left to right, tmp_k = op(tmp_(k-1), input_(k+1))
      (src/gpu/eltwise_gpu.cpp:80-94), in the first input's type: float, or the 8-bit integer type with wrap-around
      after every step; with calib / oqf != 1 ("quantized") in int, then round(r * factor), convert_char_sat, and the
      activation on the char (kernel_selector/core/actual_kernels/eltwise/eltwise_kernel_base.cpp:238-340,
      generic_eltwise_ref.cl:311-330);
    - coefficients scale the inputs of a float sum (eltwise_kernel_base.cpp:259-275).
    Integer division / modulo by zero give 0 (undefined in the reference).  strides: one (sy, sx) per input."""
    ins = [np.asarray(a) for a in inputs]
    n = len(ins)
    strides = [(1, 1)] * n if strides is None else [tuple(s) for s in strides]
    if any(s != (1, 1) for s in strides):
        B, F = ins[0].shape[0], ins[0].shape[1]
        Y, X = ins[0].shape[2] // strides[0][0], ins[0].shape[3] // strides[0][1]
    else:
        B, F, Y, X = (max(a.shape[d] for a in ins) for d in range(4))

    def read(i):
        a, (sy, sx) = ins[i], strides[i]
        return a[np.ix_(np.arange(B) % a.shape[0], np.arange(F) % a.shape[1], (np.arange(Y) * sy) % a.shape[2],
                        (np.arange(X) * sx) % a.shape[3])]

    dt = ins[0].dtype
    quantized = dt != np.float32 and (calib is not None or oqf != 1.0)
    if dt == np.float32:
        def op(a, b):
            with np.errstate(all="ignore"):
                return {"sum": lambda: a + b, "sub": lambda: a - b, "max": lambda: np.fmax(a, b), "prod": lambda: a * b,
                        "div": lambda: a / b, "min": lambda: np.fmin(a, b), "pow": lambda: np.power(a, b),
                        "mod": lambda: np.fmod(a, b)}[mode]().astype(np.float32)
        v = read(0).astype(np.float32)
        if coefficients is not None:
            v = v * np.float32(coefficients[0])
        for i in range(1, n):
            w = read(i).astype(np.float32)
            if coefficients is not None:
                w = w * np.float32(coefficients[i])
            v = op(v, w)
        if relu:
            v = np.maximum(v, 0) + np.float32(slope) * np.minimum(v, 0)
        return v.astype(np.float32)

    def trunc_div(a, b):
        q = np.abs(a) // np.where(b == 0, 1, np.abs(b))
        return np.where(b == 0, 0, np.sign(a) * np.sign(b) * q)

    def iop(a, b):
        if mode == "div":
            return trunc_div(a, b)
        if mode == "mod":
            return np.where(b == 0, 0, a - trunc_div(a, b) * b)
        return {"sum": lambda: a + b, "sub": lambda: a - b, "max": lambda: np.maximum(a, b), "prod": lambda: a * b,
                "min": lambda: np.minimum(a, b)}[mode]()
    v = read(0).astype(np.int64)
    for i in range(1, n):
        # an operand of another type is cast to the unit type first (float -> char goes toward zero)
        v = iop(v, np.trunc(read(i)).astype(np.int64).astype(dt).astype(np.int64))
        # arithmetic in the unit type wraps; the quantized form computes in int (a product of four uint8 values can
        # leave its range: undefined in C, two's-complement wrap-around on the hardware)
        v = v.astype(np.int32 if quantized else dt).astype(np.int64)
    if quantized:
        f = np.float32(oqf) if calib is None else np.asarray(calib, np.float32).reshape(1, -1, 1, 1)
        v = np.clip(_round_half_away(v.astype(np.float32) * f), -128, 127).astype(np.int64)
    if relu:
        v = np.maximum(v, 0) + int(slope) * np.minimum(v, 0)
    return v.astype(dt)


def eltwise_sum(a, b, calib=None, oqf=1.0, relu=False):
    """Stand-alone element-wise sum of two int8 tensors in its quantized form (reference
    kernel_selector/core/cl_kernels/generic_eltwise_ref.cl:311-330): int sum, round((float)sum * factor) half away from
    zero with the factor per feature (calib) or per tensor (oqf), saturation to char, then the activation on the char."""
    s = a.astype(np.int32) + b.astype(np.int32)
    f = np.float32(oqf) if calib is None else np.asarray(calib, np.float32).reshape(1, -1, 1, 1)
    v = s.astype(np.float32) * f
    c = np.clip(_round_half_away(v), -128, 127).astype(np.int8)
    return np.maximum(c, 0) if relu else c
