"""ctypes binding of the thin C-ABI HIP layer (include/cldnn_hip.h).

Only plumbing lives here: handles, structure mirrors and numpy <-> device copies.
All arithmetic runs in the HIP kernels of libcldnn_hip.so; if the library or a GPU is
missing, calls raise -- there is no host fallback.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcldnn_hip.so")

S8, U8, I32, F32, NO_TYPE = 0, 1, 2, 3, -1
BFYX, YXFB, BYXF, FS_B_YX_FSV16, B_FS_YX_FSV4 = 0, 1, 2, 3, 4
ACT_NONE, ACT_RELU, ACT_RELU_SLOPE, ACT_CLAMP = 0, 1, 2, 3
IMPL_AUTO, IMPL_REF, IMPL_MFMA, IMPL_DEPTHWISE = 0, 1, 2, 3

NP_OF = {S8: np.int8, U8: np.uint8, I32: np.int32, F32: np.float32}
DT_OF = {np.dtype(np.int8): S8, np.dtype(np.uint8): U8, np.dtype(np.int32): I32, np.dtype(np.float32): F32}
DT_NAME = {"s8": S8, "i8": S8, "u8": U8, "i32": I32, "f32": F32}
ACT_NAME = {"none": ACT_NONE, "relu": ACT_RELU, "relu_slope": ACT_RELU_SLOPE, "clamp": ACT_CLAMP}
FMT_NAME = {"bfyx": BFYX, "yxfb": YXFB, "byxf": BYXF, "fs_b_yx_fsv16": FS_B_YX_FSV16, "b_fs_yx_fsv4": B_FS_YX_FSV4}


class HipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("cldnn_hip status %d: %s" % (status, message))
        self.status = status


class Tensor(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "dtype", "format", "b", "f", "y", "x",
        "pad_lo_b", "pad_lo_f", "pad_lo_y", "pad_lo_x", "pad_hi_b", "pad_hi_f", "pad_hi_y", "pad_hi_x")]

    @staticmethod
    def make(dtype, fmt, b, f, y, x, pad_y=0, pad_x=0, pad_hi_y=None, pad_hi_x=None):
        t = Tensor()
        t.dtype = DT_NAME.get(dtype, dtype) if isinstance(dtype, str) else dtype
        t.format = FMT_NAME.get(fmt, fmt) if isinstance(fmt, str) else fmt
        t.b, t.f, t.y, t.x = b, f, y, x
        t.pad_lo_y, t.pad_lo_x = pad_y, pad_x
        t.pad_hi_y = pad_y if pad_hi_y is None else pad_hi_y
        t.pad_hi_x = pad_x if pad_hi_x is None else pad_hi_x
        return t

    @property
    def shape(self):
        return (self.b, self.f, self.y, self.x)


class ConvDesc(C.Structure):
    _fields_ = [
        ("input", Tensor), ("output", Tensor), ("eltw", Tensor),
        ("weights_dtype", C.c_int32), ("bias_dtype", C.c_int32),
        ("ofm", C.c_int32), ("ifm", C.c_int32), ("fy", C.c_int32), ("fx", C.c_int32),
        ("stride_y", C.c_int32), ("stride_x", C.c_int32), ("dilation_y", C.c_int32), ("dilation_x", C.c_int32),
        ("pad_y", C.c_int32), ("pad_x", C.c_int32), ("groups", C.c_int32),
        ("has_wqf", C.c_int32), ("has_calib", C.c_int32),
        ("input_quantization_factor", C.c_float), ("output_quantization_factor", C.c_float),
        ("activation", C.c_int32), ("activation_m", C.c_float), ("activation_n", C.c_float),
        ("fused", C.c_int32), ("non_conv_scale", C.c_float),
        ("eltw_activation", C.c_int32), ("eltw_activation_m", C.c_float), ("eltw_activation_n", C.c_float),
        ("has_eltw_calib", C.c_int32), ("eltw_stride_y", C.c_int32), ("eltw_stride_x", C.c_int32),
        ("second_input_in_output", C.c_int32), ("round_to_even", C.c_int32),
        ("impl", C.c_int32), ("tile_override", C.c_int32),
        ("pad_end_delta_y", C.c_int32), ("pad_end_delta_x", C.c_int32), ("fully_connected", C.c_int32),
        ("conv_saturate", C.c_int32),
        ("sibling_split", C.c_int32),
        ("sibling_activation", C.c_int32),
        ("sibling_activation_m", C.c_float),
        ("sibling_activation_n", C.c_float),
    ]


class PoolingDesc(C.Structure):
    _fields_ = [("input", Tensor), ("output", Tensor)] + [(n, C.c_int32) for n in (
        "mode", "divider", "size_y", "size_x", "stride_y", "stride_x", "pad_y", "pad_x")]


ELTWISE_MAX_INPUTS = 4
ELTWISE_MODE = {"sum": 0, "sub": 1, "max": 2, "prod": 3, "div": 4, "min": 5, "pow": 6, "mod": 7}


class EltwiseDesc(C.Structure):
    _fields_ = [("mode", C.c_int32), ("n_inputs", C.c_int32), ("inputs", Tensor * ELTWISE_MAX_INPUTS),
                ("stride_y", C.c_int32 * ELTWISE_MAX_INPUTS), ("stride_x", C.c_int32 * ELTWISE_MAX_INPUTS),
                ("has_coefficients", C.c_int32), ("coefficients", C.c_float * ELTWISE_MAX_INPUTS), ("output", Tensor),
                ("quantized", C.c_int32), ("output_quantization_factor", C.c_float), ("activation", C.c_int32),
                ("m", C.c_float), ("n", C.c_float)]


class ConvInfo(C.Structure):
    _fields_ = [
        ("impl", C.c_int32), ("tile_index", C.c_int32), ("tile_pixels", C.c_int32), ("tile_ofm", C.c_int32),
        ("grid", C.c_int32), ("block", C.c_int32), ("lds_bytes", C.c_int32),
        ("ops", C.c_int64), ("bytes", C.c_int64), ("kernel_name", C.c_char * 96),
    ]


class EngineInfo(C.Structure):
    _fields_ = [
        ("cores_count", C.c_uint32), ("core_frequency", C.c_uint32),
        ("max_work_group_size", C.c_uint64), ("max_local_mem_size", C.c_uint64),
        ("max_global_mem_size", C.c_uint64), ("max_alloc_mem_size", C.c_uint64),
        ("wavefront_size", C.c_uint32), ("xcd_count", C.c_uint32),
        ("name", C.c_char * 64), ("arch", C.c_char * 32),
    ]


EVENT_HANDLER = C.CFUNCTYPE(None, C.c_void_p)

# name -> (restype, argtypes); the single source of truth for what the library must export
SIGNATURES = {
    "cldnn_hip_last_error": (C.c_char_p, []),
    "cldnn_hip_device_count": (C.c_uint32, []),
    "cldnn_hip_engine_create": (C.c_int32, [C.c_uint32, C.c_uint32, C.POINTER(C.c_void_p)]),
    "cldnn_hip_engine_retain": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_engine_release": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_engine_get_info": (C.c_int32, [C.c_void_p, C.POINTER(EngineInfo)]),
    "cldnn_hip_engine_stream": (C.c_void_p, [C.c_void_p]),
    "cldnn_hip_engine_flush": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_engine_finish": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_engine_used_memory": (C.c_int64, [C.c_void_p]),
    "cldnn_hip_engine_max_used_memory": (C.c_int64, [C.c_void_p]),
    "cldnn_hip_buffer_alloc": (C.c_int32, [C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p)]),
    "cldnn_hip_buffer_retain": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_buffer_release": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_buffer_lock": (C.c_void_p, [C.c_void_p]),
    "cldnn_hip_buffer_unlock": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_buffer_fill": (C.c_int32, [C.c_void_p, C.c_uint8]),
    "cldnn_hip_buffer_device_ptr": (C.c_void_p, [C.c_void_p]),
    "cldnn_hip_buffer_size": (C.c_size_t, [C.c_void_p]),
    "cldnn_hip_buffer_write": (C.c_int32, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t]),
    "cldnn_hip_buffer_read": (C.c_int32, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t]),
    "cldnn_hip_event_create_user": (C.c_int32, [C.c_void_p, C.c_uint32, C.POINTER(C.c_void_p)]),
    "cldnn_hip_event_record": (C.c_int32, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "cldnn_hip_event_record_begin": (C.c_int32, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "cldnn_hip_event_record_end": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_event_create_deferred": (C.c_int32, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "cldnn_hip_event_record_deferred": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_event_retain": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_event_release": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_event_wait": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_event_is_set": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_event_is_user": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_event_set": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_event_add_handler": (C.c_int32, [C.c_void_p, EVENT_HANDLER, C.c_void_p]),
    "cldnn_hip_event_elapsed_ns": (C.c_int32, [C.c_void_p, C.POINTER(C.c_uint64)]),
    "cldnn_hip_engine_wait_events": (C.c_int32, [C.c_void_p, C.POINTER(C.c_void_p), C.c_size_t]),
    "cldnn_hip_tensor_bytes": (C.c_size_t, [C.POINTER(Tensor)]),
    "cldnn_hip_tensor_offset": (C.c_int64, [C.POINTER(Tensor), C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    "cldnn_hip_reorder": (C.c_int32, [C.c_void_p, C.c_void_p, C.POINTER(Tensor), C.c_void_p, C.POINTER(Tensor)]),
    "cldnn_hip_copy_region": (C.c_int32, [C.c_void_p, C.c_void_p, C.POINTER(Tensor), C.c_void_p, C.POINTER(Tensor), C.c_int32, C.c_int32,
                                          C.c_int32, C.c_int32]),
    "cldnn_hip_activation": (C.c_int32, [C.c_void_p, C.c_void_p, C.POINTER(Tensor), C.c_void_p, C.POINTER(Tensor),
                                         C.c_int32, C.c_float, C.c_float]),
    "cldnn_hip_eltwise_sum": (C.c_int32, [C.c_void_p, C.c_void_p, C.POINTER(Tensor), C.c_void_p, C.POINTER(Tensor),
                                          C.c_void_p, C.POINTER(Tensor), C.c_int32, C.c_void_p, C.c_float, C.c_int32,
                                          C.c_float, C.c_float]),
    "cldnn_hip_eltwise": (C.c_int32, [C.c_void_p, C.POINTER(EltwiseDesc), C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p]),
    "cldnn_hip_conv_create": (C.c_int32, [C.c_void_p, C.POINTER(ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p,
                                          C.c_void_p, C.c_void_p, C.POINTER(C.c_void_p)]),
    "cldnn_hip_conv_tune": (C.c_int32, [C.c_void_p, C.POINTER(ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                        C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_float), C.POINTER(C.c_float),
                                        C.POINTER(C.c_float)]),
    "cldnn_hip_conv_release": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_conv_enqueue": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "cldnn_hip_conv_enqueue_static_scratch": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "cldnn_hip_conv_chain_create": (C.c_int32, [C.c_void_p, C.c_int32, C.POINTER(ConvDesc), C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                                C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                                C.POINTER(C.c_int32), C.POINTER(C.c_void_p)]),
    "cldnn_hip_conv_chain_release": (C.c_int32, [C.c_void_p]),
    "cldnn_hip_conv_chain_enqueue": (C.c_int32, [C.c_void_p, C.c_void_p, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p)]),
    "cldnn_hip_conv_chain_get_info": (C.c_int32, [C.c_void_p, C.POINTER(ConvInfo)]),
    "cldnn_hip_conv_accumulators": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "cldnn_hip_conv_get_info": (C.c_int32, [C.c_void_p, C.POINTER(ConvInfo)]),
    "cldnn_hip_conv_out_extent": (C.c_int32, [C.c_int32] * 5),
    "cldnn_hip_pooling": (C.c_int32, [C.c_void_p, C.POINTER(PoolingDesc), C.c_void_p, C.c_void_p]),
    "cldnn_hip_pooling_out_extent": (C.c_int32, [C.c_int32] * 4),
    "cldnn_hip_tile_config_count": (C.c_int32, []),
    "cldnn_hip_tile_config_name": (C.c_char_p, [C.c_int32]),
}

_lib = None


def lib():
    """Load libcldnn_hip.so (raises if it has not been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OSError("%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'`" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def check(status):
    if status != 0:
        raise HipError(status, lib().cldnn_hip_last_error().decode())


class Engine:
    def __init__(self, device=0, profiling=False):
        h = C.c_void_p()
        check(lib().cldnn_hip_engine_create(device, int(profiling), C.byref(h)))
        self.h = h

    def info(self):
        i = EngineInfo()
        check(lib().cldnn_hip_engine_get_info(self.h, C.byref(i)))
        return i

    def finish(self):
        check(lib().cldnn_hip_engine_finish(self.h))

    @property
    def stream(self):
        return lib().cldnn_hip_engine_stream(self.h)

    def close(self):
        if self.h:
            check(lib().cldnn_hip_engine_release(self.h))
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Buffer:
    """Device buffer holding one tensor."""

    def __init__(self, engine, tensor):
        self.engine, self.tensor = engine, tensor
        self.nbytes = lib().cldnn_hip_tensor_bytes(C.byref(tensor))
        if self.nbytes == 0:
            raise HipError(-2, lib().cldnn_hip_last_error().decode())
        h = C.c_void_p()
        check(lib().cldnn_hip_buffer_alloc(engine.h, self.nbytes, C.byref(h)))
        self.h = h

    @property
    def ptr(self):
        return lib().cldnn_hip_buffer_device_ptr(self.h)

    def write_raw(self, arr):
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes == self.nbytes, (arr.nbytes, self.nbytes)
        check(lib().cldnn_hip_buffer_write(self.h, 0, arr.ctypes.data, arr.nbytes))

    def read_raw(self):
        out = np.empty(self.nbytes // np.dtype(NP_OF[self.tensor.dtype]).itemsize, NP_OF[self.tensor.dtype])
        check(lib().cldnn_hip_buffer_read(self.h, 0, out.ctypes.data, out.nbytes))
        return out

    def close(self):
        if self.h:
            check(lib().cldnn_hip_buffer_release(self.h))
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Window:
    """Feature slices [first / 16, (first + features) / 16) of an fs_b_yx_fsv16 Buffer as a tensor of its own: the feature
    slice is the outermost axis of that layout, so a range of slices is contiguous memory."""

    def __init__(self, buf, first, features):
        t = buf.tensor
        assert t.format == FS_B_YX_FSV16 and first % 16 == 0 and first + features <= t.f and not (t.pad_lo_f or t.pad_hi_f)
        assert first + features == t.f or features % 16 == 0
        self.buf, self.engine = buf, buf.engine
        self.tensor = Tensor.make(t.dtype, t.format, t.b, features, t.y, t.x, t.pad_lo_y, t.pad_lo_x, t.pad_hi_y, t.pad_hi_x)
        self.nbytes = lib().cldnn_hip_tensor_bytes(C.byref(self.tensor))
        self.offset = (first // 16) * (buf.nbytes // (-(-t.f // 16)))

    @property
    def ptr(self):
        return self.buf.ptr + self.offset

    def close(self):
        pass  # the Buffer owns the memory


def reorder(engine, src, dst):
    check(lib().cldnn_hip_reorder(engine.h, src.ptr, C.byref(src.tensor), dst.ptr, C.byref(dst.tensor)))


POOL_MAX, POOL_AVERAGE = 0, 1
POOL_DIV_FIXED, POOL_DIV_VALID, POOL_DIV_PADDED = 0, 1, 2


def pool_forward(engine, x, mode, size, stride=(1, 1), pad=(0, 0), *, fmt="bfyx", in_pad=(0, 0), out_pad=(0, 0), out_size=None,
                 global_pooling=False):
    """numpy in, numpy out through cldnn_hip_pooling; arguments as oracle.refconv.pool (mode "max" / "average" /
    "average_no_padding", (y, x) pairs)."""
    L = lib()
    x = np.ascontiguousarray(x)
    xin = upload(engine, x, fmt, in_pad)
    t = xin.tensor
    if global_pooling:
        size = (t.y, t.x)
    if out_size is None:
        out_size = (L.cldnn_hip_pooling_out_extent(t.y, pad[0], size[0], stride[0]),
                    L.cldnn_hip_pooling_out_extent(t.x, pad[1], size[1], stride[1]))
    d = PoolingDesc()
    d.input = t
    d.output = Tensor.make(t.dtype, t.format, t.b, t.f, out_size[0], out_size[1], out_pad[0], out_pad[1])
    d.mode = POOL_MAX if mode == "max" else POOL_AVERAGE
    overhang = (out_size[0] - 1) * stride[0] + size[0] > t.y + 2 * pad[0] or (out_size[1] - 1) * stride[1] + size[1] > t.x + 2 * pad[1]
    d.divider = POOL_DIV_VALID if mode == "average_no_padding" else (POOL_DIV_PADDED if mode == "average" and overhang else POOL_DIV_FIXED)
    d.size_y, d.size_x, d.stride_y, d.stride_x, d.pad_y, d.pad_x = size[0], size[1], stride[0], stride[1], pad[0], pad[1]
    out = Buffer(engine, d.output)
    check(L.cldnn_hip_pooling(engine.h, C.byref(d), xin.ptr, out.ptr))
    res = download(engine, out)
    out.close()
    xin.close()
    return res


def eltwise_forward(engine, inputs, mode="sum", strides=None, calib=None, oqf=1.0, relu=False, slope=0.0, coefficients=None, *,
                    fmt="bfyx", in_pad=(0, 0), out_pad=(0, 0)):
    """numpy in, numpy out through cldnn_hip_eltwise; arguments as oracle.refconv.eltwise."""
    L = lib()
    ins = [np.ascontiguousarray(a) for a in inputs]
    n = len(ins)
    strides = [(1, 1)] * n if strides is None else [tuple(s) for s in strides]
    if any(s != (1, 1) for s in strides):
        shape = (ins[0].shape[0], ins[0].shape[1], ins[0].shape[2] // strides[0][0], ins[0].shape[3] // strides[0][1])
    else:
        shape = tuple(max(a.shape[d] for a in ins) for d in range(4))
    bufs = [upload(engine, a, fmt, in_pad) for a in ins]
    d = EltwiseDesc()
    d.mode, d.n_inputs = ELTWISE_MODE[mode], n
    for i in range(min(n, ELTWISE_MAX_INPUTS)):
        d.inputs[i] = bufs[i].tensor
        d.stride_y[i], d.stride_x[i] = strides[i]
        d.coefficients[i] = 1.0 if coefficients is None else coefficients[i]
    d.has_coefficients = coefficients is not None
    t = bufs[0].tensor
    d.output = Tensor.make(t.dtype, t.format, shape[0], shape[1], shape[2], shape[3], out_pad[0], out_pad[1])
    d.quantized = ins[0].dtype != np.float32 and (calib is not None or oqf != 1.0)
    d.output_quantization_factor = oqf
    d.activation = ACT_NONE if not relu else (ACT_RELU if slope == 0.0 else ACT_RELU_SLOPE)
    d.m = slope
    cal = None
    if calib is not None:
        cal = Buffer(engine, Tensor.make(F32, BFYX, 1, 1, 1, len(calib)))
        cal.write_raw(np.asarray(calib, np.float32))
    out = Buffer(engine, d.output)
    ptrs = (C.c_void_p * ELTWISE_MAX_INPUTS)(*[b.ptr for b in bufs[:ELTWISE_MAX_INPUTS]])
    try:
        check(L.cldnn_hip_eltwise(engine.h, C.byref(d), ptrs, cal.ptr if cal else None, out.ptr))
        return download(engine, out)
    finally:
        for b in bufs + [out] + ([cal] if cal else []):
            b.close()


def upload(engine, arr, fmt="bfyx", pad=(0, 0)):
    """numpy [B,F,Y,X] -> device buffer in `fmt` (through the device reorder kernel)."""
    arr = np.ascontiguousarray(arr)
    b, f, y, x = arr.shape
    dt = DT_OF[arr.dtype]
    plain = Buffer(engine, Tensor.make(dt, BFYX, b, f, y, x))
    plain.write_raw(arr)
    fmt_id = FMT_NAME[fmt] if isinstance(fmt, str) else fmt
    if fmt_id == BFYX and pad == (0, 0):
        return plain
    dst = Buffer(engine, Tensor.make(dt, fmt_id, b, f, y, x, pad[0], pad[1]))
    reorder(engine, plain, dst)
    engine.finish()
    plain.close()
    return dst


def download(engine, buf):
    """device buffer in any format -> numpy [B,F,Y,X]"""
    t = buf.tensor
    if t.format == BFYX and not any((t.pad_lo_y, t.pad_lo_x, t.pad_hi_y, t.pad_hi_x, t.pad_lo_f, t.pad_hi_f)):
        engine.finish()
        return buf.read_raw().reshape(t.b, t.f, t.y, t.x)
    plain = Buffer(engine, Tensor.make(t.dtype, BFYX, t.b, t.f, t.y, t.x))
    reorder(engine, buf, plain)
    engine.finish()
    out = plain.read_raw().reshape(t.b, t.f, t.y, t.x)
    plain.close()
    return out


class Conv:
    """One convolution / fused_conv_eltwise object of the C-ABI."""

    def __init__(self, engine, desc, weights, bias=None, wqf=None, calib=None, eltw_calib=None):
        self.engine, self.desc = engine, desc
        keep = []

        def p(a, dt=None):
            if a is None:
                return None
            a = np.ascontiguousarray(a, dtype=dt)
            keep.append(a)
            return a.ctypes.data

        h = C.c_void_p()
        check(lib().cldnn_hip_conv_create(engine.h, C.byref(desc), p(weights), p(bias), p(wqf, np.float32),
                                          p(calib, np.float32), p(eltw_calib, np.float32), C.byref(h)))
        self.h = h

    def info(self):
        i = ConvInfo()
        check(lib().cldnn_hip_conv_get_info(self.h, C.byref(i)))
        return i

    def enqueue(self, src, dst, eltw=None):
        check(lib().cldnn_hip_conv_enqueue(self.h, src.ptr, dst.ptr, eltw.ptr if eltw is not None else None))

    def enqueue_static_scratch(self, src, dst, eltw=None):
        """the entry point that allocates nothing: scratch from the array inside the code object"""
        check(lib().cldnn_hip_conv_enqueue_static_scratch(self.h, src.ptr, dst.ptr, eltw.ptr if eltw is not None else None))

    def accumulators(self, src):
        d = self.desc
        t = Tensor.make(I32, BFYX, d.output.b, d.output.f, d.output.y, d.output.x)
        acc = Buffer(self.engine, t)
        check(lib().cldnn_hip_conv_accumulators(self.h, src.ptr, acc.ptr))
        out = download(self.engine, acc)
        acc.close()
        return out

    def close(self):
        if self.h:
            check(lib().cldnn_hip_conv_release(self.h))
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class ConvChain:
    """Two or three convolutions executed as one launch (cldnn_hip_conv_chain_*): stage k + 1 is a 1x1 convolution that
    reads stage k's result.  stages: list of (desc, weights, bias, wqf, calib, eltw_calib); keep[k] False: stage k's
    result is never written.  Raises HipError (CLDNN_HIP_UNSUPPORTED_FORMAT) when the stages cannot be chained."""

    def __init__(self, engine, stages, keep=None):
        self.engine, n = engine, len(stages)
        self.n = n
        hold = []

        def column(i, dt=None):
            arr = (C.c_void_p * n)()
            for k, st in enumerate(stages):
                a = st[i] if i < len(st) else None
                if a is not None:
                    a = np.ascontiguousarray(a, dtype=dt)
                    hold.append(a)
                    arr[k] = a.ctypes.data
            return arr

        descs = (ConvDesc * n)(*[st[0] for st in stages])
        keep_arr = (C.c_int32 * n)(*[1 if (keep is None or keep[k]) else 0 for k in range(n)])
        h = C.c_void_p()
        check(lib().cldnn_hip_conv_chain_create(engine.h, n, descs, column(1), column(2), column(3, np.float32), column(4, np.float32),
                                                column(5, np.float32), keep_arr, C.byref(h)))
        self.h = h

    def info(self):
        i = ConvInfo()
        check(lib().cldnn_hip_conv_chain_get_info(self.h, C.byref(i)))
        return i

    def pointers(self, outs, eltws=None):
        """device pointer arrays for enqueue_raw (entries may be None)"""
        o = (C.c_void_p * self.n)(*[None if b is None else b.ptr for b in outs])
        e = (C.c_void_p * self.n)(*[None if (eltws is None or eltws[k] is None) else eltws[k].ptr for k in range(self.n)])
        return o, e

    def enqueue(self, src, outs, eltws=None):
        o, e = self.pointers(outs, eltws)
        check(lib().cldnn_hip_conv_chain_enqueue(self.h, src.ptr, o, e))

    def close(self):
        if self.h:
            check(lib().cldnn_hip_conv_chain_release(self.h))
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def tile_config_name(row):
    """Name of row `row` (0-based) of the built-in tile table."""
    name = lib().cldnn_hip_tile_config_name(row)
    return None if name is None else name.decode()


def conv_tune(engine, desc, w, bias=None, wqf=None, calib=None, eltw_calib=None, runs=20):
    """cldnn_hip_conv_tune: -> (best row or -1, its microseconds, microseconds of the table's own choice, per-row list)"""
    L = lib()
    keep = [np.ascontiguousarray(w)] + [None if a is None else np.ascontiguousarray(a) for a in (bias, wqf, calib, eltw_calib)]
    ptr = [None if a is None else a.ctypes.data_as(C.c_void_p) for a in keep]
    best, best_us, default_us = C.c_int32(-1), C.c_float(0), C.c_float(0)
    rows = (C.c_float * L.cldnn_hip_tile_config_count())()
    check(L.cldnn_hip_conv_tune(engine.h, C.byref(desc), ptr[0], ptr[1], ptr[2], ptr[3], ptr[4], runs, C.byref(best), C.byref(best_us),
                                C.byref(default_us), rows))
    return best.value, best_us.value, default_us.value, list(rows)


def conv_desc(x_t, w_shape, out_dt, *, stride=(1, 1), pad=(0, 0), dilation=(1, 1), groups=1, out_fmt=None,
              out_pad=(0, 0), bias_dt=NO_TYPE, w_dt=S8, has_wqf=False, has_calib=False, iqf=1.0, oqf=1.0,
              act="none", act_m=0.0, act_n=0.0, eltw_t=None, non_conv_scale=1.0, eltw_act="none", eltw_m=0.0,
              eltw_n=0.0, has_eltw_calib=False, eltw_stride=(1, 1), in_place=False, round_even=False,
              impl=IMPL_AUTO, tile=0, pad_end=None, fc=False, conv_saturate=0, sibling_split=0, sibling_act="none",
              sibling_act_m=0.0, sibling_act_n=0.0):
    """Fill a ConvDesc from an input Tensor and the weight shape [OFM, IFM/groups, FY, FX].
    pad = zero padding on the low side (y, x); pad_end = on the high side (default: the same)."""
    L = lib()
    ofm, ifm_g, fy, fx = w_shape
    d = ConvDesc()
    d.input = x_t
    pad_end = pad if pad_end is None else pad_end
    oh, ow = out_extent(x_t.y, pad[0], pad_end[0], fy, dilation[0], stride[0]), out_extent(x_t.x, pad[1], pad_end[1], fx, dilation[1], stride[1])
    out_dt = DT_NAME[out_dt] if isinstance(out_dt, str) else out_dt
    d.output = Tensor.make(out_dt, x_t.format if out_fmt is None else out_fmt, x_t.b, ofm, oh, ow, out_pad[0], out_pad[1])
    d.weights_dtype, d.bias_dtype = w_dt, bias_dt
    d.ofm, d.ifm, d.fy, d.fx = ofm, ifm_g * groups, fy, fx
    d.stride_y, d.stride_x, d.dilation_y, d.dilation_x = stride[0], stride[1], dilation[0], dilation[1]
    d.pad_y, d.pad_x, d.groups = pad[0], pad[1], groups
    d.has_wqf, d.has_calib = int(has_wqf), int(has_calib)
    d.input_quantization_factor, d.output_quantization_factor = iqf, oqf
    d.activation = ACT_NAME[act] if isinstance(act, str) else act
    d.activation_m, d.activation_n = act_m, act_n
    d.fused = int(eltw_t is not None or in_place)
    if eltw_t is not None:
        d.eltw = eltw_t
    d.non_conv_scale = non_conv_scale
    d.eltw_activation = ACT_NAME[eltw_act] if isinstance(eltw_act, str) else eltw_act
    d.eltw_activation_m, d.eltw_activation_n = eltw_m, eltw_n
    d.has_eltw_calib = int(has_eltw_calib)
    d.eltw_stride_y, d.eltw_stride_x = eltw_stride
    d.second_input_in_output = int(in_place)
    d.round_to_even = int(round_even)
    d.impl, d.tile_override = impl, tile
    d.pad_end_delta_y, d.pad_end_delta_x = pad_end[0] - pad[0], pad_end[1] - pad[1]
    d.fully_connected = int(fc)
    d.conv_saturate = int(conv_saturate)
    d.sibling_split = int(sibling_split)
    d.sibling_activation = ACT_NAME[sibling_act] if isinstance(sibling_act, str) else sibling_act
    d.sibling_activation_m, d.sibling_activation_n = sibling_act_m, sibling_act_n
    return d


def out_extent(n, pad_lo, pad_hi, filt, dil, stride):
    """output extent along one axis; a window larger than the padded input gives 1"""
    wnd, span = (filt - 1) * dil + 1, n + pad_lo + pad_hi
    return 1 if wnd > span else (span - wnd) // stride + 1


def conv_forward(engine, x, w, bias=None, wqf=None, calib=None, *, stride=(1, 1), pad=(0, 0), dilation=(1, 1),
                 groups=1, out_dt=None, iqf=1.0, oqf=1.0, act="none", act_m=0.0, act_n=0.0, eltw=None,
                 non_conv_scale=1.0, eltw_act="none", eltw_m=0.0, eltw_n=0.0, eltw_calib=None, eltw_stride=(1, 1),
                 round_even=False, fmt="bfyx", in_pad=(0, 0), out_pad=(0, 0), impl=IMPL_AUTO, tile=0,
                 want_acc=False, want_info=False, pad_end=None, fc=False, in_place=False, conv_saturate=0, sibling_split=0,
                 sibling_act="none", sibling_act_m=0.0, sibling_act_n=0.0):
    """numpy in, numpy out: upload (reordering to `fmt`), run the HIP convolution, download.

    Argument meaning follows oracle.refconv.conv so that parity tests can call both alike.  in_place: the residual
    operand `eltw` (of the output's type and size) is put into the output buffer and read from there
    (second_input_in_output).
    """
    x = np.ascontiguousarray(x)
    w = np.ascontiguousarray(w)
    xin = upload(engine, x, fmt, in_pad)
    if out_dt is None:
        out_dt = DT_OF[x.dtype]
    e_buf = None
    # a first layer reads b_fs_yx_fsv4 and writes the blocked layout the rest of the network runs in
    first_layer = FMT_NAME.get(fmt, fmt) == B_FS_YX_FSV4
    if eltw is not None and not in_place:
        e_buf = upload(engine, np.ascontiguousarray(eltw), "fs_b_yx_fsv16" if first_layer else fmt)
    bias_dt = NO_TYPE if bias is None else DT_OF[np.asarray(bias).dtype]
    d = conv_desc(xin.tensor, w.shape, out_dt, stride=stride, pad=pad, dilation=dilation, groups=groups,
                  out_fmt=FS_B_YX_FSV16 if first_layer else None, out_pad=out_pad, bias_dt=bias_dt, w_dt=DT_OF[w.dtype], has_wqf=wqf is not None,
                  has_calib=calib is not None, iqf=iqf, oqf=oqf, act=act, act_m=act_m, act_n=act_n,
                  eltw_t=None if e_buf is None else e_buf.tensor, non_conv_scale=non_conv_scale, eltw_act=eltw_act,
                  eltw_m=eltw_m, eltw_n=eltw_n, has_eltw_calib=eltw_calib is not None, eltw_stride=eltw_stride,
                  round_even=round_even, impl=impl, tile=tile, pad_end=pad_end, fc=fc, in_place=in_place,
                  conv_saturate=conv_saturate, sibling_split=sibling_split, sibling_act=sibling_act,
                  sibling_act_m=sibling_act_m, sibling_act_n=sibling_act_n)
    c = Conv(engine, d, w, bias, wqf, calib, eltw_calib)
    if in_place:
        out = upload(engine, np.ascontiguousarray(eltw), "fs_b_yx_fsv16" if first_layer else fmt, out_pad)
        assert bytes(out.tensor) == bytes(d.output), "the residual must have the output's type, size and padding"
    else:
        out = Buffer(engine, d.output)
    c.enqueue(xin, out, e_buf)
    res = [download(engine, out)]
    if want_acc:
        res.append(c.accumulators(xin))
    if want_info:
        res.append(c.info())
    c.close()
    out.close()
    xin.close()
    if e_buf is not None:
        e_buf.close()
    return res[0] if len(res) == 1 else tuple(res)
