"""ctypes binding of the clDNN-compatible C API (include/api/C/cldnn.h, built as libclDNN.so).

The classes carry the names and argument order of the reference's C++ wrappers
(api/CPP/{tensor,layout,memory,engine,topology,network}.hpp, api/CPP/convolution.hpp:38-700,
api_extension/CPP/fused_conv_eltwise.hpp:37-160), so a test written against them reads like the
reference's own tests.  Nothing here computes: every call goes to the shared library, and the
library fails loudly when there is no GPU.
"""
import ctypes as C
import json
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libclDNN.so")

# ------------------------------------------------------------------------------------------ C types
SUCCESS, ERROR, INVALID_ARG, OUT_OF_RESOURCES, DEVICE_ERROR = 0, -1, -2, -3, -4
UNSUPPORTED_SIZE, UNSUPPORTED_FORMAT, DIMENSION_MISMATCH = -5, -6, -7


class format:  # noqa: N801  (reference spelling)
    yxfb, byxf, bfyx, fyxb, b_fs_yx_fsv4, fs_b_yx_fsv16, any = 0, 1, 2, 3, 31, 35, -1


class data_types:  # noqa: N801
    i8, f16, f32, u8, i32, i64 = 1, 2 | 0x80, 4 | 0x80, 1 | 0x40, 4, 8


NP_OF = {data_types.i8: np.int8, data_types.u8: np.uint8, data_types.i32: np.int32, data_types.f32: np.float32}
DT_OF = {np.dtype(v): k for k, v in NP_OF.items()}


class activation_func:  # noqa: N801
    none, logistic, hyperbolic_tan, relu, relu_negative_slope, clamp = 0, 1, 2, 3, 4, 5
    softrelu, abs, linear, square, sqrt, elu, negative = 6, 7, 8, 9, 10, 11, 25


class pooling_mode:  # noqa: N801
    max, average, average_no_padding, max_with_argmax, bilinear = range(5)


class eltwise_mode:  # noqa: N801
    sum, sub, max, prod, div, min, pow, mod = range(8)


class build_option_type:  # noqa: N801
    fusing, optimize_data, debug, outputs, tuning_config, graph_dumps_dir, learning_config = range(7)


class c_tensor(C.Structure):
    _fields_ = [("batch_num", C.c_size_t), ("feature_num", C.c_size_t), ("spatial_num", C.c_size_t),
                ("local_num", C.c_size_t), ("sizes", C.c_int32 * 8)]


class c_padding(C.Structure):
    _fields_ = [("lower_size", c_tensor), ("upper_size", c_tensor), ("filling_value", C.c_float)]


class c_layout(C.Structure):
    _fields_ = [("data_type", C.c_size_t), ("format", C.c_int32), ("size", c_tensor), ("padding", c_padding)]


class c_float_arr(C.Structure):
    _fields_ = [("data", C.POINTER(C.c_float)), ("size", C.c_size_t)]


class c_tensor_arr(C.Structure):
    _fields_ = [("data", C.POINTER(c_tensor)), ("size", C.c_size_t)]


class c_id_arr(C.Structure):
    _fields_ = [("data", C.POINTER(C.c_char_p)), ("size", C.c_size_t)]


class c_optional_dt(C.Structure):
    _fields_ = [("data_type", C.c_int), ("enabled", C.c_char)]


_BASE = [("type", C.c_void_p), ("id", C.c_char_p), ("input", c_id_arr), ("output_padding", c_padding),
         ("output_data_type", c_optional_dt)]


class c_primitive_desc(C.Structure):
    _fields_ = _BASE


class c_input_layout_desc(C.Structure):
    _fields_ = _BASE + [("layout", c_layout)]


class c_data_desc(C.Structure):
    _fields_ = _BASE + [("mem", C.c_void_p)]


class c_reorder_desc(C.Structure):
    _fields_ = _BASE + [("output_format", C.c_int), ("mean_subtract", C.c_char_p), ("subtract_per_feature", c_float_arr),
                        ("mean_mode", C.c_int)]


class c_act_params(C.Structure):
    _fields_ = [("a", C.c_float), ("b", C.c_float)]


class c_activation_desc(C.Structure):
    _fields_ = _BASE + [("activation_func", C.c_int), ("additional_params", c_act_params),
                        ("additional_params_input", C.c_char_p)]


class c_pooling_desc(C.Structure):
    _fields_ = _BASE + [("argmax", C.c_char_p), ("mode", C.c_int32), ("global_pooling", C.c_int8), ("input_offset", c_tensor),
                        ("stride", c_tensor), ("size", c_tensor), ("with_output_size", C.c_uint32), ("output_size", c_tensor)]


class c_fully_connected_desc(C.Structure):
    _fields_ = _BASE + [("with_activation", C.c_uint32), ("activation_negative_slope", C.c_float), ("weights", C.c_char_p),
                        ("bias", C.c_char_p), ("weights_quantization_factors", C.c_char_p), ("output_calibration_factors", C.c_char_p),
                        ("input_quantization_factor", C.c_float), ("output_quantization_factor", C.c_float)]


_ELTW = [("output_calibration_factors", C.c_char_p), ("output_quantization_factor", C.c_float), ("mode", C.c_int32),
         ("coefficients", c_float_arr), ("with_activation", C.c_uint32), ("activation_negative_slope", C.c_float),
         ("stride", c_tensor_arr)]


class c_eltwise_desc(C.Structure):
    _fields_ = _BASE + _ELTW


_CONV = [("input_offset", c_tensor), ("stride", c_tensor), ("dilation", c_tensor), ("with_activation", C.c_uint32),
         ("activation_negative_slope", C.c_float), ("split", C.c_uint32), ("with_output_size", C.c_uint32),
         ("output_size", c_tensor), ("weights", c_id_arr), ("bias", c_id_arr), ("weights_quantization_factors", c_id_arr),
         ("output_calibration_factors", c_id_arr), ("input_quantization_factor", C.c_float),
         ("output_quantization_factor", C.c_float)]


class c_convolution_desc(C.Structure):
    _fields_ = _BASE + _CONV + [("groups", C.c_uint32), ("padding_above", c_tensor), ("padding_below", c_tensor)]


class c_conv_data(C.Structure):
    _fields_ = _CONV


class c_eltw_data(C.Structure):
    _fields_ = _ELTW


class c_fused_conv_eltwise_desc(C.Structure):
    _fields_ = _BASE + [("conv", c_conv_data), ("eltw", c_eltw_data), ("non_conv_scale", C.c_float),
                        ("second_input_in_output", C.c_uint8)]


class c_engine_configuration(C.Structure):
    _fields_ = [("enable_profiling", C.c_uint32), ("meaningful_kernels_names", C.c_uint32), ("dump_custom_program", C.c_uint32),
                ("compiler_options", C.c_char_p), ("single_kernel_name", C.c_char_p), ("enable_parallelisation", C.c_uint32),
                ("engine_log", C.c_char_p), ("sources_dumps_dir", C.c_char_p), ("priority_mode", C.c_int16),
                ("throttle_mode", C.c_int16), ("enable_memory_pool", C.c_uint32), ("context", C.c_void_p),
                ("tuning_cache_path", C.c_char_p)]


class c_engine_info(C.Structure):
    _fields_ = [("cores_count", C.c_uint32), ("core_frequency", C.c_uint32), ("max_work_group_size", C.c_uint64),
                ("max_local_mem_size", C.c_uint64), ("max_global_mem_size", C.c_uint64), ("max_alloc_mem_size", C.c_uint64),
                ("max_image2d_width", C.c_uint64), ("max_image2d_height", C.c_uint64), ("supports_fp16", C.c_uint8),
                ("supports_fp16_denorms", C.c_uint8), ("supports_subgroups_short", C.c_uint8), ("supports_image", C.c_uint8),
                ("supports_imad", C.c_uint8), ("supports_immad", C.c_uint8)]


class c_version(C.Structure):
    _fields_ = [("major", C.c_int32), ("minor", C.c_int32), ("build", C.c_int32), ("revision", C.c_int32)]


class c_profiling_interval(C.Structure):
    _fields_ = [("name", C.c_char_p), ("nanoseconds", C.c_uint64)]


class c_build_option(C.Structure):
    _fields_ = [("type", C.c_int32), ("data", C.c_void_p)]


class c_network_output(C.Structure):
    _fields_ = [("event", C.c_void_p), ("memory", C.c_void_p)]


_ST = C.POINTER(C.c_int32)
_H = C.c_void_p
_NAMES = [_H, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t), _ST]
EVENT_HANDLER = C.CFUNCTYPE(None, C.c_void_p)

# name -> (restype, argtypes); every function declared in include/api/C/cldnn.h and primitives.h
SIGNATURES = {
    "cldnn_get_version": (c_version, [_ST]),
    "cldnn_create_topology": (_H, [_ST]),
    "cldnn_add_primitive": (None, [_H, C.c_void_p, _ST]),
    "cldnn_change_input_layout": (None, [_H, C.c_char_p, c_layout, _ST]),
    "cldnn_get_primitive_ids": (None, _NAMES),
    "cldnn_retain_topology": (None, [_H, _ST]),
    "cldnn_release_topology": (None, [_H, _ST]),
    "cldnn_get_engine_count": (C.c_uint32, [C.c_int32, _ST]),
    "cldnn_release_pending_memory": (None, [_H, _ST]),
    "cldnn_create_engine": (_H, [C.c_int32, C.c_uint32, C.POINTER(c_engine_configuration), _ST]),
    "cldnn_retain_engine": (None, [_H, _ST]),
    "cldnn_release_engine": (None, [_H, _ST]),
    "cldnn_get_engine_info": (c_engine_info, [_H, _ST]),
    "cldnn_get_engine_type": (C.c_int32, [_H, _ST]),
    "cldnn_get_temp_used_device_memory_size": (C.c_int64, [_H, _ST]),
    "cldnn_get_max_used_device_memory_size": (C.c_int64, [_H, _ST]),
    "cldnn_create_user_event": (_H, [_H, _ST]),
    "cldnn_is_user_event": (C.c_int32, [_H, _ST]),
    "cldnn_retain_event": (None, [_H, _ST]),
    "cldnn_release_event": (None, [_H, _ST]),
    "cldnn_wait_for_event": (None, [_H, _ST]),
    "cldnn_set_event": (None, [_H, _ST]),
    "cldnn_add_event_handler": (None, [_H, EVENT_HANDLER, C.c_void_p, _ST]),
    "cldnn_get_event_profiling_info": (None, [_H, C.POINTER(c_profiling_interval), C.c_size_t, C.POINTER(C.c_size_t), _ST]),
    "cldnn_build_program": (_H, [_H, _H, C.POINTER(c_build_option), C.c_size_t, _ST]),
    "cldnn_retain_program": (None, [_H, _ST]),
    "cldnn_release_program": (None, [_H, _ST]),
    "cldnn_build_network": (_H, [_H, _H, C.POINTER(c_build_option), C.c_size_t, _ST]),
    "cldnn_allocate_network": (_H, [_H, _ST]),
    "cldnn_retain_network": (None, [_H, _ST]),
    "cldnn_release_network": (None, [_H, _ST]),
    "cldnn_set_network_input": (None, [_H, C.c_char_p, _H, _ST]),
    "cldnn_get_primitive_info": (None, [_H, C.c_char_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t), _ST]),
    "cldnn_get_network_engine": (_H, [_H, _ST]),
    "cldnn_get_network_program": (_H, [_H, _ST]),
    "cldnn_get_network_output_names": (None, _NAMES),
    "cldnn_get_network_executed_primitive_names": (None, _NAMES),
    "cldnn_get_network_all_primitive_names": (None, _NAMES),
    "cldnn_get_network_all_primitive_org_names": (None, _NAMES),
    "cldnn_execute_network": (None, [_H, C.POINTER(C.c_void_p), C.c_size_t, _ST]),
    "cldnn_get_network_output": (c_network_output, [_H, C.c_char_p, _ST]),
    "cldnn_get_network_output_memory": (_H, [_H, C.c_char_p, _ST]),
    "cldnn_get_network_output_event": (_H, [_H, C.c_char_p, _ST]),
    "cldnn_allocate_memory": (_H, [_H, c_layout, _ST]),
    "cldnn_attach_memory": (_H, [c_layout, C.c_void_p, C.c_size_t, _ST]),
    "cldnn_is_the_same_buffer": (C.c_int32, [_H, _H, _ST]),
    "cldnn_retain_memory": (None, [_H, _ST]),
    "cldnn_release_memory": (None, [_H, _ST]),
    "cldnn_lock_memory": (C.c_void_p, [_H, _ST]),
    "cldnn_unlock_memory": (None, [_H, _ST]),
    "cldnn_get_memory_layout": (c_layout, [_H, _ST]),
    "cldnn_get_memory_engine": (_H, [_H, _ST]),
    "cldnn_get_last_error_message": (C.c_char_p, []),
    "cldnn_plan_topology": (None, [_H, C.POINTER(c_build_option), C.c_size_t, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t), _ST]),
    "cldnn_input_layout_type_id": (C.c_void_p, [_ST]),
    "cldnn_data_type_id": (C.c_void_p, [_ST]),
    "cldnn_reorder_type_id": (C.c_void_p, [_ST]),
    "cldnn_activation_type_id": (C.c_void_p, [_ST]),
    "cldnn_eltwise_type_id": (C.c_void_p, [_ST]),
    "cldnn_convolution_type_id": (C.c_void_p, [_ST]),
    "cldnn_fused_conv_eltwise_type_id": (C.c_void_p, [_ST]),
    "cldnn_pooling_type_id": (C.c_void_p, [_ST]),
    "cldnn_concatenation_type_id": (C.c_void_p, [_ST]),
    "cldnn_fully_connected_type_id": (C.c_void_p, [_ST]),
}

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is not built: run `python -c 'import __graft_entry__ as g; g.build()'`")
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            f = getattr(l, name)
            f.restype, f.argtypes = res, args
        _lib = l
    return _lib


class error(RuntimeError):  # noqa: N801
    def __init__(self, status, message):
        super().__init__(f"[{status}] {message}")
        self.status = status


def _call(name, *args):
    st = C.c_int32(0)
    r = getattr(lib(), name)(*args, C.byref(st))
    if st.value != SUCCESS:
        raise error(st.value, lib().cldnn_get_last_error_message().decode())
    return r


def _names(fn, handle):
    need = C.c_size_t(0)
    st = C.c_int32(0)
    getattr(lib(), fn)(handle, None, 0, C.byref(need), C.byref(st))  # size query: reports INVALID_ARG and the size
    buf = C.create_string_buffer(need.value)
    _call(fn, handle, buf, need.value, C.byref(need))
    return [s.decode() for s in buf.raw[: need.value].split(b"\0") if s]


# ------------------------------------------------------------------------------------------ value types
def tensor(b=1, f=1, x=1, y=1, default=1):
    """cldnn::tensor(batch, feature, x, y) (reference api/CPP/tensor.hpp:382-399)."""
    t = c_tensor(1, 1, 3, 2)
    for i in range(8):
        t.sizes[i] = default
    t.sizes[0], t.sizes[1], t.sizes[2], t.sizes[3] = b, f, x, y
    return t


def spatial(x, y, default=1):
    return tensor(default, default, x, y, default)


def padding(lower=(0, 0, 0, 0), upper=None, filling_value=0.0):
    """cldnn::padding{ {b, f, y, x} lower, upper } in the reference's bfyx argument order."""
    upper = lower if upper is None else upper
    lo = tensor(lower[0], lower[1], lower[3], lower[2], 0)
    hi = tensor(upper[0], upper[1], upper[3], upper[2], 0)
    return c_padding(lo, hi, filling_value)


def layout(data_type, fmt, size, pad=None):
    return c_layout(data_type, fmt, size, pad if pad is not None else padding())


def _layout_shape(l):
    """numpy shape + axis order of the padded buffer of a plain (unblocked) layout."""
    s, lo, hi = l.size.sizes, l.padding.lower_size.sizes, l.padding.upper_size.sizes
    dim = {"b": 0, "f": 1, "x": 2, "y": 3}
    order = {format.bfyx: "bfyx", format.yxfb: "yxfb", format.byxf: "byxf"}[l.format]
    full = [lo[dim[c]] + s[dim[c]] + hi[dim[c]] for c in order]
    inner = tuple(slice(lo[dim[c]], lo[dim[c]] + s[dim[c]]) for c in order)
    return order, full, inner


class engine:  # noqa: N801
    """cldnn::engine (reference api/CPP/engine.hpp:96-190)."""

    def __init__(self, engine_num=0, enable_profiling=False, enable_memory_pool=True, enable_parallelisation=False, _handle=None):
        if _handle is not None:
            self.h = _handle
            return
        cfg = c_engine_configuration()
        cfg.enable_profiling = 1 if enable_profiling else 0
        cfg.enable_memory_pool = 1 if enable_memory_pool else 0  # the reference's default is on (api/CPP/engine.hpp:66)
        cfg.enable_parallelisation = 1 if enable_parallelisation else 0  # independent branches on a second stream
        self.h = _call("cldnn_create_engine", 0, engine_num, C.byref(cfg))

    @staticmethod
    def engine_count():
        return _call("cldnn_get_engine_count", 0)

    def get_info(self):
        return _call("cldnn_get_engine_info", self.h)

    def get_temp_used_device_memory_size(self):
        return _call("cldnn_get_temp_used_device_memory_size", self.h)

    def get_max_used_device_memory_size(self):
        return _call("cldnn_get_max_used_device_memory_size", self.h)

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None:
            st = C.c_int32(0)
            _lib.cldnn_release_engine(self.h, C.byref(st))
            self.h = None


class memory:  # noqa: N801
    """cldnn::memory (reference api/CPP/memory.hpp:40-180)."""

    def __init__(self, handle, keepalive=None):
        self.h = handle
        self._keep = keepalive

    @staticmethod
    def allocate(eng, lay):
        return memory(_call("cldnn_allocate_memory", eng.h, lay))

    @staticmethod
    def attach(lay, array):
        assert array.flags["C_CONTIGUOUS"]
        return memory(_call("cldnn_attach_memory", lay, array.ctypes.data_as(C.c_void_p), array.nbytes), keepalive=array)

    def get_layout(self):
        return _call("cldnn_get_memory_layout", self.h)

    def is_the_same_buffer(self, other):
        return bool(_call("cldnn_is_the_same_buffer", self.h, other.h))

    def pointer(self):
        return _pointer(self)

    # numpy conveniences for plain layouts ----------------------------------------------------------
    def write(self, array_bfyx):
        """Store a (b, f, y, x) array into the buffer, whatever its plain format and padding."""
        l = self.get_layout()
        order, full, inner = _layout_shape(l)
        src = np.ascontiguousarray(array_bfyx, dtype=NP_OF[l.data_type]).transpose(["bfyx".index(c) for c in order])
        with self.pointer() as p:
            buf = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(int(np.prod(full)) * src.itemsize,))
            view = buf.view(src.dtype).reshape(full)
            view[inner] = src

    def read(self):
        """The logical (b, f, y, x) contents of a plain-format buffer."""
        l = self.get_layout()
        order, full, inner = _layout_shape(l)
        dt = np.dtype(NP_OF[l.data_type])
        with self.pointer() as p:
            buf = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(int(np.prod(full)) * dt.itemsize,))
            view = buf.view(dt).reshape(full)[inner].copy()
        return np.ascontiguousarray(view.transpose([order.index(c) for c in "bfyx"]))

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None:
            st = C.c_int32(0)
            _lib.cldnn_release_memory(self.h, C.byref(st))
            self.h = None


class _pointer:
    """cldnn::pointer<T>: lock on entry, unlock on exit (reference api/CPP/memory.hpp:182-260)."""

    def __init__(self, mem):
        self.mem = mem

    def __enter__(self):
        return _call("cldnn_lock_memory", self.mem.h)

    def __exit__(self, *a):
        _call("cldnn_unlock_memory", self.mem.h)


def make_memory(eng, array_bfyx, fmt=format.bfyx, pad=None):
    """Allocate engine memory of the array's type and (b, f, y, x) shape and fill it."""
    a = np.asarray(array_bfyx)
    b, f, y, x = a.shape
    m = memory.allocate(eng, layout(DT_OF[a.dtype], fmt, tensor(b, f, x, y), pad))
    m.write(a)
    return m


class event:  # noqa: N801
    def __init__(self, handle):
        self.h = handle

    @staticmethod
    def create_user_event(eng):
        return event(_call("cldnn_create_user_event", eng.h))

    def wait(self):
        _call("cldnn_wait_for_event", self.h)

    def set(self):
        _call("cldnn_set_event", self.h)

    def is_user_event(self):
        return bool(_call("cldnn_is_user_event", self.h))

    def get_profiling_info(self):
        arr = (c_profiling_interval * 3)()
        n = C.c_size_t(0)
        _call("cldnn_get_event_profiling_info", self.h, arr, 3, C.byref(n))
        return {arr[i].name.decode(): arr[i].nanoseconds for i in range(n.value)}

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None:
            st = C.c_int32(0)
            _lib.cldnn_release_event(self.h, C.byref(st))
            self.h = None


# ------------------------------------------------------------------------------------------ primitives
def _ids(names, keep):
    names = [names] if isinstance(names, str) else list(names or [])
    arr = (C.c_char_p * max(len(names), 1))(*[n.encode() for n in names])
    keep.append(arr)
    return c_id_arr(C.cast(arr, C.POINTER(C.c_char_p)), len(names))


class _primitive:
    type_fn = None
    desc = None

    def _base(self, d, prim_id, inputs, output_padding=None, output_data_type=None):
        self._keep = []
        self.id = prim_id
        d.type = _call(self.type_fn)
        d.id = prim_id.encode()
        d.input = _ids(inputs, self._keep)
        d.output_padding = output_padding if output_padding is not None else padding()
        if output_data_type is not None:
            d.output_data_type = c_optional_dt(output_data_type, b"\x01")
        self.dto = d


class input_layout(_primitive):  # noqa: N801
    type_fn = "cldnn_input_layout_type_id"

    def __init__(self, prim_id, lay):
        d = c_input_layout_desc()
        self._base(d, prim_id, [])
        d.layout = lay


class data(_primitive):  # noqa: N801
    type_fn = "cldnn_data_type_id"

    def __init__(self, prim_id, mem):
        d = c_data_desc()
        self._base(d, prim_id, [])
        d.mem = mem.h
        self._keep.append(mem)


class reorder(_primitive):  # noqa: N801
    """reorder(id, input, output_format, output_data_type) or reorder(id, input, layout)
    (reference api/CPP/reorder.hpp:52-160)."""
    type_fn = "cldnn_reorder_type_id"

    def __init__(self, prim_id, inp, fmt_or_layout, output_data_type=None, output_padding=None):
        d = c_reorder_desc()
        if isinstance(fmt_or_layout, c_layout):
            fmt, output_data_type = fmt_or_layout.format, fmt_or_layout.data_type
            output_padding = fmt_or_layout.padding if output_padding is None else output_padding
        else:
            fmt = fmt_or_layout
        self._base(d, prim_id, [inp], output_padding, output_data_type)
        d.output_format = fmt
        d.mean_subtract = b""
        d.mean_mode = 0


class activation(_primitive):  # noqa: N801
    type_fn = "cldnn_activation_type_id"

    def __init__(self, prim_id, inp, func, params=(0.0, 0.0), output_padding=None):
        d = c_activation_desc()
        self._base(d, prim_id, [inp], output_padding)
        d.activation_func = func
        d.additional_params = c_act_params(*params)
        d.additional_params_input = b""


class concatenation_axis:  # noqa: N801
    along_b, along_f, along_x, along_y = 0, 1, 2, 3


class c_concatenation_desc(C.Structure):
    _fields_ = _BASE + [("axis", C.c_int32)]


class concatenation(_primitive):  # noqa: N801
    """concatenation(id, inputs, axis) (reference api/CPP/concatenation.hpp:54-92)."""
    type_fn = "cldnn_concatenation_type_id"

    def __init__(self, prim_id, inputs, axis, output_padding=None):
        d = c_concatenation_desc()
        self._base(d, prim_id, list(inputs), output_padding)
        d.axis = axis


class pooling(_primitive):  # noqa: N801
    """pooling(id, input, mode, size, stride, input_offset) or, without a size, global pooling over the whole plane;
    output_size = the reference's create_with_output_size (api/CPP/pooling.hpp:59-190)."""
    type_fn = "cldnn_pooling_type_id"

    def __init__(self, prim_id, inp, mode, size=None, stride=None, input_offset=None, output_size=None, output_padding=None):
        d = c_pooling_desc()
        self._base(d, prim_id, [inp], output_padding)
        d.argmax = b""
        d.mode = mode
        d.global_pooling = 1 if size is None else 0
        d.size = size if size is not None else tensor(0, 0, 0, 0, 0)
        d.stride = stride if stride is not None else tensor(1, 1, 1, 1)
        d.input_offset = input_offset if input_offset is not None else tensor(0, 0, 0, 0, 0)
        d.with_output_size = 0 if output_size is None else 1
        d.output_size = output_size if output_size is not None else tensor(0, 0, 0, 0, 0)


class fully_connected(_primitive):  # noqa: N801
    """fully_connected(id, input, weights, bias, [w_quantization_factor, [output_calibration_factors,] i_quantization_factor,
    [o_quantization_factor]], with_activation, activation_slp) (reference api/CPP/fully_connected.hpp:60-150)."""
    type_fn = "cldnn_fully_connected_type_id"

    def __init__(self, prim_id, inp, weights, bias="", w_quantization_factor="", output_calibration_factors="",
                 i_quantization_factor=1.0, o_quantization_factor=1.0, with_activation=False, activation_slp=0.0, output_padding=None):
        d = c_fully_connected_desc()
        self._base(d, prim_id, [inp], output_padding)
        d.with_activation, d.activation_negative_slope = int(with_activation), activation_slp
        d.weights, d.bias = weights.encode(), (bias or "").encode()
        d.weights_quantization_factors = (w_quantization_factor or "").encode()
        d.output_calibration_factors = (output_calibration_factors or "").encode()
        d.input_quantization_factor, d.output_quantization_factor = i_quantization_factor, o_quantization_factor


def _eltw_fields(e, keep, output_calibration_factors, oqf, mode, with_activation, slope, stride):
    e.output_calibration_factors = (output_calibration_factors or "").encode()
    e.output_quantization_factor = oqf
    e.mode = mode
    e.with_activation = 1 if with_activation else 0
    e.activation_negative_slope = slope
    if stride:
        arr = (c_tensor * len(stride))(*stride)
        keep.append(arr)
        e.stride = c_tensor_arr(C.cast(arr, C.POINTER(c_tensor)), len(stride))


class eltwise(_primitive):  # noqa: N801
    """eltwise(id, input, input2, [stride], mode, with_activation, slope) and the quantized form with
    output_calibration_factors / output_quantization_factor (reference api/CPP/eltwise.hpp:78-260)."""
    type_fn = "cldnn_eltwise_type_id"

    def __init__(self, prim_id, inp, *args, **kw):
        """eltwise(id, input, input2, mode, with_activation, activation_slp, ...) or, with the list of all inputs,
        eltwise(id, [inputs], mode, with_activation, activation_slp, ...); keywords: output_calibration_factors,
        output_quantization_factor, stride (one tensor per input), coefficients, output_padding, output_data_type."""
        several = isinstance(inp, (list, tuple))
        names = ([] if several else ["inp2"]) + ["mode", "with_activation", "activation_slp", "output_calibration_factors",
                                                 "output_quantization_factor", "stride", "output_padding", "output_data_type", "coefficients"]
        if len(args) > len(names):
            raise TypeError("eltwise: too many positional arguments")
        for k, v in zip(names, args):
            if k in kw:
                raise TypeError("eltwise: argument %s given twice" % k)
            kw[k] = v
        unknown = set(kw) - set(names) - {"inp2"}
        if unknown:
            raise TypeError("eltwise: unknown argument(s) %s" % sorted(unknown))
        inputs = list(inp) if several else [inp, kw["inp2"]]
        mode, with_activation, activation_slp = kw.get("mode", eltwise_mode.sum), kw.get("with_activation", False), kw.get("activation_slp", 0.0)
        output_calibration_factors, output_quantization_factor = kw.get("output_calibration_factors", ""), kw.get("output_quantization_factor", 1.0)
        stride, output_padding, output_data_type = kw.get("stride"), kw.get("output_padding"), kw.get("output_data_type")
        coefficients = kw.get("coefficients")
        if coefficients:
            # reference api/CPP/eltwise.hpp:303-310
            if mode == eltwise_mode.sum and len(coefficients) != len(inputs):
                raise ValueError("Invalid eltwise sum coefficients count (should be equal to 0 or input.size)")
            if mode != eltwise_mode.sum:
                raise ValueError("Only eltwise sum operation supports blob-wise coefficients")
        d = c_eltwise_desc()
        self._base(d, prim_id, inputs, output_padding, output_data_type)
        if coefficients:
            arr = (C.c_float * len(coefficients))(*coefficients)
            self._keep.append(arr)
            d.coefficients = c_float_arr(C.cast(arr, C.POINTER(C.c_float)), len(coefficients))
        _eltw_fields(d, self._keep, output_calibration_factors, output_quantization_factor, mode, with_activation,
                     activation_slp, stride)


def _conv_fields(c, keep, weights, bias, w_quantization_factor, output_calibration_factors, i_quantization_factor,
                 output_quantization_factor, stride, input_offset, dilation, with_activation, slope, output_size):
    c.input_offset = input_offset if input_offset is not None else tensor(0, 0, 0, 0, 0)
    c.stride = stride if stride is not None else tensor(1, 1, 1, 1)
    c.dilation = dilation if dilation is not None else tensor(1, 1, 1, 1)
    c.with_activation = 1 if with_activation else 0
    c.activation_negative_slope = slope
    c.weights = _ids(weights, keep)
    c.split = c.weights.size
    c.bias = _ids(bias, keep)
    c.weights_quantization_factors = _ids(w_quantization_factor, keep)
    c.output_calibration_factors = _ids(output_calibration_factors, keep)
    c.input_quantization_factor = i_quantization_factor
    c.output_quantization_factor = output_quantization_factor
    if output_size is not None:
        c.with_output_size = 1
        c.output_size = output_size
    else:
        c.output_size = tensor(0, 0, 0, 0, 0)


class convolution(_primitive):  # noqa: N801
    """The reference's constructor families in one signature (api/CPP/convolution.hpp:38-700):
    weights/bias lists, optional w_quantization_factor, output_calibration_factors,
    i_quantization_factor / output_quantization_factor, stride, input_offset, dilation,
    with_activation / activation_slp, groups, with_output_size, padding_above / padding_below."""
    type_fn = "cldnn_convolution_type_id"

    def __init__(self, prim_id, inp, weights, bias=None, w_quantization_factor=None, output_calibration_factors=None,
                 i_quantization_factor=1.0, output_quantization_factor=1.0, stride=None, input_offset=None, dilation=None,
                 with_activation=False, activation_slp=0.0, groups=1, output_size=None, padding_above=None,
                 padding_below=None, output_padding=None, output_data_type=None):
        d = c_convolution_desc()
        self._base(d, prim_id, [inp], output_padding, output_data_type)
        _conv_fields(d, self._keep, weights, bias, w_quantization_factor, output_calibration_factors, i_quantization_factor,
                     output_quantization_factor, stride, input_offset, dilation, with_activation, activation_slp, output_size)
        d.groups = groups
        d.padding_above = padding_above if padding_above is not None else tensor(0, 0, 0, 0, 0)
        d.padding_below = padding_below if padding_below is not None else tensor(0, 0, 0, 0, 0)


class fused_conv_eltwise(_primitive):  # noqa: N801
    """fused_conv_eltwise(id, input, input2, eltw_mode, weights, bias, conv_w_quantization_factor,
    conv_output_calibration_factors, conv_i_quantization_factor, non_conv_scale, eltw_output_calibration_factors,
    eltw_stride, stride, input_offset, dilation, conv_with_activation, conv_activation_slp, eltw_with_activation,
    eltw_activation_slp) (reference api_extension/CPP/fused_conv_eltwise.hpp:37-110)."""
    type_fn = "cldnn_fused_conv_eltwise_type_id"

    def __init__(self, prim_id, inp, inp2, eltw_mode, weights, bias=None, conv_w_quantization_factor=None,
                 conv_output_calibration_factors=None, conv_i_quantization_factor=1.0, non_conv_scale=1.0,
                 eltw_output_calibration_factors="", eltw_stride=None, stride=None, input_offset=None, dilation=None,
                 conv_with_activation=False, conv_activation_slp=0.0, eltw_with_activation=False, eltw_activation_slp=0.0,
                 output_padding=None, output_data_type=None, conv_output_quantization_factor=1.0):
        d = c_fused_conv_eltwise_desc()
        self._base(d, prim_id, [inp, inp2], output_padding, output_data_type)
        _conv_fields(d.conv, self._keep, weights, bias, conv_w_quantization_factor, conv_output_calibration_factors,
                     conv_i_quantization_factor, conv_output_quantization_factor, stride, input_offset, dilation,
                     conv_with_activation, conv_activation_slp, None)
        _eltw_fields(d.eltw, self._keep, eltw_output_calibration_factors, 1.0, eltw_mode, eltw_with_activation,
                     eltw_activation_slp, eltw_stride)
        d.non_conv_scale = non_conv_scale
        d.second_input_in_output = 0


# ------------------------------------------------------------------------------------------ topology / network
class topology:  # noqa: N801
    def __init__(self, *prims):
        self.h = _call("cldnn_create_topology")
        self._keep = []
        self.add(*prims)

    def add(self, *prims):
        for p in prims:
            _call("cldnn_add_primitive", self.h, C.byref(p.dto))
            self._keep.append(p)
        return self

    def change_input_layout(self, prim_id, lay):
        _call("cldnn_change_input_layout", self.h, prim_id.encode(), lay)

    def get_primitive_ids(self):
        return _names("cldnn_get_primitive_ids", self.h)

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None:
            st = C.c_int32(0)
            _lib.cldnn_release_topology(self.h, C.byref(st))
            self.h = None


class tuning_mode:  # noqa: N801
    tuning_disabled, tuning_use_cache, tuning_tune_and_cache = range(3)


class c_tuning_config(C.Structure):
    _fields_ = [("mode", C.c_int32), ("cache_file_path", C.c_char_p)]


class build_options:  # noqa: N801
    """optimize_data, outputs, tuning_config=(tuning_mode, cache file path) (reference api/CPP/program.hpp:68-135)"""

    def __init__(self, optimize_data=False, outputs=None, tuning_config=None):
        self.optimize_data = optimize_data
        self.outputs = outputs
        self.tuning_config = tuning_config

    def _c(self):
        keep, opts = [], []
        if self.optimize_data:
            opts.append(c_build_option(build_option_type.optimize_data, None))
        if self.outputs is not None:
            arr = _ids(self.outputs, keep)
            keep.append(arr)
            opts.append(c_build_option(build_option_type.outputs, C.cast(C.pointer(arr), C.c_void_p)))
        if self.tuning_config is not None:
            t = c_tuning_config(self.tuning_config[0], (self.tuning_config[1] or "").encode())
            keep.append(t)
            opts.append(c_build_option(build_option_type.tuning_config, C.cast(C.pointer(t), C.c_void_p)))
        carr = (c_build_option * max(len(opts), 1))(*opts)
        return carr, len(opts), keep


def plan(topo, options=None):
    """The graph cldnn_build_program would execute, as a list of dicts; needs no GPU."""
    carr, n, keep = (options or build_options())._c()
    need = C.c_size_t(0)
    st = C.c_int32(0)
    lib().cldnn_plan_topology(topo.h, carr, n, None, 0, C.byref(need), C.byref(st))
    if need.value == 0:
        raise error(st.value, lib().cldnn_get_last_error_message().decode())
    buf = C.create_string_buffer(need.value)
    _call("cldnn_plan_topology", topo.h, carr, n, buf, need.value, C.byref(need))
    return json.loads(buf.value.decode())


class network_output:  # noqa: N801
    def __init__(self, ev, mem):
        self._event, self._memory = ev, mem

    def get_event(self):
        return self._event

    def get_memory(self):
        self._event.wait()
        return self._memory


class network:  # noqa: N801
    """cldnn::network(engine, topology, build_options) (reference api/CPP/network.hpp:62-290)."""

    def __init__(self, eng, topo, options=None):
        carr, n, keep = (options or build_options())._c()
        self.h = _call("cldnn_build_network", eng.h, topo.h, carr, n)
        self._engine, self._topology = eng, topo

    def set_input_data(self, prim_id, mem):
        _call("cldnn_set_network_input", self.h, prim_id.encode(), mem.h)

    def get_output_ids(self):
        return _names("cldnn_get_network_output_names", self.h)

    def get_executed_primitive_ids(self):
        return _names("cldnn_get_network_executed_primitive_names", self.h)

    def get_all_primitive_ids(self):
        return _names("cldnn_get_network_all_primitive_names", self.h)

    def get_all_primitive_org_ids(self):
        return _names("cldnn_get_network_all_primitive_org_names", self.h)

    def get_primitive_info(self, prim_id):
        need = C.c_size_t(0)
        st = C.c_int32(0)
        lib().cldnn_get_primitive_info(self.h, prim_id.encode(), None, 0, C.byref(need), C.byref(st))
        if need.value == 0:
            raise error(st.value, lib().cldnn_get_last_error_message().decode())
        buf = C.create_string_buffer(need.value)
        _call("cldnn_get_primitive_info", self.h, prim_id.encode(), buf, need.value, C.byref(need))
        return json.loads(buf.value.decode())

    def execute(self, dependencies=()):
        deps = (C.c_void_p * max(len(dependencies), 1))(*[e.h for e in dependencies])
        _call("cldnn_execute_network", self.h, deps, len(dependencies))
        out = {}
        for name in self.get_output_ids():
            o = _call("cldnn_get_network_output", self.h, name.encode())
            out[name] = network_output(event(o.event), memory(o.memory))
        return out

    def __del__(self):
        if getattr(self, "h", None) and _lib is not None:
            st = C.c_int32(0)
            _lib.cldnn_release_network(self.h, C.byref(st))
            self.h = None
