"""Host side of the clDNN-compatible API on the CPU: symbol coverage, object handling, error behaviour
and the graph passes (output layout, dependency order, activation fusing, conv+eltwise fusing, the
fs_b_yx_fsv16 layout rule, border preparation), observed through the engine-less planning call.

The checks follow what the reference asserts in tests/test_cases/topology_test.cpp,
tests/test_cases/fused_conv_eltwise_gpu_test.cpp:31-100 (graph shape after fusing) and
src/convolution.cpp:32-130 (output layout, argument validation).
"""
import ctypes as C
import os
import re

import numpy as np
import pytest

from cldnn_amd import api as cl
from oracle import refconv as rc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F = cl.format
DT = cl.data_types


def header_functions():
    names = []
    for h in ("include/api/C/cldnn.h", "include/api/C/primitives.h"):
        src = open(os.path.join(ROOT, h)).read()
        names += re.findall(r"^CLDNN_API[^;(]*?\b(cldnn_\w+)\s*\(", src, re.M)
        names += [f"cldnn_{t}_type_id" for t in re.findall(r"^CLDNN_DECLARE_PRIMITIVE_TYPE_ID\((\w+)\);", src, re.M)]
    return names


def test_library_exports_every_declared_function():
    names = header_functions()
    assert len(names) > 60
    l = C.CDLL(cl.LIB_PATH)
    for n in names:
        assert hasattr(l, n), n


def test_binding_covers_header():
    assert sorted(header_functions()) == sorted(cl.SIGNATURES)


def test_headers_compile_as_c_and_cpp(tmp_path):
    """The public headers stand alone: C99 and C++14 translation units that include all of them build."""
    incs = ["api/C/cldnn.h", "api/C/input_layout.h", "api/C/data.h", "api/C/reorder.h", "api/C/activation.h",
            "api/C/eltwise.h", "api/C/convolution.h", "api_extension/C/fused_conv_eltwise.h"]
    body = "".join(f'#include "{i}"\n' for i in incs) + "int main(void) { struct cldnn_convolution_desc d; (void)d; return 0; }\n"
    for name, cc, std in (("a.c", "gcc", "-std=c99"), ("a.cpp", "g++", "-std=c++14")):
        p = tmp_path / name
        p.write_text(body)
        rc_ = os.system(f"{cc} {std} -Wall -Werror -fsyntax-only -I{ROOT}/include {p}")
        assert rc_ == 0, name


def test_cpp_api_program_builds_and_needs_a_gpu():
    """The C++ wrappers (include/api/CPP) compile into the reference-style test program; without a GPU it stops at
    engine creation with the library's message instead of computing anything on the host."""
    import subprocess
    import torch
    r = subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "cpp"), "conv_network_test"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    if not torch.cuda.is_available():
        r = subprocess.run([os.path.join(ROOT, "tests", "cpp", "conv_network_test")], capture_output=True, text=True)
        assert r.returncode == 2 and "no HIP device" in r.stdout, r.stdout + r.stderr


def test_version():
    v = cl._call("cldnn_get_version")
    assert (v.major, v.minor) == (1, 4)


def test_engine_needs_a_gpu_or_works():
    import torch
    if torch.cuda.is_available():
        assert cl.engine.engine_count() >= 1
    else:
        assert cl.engine.engine_count() == 0
        with pytest.raises(cl.error) as e:
            cl.engine()
        assert e.value.status == cl.DEVICE_ERROR and "no host fallback" in str(e.value)


def test_null_handles_are_invalid_arg():
    st = C.c_int32(0)
    cl.lib().cldnn_retain_engine(None, C.byref(st))
    assert st.value == cl.INVALID_ARG
    cl.lib().cldnn_execute_network(None, None, 0, C.byref(st))
    assert st.value == cl.INVALID_ARG
    assert b"null" in cl.lib().cldnn_get_last_error_message()


def attach(arr, shape_bfxy=None, fmt=F.bfyx):
    a = np.ascontiguousarray(arr)
    if shape_bfxy is None:
        b, f, y, x = a.shape
        shape_bfxy = (b, f, x, y)
    return cl.memory.attach(cl.layout(cl.DT_OF[a.dtype], fmt, cl.tensor(*shape_bfxy)), a)


def vec(n, dtype=np.float32, value=1):
    return attach(np.full(n, value, dtype), (1, 1, n, 1))


def test_attached_memory():
    a = np.arange(24, dtype=np.int8).reshape(1, 2, 3, 4)
    m = attach(a)
    l = m.get_layout()
    assert (l.data_type, l.format, list(l.size.sizes[:4])) == (DT.i8, F.bfyx, [1, 2, 4, 3])
    assert m.is_the_same_buffer(m)
    np.testing.assert_array_equal(m.read(), a)
    with pytest.raises(cl.error):  # buffer smaller than the layout
        cl._call("cldnn_attach_memory", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 2, 4, 4)), a.ctypes.data_as(C.c_void_p), a.nbytes)


def conv_topology(B=2, IFM=16, H=12, W=10, OFM=8, FY=3, FX=3, in_fmt=F.bfyx, in_dt=DT.i8, quant=True, **kw):
    w = np.ones((OFM, IFM // kw.get("groups", 1), FY, FX), np.int8)
    t = cl.topology(cl.input_layout("in", cl.layout(in_dt, in_fmt, cl.tensor(B, IFM, W, H))), cl.data("w", attach(w)),
                    cl.data("q", vec(OFM)), cl.data("c", vec(OFM)))
    q = dict(w_quantization_factor=["q"], output_calibration_factors=["c"]) if quant else {}
    t.add(cl.convolution("conv", "in", ["w"], **q, **kw))
    return t


def by_id(nodes):
    return {n["id"]: n for n in nodes}


# ------------------------------------------------------------------------------------------ topology object
def test_topology_ids_and_errors():
    t = conv_topology()
    assert t.get_primitive_ids() == ["in", "w", "q", "c", "conv"]
    with pytest.raises(cl.error) as e:
        t.add(cl.activation("conv", "in", cl.activation_func.relu))
    assert e.value.status == cl.INVALID_ARG and "already contains" in str(e.value)
    with pytest.raises(cl.error):
        t.change_input_layout("conv", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 1, 1, 1)))
    t.change_input_layout("in", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 16, 20, 20)))
    assert by_id(cl.plan(t))["conv"]["size"] == [1, 8, 18, 18]


def test_unknown_dependency_is_reported():
    t = cl.topology(cl.input_layout("in", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 16, 4, 4))),
                    cl.activation("a", "nope", cl.activation_func.relu))
    with pytest.raises(cl.error) as e:
        cl.plan(t)
    assert "unknown primitive nope" in str(e.value)


def test_weights_count_must_match_split():
    x = cl.input_layout("in", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 16, 4, 4)))
    with pytest.raises(cl.error):
        cl.topology(x, cl.convolution("conv", "in", ["w"], bias=["b0", "b1"]))


# ------------------------------------------------------------------------------------------ output layout
@pytest.mark.parametrize("H,W,FY,FX,sy,sx,py,px,dy,dx", [
    (12, 10, 3, 3, 1, 1, 0, 0, 1, 1), (12, 10, 3, 3, 1, 1, 1, 1, 1, 1), (224, 224, 7, 7, 2, 2, 3, 3, 1, 1),
    (56, 56, 1, 1, 2, 2, 0, 0, 1, 1), (9, 11, 5, 3, 2, 1, 2, 1, 1, 1), (15, 15, 3, 3, 1, 1, 2, 2, 2, 2),
    (7, 9, 3, 3, 3, 2, 0, 1, 1, 1)])
def test_conv_output_layout(H, W, FY, FX, sy, sx, py, px, dy, dx):
    t = conv_topology(H=H, W=W, FY=FY, FX=FX, stride=cl.tensor(1, 1, sx, sy), input_offset=cl.tensor(0, 0, -px, -py, 0),
                      dilation=cl.tensor(1, 1, dx, dy))
    n = by_id(cl.plan(t))["conv"]
    # format and data type follow the input, the feature count the weights (reference src/convolution.cpp:113-129)
    assert n["format"] == F.bfyx and n["data_type"] == DT.i8
    assert n["size"] == [2, 8, rc.out_extent(W, px, FX, dx, sx), rc.out_extent(H, py, FY, dy, sy)]
    # closed form for the cases without a partial last window
    if (W + 2 * px - ((FX - 1) * dx + 1)) % sx == 0:
        assert n["size"][2] == (W + 2 * px - ((FX - 1) * dx + 1)) // sx + 1


def test_conv_output_type_override_and_padding():
    t = conv_topology(output_data_type=DT.u8, output_padding=cl.padding((0, 0, 2, 1)))
    n = by_id(cl.plan(t))["conv"]
    assert n["data_type"] == DT.u8
    assert n["pad_lower"] == [0, 0, 1, 2] and n["pad_upper"] == [0, 0, 1, 2]


def test_user_output_size_must_agree():
    ok = conv_topology(output_size=cl.tensor(2, 8, 8, 10))
    assert by_id(cl.plan(ok))["conv"]["size"] == [2, 8, 8, 10]
    with pytest.raises(cl.error):
        cl.plan(conv_topology(output_size=cl.tensor(2, 8, 9, 10)))


@pytest.mark.parametrize("kw,msg", [
    (dict(stride=cl.tensor(1, 1, 0, 1)), "stride"),
    (dict(dilation=cl.tensor(1, 1, 1, 0)), "dilation"),
    (dict(input_offset=cl.tensor(0, 1, 0, 0, 0)), "input offset"),
    (dict(groups=3), "feature count"),
    (dict(padding_above=cl.tensor(0, 0, -1, 0, 0)), "cannot be negative"),
    (dict(padding_below=cl.tensor(0, 1, 0, 0, 0)), "batch or feature"),
])
def test_conv_argument_validation(kw, msg):
    with pytest.raises(cl.error) as e:
        cl.plan(conv_topology(**kw))
    assert msg in str(e.value)


def test_padding_above_below_output_size():
    """reference tests basic_convolution_sym / asym_input_padding (convolution_gpu_test.cpp:1064-1257): zeros above
    (in front of) and below (behind) the input; the symmetric case equals a negative input offset"""
    # 12 x 10 input, 3x3 filter: (12 + 1 + 2 - 3) + 1 = 13 rows, (10 + 2 + 3 - 3) + 1 = 13 columns
    t = conv_topology(padding_above=cl.tensor(0, 0, 2, 1, 0), padding_below=cl.tensor(0, 0, 3, 2, 0))
    assert by_id(cl.plan(t))["conv"]["size"] == [2, 8, 13, 13]
    sym = conv_topology(padding_above=cl.tensor(0, 0, 1, 1, 0), padding_below=cl.tensor(0, 0, 1, 1, 0))
    off = conv_topology(input_offset=cl.tensor(0, 0, -1, -1, 0))
    assert by_id(cl.plan(sym))["conv"]["size"] == by_id(cl.plan(off))["conv"]["size"] == [2, 8, 10, 12]
    # together with an input offset (reference ..._with_input_offset, :1259-1478)
    both = conv_topology(input_offset=cl.tensor(0, 0, -1, -2, 0), padding_above=cl.tensor(0, 0, 1, 0, 0),
                         padding_below=cl.tensor(0, 0, 0, 1, 0))
    assert by_id(cl.plan(both))["conv"]["size"] == [2, 8, 11, 15]


def test_split_convolution_layout():
    """split = one weights primitive per part; output features = parts x weights.batch (reference src/convolution.cpp:103)"""
    w = np.ones((4, 8, 1, 1), np.int8)
    t = cl.topology(cl.input_layout("in", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 16, 4, 4))),
                    cl.data("w0", attach(w)), cl.data("w1", attach(w)), cl.convolution("conv", "in", ["w0", "w1"]))
    assert by_id(cl.plan(t))["conv"]["size"] == [1, 8, 4, 4]
    bad = cl.topology(cl.input_layout("in", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 16, 4, 4))),
                      cl.data("w0", attach(w)), cl.data("w1", attach(w)), cl.convolution("conv", "in", ["w0", "w1"], groups=2))
    with pytest.raises(cl.error) as e:
        cl.plan(bad)
    assert "split and groups" in str(e.value)


def test_weights_feature_mismatch():
    t = cl.topology(cl.input_layout("in", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 16, 4, 4))),
                    cl.data("w", attach(np.ones((8, 12, 1, 1), np.int8))), cl.convolution("conv", "in", ["w"]))
    with pytest.raises(cl.error) as e:
        cl.plan(t)
    assert e.value.status == cl.DIMENSION_MISMATCH


# ------------------------------------------------------------------------------------------ dependency order
def test_dependency_order_of_convolution():
    """input, weights, bias, quantization factors, calibration factors (reference src/gpu/convolution_gpu.cpp:37-69)."""
    t = cl.topology(cl.input_layout("in", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 16, 4, 4))),
                    cl.data("calib", vec(8)), cl.data("bias", vec(8, np.int32)), cl.data("wq", vec(8)),
                    cl.data("weights", attach(np.ones((8, 16, 1, 1), np.int8))),
                    cl.convolution("conv", "in", ["weights"], ["bias"], ["wq"], ["calib"]))
    nodes = cl.plan(t)
    assert by_id(nodes)["conv"]["deps"] == ["in", "weights", "bias", "wq", "calib"]
    order = [n["id"] for n in nodes]
    assert all(order.index(d) < order.index("conv") for d in by_id(nodes)["conv"]["deps"])
    assert [n["id"] for n in nodes if n["is_output"]] == ["conv"]


def test_outputs_option():
    t = conv_topology()
    t.add(cl.activation("relu", "conv", cl.activation_func.relu))
    assert [n["id"] for n in cl.plan(t) if n["is_output"]] == ["relu"]
    assert [n["id"] for n in cl.plan(t, cl.build_options(outputs=["conv", "relu"])) if n["is_output"]] == ["conv", "relu"]
    with pytest.raises(cl.error):
        cl.plan(t, cl.build_options(outputs=["nope"]))


# ------------------------------------------------------------------------------------------ fusing passes
def two_convs(second_fy=3, act=cl.activation_func.relu, params=(0.0, 0.0)):
    t = conv_topology(input_offset=cl.tensor(0, 0, -1, -1, 0))
    t.add(cl.activation("relu", "conv", act, params),
          cl.data("w2", attach(np.ones((8, 8, second_fy, second_fy), np.int8))),
          cl.convolution("conv2", "relu", ["w2"], w_quantization_factor=["q"], output_calibration_factors=["c"],
                         input_offset=cl.tensor(0, 0, -(second_fy // 2), -(second_fy // 2), 0)))
    return t


def test_activation_is_folded_into_convolution():
    plain = by_id(cl.plan(two_convs()))
    assert "relu" in plain and plain["conv"]["fused_activation"] == cl.activation_func.none
    opt = by_id(cl.plan(two_convs(), cl.build_options(optimize_data=True)))
    assert "relu" not in opt
    assert opt["conv"]["fused_activation"] == cl.activation_func.relu
    assert opt["conv2_fsv16"]["deps"][0] == "conv"


def test_clamp_parameters_survive_folding():
    opt = by_id(cl.plan(two_convs(act=cl.activation_func.clamp, params=(-3.0, 5.0)), cl.build_options(optimize_data=True)))
    assert opt["conv"]["fused_activation"] == cl.activation_func.clamp
    assert opt["conv"]["fused_activation_params"] == [-3.0, 5.0]


def test_activation_with_two_consumers_of_the_conv_is_kept():
    t = two_convs()
    t.add(cl.activation("other", "conv", cl.activation_func.relu))
    opt = by_id(cl.plan(t, cl.build_options(optimize_data=True)))
    assert "relu" in opt and opt["conv"]["fused_activation"] == cl.activation_func.none


def test_unsupported_activation_is_not_folded():
    opt = by_id(cl.plan(two_convs(act=cl.activation_func.logistic), cl.build_options(optimize_data=True)))
    assert "relu" in opt and opt["conv"]["fused_activation"] == cl.activation_func.none


def residual_block(fy=1, stride=1, with_activation=True, eltw_strides=None, in_fmt=F.bfyx, sum_calib="c", dt=None, groups=1,
                   quantized=True):
    """conv(3x3) -> [conv 1x1 | 3x3] + shortcut -> eltwise sum (+relu): the tail of a ResNet block."""
    B, Cn, H, W = 2, 16, 8, 8
    w1 = attach(np.ones((Cn, Cn, 3, 3), np.int8))
    w2 = attach(np.ones((Cn, Cn // groups, fy, fy), np.int8))
    q2 = dict(w_quantization_factor=["q"], output_calibration_factors=["c"]) if quantized else {}
    t = cl.topology(cl.input_layout("in", cl.layout(DT.i8 if dt is None else dt, in_fmt, cl.tensor(B, Cn, W, H))),
                    cl.data("w1", w1), cl.data("w2", w2), cl.data("q", vec(Cn)), cl.data("c", vec(Cn)),
                    cl.convolution("conv1", "in", ["w1"], w_quantization_factor=["q"], output_calibration_factors=["c"],
                                   input_offset=cl.tensor(0, 0, -1, -1, 0), with_activation=True),
                    cl.convolution("conv2", "conv1", ["w2"], input_offset=cl.tensor(0, 0, -(fy // 2), -(fy // 2), 0),
                                   stride=cl.tensor(1, 1, stride, stride), groups=groups, **q2),
                    cl.eltwise("sum", "in", "conv2", cl.eltwise_mode.sum, with_activation, 0.0, output_calibration_factors=sum_calib,
                               stride=eltw_strides),
                    cl.activation("out", "sum", cl.activation_func.none))
    return t


def test_conv_eltwise_fusing():
    opt = cl.plan(residual_block(), cl.build_options(optimize_data=True))
    ids = [n["id"] for n in opt]
    assert "conv2" not in ids and "sum" not in ids
    f = by_id(opt)["conv2_fused_sum"]
    assert f["type"] == "fused_conv_eltwise"
    # input, second input, then the convolution's constants, then the eltwise calibration
    assert f["deps"][2:] == ["w2", "q", "c", "c"]
    assert f["eltw_calib"] == "c"
    # both data inputs were moved into the blocked layout
    assert f["deps"][0] == "conv1" and f["deps"][1].startswith("in_to_fsv16")
    assert f["format"] == F.fs_b_yx_fsv16


@pytest.mark.parametrize("kw", [dict(fy=3), dict(with_activation=False, sum_calib=""), dict(with_activation=False, dt=DT.u8)],
                         ids=["3x3", "no_activation_unquantized", "no_activation_u8"])
def test_conv_eltwise_not_fused(kw):
    ids = [n["id"] for n in cl.plan(residual_block(**kw), cl.build_options(optimize_data=True))]
    assert "conv2" in ids and "sum" in ids


def test_int8_convolutions_that_stay_on_the_plain_kernel_are_not_fused():
    """the reference fuses int8 convolutions only in its blocked int8 formats (prepare_primitive_fusing.cpp:197-205); here
    that means the ones the layout rule runs in fs_b_yx_fsv16 on the matrix-core kernels.  An unquantized int8 1x1
    convolution stays on the one-thread-per-output kernel, and its relu sum stays a primitive of its own (the sum then
    adds to the int8 tensor the convolution wrote, not to an accumulator)."""
    opt = by_id(cl.plan(residual_block(quantized=False), cl.build_options(optimize_data=True)))
    assert "conv2" in opt and "sum" in opt and "conv2_fused_sum" not in opt
    assert opt["conv2"]["type"] == "convolution" and opt["sum"]["type"] == "eltwise"


def test_grouped_quantized_convolution_is_blocked_and_fused():
    """a grouped (not depthwise) quantized convolution runs on the matrix-core kernels too (block-diagonal weights), so
    the layout rule blocks it and the fusing pass treats it like any other blocked convolution"""
    opt = by_id(cl.plan(residual_block(groups=2), cl.build_options(optimize_data=True)))
    assert "conv2_fused_sum" in opt and opt["conv2_fused_sum"]["format"] == F.fs_b_yx_fsv16


def test_sum_without_activation_is_fused_with_the_saturation_kept():
    """the reference leaves a sum without activation stand-alone (prepare_primitive_fusing.cpp:181-337 wants the relu); a
    quantized s8 one is fused here with the one difference of the two forms -- the stand-alone sum adds to the
    convolution's saturated int8 output -- kept inside the kernel"""
    opt = by_id(cl.plan(residual_block(with_activation=False), cl.build_options(optimize_data=True)))
    f = opt["conv2_fused_sum"]
    assert f["type"] == "fused_conv_eltwise" and f["conv_saturate"] == 1 and f["eltw_calib"] == "c"
    assert "conv_saturate" not in by_id(cl.plan(residual_block(), cl.build_options(optimize_data=True)))["conv2_fused_sum"]
    assert "sum" in by_id(cl.plan(residual_block(with_activation=False)))  # as written without optimize_data


def downsampling_junction(size=8, user_stride=(2, 2), second_user="conv", mid_filter=3):
    """the place where a Caffe-form ResNet halves its resolution: a residual sum whose users are the two stride-2 1x1
    convolutions of the next block"""
    Cn = 16
    w1, w3 = attach(np.ones((Cn, Cn, 1, 1), np.int8)), attach(np.ones((Cn, Cn, mid_filter, mid_filter), np.int8))
    conv = lambda i, src, w, **kw: cl.convolution(i, src, [w], None, ["q"], ["c"], **kw)  # noqa: E731
    t = cl.topology(cl.input_layout("in", cl.layout(DT.i8, F.bfyx, cl.tensor(1, Cn, size, size))), cl.data("w1", w1), cl.data("w3", w3),
                    cl.data("q", vec(Cn)), cl.data("c", vec(Cn)),
                    conv("a", "in", "w1", with_activation=True),
                    conv("b", "a", "w3", with_activation=True, input_offset=cl.tensor(0, 0, -(mid_filter // 2), -(mid_filter // 2), 0)),
                    conv("c_", "b", "w1"),
                    cl.eltwise("res", "in", "c_", cl.eltwise_mode.sum, True, 0.0, output_calibration_factors="c"),
                    conv("down1", "res", "w1", stride=cl.tensor(1, 1, 2, 2)))
    if second_user == "conv":
        t.add(conv("down2", "res", "w1", stride=cl.tensor(1, 1, user_stride[0], user_stride[1])))
    elif second_user == "pool":
        t.add(cl.pooling("down2", "res", cl.pooling_mode.max, cl.tensor(1, 1, 2, 2), cl.tensor(1, 1, 2, 2)))
    return t


def conv_node(nodes, i):
    """an output convolution of the blocked path is followed by a reorder that takes over its id"""
    return nodes.get(i + "_fsv16", nodes[i])


def test_eltwise_shrinking_and_stride_removal():
    """reference src/graph_optimizer/eltwise_shrinking.cpp, eltwise_remove_stride.cpp: the sum computes only what the
    stride-2 users read, and the branch before it shrinks back to the first convolution that can take the stride"""
    plain = by_id(cl.plan(downsampling_junction()))
    assert plain["res"]["size"][2:] == [8, 8] and plain["b"]["stride"][2:] == [1, 1] and plain["down1"]["stride"][2:] == [2, 2]
    opt = by_id(cl.plan(downsampling_junction(), cl.build_options(optimize_data=True)))
    f = opt["c__fused_res"]
    assert f["size"][2:] == [4, 4] and f["stride"][2:] == [1, 1] and f["eltw_stride"][2:] == [2, 2]
    assert opt["b"]["stride"][2:] == [2, 2] and opt["b"]["size"][2:] == [4, 4]
    assert opt["a"]["size"][2:] == [8, 8]
    assert conv_node(opt, "down1")["stride"][2:] == [1, 1] and conv_node(opt, "down2")["stride"][2:] == [1, 1]
    assert opt["down1"]["size"] == plain["down1"]["size"] and opt["down2"]["size"] == plain["down2"]["size"]


@pytest.mark.parametrize("kw", [dict(user_stride=(1, 1)), dict(user_stride=(2, 1)), dict(second_user="pool"), dict(size=7)],
                         ids=["a_user_of_stride_1", "users_differ", "a_user_is_no_convolution", "odd_size"])
def test_eltwise_not_shrunk(kw):
    opt = by_id(cl.plan(downsampling_junction(**kw), cl.build_options(optimize_data=True)))
    f = opt["c__fused_res"]
    assert f["size"][2:] == [kw.get("size", 8)] * 2 and f["eltw_stride"] is None
    assert conv_node(opt, "down1")["stride"][2:] == [2, 2] and opt["b"]["stride"][2:] == [1, 1]


def test_eltwise_stride_stays_where_no_convolution_takes_it():
    """a 1x1 convolution in the middle of the branch cannot absorb the stride: the sum stays strided on that input
    and the closing convolution takes the stride when the two are fused"""
    opt = by_id(cl.plan(downsampling_junction(mid_filter=1), cl.build_options(optimize_data=True)))
    f = opt["c__fused_res"]
    assert f["size"][2:] == [4, 4] and f["stride"][2:] == [2, 2] and f["eltw_stride"][2:] == [2, 2]
    assert opt["b"]["size"][2:] == [8, 8] and conv_node(opt, "down1")["stride"][2:] == [1, 1]


def test_conv_eltwise_fusing_reaches_every_block_of_a_chain():
    """three residual blocks in a row: each sum reads the previous (fused) block's output and its own closing 1x1
    convolution; every one of them fuses (the fused node keeps the sum's place in the execution order)"""
    w = np.ones((16, 16, 1, 1), np.int8)
    t = cl.topology(cl.input_layout("in", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 16, 4, 4))), cl.data("w", attach(w)), cl.data("q", vec(16)),
                    cl.data("c", vec(16)))
    cur = "in"
    for i in range(3):
        t.add(cl.convolution(f"mid{i}", cur, ["w"], None, ["q"], ["c"], with_activation=True),
              cl.convolution(f"close{i}", f"mid{i}", ["w"], None, ["q"], ["c"]),
              cl.eltwise(f"sum{i}", cur, f"close{i}", cl.eltwise_mode.sum, with_activation=True))
        cur = f"sum{i}"
    t.add(cl.reorder("out", cur, F.bfyx, DT.i8))
    ids = [n["id"] for n in cl.plan(t, cl.build_options(optimize_data=True))]
    assert [i for i in ids if "_fused_" in i] == ["close0_fused_sum0", "close1_fused_sum1", "close2_fused_sum2"]
    assert not any(i.startswith("sum") for i in ids)


def test_conv_eltwise_fusing_moves_eltwise_stride_into_the_conv():
    """A strided eltwise after a 1x1 convolution: the convolution takes the stride, the shortcut keeps its own
    (reference src/graph_optimizer/prepare_primitive_fusing.cpp:300-318)."""
    B, Cn, H, W = 1, 16, 8, 8
    t = cl.topology(cl.input_layout("in", cl.layout(DT.i8, F.bfyx, cl.tensor(B, Cn, W, H))),
                    cl.input_layout("short", cl.layout(DT.i8, F.bfyx, cl.tensor(B, Cn, W, H))),
                    cl.data("w", attach(np.ones((Cn, Cn, 1, 1), np.int8))), cl.data("q", vec(Cn)),
                    cl.convolution("conv", "in", ["w"], w_quantization_factor=["q"], output_calibration_factors=["q"]))
    # both inputs subsampled by 2 -> output 4x4
    t.add(cl.eltwise("sum", "short", "conv", cl.eltwise_mode.sum, True, 0.0, stride=[cl.tensor(1, 1, 2, 2), cl.tensor(1, 1, 2, 2)]))
    t.add(cl.activation("out", "sum", cl.activation_func.none))
    nodes = cl.plan(t, cl.build_options(optimize_data=True))
    f = by_id(nodes)["conv_fused_sum"]
    assert f["stride"][2:] == [2, 2] and f["eltw_stride"][2:] == [2, 2]
    assert f["size"] == [1, 16, 4, 4]
    unfused = by_id(cl.plan(t))  # left unfused, the stand-alone eltwise does the sub-sampling
    assert unfused["sum"]["type"] == "eltwise" and unfused["sum"]["size"] == [1, 16, 4, 4] and unfused["conv"]["size"] == [1, 16, 8, 8]


# ------------------------------------------------------------------------------------------ layout rule
def test_layout_rule_blocks_quantized_int8_convolutions():
    plain = by_id(cl.plan(conv_topology()))
    assert plain["conv"]["format"] == F.bfyx and not any("fsv16" in k for k in plain)
    opt = cl.plan(conv_topology(), cl.build_options(optimize_data=True))
    ids = [n["id"] for n in opt]
    # reorder in, convolution under an internal id, reorder back under the user's id
    assert ids[-3:] == ["in_to_fsv16_0", "conv_fsv16", "conv"]
    o = by_id(opt)
    assert o["in_to_fsv16_0"]["format"] == F.fs_b_yx_fsv16 and o["conv_fsv16"]["format"] == F.fs_b_yx_fsv16
    assert o["conv"]["type"] == "reorder" and o["conv"]["format"] == F.bfyx and o["conv"]["is_output"]
    assert not o["conv_fsv16"]["is_output"] and o["conv"]["org_id"] == "conv"


def test_layout_rule_keeps_user_blocked_tensors():
    opt = cl.plan(conv_topology(in_fmt=F.fs_b_yx_fsv16), cl.build_options(optimize_data=True))
    assert [n["id"] for n in opt][-1] == "conv" and by_id(opt)["conv"]["type"] == "convolution"
    assert by_id(opt)["conv"]["format"] == F.fs_b_yx_fsv16


@pytest.mark.parametrize("kw", [dict(quant=False), dict(in_dt=DT.f32), dict(IFM=16, OFM=8, groups=2, quant=False)])
def test_layout_rule_leaves_other_convolutions_alone(kw):
    if kw.get("in_dt") == DT.f32:
        kw = dict(kw, quant=False)
    opt = cl.plan(conv_topology(**kw), cl.build_options(optimize_data=True))
    assert not any("fsv16" in n["id"] for n in opt)
    assert by_id(opt)["conv"]["format"] == F.bfyx


def test_layout_rule_takes_grouped_quantized_convolutions():
    opt = by_id(cl.plan(conv_topology(IFM=16, OFM=8, groups=2), cl.build_options(optimize_data=True)))
    assert opt["conv_fsv16"]["type"] == "convolution" and opt["conv_fsv16"]["format"] == F.fs_b_yx_fsv16


def test_layout_rule_takes_depthwise():
    opt = cl.plan(conv_topology(IFM=16, OFM=16, groups=16), cl.build_options(optimize_data=True))
    assert by_id(opt)["conv_fsv16"]["format"] == F.fs_b_yx_fsv16


def test_layout_rule_first_layer_reads_fsv4():
    """A quantized convolution with at most 4 input features takes its input in b_fs_yx_fsv4 (the format the reference
    has for first layers) and already writes fs_b_yx_fsv16."""
    opt = by_id(cl.plan(conv_topology(IFM=3, OFM=64, FY=7, FX=7, H=32, W=32, stride=cl.tensor(1, 1, 2, 2),
                                      input_offset=cl.tensor(0, 0, -3, -3, 0)), cl.build_options(optimize_data=True)))
    assert opt["in_to_fsv4_0"]["format"] == F.b_fs_yx_fsv4 and opt["in_to_fsv4_0"]["pad_lower"] == [0, 0, 3, 3]
    assert opt["conv_fsv16"]["format"] == F.fs_b_yx_fsv16 and opt["conv_fsv16"]["deps"][0] == "in_to_fsv4_0"
    assert opt["conv"]["format"] == F.bfyx
    # 11x11 filters are more than the first-layer kernel holds: the general blocked layout is used
    opt = by_id(cl.plan(conv_topology(IFM=3, OFM=64, FY=11, FX=11, H=32, W=32), cl.build_options(optimize_data=True)))
    assert "in_to_fsv16_0" in opt


def test_one_reorder_serves_all_blocked_consumers():
    opt = cl.plan(residual_block(), cl.build_options(optimize_data=True))
    assert sum(n["id"].startswith("in_to_fsv16") for n in opt) == 1
    o = by_id(opt)
    assert o["conv1"]["deps"][0] == o["conv2_fused_sum"]["deps"][1]


def test_border_preparation():
    """The producer of a padded blocked convolution's input carries the zero border physically
    (reference src/graph_optimizer/prepare_padding.cpp:26-124)."""
    o = by_id(cl.plan(two_convs(), cl.build_options(optimize_data=True)))
    assert o["in_to_fsv16_0"]["pad_lower"] == [0, 0, 1, 1] and o["in_to_fsv16_0"]["pad_upper"] == [0, 0, 1, 1]
    assert o["conv"]["pad_lower"] == [0, 0, 1, 1]          # conv2 is 3x3 with offset -1
    o = by_id(cl.plan(two_convs(second_fy=1), cl.build_options(optimize_data=True)))
    assert o["conv"]["pad_lower"] == [0, 0, 0, 0]          # a 1x1 consumer needs no border


def test_border_for_strided_window_covers_the_last_tap():
    t = conv_topology(H=9, W=9, FY=3, FX=3, stride=cl.tensor(1, 1, 2, 2), input_offset=cl.tensor(0, 0, -1, -1, 0))
    o = by_id(cl.plan(t, cl.build_options(optimize_data=True)))
    r = o["in_to_fsv16_0"]
    OW = o["conv_fsv16"]["size"][2]
    last = (OW - 1) * 2 - 1 + 2  # leftmost tap of the last window + filter reach
    assert r["pad_lower"][2] == 1 and r["pad_upper"][2] == max(0, last - 8)


# ------------------------------------------------------------------------------------------ concatenation
def two_branch_topology(f1=32, f2=16, axis=cl.concatenation_axis.along_f, quantized=True, in_fmt=F.bfyx, batch=2, tail=True, out=None):
    """in -> conv a (f1 features), conv b (f2 features) -> concatenation -> [1x1 conv]"""
    Cn, H, W = 16, 6, 5
    q = dict(w_quantization_factor=None, output_calibration_factors=None)
    prims = [cl.input_layout("in", cl.layout(DT.i8, in_fmt, cl.tensor(batch, Cn, W, H)))]
    for name, f in (("a", f1), ("b", f2)):
        prims += [cl.data("w" + name, attach(np.ones((f, Cn, 3, 3), np.int8))), cl.data("q" + name, vec(f)), cl.data("c" + name, vec(f))]
        q = dict(w_quantization_factor=["q" + name], output_calibration_factors=["c" + name]) if quantized else {}
        prims.append(cl.convolution(name, "in", ["w" + name], input_offset=cl.tensor(0, 0, -1, -1, 0), with_activation=True, **q))
    prims.append(cl.concatenation("cat", ["a", "b"], axis))
    if tail:
        n = f1 + f2 if axis == cl.concatenation_axis.along_f else f1
        prims += [cl.data("wt", attach(np.ones((8, n, 1, 1), np.int8))), cl.data("qt", vec(8)), cl.data("ct", vec(8)),
                  cl.convolution("tail", "cat", ["wt"], w_quantization_factor=["qt"], output_calibration_factors=["ct"])]
    return cl.topology(*prims)


@pytest.mark.parametrize("axis,sizes,want", [(cl.concatenation_axis.along_f, [(2, 3, 5, 4), (2, 7, 5, 4), (2, 1, 5, 4)], [2, 11, 5, 4]),
                                             (cl.concatenation_axis.along_b, [(1, 3, 5, 4), (4, 3, 5, 4)], [5, 3, 5, 4]),
                                             (cl.concatenation_axis.along_x, [(2, 3, 5, 4), (2, 3, 2, 4)], [2, 3, 7, 4]),
                                             (cl.concatenation_axis.along_y, [(2, 3, 5, 4), (2, 3, 5, 9)], [2, 3, 5, 13])],
                         ids=["f", "b", "x", "y"])
def test_concatenation_layout(axis, sizes, want):
    """reference src/concatenation.cpp:31-54: the sizes add up along the axis, format and type follow the first input"""
    prims = [cl.input_layout("i%d" % k, cl.layout(DT.f32, F.bfyx, cl.tensor(*s))) for k, s in enumerate(sizes)]
    prims.append(cl.concatenation("cat", ["i%d" % k for k in range(len(sizes))], axis))
    n = by_id(cl.plan(cl.topology(*prims)))["cat"]
    assert n["type"] == "concatenation" and n["size"] == want and n["format"] == F.bfyx and n["data_type"] == DT.f32
    assert n["deps"] == ["i%d" % k for k in range(len(sizes))] and n["in_place"] is False


def test_concatenation_inputs_must_agree():
    a = cl.input_layout("a", cl.layout(DT.f32, F.bfyx, cl.tensor(2, 3, 5, 4)))
    with pytest.raises(cl.error, match="same size along the other axes") as e:
        cl.plan(cl.topology(a, cl.input_layout("b", cl.layout(DT.f32, F.bfyx, cl.tensor(2, 3, 6, 4))),
                            cl.concatenation("cat", ["a", "b"], cl.concatenation_axis.along_f)))
    assert e.value.status == cl.DIMENSION_MISMATCH
    with pytest.raises(cl.error, match="differ in data type"):
        cl.plan(cl.topology(a, cl.input_layout("b", cl.layout(DT.i8, F.bfyx, cl.tensor(2, 3, 5, 4))),
                            cl.concatenation("cat", ["a", "b"], cl.concatenation_axis.along_f)))
    with pytest.raises(cl.error, match="axis must be b, f, x or y"):
        cl.plan(cl.topology(a, cl.concatenation("cat", ["a"], 4)))  # along_z: five-dimensional tensors only


def test_concatenation_in_place_of_blocked_convolutions():
    """reference prepare_buffer_fusing.cpp:38-140: the producers write into the concatenation's buffer.  Here that holds
    where an input's place is one contiguous piece of the buffer: feature slices of fs_b_yx_fsv16"""
    opt = by_id(cl.plan(two_branch_topology(), cl.build_options(optimize_data=True)))
    cat, a, b = opt["cat"], opt["a"], opt["b"]
    assert cat["format"] == F.fs_b_yx_fsv16 and cat["in_place"] is True and cat["size"] == [2, 48, 5, 6]
    assert a["concat_into"] == "cat" and a["concat_offset"] == 0
    # b starts behind a's two feature slices: 2 slices x batch 2 x 6 rows x 5 pixels x 16 bytes (no border: the tail is 1x1)
    assert b["concat_into"] == "cat" and b["concat_offset"] == 2 * 2 * 6 * 5 * 16
    # without the graph optimisations nothing is shared
    plain = by_id(cl.plan(two_branch_topology()))
    assert plain["cat"]["in_place"] is False and "concat_into" not in plain["a"]


@pytest.mark.parametrize("kw,why", [(dict(f1=24), "24 features do not fill their last slice"),
                                    (dict(axis=cl.concatenation_axis.along_x, f2=32), "x is not the outermost axis"),
                                    (dict(quantized=False), "plain kernel, bfyx at batch 2: features are not outermost")],
                         ids=["ragged_slice", "along_x", "bfyx_batch2"])
def test_concatenation_not_in_place(kw, why):
    opt = by_id(cl.plan(two_branch_topology(**kw), cl.build_options(optimize_data=True)))
    assert opt["cat"]["in_place"] is False, why
    assert "concat_into" not in opt["a"] and "concat_into" not in opt["b"]


def test_concatenation_in_place_needs_private_intermediate_inputs():
    # an input that is an output keeps its own buffer (reference :95-99)
    t = two_branch_topology(in_fmt=F.fs_b_yx_fsv16)
    opt = by_id(cl.plan(t, cl.build_options(optimize_data=True, outputs=["a", "tail"])))
    assert opt["a"]["is_output"] and opt["cat"]["in_place"] is False
    # ... unless the application sees a copy in its own format: then the blocked tensor behind it is an intermediate one
    opt = by_id(cl.plan(two_branch_topology(), cl.build_options(optimize_data=True, outputs=["a", "tail"])))
    assert opt["a"]["type"] == "reorder" and opt["a_fsv16"]["concat_into"] == "cat" and opt["cat"]["in_place"] is True
    # bfyx at batch 1: the features are the outermost axis, so the plain path shares too; one border for the whole group
    opt = by_id(cl.plan(two_branch_topology(quantized=False, batch=1), cl.build_options(optimize_data=True)))
    assert opt["cat"]["in_place"] is True and opt["b"]["concat_offset"] == 32 * 6 * 5
    assert opt["a"]["pad_lower"] == opt["b"]["pad_lower"] == opt["cat"]["pad_lower"]
    # user memory is never a window into something else
    prims = [cl.input_layout("i%d" % k, cl.layout(DT.i8, F.bfyx, cl.tensor(1, 16, 5, 4))) for k in range(2)]
    prims.append(cl.concatenation("cat", ["i0", "i1"], cl.concatenation_axis.along_f))
    assert by_id(cl.plan(cl.topology(*prims), cl.build_options(optimize_data=True)))["cat"]["in_place"] is False
