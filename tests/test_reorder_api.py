"""reorder at the edges of the convolution path through the clDNN API, on the reference's own tables
(tests/test_cases/reorder_gpu_test.cpp): layout changes, float -> int8 towards zero, uint8 -> float."""
import numpy as np
import pytest

from cldnn_amd import api as cl

pytestmark = pytest.mark.gpu
DT, F = cl.data_types, cl.format


def run(topo, feed, outputs=None):
    eng = feed.pop("_engine")
    net = cl.network(eng, topo, cl.build_options(outputs=outputs))
    for k, v in feed.items():
        net.set_input_data(k, v)
    return net.execute()


def raw_memory(eng, flat, dtype, fmt, tensor):
    """memory whose buffer holds `flat` in storage order (what set_values does in the reference's tests)"""
    m = cl.memory.allocate(eng, cl.layout(cl.DT_OF[np.dtype(dtype)], fmt, cl.tensor(*tensor)))
    b, f, x, y = tensor
    a = np.array(flat, dtype)
    logical = {F.yxfb: lambda: a.reshape(y, x, f, b).transpose(3, 2, 0, 1), F.byxf: lambda: a.reshape(b, y, x, f).transpose(0, 3, 1, 2),
               F.bfyx: lambda: a.reshape(b, f, y, x)}[fmt]()
    m.write(np.ascontiguousarray(logical))
    return m


def test_basic_yxfb_to_bfyx():
    """reorder_gpu_f32.basic (:37-114)"""
    eng = cl.engine()
    src = [1, 0, 5, 1.5, 2, 0, 6, 5.2, 3, 0.5, 7, 12, 4, -0.5, 8, 8]
    m = raw_memory(eng, src, np.float32, F.yxfb, (2, 2, 2, 2))
    topo = cl.topology(cl.input_layout("input", m.get_layout()), cl.reorder("reorder", "input", cl.layout(DT.f32, F.bfyx, cl.tensor(2, 2, 2, 2))))
    outs = run(topo, {"_engine": eng, "input": m})
    assert list(outs) == ["reorder"]
    got = outs["reorder"].get_memory().read()   # logical [b, f, y, x] = the bfyx buffer
    np.testing.assert_array_equal(got.ravel(), np.array([1, 2, 3, 4, 5, 6, 7, 8, 0, 0, 0.5, -0.5, 1.5, 5.2, 12, 8], np.float32))


def test_basic_convert_int8():
    """reorder_gpu.basic_convert_int8 (:563-610): float -> int8 drops the fraction (-2.5 -> -2, -6.99 -> -6), and back"""
    eng = cl.engine()
    m = raw_memory(eng, [1.0, -2.5, 3.1, -4.0, 5.03, -6.99, 7.0, -8.0, 9.0], np.float32, F.byxf, (1, 1, 3, 3))
    topo = cl.topology(cl.input_layout("input", m.get_layout()),
                       cl.reorder("reorder_input", "input", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 1, 3, 3))),
                       cl.reorder("reorder2", "reorder_input", m.get_layout()))
    outs = run(topo, {"_engine": eng, "input": m}, outputs=["reorder2"])
    got = outs["reorder2"].get_memory().read()
    assert got.dtype == np.float32
    np.testing.assert_array_equal(got.ravel(), np.array([1, -2, 3, -4, 5, -6, 7, -8, 9], np.float32))


def test_basic_convert_uint8_byxf_to_fp32_bfyx():
    """reorder_gpu.basic_convert_uint8rgbabyxf_to_fp32_bfyx (:612-728), the reorder part: element (y, x, f) of the byxf
    image lands at f * 25 + y * 5 + x"""
    eng = cl.engine()
    src = (list(range(1, 21)) + list(range(55, 35, -1)) + list(range(101, 121)) + list(range(155, 135, -1)) + list(range(255, 235, -1)))
    m = raw_memory(eng, src, np.uint8, F.byxf, (1, 4, 5, 5))
    topo = cl.topology(cl.input_layout("input", m.get_layout()), cl.reorder("reorder_input", "input", cl.layout(DT.f32, F.bfyx, cl.tensor(1, 4, 5, 5))))
    got = run(topo, {"_engine": eng, "input": m})["reorder_input"].get_memory().read().ravel()
    assert got.dtype == np.float32 and got.size == 100 and got[0] == 1.0
    for i, v in enumerate(src):
        f, x, y = i % 4, (i // 4) % 5, i // 20
        assert got[x + y * 5 + f * 25] == float(v)


@pytest.mark.parametrize("src_fmt,dst_fmt", [(F.yxfb, F.bfyx), (F.bfyx, F.yxfb)])
def test_input_padding(src_fmt, dst_fmt):
    """reorder_gpu_f32.basic_yxfb_to_bfyx_input_padding / basic_bfyx_to_yxfb_input_padding (:730-887): a padded
    intermediate tensor between two reorders does not change the values"""
    eng = cl.engine()
    x = (np.arange(16, dtype=np.float32) * 1.5 - 7).reshape(2, 2, 2, 2)
    m = cl.make_memory(eng, x, src_fmt)
    topo = cl.topology(cl.input_layout("input", m.get_layout()),
                       cl.reorder("reorder", "input", src_fmt, DT.f32, output_padding=cl.padding([0, 0, 2, 1], [0, 0, 1, 2])),
                       cl.reorder("reorder2", "reorder", dst_fmt, DT.f32))
    got = run(topo, {"_engine": eng, "input": m})["reorder2"].get_memory().read()
    np.testing.assert_array_equal(got, x)
