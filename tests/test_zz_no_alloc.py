"""The entry point that allocates nothing, cldnn_hip_conv_enqueue_static_scratch, against cldnn_hip_conv_enqueue.

The small-batch kernel gathers the activations of a filter wider than one tap into a scratch buffer; the plain entry
point uses the buffer the convolution object allocated, this one a fixed array inside the library's code object.
Results must be identical (int8: bit-exact), also on a second call with a smaller input right behind the first,
which finds the first call's bytes in the array."""
import numpy as np
import pytest

from cldnn_amd import hip
from oracle import refconv as rc

pytestmark = pytest.mark.gpu


def problem(seed, B, IFM, H, W, OFM, FY, FX, in_dt=np.uint8):
    r = np.random.default_rng(seed)
    lo, hi = (0, 256) if in_dt == np.uint8 else (-128, 128)
    x = r.integers(lo, hi, (B, IFM, H, W)).astype(in_dt)
    w = r.integers(-127, 128, (OFM, IFM, FY, FX)).astype(np.int8)
    bias = r.integers(-1000, 1001, OFM).astype(np.int32)
    wqf = np.ones(OFM, np.float32)
    calib = (40.0 / (np.sqrt(IFM * FY * FX) * 147.4 * 73.3) * r.uniform(0.5, 2.0, OFM)).astype(np.float32)
    return x, w, bias, wqf, calib


def gemv_row():
    L = hip.lib()
    names = [L.cldnn_hip_tile_config_name(i).decode() for i in range(L.cldnn_hip_tile_config_count())]
    return names.index("gemv_p16_f16") + 1


def build(eng, shape, seed, tile):
    B, IFM, H, W, OFM, FY, FX = shape
    x, w, bias, wqf, calib = problem(seed, B, IFM, H, W, OFM, FY, FX)
    xin = hip.upload(eng, x, "fs_b_yx_fsv16")
    d = hip.conv_desc(xin.tensor, w.shape, "s8", bias_dt=hip.I32, has_wqf=True, has_calib=True, act="relu", tile=tile)
    conv = hip.Conv(eng, d, w, bias, wqf, calib)
    ref = rc.conv(x, w, bias, wqf=wqf, calib=calib, out_dt="s8", act="relu")
    return conv, xin, d, ref


def device_free_bytes():
    """hipMemGetInfo through the HIP runtime the library itself is linked against"""
    import ctypes as C
    rt = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(0), C.c_size_t(0)
    assert rt.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_static_scratch_equals_allocated_scratch_twice_in_a_row():
    eng = hip.Engine()
    tile = gemv_row()
    # a fully_connected-like convolution over a 7x7 plane (gathered), then a smaller one of the same kind
    cases = [build(eng, (16, 512, 7, 7, 128, 7, 7), 5, tile), build(eng, (5, 64, 7, 7, 70, 7, 7), 6, tile)]
    outs = []
    for conv, xin, d, ref in cases:
        assert b"conv_gemv" in conv.info().kernel_name
        a, b = hip.Buffer(eng, d.output), hip.Buffer(eng, d.output)
        outs.append((a, b))
    # the two static calls back to back on the stream, the second with the smaller input; after a warm-up call (code
    # object loading is not the entry point's doing) they leave the device's free memory where it was
    cases[0][0].enqueue_static_scratch(cases[0][1], outs[0][1])
    eng.finish()
    free_before = device_free_bytes()
    for (conv, xin, d, ref), (a, b) in zip(cases, outs):
        conv.enqueue_static_scratch(xin, b)
    eng.finish()
    assert device_free_bytes() == free_before, "the entry point that allocates nothing changed the device's free memory"
    for (conv, xin, d, ref), (a, b) in zip(cases, outs):
        conv.enqueue(xin, a)
    eng.finish()
    for (conv, xin, d, ref), (a, b) in zip(cases, outs):
        plain, static = hip.download(eng, a), hip.download(eng, b)
        assert static.dtype == np.int8 and np.array_equal(static, plain), "static scratch differs from the allocated one"
        assert np.array_equal(static, ref), "static scratch differs from the oracle"
    # once more in the other order: the larger input finds the smaller one's bytes in the array
    for (conv, xin, d, ref), (a, b) in reversed(list(zip(cases, outs))):
        b.write_raw(np.zeros(b.nbytes, np.uint8))
        conv.enqueue_static_scratch(xin, b)
    eng.finish()
    for (conv, xin, d, ref), (a, b) in zip(cases, outs):
        assert np.array_equal(hip.download(eng, b), ref)
    for (conv, xin, d, ref), (a, b) in zip(cases, outs):
        conv.close(), xin.close(), a.close(), b.close()
    eng.close()


def test_static_scratch_serves_kernels_without_scratch_and_refuses_what_does_not_fit():
    eng = hip.Engine()
    # a tile kernel has no scratch: the entry point is the plain enqueue
    conv, xin, d, ref = build(eng, (2, 64, 14, 14, 64, 3, 3), 7, 0)
    out = hip.Buffer(eng, d.output)
    conv.enqueue_static_scratch(xin, out)
    eng.finish()
    out2 = hip.Buffer(eng, d.output)
    conv.enqueue(xin, out2)
    eng.finish()
    assert np.array_equal(hip.download(eng, out), hip.download(eng, out2))
    assert np.array_equal(hip.download(eng, out), ref)
    conv.close(), xin.close(), out.close(), out2.close()
    # 160 output pixels x 392 K-steps gather 4240 KiB: more than the array holds
    B, IFM, OFM = 160, 512, 64
    x = np.zeros((B, IFM, 7, 7), np.uint8)
    w = np.ones((OFM, IFM, 7, 7), np.int8)
    xin = hip.upload(eng, x, "fs_b_yx_fsv16")
    d = hip.conv_desc(xin.tensor, w.shape, "s8", has_wqf=True, has_calib=True, tile=gemv_row())
    conv = hip.Conv(eng, d, w, None, np.ones(OFM, np.float32), np.ones(OFM, np.float32))
    out = hip.Buffer(eng, d.output)
    with pytest.raises(hip.HipError) as err:
        conv.enqueue_static_scratch(xin, out)
    assert "static scratch" in str(err.value)
    conv.enqueue(xin, out)  # the allocating entry point still takes it
    eng.finish()
    conv.close(), xin.close(), out.close()
    eng.close()
