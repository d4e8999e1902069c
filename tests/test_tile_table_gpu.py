"""The built-in tile table (mfma_choose) against the device.

cldnn_hip_conv_tune measures every applicable row of the table on the device and reports the fastest one beside the
table's own choice.  Two groups of layer shapes:

  * the layers of the benchmark networks at the benchmark batch (VGG-16 at 16, ResNet-50 at 32), where the table was
    fitted by sweeps: a change of the table or of a kernel that makes the table's row lose there is a regression;
  * shapes that none of the benchmark networks has (inception / DenseNet / detection-head like), which fall into
    whatever branch covers them.

Each shape is tuned several times and every row takes the median of its passes, so that one noisy pass of a 5-40 us
kernel on a shared box does not decide the test; a shape that fails is measured once more with seven passes before it
counts.  The table's row may be 15 % + 0.5 us slower than the best row."""
import numpy as np
import pytest

from cldnn_amd import hip

pytestmark = pytest.mark.gpu

PASSES, RUNS = 3, 30

# batch, input features, height = width, output features, filter, stride
OTHER = [
    (8, 192, 35, 64, 1, 1),
    (8, 64, 73, 96, 3, 1),
    (4, 288, 17, 384, 3, 2),
    (16, 480, 14, 192, 1, 1),
    (2, 256, 64, 256, 3, 1),
    (1, 128, 128, 128, 3, 1),
    (32, 160, 17, 320, 3, 2),
    (16, 832, 7, 384, 1, 1),
    (4, 96, 28, 208, 3, 1),
    (24, 1024, 10, 256, 1, 1),
    # the benchmark networks at other batch sizes
    (32, 256, 28, 512, 3, 1),
    (32, 512, 28, 512, 3, 1),
    (32, 512, 14, 512, 3, 1),
    (8, 512, 28, 512, 3, 1),
    (8, 256, 56, 256, 3, 1),
    (16, 256, 14, 256, 3, 1),
    (64, 64, 56, 64, 3, 1),
    (64, 256, 14, 1024, 1, 1),
]
VGG16_B16 = [
    (16, 64, 224, 64, 3, 1),
    (16, 64, 112, 128, 3, 1),
    (16, 128, 112, 128, 3, 1),
    (16, 128, 56, 256, 3, 1),
    (16, 256, 56, 256, 3, 1),
    (16, 256, 28, 512, 3, 1),
    (16, 512, 28, 512, 3, 1),
    (16, 512, 14, 512, 3, 1),
]
RESNET50_B32 = [
    (32, 64, 56, 64, 3, 1),
    (32, 64, 56, 256, 1, 1),
    (32, 256, 56, 64, 1, 1),
    (32, 128, 56, 128, 3, 2),
    (32, 128, 28, 128, 3, 1),
    (32, 128, 28, 512, 1, 1),
    (32, 512, 28, 128, 1, 1),
    (32, 256, 28, 256, 3, 2),
    (32, 256, 14, 256, 3, 1),
    (32, 256, 14, 1024, 1, 1),
    (32, 1024, 14, 256, 1, 1),
    (32, 512, 14, 512, 3, 2),
    (32, 512, 7, 512, 3, 1),
    (32, 512, 7, 2048, 1, 1),
    (32, 2048, 7, 512, 1, 1),
]


def shape_id(s):
    return "b%d_%dx%dx%d_to_%d_k%d_s%d" % (s[0], s[1], s[2], s[2], s[3], s[4], s[5])


def tuned(shape, passes=PASSES):
    """-> (median microseconds of the table's row, {row index: median microseconds})"""
    B, IFM, HW, OFM, K, S = shape
    eng = hip.Engine(0, profiling=True)
    r = np.random.default_rng(9)
    pad = K // 2
    x_t = hip.Tensor.make(hip.U8, hip.FS_B_YX_FSV16, B, IFM, HW, HW, pad, pad)
    w = r.integers(-127, 128, (OFM, IFM, K, K)).astype(np.int8)
    bias = r.integers(-1000, 1001, OFM).astype(np.int32)
    wqf = np.ones(OFM, np.float32)
    calib = np.exp(r.uniform(np.log(1e-4), np.log(1e-2), OFM)).astype(np.float32)
    desc = hip.conv_desc(x_t, w.shape, "s8", stride=(S, S), pad=(pad, pad), bias_dt=hip.I32, has_wqf=True, has_calib=True, act="relu")
    default, rows = [], []
    for _ in range(passes):
        _, _, default_us, row_us = hip.conv_tune(eng, desc, w, bias, wqf, calib, runs=RUNS)
        default.append(default_us)
        rows.append(row_us)
    eng.close()
    rows = np.median(np.asarray(rows), axis=0)
    return float(np.median(default)), {i: float(t) for i, t in enumerate(rows) if t > 0}


@pytest.mark.parametrize("shape", VGG16_B16 + RESNET50_B32 + OTHER, ids=shape_id)
def test_table_choice_is_close_to_the_tuned_one(shape):
    default_us, rows = tuned(shape)
    assert len(rows) >= 3, rows  # several rows of the table take the shape
    best = min(rows, key=rows.get)
    if default_us > 1.15 * rows[best] + 0.5:
        # a second opinion before the verdict: more passes (a neighbour's burst on a shared box outlasts three)
        default_us, rows = tuned(shape, passes=7)
        best = min(rows, key=rows.get)
    ratio = default_us / rows[best]
    print("%s: the table's row %.1f us, best row %s %.1f us, ratio %.3f" % (shape_id(shape), default_us, hip.tile_config_name(best), rows[best], ratio))
    assert default_us <= 1.15 * rows[best] + 0.5, "the table's row takes %.1f us, row %s takes %.1f us (all rows: %s)" % (
        default_us, hip.tile_config_name(best), rows[best], {hip.tile_config_name(i): round(t, 1) for i, t in rows.items()})
