"""The built-in tile table (mfma_choose) on layer shapes that none of the three benchmark networks has.

The table was fitted by sweeps over the layers of ResNet-50, VGG-16 and MobileNet-v2; other shapes fall into whatever
branch covers them.  cldnn_hip_conv_tune measures every applicable row of the table on the device and reports the
fastest one beside the table's own choice: the choice must stay within a factor of the best on these shapes too (a
gross misselection, not a few percent, is what this guards against; run-time tuning covers the rest)."""
import numpy as np
import pytest

from cldnn_amd import hip

pytestmark = pytest.mark.gpu

# batch, input features, height = width, output features, filter, stride -- inception / DenseNet / detection-head like
SHAPES = [
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
]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "b%d_%dx%dx%d_to_%d_k%d_s%d" % (s[0], s[1], s[2], s[2], s[3], s[4], s[5]))
def test_table_choice_is_close_to_the_tuned_one(shape):
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
    best, best_us, default_us, rows = hip.conv_tune(eng, desc, w, bias, wqf, calib, runs=30)
    measured = [t for t in rows if t > 0]
    assert len(measured) >= 3, rows  # several rows of the table take the shape
    assert best_us > 0 and default_us > 0
    assert default_us <= 1.35 * best_us + 1.0, "the table's row takes %.1f us, row %d takes %.1f us (all rows: %s)" % (
        default_us, best, best_us, ["%.1f" % t for t in rows])
    eng.close()
