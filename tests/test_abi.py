"""CPU-side checks of the C-ABI library: it loads, exports every symbol that
include/cldnn_hip.h declares, and its host-only entry points behave."""
import ctypes as C
import os
import re

import pytest

from cldnn_amd import hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "cldnn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cldnn_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = C.CDLL(hip.LIB_PATH)
    names = declared_symbols()
    assert len(names) > 40
    for n in names:
        assert hasattr(L, n), "missing export: " + n


def test_binding_covers_the_header():
    assert set(hip.SIGNATURES) == set(declared_symbols())


def test_out_extent_and_tensor_math_without_gpu():
    L = hip.lib()
    assert L.cldnn_hip_conv_out_extent(224, 3, 7, 1, 2) == 112
    assert L.cldnn_hip_conv_out_extent(56, 1, 3, 1, 1) == 56
    assert L.cldnn_hip_conv_out_extent(2, 0, 3, 1, 2) == 1  # window larger than the input
    t = hip.Tensor.make("u8", "fs_b_yx_fsv16", 2, 40, 5, 7, 1, 1)
    # 40 features -> 3 slices of 16; padded plane 7 x 9
    assert L.cldnn_hip_tensor_bytes(C.byref(t)) == 3 * 2 * 7 * 9 * 16
    assert L.cldnn_hip_tensor_offset(C.byref(t), 0, 0, 0, 0) == (1 * 9 + 1) * 16
    assert L.cldnn_hip_tensor_offset(C.byref(t), 1, 17, 2, 3) == (1 * 2 + 1) * 7 * 9 * 16 + (3 * 9 + 4) * 16 + 1
    t2 = hip.Tensor.make("f32", "bfyx", 2, 3, 4, 5, 1, 2)
    assert L.cldnn_hip_tensor_bytes(C.byref(t2)) == 2 * 3 * 6 * 9 * 4
    assert L.cldnn_hip_tensor_offset(C.byref(t2), 1, 2, 3, 4) == ((1 * 3 + 2) * 6 + 4) * 9 + 6


def test_tile_table_is_listed():
    L = hip.lib()
    n = L.cldnn_hip_tile_config_count()
    assert n >= 4
    names = [L.cldnn_hip_tile_config_name(i).decode() for i in range(n)]
    assert len(set(names)) == n
    assert L.cldnn_hip_tile_config_name(n) is None


def test_no_device_fails_loudly():
    L = hip.lib()
    if L.cldnn_hip_device_count() > 0:
        pytest.skip("a HIP device is present")
    with pytest.raises(hip.HipError) as ei:
        hip.Engine()
    assert ei.value.status == -4
    assert "no HIP device" in str(ei.value)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asking for more ends with a message and a non-zero status before anything is loaded"""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in r.stderr and r.stdout.strip() == ""
