"""Tuning cache (build option tuning_config; reference kernel_selector/core/auto_tuner.cpp, src/gpu/kernel_runner.cpp): the
file format and its errors without a GPU; on the GPU tune_and_cache fills the file, use_cache applies it, and neither
changes a result."""
import json

import numpy as np
import pytest

from cldnn_amd import api as cl, hip
from oracle import refconv as rc

DT, F = cl.data_types, cl.format


def tile_config_count():
    return hip.lib().cldnn_hip_tile_config_count()


def tile_config_name(row):
    return hip.lib().cldnn_hip_tile_config_name(row).decode()


def attach(a):
    a = np.ascontiguousarray(a)
    b, f, y, x = a.shape
    return cl.memory.attach(cl.layout(cl.DT_OF[a.dtype], F.bfyx, cl.tensor(b, f, x, y)), a)


def small_topology(mem=attach):
    w = np.ones((64, 64, 1, 1), np.int8)
    one = np.ones((1, 1, 1, 64), np.float32)
    return cl.topology(cl.input_layout("in", cl.layout(DT.i8, F.bfyx, cl.tensor(1, 64, 8, 8))), cl.data("w", mem(w)), cl.data("q", mem(one)),
                       cl.convolution("conv", "in", ["w"], None, ["q"], ["q"], with_activation=True))


def test_use_cache_needs_a_readable_file(tmp_path):
    """reference auto_tuner.cpp:40-46"""
    missing = str(tmp_path / "none.json")
    with pytest.raises(cl.error, match="could not be read! Must provide a valid cache file in USE_CACHE mode"):
        cl.plan(small_topology(), cl.build_options(optimize_data=True, tuning_config=(cl.tuning_mode.tuning_use_cache, missing)))
    # tune_and_cache starts from nothing
    cl.plan(small_topology(), cl.build_options(optimize_data=True, tuning_config=(cl.tuning_mode.tuning_tune_and_cache, missing)))


@pytest.mark.parametrize("text,ok", [("", True), ("{}", True), ('{"256": {}}', True),
                                      ('{"256": {"conv;in=x": ["bdir 64x64", 9], "other \\"quoted\\"": ["table", -1]}, "304": {}}', True),
                                      ('{"256": {"k": ["name"]}}', False), ('{"256": [1]}', False), ('{"256": {"k": ["n", 1]}', False)])
def test_cache_file_format(tmp_path, text, ok):
    """{ "<compute units>": { "<signature>": ["<row name>", <row>] } } as the reference's cache.json"""
    path = tmp_path / "cache.json"
    path.write_text(text)
    opts = cl.build_options(optimize_data=True, tuning_config=(cl.tuning_mode.tuning_use_cache, str(path)))
    if ok:
        assert len(cl.plan(small_topology(), opts)) > 0
    else:
        with pytest.raises(cl.error, match="tuning cache"):
            cl.plan(small_topology(), opts)


@pytest.mark.gpu
def test_tune_and_cache_then_use_cache(tmp_path):
    path = str(tmp_path / "cache.json")
    r = np.random.default_rng(3)
    x = r.integers(-128, 128, (2, 64, 14, 14)).astype(np.int8)
    w1 = r.integers(-127, 128, (64, 64, 3, 3)).astype(np.int8)
    w2 = r.integers(-127, 128, (256, 64, 1, 1)).astype(np.int8)
    c1, c2 = (r.uniform(1e-3, 4e-3, n).astype(np.float32) for n in (64, 256))
    # the second convolution has a stride, so the two cannot run as a chain: every node is a launch with a row of its own
    ref = rc.conv(rc.conv(x, w1, None, wqf=np.ones(64, np.float32), calib=c1, pad=(1, 1), out_dt="s8", act="relu"),
                  w2, None, wqf=np.ones(256, np.float32), calib=c2, stride=(2, 2), out_dt="s8", act="relu")

    def run(eng, opts):
        vec = lambda v: cl.make_memory(eng, np.asarray(v, np.float32).reshape(1, 1, 1, -1))  # noqa: E731
        topo = cl.topology(cl.input_layout("in", cl.layout(DT.i8, F.bfyx, cl.tensor(2, 64, 14, 14))),
                           cl.data("w1", cl.make_memory(eng, w1)), cl.data("w2", cl.make_memory(eng, w2)),
                           cl.data("q1", vec(np.ones(64))), cl.data("q2", vec(np.ones(256))), cl.data("c1", vec(c1)), cl.data("c2", vec(c2)),
                           cl.convolution("a", "in", ["w1"], None, ["q1"], ["c1"], input_offset=cl.tensor(0, 0, -1, -1, 0), with_activation=True),
                           cl.convolution("b", "a", ["w2"], None, ["q2"], ["c2"], stride=cl.tensor(1, 1, 2, 2), with_activation=True))
        net = cl.network(eng, topo, opts)
        net.set_input_data("in", cl.make_memory(eng, x))
        out = net.execute()["b"].get_memory().read()
        return out, {i: net.get_primitive_info(i)["kernel"] for i in ("a", "b_fsv16")}

    plain_eng = cl.engine()
    tune = cl.build_options(optimize_data=True, tuning_config=(cl.tuning_mode.tuning_tune_and_cache, path))
    with pytest.raises(cl.error, match="profiling enabled in tune_and_cache mode"):
        run(plain_eng, tune)
    out, tuned_kernels = run(cl.engine(enable_profiling=True), tune)
    np.testing.assert_array_equal(out, ref)
    cache = json.load(open(path))
    assert list(cache) == [str(plain_eng.get_info().cores_count)]
    entries = cache[list(cache)[0]]
    assert len(entries) == 2 and all(k.startswith("conv;in=") for k in entries)
    for name, row in entries.values():
        assert (row == -1 and name == "table") or name == tile_config_name(row)

    use = cl.build_options(optimize_data=True, tuning_config=(cl.tuning_mode.tuning_use_cache, path))
    out, used_kernels = run(plain_eng, use)
    np.testing.assert_array_equal(out, ref)
    assert used_kernels == tuned_kernels
    # the file decides: name another row for the second convolution and it runs on that row; a stale name is ignored
    key_b = [k for k in entries if "256x64x1x1" in k][0]
    # the table's own choice
    default_kernel = run(plain_eng, cl.build_options(optimize_data=True))[1]["b_fsv16"]
    forced = None
    for row in range(tile_config_count()):
        entries[key_b] = [tile_config_name(row), row]
        json.dump(cache, open(path, "w"))
        try:
            out, k = run(plain_eng, use)
        except cl.error:
            continue  # this row does not take the shape
        np.testing.assert_array_equal(out, ref)
        if k["b_fsv16"] != default_kernel:
            forced = k["b_fsv16"]
            break
    assert forced is not None
    entries[key_b] = ["no such row", 3]
    json.dump(cache, open(path, "w"))
    assert run(plain_eng, use)[1]["b_fsv16"] == default_kernel


@pytest.mark.gpu
def test_a_tuned_program_keeps_its_pairs_and_chains(tmp_path):
    """The reference's tuning composes with every graph pass (src/program.cpp:305-309, kernel_selector.cpp:148-207); here
    two convolutions of one input still run as one launch (whose row the cache decides) and a 3x3 with the 1x1 behind it
    still run as a chain (which has no rows), with the same bits as the untuned program."""
    path = str(tmp_path / "cache.json")
    r = np.random.default_rng(5)
    x = r.integers(-128, 128, (2, 64, 14, 14)).astype(np.int8)
    wp = r.integers(-127, 128, (256, 64, 1, 1)).astype(np.int8)
    wq = r.integers(-127, 128, (64, 64, 1, 1)).astype(np.int8)
    wa = r.integers(-127, 128, (64, 64, 3, 3)).astype(np.int8)
    wb = r.integers(-127, 128, (256, 64, 1, 1)).astype(np.int8)
    cp, cq, ca, cb = (r.uniform(1e-3, 4e-3, n).astype(np.float32) for n in (256, 64, 64, 256))
    one = lambda n: np.ones(n, np.float32)  # noqa: E731
    ref_p = rc.conv(x, wp, None, wqf=one(256), calib=cp, out_dt="s8")
    q = rc.conv(x, wq, None, wqf=one(64), calib=cq, out_dt="s8", act="relu")
    a = rc.conv(q, wa, None, wqf=one(64), calib=ca, pad=(1, 1), out_dt="s8", act="relu")
    ref_b = rc.conv(a, wb, None, wqf=one(256), calib=cb, out_dt="s8", act="relu")

    def run(eng, opts):
        vec = lambda v: cl.make_memory(eng, np.asarray(v, np.float32).reshape(1, 1, 1, -1))  # noqa: E731
        topo = cl.topology(cl.input_layout("in", cl.layout(DT.i8, F.bfyx, cl.tensor(2, 64, 14, 14))),
                           cl.data("wp", cl.make_memory(eng, wp)), cl.data("wq", cl.make_memory(eng, wq)),
                           cl.data("wa", cl.make_memory(eng, wa)), cl.data("wb", cl.make_memory(eng, wb)),
                           cl.data("q256", vec(one(256))), cl.data("q64", vec(one(64))),
                           cl.data("cp", vec(cp)), cl.data("cq", vec(cq)), cl.data("ca", vec(ca)), cl.data("cb", vec(cb)),
                           cl.convolution("p", "in", ["wp"], None, ["q256"], ["cp"]),
                           cl.convolution("q", "in", ["wq"], None, ["q64"], ["cq"], with_activation=True),
                           cl.convolution("a", "q", ["wa"], None, ["q64"], ["ca"], input_offset=cl.tensor(0, 0, -1, -1, 0), with_activation=True),
                           cl.convolution("b", "a", ["wb"], None, ["q256"], ["cb"], with_activation=True))
        net = cl.network(eng, topo, opts)
        net.set_input_data("in", cl.make_memory(eng, x))
        outs = net.execute()
        info = {i: net.get_primitive_info(i) for i in net.get_all_primitive_ids()}
        return outs["p"].get_memory().read(), outs["b"].get_memory().read(), info

    eng = cl.engine(enable_profiling=True)
    plain = run(eng, cl.build_options(optimize_data=True, outputs=["p", "b"]))
    tuned = run(eng, cl.build_options(optimize_data=True, outputs=["p", "b"], tuning_config=(cl.tuning_mode.tuning_tune_and_cache, path)))
    used = run(eng, cl.build_options(optimize_data=True, outputs=["p", "b"], tuning_config=(cl.tuning_mode.tuning_use_cache, path)))
    for got_p, got_b, info in (plain, tuned, used):
        np.testing.assert_array_equal(got_p, ref_p)
        np.testing.assert_array_equal(got_b, ref_b)
        pair = [i for i, d in info.items() if d.get("launches_also")]
        assert len(pair) == 1 and info[pair[0]]["launches_also"] in ("q", "p_fsv16"), {i: d.get("launches_also") for i, d in info.items()}
        assert info["b_fsv16"]["kernel"] == "in the chain of a"
    entries = list(json.load(open(path)).values())[0]
    assert any(";pair=" in k for k in entries), list(entries)
    assert not any("3x3" in k for k in entries), "a chain has no row to tune"
