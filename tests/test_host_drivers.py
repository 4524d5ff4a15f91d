"""The tuning drivers (optimize_*.py): key construction, log append and replay,
with a host-side cost function instead of the GPU."""
import argparse
import json
import os

import numpy as np

from flextensor_amd.optimize import (common, optimize_conv2d, optimize_depthwise_conv2d, optimize_gemm,
                                     optimize_gemm_conv2d)
from flextensor_amd.scheduler import schedule_with_config
from flextensor_amd.task import TASK_TABLE
from flextensor_amd.tuned import load, lookup
from flextensor_amd.utils import Config


def parse(argv):
    p = argparse.ArgumentParser()
    common.init_arg_parser(p)
    return p.parse_args(argv)


def test_arg_parser_has_reference_flags():
    a = parse([])
    for flag in ("from_", "to", "log", "test", "trials", "target", "device", "timeout", "parallel",
                 "use_model", "method", "slevel", "rlevel", "force_inline", "host", "target_host",
                 "device_key", "use_rpc", "fcompile", "port", "check"):
        assert hasattr(a, flag), flag
    assert a.target == "rocm" and a.method == "searching" and a.slevel == 4 and a.rlevel == 3


def test_driver_keys_are_registered():
    a = parse([])
    for i, e in enumerate(optimize_gemm.SHAPES["baseline"] + optimize_gemm.SHAPES["int8"]):
        task, trials = optimize_gemm.make_task(i, e, a)
        assert task.key in TASK_TABLE and len(trials) == 1
    mk = optimize_conv2d.make_task_for("baseline")
    for i, s in enumerate(optimize_conv2d.SHAPES["baseline"]):
        task, trials = mk(i, s, a)
        assert task.key in TASK_TABLE and len(trials) == 2
    for table in ("grouped", "dilation"):
        mk = optimize_conv2d.make_task_for(table)
        for i, shp in enumerate(optimize_conv2d.SHAPES[table]):
            assert mk(i, shp, a)[0].key in TASK_TABLE, (table, i)
    # the reference's table names (optimize_conv2d.py:17-26), every layer registered for both conv forms
    assert set(optimize_conv2d.SHAPES) >= {"yolo", "google", "squeeze", "res", "vgg-16", "vgg-19", "yolo_b8", "mobile_v2"}
    assert [len(optimize_conv2d.SHAPES[n]) for n in ("yolo", "google", "squeeze", "res", "vgg-16", "vgg-19", "mobile_v2",
                                                     "overfeat", "test")] == [15, 49, 22, 20, 9, 0, 7, 5, 1]
    for table in ("yolo", "google", "squeeze", "res", "vgg-16", "mobile_v2", "overfeat", "test"):
        mk, mk2 = optimize_conv2d.make_task_for(table), optimize_gemm_conv2d.make_task_for(table)
        for i, shp in enumerate(optimize_conv2d.SHAPES[table]):
            assert mk(i, shp, a)[0].key in TASK_TABLE and mk2(i, shp, a)[0].key in TASK_TABLE, (table, i)
    assert "conv2d_res5_(64, 256, 56, 56, 512, 1, 2, 0, 1, 1)_rocm(0)" in TASK_TABLE
    assert "conv2d_mobile_v21_(1, 16, 112, 112, 96, 3, 2, 1, 1, 16)_rocm(0)" in TASK_TABLE
    for table in ("yolo_b8", "baseline"):
        mk = optimize_gemm_conv2d.make_task_for(table)
        for i, shp in enumerate(optimize_gemm_conv2d.SHAPES[table]):
            task, trials = mk(i, shp, a)
            assert task.key in TASK_TABLE and task.key.startswith("gemm_conv2d_") and len(trials) == 4
    for i, s in enumerate(optimize_depthwise_conv2d.SHAPES["baseline"] + optimize_depthwise_conv2d.SHAPES["mobile"]):
        assert optimize_depthwise_conv2d.make_task(i, s, a)[0].key in TASK_TABLE


def test_run_driver_appends_log_and_replays(tmp_path, monkeypatch):
    np.random.seed(0)
    log = str(tmp_path / "gemm.log")

    def cost(task_key, cfg, op_pos, number):
        s, _ = schedule_with_config(task_key, cfg, op_pos=op_pos)
        return 1.0 + 1e-3 * s.specs[-1].grid[0]

    import flextensor_amd.scheduler as sch
    real = sch.schedule
    monkeypatch.setattr(sch, "schedule", lambda *a, **k: real(*a, evaluator=cost, verbose=False,
                                                               **{x: y for x, y in k.items()}))
    monkeypatch.setattr(common, "evaluate", lambda *a, **k: 0.5)
    args = parse(["--log", log, "--trials", "2", "--parallel", "2", "--warm_up", "1x4"])
    common.run_driver(args, optimize_gemm.SHAPES["baseline"], optimize_gemm.make_task, "gemm")
    entries = load(log)
    key = "gemm_gemm_(1024, 1024, 1024)_rocm(0)"
    assert list(entries) == [key]
    cfg = entries[key]
    assert isinstance(cfg, Config) and cfg.op_config_lst[0]["spatial"]
    with open(log) as f:
        lines = [l for l in f.read().splitlines() if l]
    # nothing but key:json lines: what the reference's readers parse (split(":", 1) + json.loads)
    assert len(lines) == 1 and lines[0].startswith(key + ":")
    for line in lines:
        json.loads(line.split(":", 1)[1])
    s, _ = schedule_with_config(key, cfg)
    assert s.specs[-1].kernel == "igemm_f32"


def test_shipped_tuned_log_replays_for_every_benchmark_task():
    import __graft_entry__ as g
    for key in g.BENCH_KEYS:
        cfg = lookup(key)
        assert cfg is not None, key
        s, bufs = schedule_with_config(key, cfg)
        assert s.specs and len(bufs) == 3
    assert os.path.exists(os.path.join(os.path.dirname(common.__file__), "..", "tuned", "mi355x.log"))


def test_tuned_convolution_points_carry_over_to_the_im2col_form():
    """A gemm_conv2d task without an entry of its own replays the direct
    convolution's tuned point: same kernel, same constants, no intermediates."""
    key = "gemm_conv2d_yolo5_(1, 256, 56, 56, 512, 3, 1, 1, 1, 1)_rocm(0)"
    direct = "conv2d_yolo5_(1, 256, 56, 56, 512, 3, 1, 1, 1, 1)_rocm(0)"
    assert key not in load() and direct in load()
    cfg = lookup(key)
    assert len(cfg.op_config_lst) == 4 and cfg.op_config_lst[2] == lookup(direct).op_config_lst[1]
    assert cfg.graph_config["inline"] == [[1, 1, 0, 0]] and cfg.graph_config["merge"] == [[0, 0, 0, 1]]
    s, _ = schedule_with_config(key, cfg)
    d, _ = schedule_with_config(direct, lookup(direct))
    assert [k.defines for k in s.specs] == [k.defines for k in d.specs] and not s.intermediates
    assert lookup("gemm_conv2d_nothing_(1,)_rocm(0)") is None
    # one input channel per group: the direct task is the depthwise operator, tuned for another kernel
    mobile = "conv2d_mobile_v21_(1, 16, 112, 112, 96, 3, 2, 1, 1, 16)_rocm(0)"
    assert mobile in load() and lookup("gemm_" + mobile) is None
    s, _ = schedule_with_config(mobile, lookup(mobile))
    assert [k.kernel for k in s.specs] == ["depthwise_f32"] and s.specs[0].defines["MFUSE"] == 1


def test_layer_tuned_at_another_batch_size_seeds_the_search():
    """lookup(similar=True): the same convolution layer at another batch lends
    its tile, K division and pipeline; only the N grid level follows the batch.
    Plain lookup() stays exact."""
    from flextensor_amd.task import register, conv2d
    args = (4, 256, 56, 56, 512, 3, 1, 1, 1, 1)
    key = "conv2d_t_%s_rocm(0)" % str(args)
    register(conv2d, "conv2d", "t", args, "rocm", 0)
    assert lookup(key) is None
    lent = lookup(key, similar=True)
    assert lent is not None and len(lent.op_config_lst) == 2
    grid, waves, reps, mfma = lent.op_config_lst[1]["spatial"][1]
    assert grid == -(-4 * 56 * 56 // (waves * reps * mfma))
    sources = [lookup("conv2d_yolo5_(1, 256, 56, 56, 512, 3, 1, 1, 1, 1)_rocm(0)"),
               lookup("conv2d_yolo_b85_(8, 256, 56, 56, 512, 3, 1, 1, 1, 1)_rocm(0)")]
    assert any(lent.op_config_lst[1]["reduce"] == s.op_config_lst[1]["reduce"] and
               lent.op_config_lst[1]["spatial"][0] == s.op_config_lst[1]["spatial"][0] for s in sources)
    s, _ = schedule_with_config(key, lent)            # it lowers for the new batch
    assert s.specs[-1].defines["N"] == 4 * 56 * 56
    # nothing to lend: another layer, a depthwise task, a malformed key
    assert lookup("conv2d_t_(4, 250, 56, 56, 512, 3, 1, 1, 1, 1)_rocm(0)", similar=True) is None
    assert lookup("conv2d_depthwise_(4, 512, 28, 28, 1, 3, 1, 1, 1)_rocm(0)", similar=True) is None
    assert lookup("not a key", similar=True) is None
