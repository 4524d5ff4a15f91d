"""The tuning drivers end to end on the device: a short search that appends
``key:json`` to a log, then the replay of that log with ``--test --check``
(flextensor/optimize/optimize_gemm.py:26-99, optimize/common.py:63-82), and
the replayed plan's output against the CPU oracle.
"""
import argparse
import json
import os
import subprocess
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
if not torch.cuda.is_available():
    pytest.skip("no GPU visible", allow_module_level=True)

from flextensor_amd.measure import seeded_inputs  # noqa: E402
from flextensor_amd.optimize import (common, optimize_conv2d, optimize_depthwise_conv2d,  # noqa: E402
                                     optimize_gemm)
from flextensor_amd.plan import build  # noqa: E402
from flextensor_amd.scheduler import schedule_with_config  # noqa: E402
from flextensor_amd.task import TASK_TABLE  # noqa: E402
from flextensor_amd.utils import Config  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = 1e-5


def parse(argv):
    p = argparse.ArgumentParser()
    common.init_arg_parser(p)
    return p.parse_args(argv)


def rel(a, b):
    b = np.asarray(b, np.float64)
    return float(np.max(np.abs(np.asarray(a, np.float64) - b)) / np.max(np.abs(b)))


def read_log(path):
    """The reference's reader: every line is key:json (optimize_gemm.py:76-82)."""
    out = []
    with open(path) as f:
        for line in f:
            name, string = line.split(":", 1)
            obj = json.loads(string)
            out.append((name, Config(obj[0], obj[1])))
    return out


def replay_output(key, configs, seed):
    _, bufs = TASK_TABLE[key].func(*TASK_TABLE[key].args)
    host = seeded_inputs(bufs, seed=seed)
    s, bufs = schedule_with_config(key, configs)
    func = build(s, bufs, "rocm")
    out = torch.full(bufs[-1].shape, -77.0, device="cuda")
    func(*[torch.from_numpy(a).cuda() for a in host], out)
    torch.cuda.synchronize()
    func.close()
    return host, out.cpu().numpy()


def search_then_replay(capsys, tmp_path, shapes, make_task, describe, index, extra=()):
    log = str(tmp_path / "driver.log")
    args = parse(["--log", log, "--trials", "2", "--warm_up", "1x4", "--parallel", "4", "--number", "10",
                  "--from_", str(index), "--to", str(index + 1)] + list(extra))
    common.run_driver(args, shapes, make_task, describe)
    text = capsys.readouterr().out
    assert "Optimize %s shape" % describe in text and "op schedules:" in text and "Use " in text
    used = float(text.split("Use ")[1].split(" ms")[0])
    assert 0 < used < 50, "the winner was timed on the device"
    entries = read_log(log)
    key = make_task(index, shapes[index], args)[0].key
    assert [k for k, _ in entries] == [key]
    # --test --check: the log replayed, timed and compared with the default-schedule kernels on the device
    common.run_driver(parse(["--test", log, "--check"]), shapes, make_task, describe)
    text = capsys.readouterr().out
    assert "Test correctness... passed!" in text, text
    assert "Test instruction stream... passed!" in text or "Test instruction stream" not in text
    cost = float(text.split(key + " use ")[1].split(" ms")[0])
    assert 0 < cost < 50
    return key, entries[0][1], log


def test_optimize_gemm_searches_logs_and_replays_on_the_device(oracle, capsys, tmp_path):
    shapes = optimize_gemm.SHAPES["pow2"]
    index = [e[1] for e in shapes].index((256, 256, 256))
    key, configs, log = search_then_replay(capsys, tmp_path, shapes, optimize_gemm.make_task, "gemm", index)
    (a, b), out = replay_output(key, configs, seed=3)
    assert rel(out, oracle.gemm_np(a, b)) <= TOL
    # the command line itself, in a process of its own: the module's __main__ with --test --check
    r = subprocess.run([sys.executable, "-m", "flextensor_amd.optimize.optimize_gemm", "--shapes", "pow2",
                        "--test", log, "--check"], cwd=ROOT, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert "Test correctness... passed!" in r.stdout and key + " use" in r.stdout


def test_optimize_conv2d_cold_search_logs_and_replays_on_the_device(oracle, capsys, tmp_path):
    shapes = optimize_conv2d.SHAPES["squeeze"]
    index = 20                                   # 1x64x13x13 -> 256, 3x3, padding 1
    key, configs, _ = search_then_replay(capsys, tmp_path, shapes, optimize_conv2d.make_task_for("squeeze"),
                                         "squeeze convolution layer", index, extra=["--cold"])
    assert len(configs.op_config_lst) == 2 and configs.graph_config["inline"]
    (x, w), out = replay_output(key, configs, seed=4)
    assert rel(out, oracle.conv2d_nchw_c(x, w, 1, 1, 1, 1)) <= TOL


def test_optimize_depthwise_searches_logs_and_replays_on_the_device(oracle, capsys, tmp_path):
    shapes = optimize_depthwise_conv2d.SHAPES["mobile"]
    index = 3                                    # 1x32x28x28, six kernels per channel, stride 2
    key, configs, _ = search_then_replay(capsys, tmp_path, shapes, optimize_depthwise_conv2d.make_task,
                                         "depthwise conv2d", index)
    (x, w), out = replay_output(key, configs, seed=5)
    assert rel(out, oracle.depthwise_nchw_c(x, w, 2, 1, 1)) <= TOL


def test_perf_path_is_written_by_the_driver(capsys, tmp_path):
    """--perf_path: the search leaves its measured batches where the offline trainer reads them."""
    shapes = optimize_gemm.SHAPES["pow2"]
    index = [e[1] for e in shapes].index((128, 128, 128))
    perf = str(tmp_path / "perf")
    args = parse(["--log", str(tmp_path / "g.log"), "--trials", "1", "--warm_up", "1x3", "--parallel", "2",
                  "--number", "5", "--from_", str(index), "--to", str(index + 1), "--perf_path", perf])
    common.run_driver(args, shapes, optimize_gemm.make_task, "gemm")
    capsys.readouterr()
    assert os.path.isdir(perf) and os.listdir(perf)


def test_polish_refines_a_log_one_knob_at_a_time(oracle, tmp_path, capsys):
    """flextensor_amd.optimize.polish: every line of the log comes out (refined or as it was),
    still a key:json line the reference's reader takes, still correct against the oracle; a line
    of a task that is not registered is copied."""
    from flextensor_amd.optimize import polish
    from flextensor_amd.templates.gfx950 import default_config
    key = "gemm_gemm_(256, 256, 256)_rocm(0)"
    ops, _ = TASK_TABLE[key].func(*TASK_TABLE[key].args)
    cfg = Config([default_config(ops[0])], {k: [] for k in default_config(ops[0])})
    foreign = "gemm_gemm_(3, 5, 7)_cuda(0):" + json.dumps(cfg)
    src, dst = tmp_path / "in.log", tmp_path / "out.log"
    src.write_text(key + ":" + json.dumps(cfg) + "\n" + foreign + "\n")
    assert polish.main(["--log", str(src), "--out", str(dst), "--number", "60", "--threshold", "0.03"]) == 0
    said = capsys.readouterr().out
    assert "entries refined" in said and key in said
    entries = read_log(str(dst))
    assert [k for k, _ in entries] == [key, "gemm_gemm_(3, 5, 7)_cuda(0)"]
    assert dst.read_text().split("\n")[1] == foreign
    host, out = replay_output(key, entries[0][1], seed=11)
    assert rel(out, oracle.gemm_f32_c(host[0], host[1])) <= TOL
    # the neighbours differ from the entry in exactly one knob
    for what, cand in polish.neighbours(key, entries[0][1]):
        a, b = json.loads(json.dumps(entries[0][1])), json.loads(json.dumps(cand))
        diff = [k for k in a[0][0] if a[0][0][k] != b[0][0][k]] + [k for k in a[1] if a[1].get(k) != b[1].get(k)]
        assert len(diff) == 1, (what, diff)
