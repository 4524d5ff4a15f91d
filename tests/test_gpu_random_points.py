"""Random points of the schedule spaces against the CPU oracle.

The hand-picked cases of test_gpu_parity.py cover the knobs one by one; here
points are drawn from the operators' own spaces (the same sub-spaces the search
walks: tile splits, K splits, pipeline depths, traversal, K division, plus the
task-level knobs and the graph-level inline flag), so that combinations nobody
thought of are run too. Points the templates refuse on the host are redrawn,
as the search does. The draw is seeded by the case, so the points are the same
in every process (and can be compiled ahead of time without a device).

Acceptance as everywhere: fp32 max|out - ref| / max|ref| <= 1e-5, int32 bit-exact.
"""
import os
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
if not torch.cuda.is_available() and os.environ.get("FT_TESTS_COMPILE_ONLY") != "1":
    pytest.skip("no GPU visible", allow_module_level=True)

from flextensor_amd.measure import seeded_inputs  # noqa: E402
from flextensor_amd.plan import build  # noqa: E402
from flextensor_amd.scheduler import schedule_with_config  # noqa: E402
from flextensor_amd.task import (TASK_TABLE, Task, register, gemm, gemm_int8, conv2d,  # noqa: E402
                                 depthwise_conv2d)
from flextensor_amd.templates import gfx950  # noqa: E402
from flextensor_amd.utils import Config  # noqa: E402

TOL = 1e-5
KEYS = ["fuse", "spatial", "reduce", "reorder", "inline", "unroll", "merge", "special"]
POINTS = 6

SHAPES = [
    ("gemm", gemm, "gemm", "gemm", (128, 96, 160)),
    ("gemm", gemm, "gemm", "gemm", (200, 136, 328)),
    ("gemm", gemm, "gemm", "gemm", (96, 80, 67)),
    ("gemm", gemm, "gemm", "gemm", (256, 512, 256)),
    ("conv", conv2d, "conv2d", "rnd", (2, 16, 14, 14, 32, 3, 1, 1, 1, 1)),
    ("conv", conv2d, "conv2d", "rnd", (1, 8, 17, 13, 24, 3, 2, 1, 1, 1)),
    ("conv", conv2d, "conv2d", "rnd", (3, 6, 11, 11, 20, 3, 1, 2, 2, 1)),
    ("conv", conv2d, "conv2d", "rnd", (2, 32, 14, 14, 64, 3, 1, 1, 1, 4)),
    ("conv", conv2d, "conv2d", "rnd", (8, 64, 7, 7, 96, 1, 1, 0, 1, 1)),
    ("conv", conv2d, "conv2d", "rnd", (1, 16, 28, 28, 32, 1, 1, 0, 1, 1)),
    ("int8", gemm_int8, "gemm", "gemm_int8", (136, 208, 72)),
    ("int8", gemm_int8, "gemm", "gemm_int8", (256, 256, 256)),
    ("int8", gemm_int8, "gemm", "gemm_int8", (80, 333, 96)),
    ("int8", gemm_int8, "gemm", "gemm_int8", (200, 320, 136)),
    ("dw", depthwise_conv2d, "conv2d", "depthwise", (2, 16, 28, 28, 1, 3, 1, 1, 1)),
    ("dw", depthwise_conv2d, "conv2d", "depthwise", (1, 8, 15, 13, 2, 3, 2, 1, 1)),
    ("dw", depthwise_conv2d, "conv2d", "depthwise", (1, 4, 28, 28, 1, 5, 2, 2, 1)),
    ("dw", depthwise_conv2d, "conv2d", "depthwise", (1, 5, 14, 28, 6, 3, 2, 1, 1)),
]
CASES = [(i, p) for i in range(len(SHAPES)) for p in range(POINTS)]


def draw(kind, key, rng):
    """One point that lowers: (Config, plan)."""
    task = TASK_TABLE[key]
    ops, _ = task.func(*task.args)
    main = ops[0]
    space = gfx950.generate_space(main)
    specials = list(task.special_space.items())
    for _ in range(5000):
        cfg = {k: [] for k in KEYS}
        for type_key, names in space.types.items():
            for name in names:
                sub = space.subspaces[name]
                cfg[type_key].append(sub.get_entity(rng.randrange(len(sub))))
        graph = {k: [] for k in KEYS}
        graph["special"] = [sp.get_entity(rng.randrange(len(sp))) for _, sp in specials]
        if kind in ("conv", "dw"):
            graph["inline"] = [[rng.choice((0, 1)), 0]]          # padding folded into the loads or materialised
            op_cfgs = [{k: [] for k in KEYS}, cfg]
        else:
            op_cfgs = [cfg]
        configs = Config(op_cfgs, graph)
        try:
            plan, _ = schedule_with_config(key, configs)
        except gfx950.InvalidConfig:
            continue
        return configs, plan
    raise AssertionError("no point of the space lowers for %s" % key)


@pytest.mark.parametrize("shape_index,point", CASES)
def test_random_point_vs_oracle(oracle, shape_index, point):
    kind, func, category, name, args = SHAPES[shape_index]
    register(func, category, name, args, "rocm", 0)
    key = Task(category, name, None, args, "rocm", 0).key
    rng = random.Random("%s %s %d" % (name, args, point))
    configs, plan = draw(kind, key, rng)
    _, bufs = TASK_TABLE[key].func(*args)
    host = seeded_inputs(bufs, seed=shape_index * 31 + point)
    func_ = build(plan, bufs, "rocm")
    tdt = {"float32": torch.float32, "int32": torch.int32}[bufs[-1].dtype]
    out = torch.full(bufs[-1].shape, -77, dtype=tdt, device="cuda")
    func_(*[torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in host], out)
    torch.cuda.synchronize()
    func_.close()
    out = out.cpu().numpy()
    what = (key, [dict((k, v) for k, v in c.items() if v) for c in configs.op_config_lst], configs.graph_config)
    if kind == "int8":
        assert np.array_equal(out, oracle.gemm_i8_c(host[0], host[1])), what
        return
    if kind == "gemm":
        ref = oracle.gemm_f32_c(host[0], host[1])
    elif kind == "conv":
        ref = oracle.conv2d_nchw_c(host[0], host[1], args[6], args[7], args[8], args[9])
    else:
        ref = oracle.depthwise_nchw_c(host[0], host[1], args[6], args[7], args[8])
    ref = np.asarray(ref, np.float64)
    err = float(np.max(np.abs(out.astype(np.float64) - ref)) / np.max(np.abs(ref)))
    assert err <= TOL, (err,) + what
