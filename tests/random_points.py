"""Points drawn at random from the operators' schedule spaces (shared by the
device parity test and the host-side check of the generated assembly).

The draw is seeded by (task, point number), so every process sees the same
points; points the templates refuse on the host are redrawn, as the search
does."""
import random

from flextensor_amd.scheduler import flatten_graph, schedule_with_config
from flextensor_amd.task import (TASK_TABLE, Task, register, gemm, gemm_int8, conv2d,
                                 depthwise_conv2d, gemm_conv2d, batch_gemm)
from flextensor_amd.templates import gfx950
from flextensor_amd.utils import Config

KEYS = ["fuse", "spatial", "reduce", "reorder", "inline", "unroll", "merge", "special"]
POINTS = 10

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
    # the im2col form: [padding, im2col, GEMM, col2img] with random inline and merge flags
    ("gconv", gemm_conv2d, "gemm_conv2d", "rnd", (2, 16, 14, 14, 32, 3, 1, 1, 1, 1)),
    ("gconv", gemm_conv2d, "gemm_conv2d", "rnd", (1, 8, 17, 13, 24, 3, 2, 1, 1, 1)),
    ("gconv", gemm_conv2d, "gemm_conv2d", "rnd", (2, 32, 14, 14, 64, 3, 1, 1, 1, 4)),
    ("bgemm", batch_gemm, "gemm", "batch_gemm", (3, 96, 80, 72)),
]
CASES = [(i, p) for i in range(len(SHAPES)) for p in range(POINTS)]


def draw(kind, key, rng):
    """One point that lowers: (Config, plan)."""
    task = TASK_TABLE[key]
    ops, _ = task.func(*task.args)
    op_lst, _ = flatten_graph(ops)
    pos = [i for i, o in enumerate(op_lst) if o.kind in gfx950.GEMM_KINDS + ("depthwise_conv2d_nchw",)][0]
    space = gfx950.generate_space(op_lst[pos])
    specials = list(task.special_space.items())
    for _ in range(5000):
        cfg = {k: [] for k in KEYS}
        for type_key, names in space.types.items():
            for name in names:
                sub = space.subspaces[name]
                cfg[type_key].append(sub.get_entity(rng.randrange(len(sub))))
        graph = {k: [] for k in KEYS}
        graph["special"] = [sp.get_entity(rng.randrange(len(sp))) for _, sp in specials]
        op_cfgs = [{k: [] for k in KEYS} for _ in op_lst]
        op_cfgs[pos] = cfg
        if kind in ("conv", "dw"):
            graph["inline"] = [[rng.choice((0, 1)), 0]]          # padding folded into the loads or materialised
        elif kind == "gconv":
            # padding and column matrix read through or materialised; col2img in the GEMM's stores or a kernel
            graph["inline"] = [[rng.choice((0, 1)), rng.choice((0, 1)), 0, 0]]
            graph["merge"] = [[0, 0, 0, rng.choice((0, 1))]]
        configs = Config(op_cfgs, graph)
        try:
            plan, _ = schedule_with_config(key, configs)
        except gfx950.InvalidConfig:
            continue
        return configs, plan
    raise AssertionError("no point of the space lowers for %s" % key)




def point(shape_index, number):
    """(kind, key, args, Config, plan) of point ``number`` of shape ``shape_index``."""
    kind, func, category, name, args = SHAPES[shape_index]
    register(func, category, name, args, "rocm", 0)
    key = Task(category, name, None, args, "rocm", 0).key
    rng = random.Random("%s %s %d" % (name, args, number))
    configs, plan = draw(kind, key, rng)
    return kind, key, args, configs, plan
