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


def _gemm_stored(trans_a, trans_b):
    """gemm with A stored [K][M] and / or B stored [N][K] (flextensor/nn/ops.py:1093-1108)."""
    def wrap(M, K, N):
        from flextensor_amd.nn import gemm as op_gemm
        from flextensor_amd.te import placeholder
        A = placeholder((K, M) if trans_a else (M, K), name="A")
        B = placeholder((N, K) if trans_b else (K, N), name="B")
        C = op_gemm(A, B, transposeA=trans_a, transposeB=trans_b)
        return [C.op], [A, B, C]
    return wrap


gemm_tn, gemm_tt, gemm_nt = _gemm_stored(True, False), _gemm_stored(True, True), _gemm_stored(False, True)


def conv2d_bias(N, C, H, W, K, k, stride=1, padding=0, dilation=1, groups=1):
    """[Padding, conv, bias] (flextensor/nn/ops.py:474-478)."""
    from flextensor_amd.nn import conv2d_nchw
    from flextensor_amd.te import placeholder
    Img = placeholder((N, C, H, W), name="Img")
    Wt = placeholder((K, C // groups, k, k), name="W")
    bias = placeholder((K,), name="bias")
    Out = conv2d_nchw(Img, Wt, bias, stride=stride, padding=padding, dilation=dilation, groups=groups)
    return [Out.op], [Img, Wt, bias, Out]


def depthwise_bias(N, C, H, W, factor, k, stride=1, padding=0, dilation=1):
    """[Padding, depthwise, bias] (flextensor/nn/ops.py:673-677)."""
    from flextensor_amd.nn import depthwise_conv2d_nchw
    from flextensor_amd.te import placeholder
    Img = placeholder((N, C, H, W), name="Img")
    Wt = placeholder((C, factor, k, k), name="W")
    bias = placeholder((C * factor,), name="bias")
    Out = depthwise_conv2d_nchw(Img, Wt, bias, stride=stride, padding=padding, dilation=dilation)
    return [Out.op], [Img, Wt, bias, Out]


# tasks built from these wrappers get the enumerated knobs of this operator family
# (register() attaches them by itself only to the stock wrappers)
FAMILY = {gemm_tn: "gemm", gemm_tt: "gemm", gemm_nt: "gemm", conv2d_bias: "conv2d_nchw",
          depthwise_bias: "depthwise_conv2d_nchw"}

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
    # stored-transposed operands, a bias stage (merged into the stores or its own kernel), a 1x1
    # convolution over one image (read as a plain matrix or gathered), an int8 GEMM with a long K
    ("gemm_tn", gemm_tn, "gemm", "rnd_tn", (160, 96, 224)),
    ("gemm_tt", gemm_tt, "gemm", "rnd_tt", (64, 128, 200)),
    ("gemm_nt", gemm_nt, "gemm", "rnd_nt", (96, 80, 136)),
    ("convb", conv2d_bias, "conv2d", "rnd_bias", (2, 32, 14, 14, 64, 3, 1, 1, 1, 4)),
    ("convb", conv2d_bias, "conv2d", "rnd_bias", (4, 6, 7, 7, 9, 3, 2, 1, 2, 3)),
    ("dwb", depthwise_bias, "conv2d", "rnd_dw_bias", (2, 16, 28, 28, 1, 3, 1, 1, 1)),
    ("conv", conv2d, "conv2d", "rnd", (1, 64, 14, 14, 96, 1, 1, 0, 1, 1)),
    ("int8", gemm_int8, "gemm", "gemm_int8", (64, 2048, 64)),
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
        elif kind in ("convb", "dwb"):
            graph["inline"] = [[rng.choice((0, 1)), 0, 0]]
            graph["merge"] = [[0, 0, rng.choice((0, 1))]]        # bias in the stores or as its own kernel
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
    for knob, values in gfx950.special_knobs(FAMILY.get(func, "")).items():
        if knob not in TASK_TABLE[key].special_space:
            TASK_TABLE[key].set_specific_space(knob, "enum", values)
    rng = random.Random("%s %s %d" % (name, args, number))
    configs, plan = draw(kind, key, rng)
    return kind, key, args, configs, plan
