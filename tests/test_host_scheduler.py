"""Task registry, search driver with a host-side cost function, config replay,
lowering invariants and error behaviour. No GPU."""
import json
import math

import numpy as np
import pytest

from flextensor_amd import scheduler as sch
from flextensor_amd.model import WalkerGroup
from flextensor_amd.scheduler import flatten_graph, schedule, schedule_with_config
from flextensor_amd.space import generate_space_intra_op
from flextensor_amd.task import TASK_TABLE, Task, register_task, gemm, conv2d
from flextensor_amd.templates import gfx950
from flextensor_amd.tuned import lookup
from flextensor_amd.utils import Config

GEMM = "gemm_gemm_(1024, 1024, 1024)_rocm(0)"
CONV = "conv2d_baseline0_(1, 64, 56, 56, 64, 3, 1, 1, 1, 1)_rocm(0)"
DW = "conv2d_depthwise_(8, 512, 28, 28, 1, 3, 1, 1, 1)_rocm(0)"
I8 = "gemm_gemm_int8_(4096, 4096, 4096)_rocm(0)"
CONV1x1 = "conv2d_baseline2_(8, 512, 7, 7, 2048, 1, 1, 0, 1, 1)_rocm(0)"


def test_task_key_format_and_registry():
    # key format of the reference: "{category}_{name}_{args}_{target}({dev})"
    t = Task("gemm", "gemm", None, (1024, 1024, 1024), "llvm", 0)
    assert t.key == "gemm_gemm_(1024, 1024, 1024)_llvm(0)"
    for k in (GEMM, CONV, DW, I8, CONV1x1):
        assert k in TASK_TABLE
    for dev in range(4):
        assert "gemm_gemm_(1024, 1024, 1024)_rocm(%d)" % dev in TASK_TABLE
    with pytest.raises(KeyError):
        schedule("gemm_gemm_(3, 3, 3)_rocm(0)")
    with pytest.raises(RuntimeError):
        t.set_specific_space("x", "range", [1, 2])
    # drivers build a func=None task for the key and look the real one up
    probe = Task("conv2d", "baseline0", None, (1, 64, 56, 56, 64, 3, 1, 1, 1, 1), "rocm", 0)
    ops, bufs = TASK_TABLE[probe.key].func(*TASK_TABLE[probe.key].args)
    assert [b.shape for b in bufs] == [(1, 64, 56, 56), (64, 64, 3, 3), (1, 64, 56, 56)]
    ops, bufs = TASK_TABLE[I8].func(*TASK_TABLE[I8].args)
    assert [b.dtype for b in bufs] == ["int8", "int8", "int32"]
    # no override unless asked
    other = Task("gemm", "gemm", lambda *a: None, (1024, 1024, 1024), "rocm", 0)
    register_task(other)
    assert TASK_TABLE[GEMM].func is gemm
    assert "lds_pad" in TASK_TABLE[GEMM].special_space


def test_unsupported_target_and_method():
    register_task(Task("gemm", "gemm", gemm, (64, 64, 64), "cuda", 0), override=True)
    with pytest.raises(RuntimeError, match="no support for target"):
        schedule("gemm_gemm_(64, 64, 64)_cuda(0)")
    with pytest.raises(RuntimeError, match="no support for target"):
        schedule_with_config("gemm_gemm_(64, 64, 64)_cuda(0)", Config([], None))
    with pytest.raises(RuntimeError, match="no support for method"):
        schedule(GEMM, method="annealing", evaluator=lambda *a: 1.0)


def test_default_lowering_of_baseline_tasks():
    for key in (GEMM, CONV, DW, I8, CONV1x1):
        s, bufs = schedule_with_config(key, Config([], None))
        assert len(bufs) == 3 and s.specs
        main = s.specs[-1]
        assert main.block[0] % 64 == 0 and main.block[0] <= 1024
        for spec in s.specs:
            assert all(g >= 1 for g in spec.grid)
    s, _ = schedule_with_config(CONV, Config([], None))
    d = s.specs[-1].defines
    assert d["MODE"] == 1 and (d["M"], d["N"], d["K"]) == (64, 3136, 576) and d["CPADH"] == 1 and d["CPADW"] == 1
    assert [a[1] for a in s.specs[-1].args] == ["in1", "in0", "out"]  # A = weight, B = image
    assert s.intermediates == {}


def test_graph_config_not_inlined_materialises_padding():
    empty = {k: [] for k in ["fuse", "spatial", "reduce", "reorder", "inline", "unroll", "merge", "special"]}
    g = dict(empty)
    g["inline"] = [[0, 0]]
    s, _ = schedule_with_config(CONV, Config([dict(empty), {}], g))
    assert [x.kernel for x in s.specs] == ["zero_pad2d_f32", "igemm_f32"]
    assert s.intermediates == {"tmp0": ((1, 64, 58, 58), "float32")}
    d = s.specs[-1].defines
    assert d["CPADH"] == 0 and d["CPADW"] == 0 and d["CH"] == 58 and d["CW"] == 58
    assert [a[1] for a in s.specs[-1].args] == ["in1", "tmp0", "out"]
    g["inline"] = [[1, 1]]
    with pytest.raises(ValueError):
        schedule_with_config(CONV, Config([dict(empty), {}], g))


def _gemm_cfg(sp0, sp1, red, stages=2, gm=4, xcd=1):
    c = {k: [] for k in ["fuse", "spatial", "reduce", "reorder", "inline", "unroll", "merge", "special"]}
    c.update(spatial=[sp0, sp1], reduce=[red], unroll=[[stages, 1]], fuse=[[gm]], reorder=[[xcd]])
    return c


def test_lowering_rejects_bad_configs():
    ok = _gemm_cfg([16, 2, 1, 32], [16, 2, 1, 32], [1, 64, 16])
    s, _ = schedule_with_config(GEMM, Config([ok], None))
    d = s.specs[0].defines
    assert (d["WAVES_M"], d["REP_M"], d["MFMA"], d["BK"], d["SPLITK"]) == (2, 1, 32, 16, 1)
    assert s.specs[0].grid == (256, 1, 1) and s.specs[0].block == (256, 1, 1)
    bad = [
        _gemm_cfg([16, 2, 1, 32], [32, 2, 1, 16], [1, 64, 16]),   # mixed MFMA edge
        _gemm_cfg([15, 2, 1, 32], [16, 2, 1, 32], [1, 64, 16]),   # wrong grid level
        _gemm_cfg([16, 2, 1, 32], [16, 2, 1, 32], [1, 64, 8]),    # K product != K
        _gemm_cfg([2, 2, 8, 32], [2, 2, 8, 32], [1, 64, 16]),     # 1024 accumulators
        _gemm_cfg([8, 8, 1, 16], [8, 8, 1, 16], [1, 64, 16]),     # 64 wavefronts
        _gemm_cfg([32, 2, 1, 16], [32, 2, 1, 16], [1, 128, 8]),   # BK < 16 with 16x16x4
        _gemm_cfg([16, 2, 1, 32], [16, 2, 1, 32], [1, 64, 16], stages=9),   # no such pipeline depth
    ]
    # tiles straight into LDS (depth 5) land in unpadded rows: a padded A tile is refused
    dtl = _gemm_cfg([16, 2, 1, 32], [16, 2, 1, 32], [1, 64, 16], stages=5)
    assert schedule_with_config(GEMM, Config([dtl], None))[0].specs[0].defines["DTL"] == 1
    padded = {k: [] for k in dtl}
    padded["special"] = [[4, -1]]
    with pytest.raises(gfx950.InvalidConfig):
        schedule_with_config(GEMM, Config([dtl], padded))
    for cfg in bad:
        with pytest.raises(gfx950.InvalidConfig):
            schedule_with_config(GEMM, Config([cfg], None))
    # split-K adds the zero-fill kernel and multiplies the grid
    s, _ = schedule_with_config(GEMM, Config([_gemm_cfg([16, 2, 1, 32], [16, 2, 1, 32], [2, 32, 16])], None))
    assert [x.kernel for x in s.specs] == ["fill_zero_f32", "igemm_f32"] and s.specs[1].grid[0] == 512
    # int8 the same (integer atomic adds), or wavefront groups that add up in LDS
    i8 = _gemm_cfg([16, 2, 4, 32], [16, 2, 4, 32], [2, 32, 64])
    s, _ = schedule_with_config(I8, Config([i8], None))
    assert [x.kernel for x in s.specs] == ["fill_zero_f32", "gemm_i8"] and s.specs[1].grid[0] == 512
    assert s.specs[1].defines["SPLITK"] == 2 and "WAVES_K" not in s.specs[1].defines
    i8["reorder"] = [[1, 1]]
    with pytest.raises(gfx950.InvalidConfig):          # 256 accumulators x 256 lanes of the second group: 256 KiB
        schedule_with_config(I8, Config([i8], None))
    i8 = _gemm_cfg([32, 2, 2, 32], [32, 2, 2, 32], [2, 32, 64])
    i8["reorder"] = [[1, 1]]
    s, _ = schedule_with_config(I8, Config([i8], None))
    assert [x.kernel for x in s.specs] == ["gemm_i8"] and s.specs[0].grid[0] == 1024
    assert s.specs[0].defines["WAVES_K"] == 2 and s.specs[0].block[0] == 2 * 2 * 2 * 64
    # ... but finished-sum stores (early stores of the last tile) need an undivided K
    g = _gemm_cfg(None, None, None)
    g.update(spatial=[], reduce=[], unroll=[], fuse=[], reorder=[], inline=[[0]], special=[[-1, 0], [4]])
    i8 = _gemm_cfg([16, 2, 4, 32], [16, 2, 4, 32], [2, 32, 64], stages=7)
    schedule_with_config(I8, Config([_gemm_cfg([16, 2, 4, 32], [16, 2, 4, 32], [1, 64, 64], stages=7)], g))
    with pytest.raises(gfx950.InvalidConfig):
        schedule_with_config(I8, Config([i8], g))


def test_k_streaming_lowering():
    """reorder [[xcd, 0, s]]: s workgroups per compute unit share the (tile, k-tile) units."""
    cfg = _gemm_cfg([8, 2, 2, 32], [8, 2, 2, 32], [1, 32, 32])          # 64 tiles x 32 k-tiles
    cfg["reorder"] = [[1, 0, 1]]
    s, _ = schedule_with_config(GEMM, Config([cfg], None))
    spec = s.specs[-1]
    assert [x.kernel for x in s.specs] == ["igemm_f32"]                  # no zero fill
    assert spec.defines["SK_PER"] == 8 and spec.grid == (256, 1, 1)      # 2048 units over 256 CUs
    slot = 256 * 4 * 16                                                  # threads x accumulators
    assert s.workspaces == {"out_parts": ((256 * 2 * slot,), "float32"), "out_count": ((64,), "int32")}
    assert [a[1] for a in spec.args] == ["in0", "in1", "out", "out_parts", "out_count"]
    cfg["reorder"] = [[1, 0, 2]]
    s, _ = schedule_with_config(GEMM, Config([cfg], None))
    assert s.specs[-1].defines["SK_PER"] == 4 and s.specs[-1].grid == (512, 1, 1)
    # excluded together with the other K splits, and for int8
    for rd, ro in (([2, 16, 32], [1, 0, 1]), ([2, 16, 32], [1, 1, 1])):
        bad = _gemm_cfg([8, 2, 2, 32], [8, 2, 2, 32], rd)
        bad["reorder"] = [ro]
        with pytest.raises(gfx950.InvalidConfig):
            schedule_with_config(GEMM, Config([bad], None))
    i8 = _gemm_cfg([16, 2, 4, 32], [16, 2, 4, 32], [1, 64, 64])
    i8["reorder"] = [[1, 0, 1]]
    with pytest.raises(gfx950.InvalidConfig):
        schedule_with_config(I8, Config([i8], None))


def _conv_bias(N, C, H, W, K, k, stride=1, padding=0, dilation=1, groups=1):
    from flextensor_amd.nn import conv2d_nchw
    from flextensor_amd.te import placeholder
    Img = placeholder((N, C, H, W), name="Img")
    Wt = placeholder((K, C // groups, k, k), name="W")
    bias = placeholder((K,), name="bias")
    Out = conv2d_nchw(Img, Wt, bias, stride=stride, padding=padding, dilation=dilation, groups=groups)
    return [Out.op], [Img, Wt, bias, Out]


def test_bias_stage_merges_into_the_convolution_or_runs_alone():
    """Graph [Padding, conv, bias]: the "merge" key decides between a bias
    epilogue in the convolution kernel and a separate elementwise kernel."""
    from flextensor_amd.task import register
    from flextensor_amd.space import generate_space_inter_op
    args = (2, 16, 14, 14, 32, 3, 1, 1, 1, 1)
    register(_conv_bias, "conv2d", "bias", args, "rocm", 0)
    key = Task("conv2d", "bias", None, args, "rocm", 0).key
    ops, bufs = _conv_bias(*args)
    op_lst, down = flatten_graph(ops)
    assert [o.kind for o in op_lst] == ["zero_pad2d", "conv2d_nchw", "bias_add_nchw"]
    gs = generate_space_inter_op(op_lst, down)
    assert gs.subspaces["merge"].static_entities == [[0, 0, 1], [0, 0, 0]] or \
        sorted(gs.subspaces["merge"].static_entities) == [[0, 0, 0], [0, 0, 1]]
    # default: merged -> one kernel with the bias as fourth buffer
    s, _ = schedule_with_config(key, Config([], None))
    assert [x.kernel for x in s.specs] == ["igemm_f32"]
    assert s.specs[0].defines["HAS_BIAS"] == 1 and [a[1] for a in s.specs[0].args] == ["in1", "in0", "out", "in2"]
    # not merged -> convolution into a temporary, then the bias kernel
    g = {k: [] for k in ["fuse", "spatial", "reduce", "reorder", "inline", "unroll", "merge", "special"]}
    g["inline"], g["merge"] = [[1, 0, 0]], [[0, 0, 0]]
    s, _ = schedule_with_config(key, Config([], g))
    assert [x.kernel for x in s.specs] == ["igemm_f32", "bias_add_nchw_f32"]
    assert "HAS_BIAS" not in s.specs[0].defines and s.specs[0].args[2] == ("buf", "tmp1")
    assert [a[1] for a in s.specs[1].args[:3]] == ["tmp1", "in2", "out"] and "tmp1" in s.intermediates
    # a flag on an op that cannot merge is refused
    g["merge"] = [[0, 1, 0]]
    with pytest.raises(gfx950.InvalidConfig):
        schedule_with_config(key, Config([], g))
    # the search handles the three-op graph (host cost: fewer kernels is cheaper)
    np.random.seed(5)
    s, bufs2, configs = schedule(key, op_trial=2, graph_trial=2, parallel=2, warm_up=(1, 4), verbose=False,
                                 evaluator=lambda k, c, p, n: 1.0 + len(schedule_with_config(k, c, op_pos=p)[0].specs))
    assert len(configs.op_config_lst) == 3 and configs.graph_config["merge"][0] == [0, 0, 1]
    assert [x.kernel for x in s.specs] == ["igemm_f32"]


def test_gemm_conv2d_graph_flags_choose_the_kernel_sequence():
    """Graph [Padding, Img2Col, ComputeGemm, Col2Img] (flextensor/nn/ops.py:982-1044):
    inline and merge flags decide which stages exist as kernels; with everything
    folded the plan is the direct convolution's kernel."""
    from flextensor_amd.space import generate_space_inter_op
    key = Task("gemm_conv2d", "yolo5", None, (1, 256, 56, 56, 512, 3, 1, 1, 1, 1), "rocm", 0).key
    conv_key = Task("conv2d", "yolo5", None, (1, 256, 56, 56, 512, 3, 1, 1, 1, 1), "rocm", 0).key
    task = TASK_TABLE[key]
    ops, bufs = task.func(*task.args)
    op_lst, down = flatten_graph(ops)
    assert [(o.name, o.kind) for o in op_lst] == [("Padding", "zero_pad2d"), ("Img2Col", "im2col_nchw"),
                                                   ("ComputeGemm", "col_gemm"), ("Col2Img", "col2img_nchw")]
    assert op_lst[1].output(0).shape == (1, 2304, 3136) and op_lst[2].output(0).shape == (1, 512, 3136)
    assert bufs[-1].shape == (1, 512, 56, 56)
    gs = generate_space_inter_op(op_lst, down, special_space=task.special_space)
    assert sorted(gs.subspaces["inline"].static_entities) == [[0, 0, 0, 0], [0, 1, 0, 0], [1, 0, 0, 0], [1, 1, 0, 0]]
    assert sorted(gs.subspaces["merge"].static_entities) == [[0, 0, 0, 0], [0, 0, 0, 1]]
    # defaults: one implicit-GEMM kernel, the same source and constants as conv2d's
    s, _ = schedule_with_config(key, Config([], None))
    c, _ = schedule_with_config(conv_key, Config([], None))
    assert [x.kernel for x in s.specs] == ["igemm_f32"] and not s.intermediates
    assert s.specs[0].defines == c.specs[0].defines and s.specs[0].grid == c.specs[0].grid

    def plan(inline, merge):
        g = {k: [] for k in ["fuse", "spatial", "reduce", "reorder", "inline", "unroll", "merge", "special"]}
        g["inline"], g["merge"] = [inline], [merge]
        return schedule_with_config(key, Config([], g))[0]

    s = plan([1, 1, 0, 0], [0, 0, 0, 0])
    assert [x.kernel for x in s.specs] == ["igemm_f32", "col2img_nchw_f32"]
    assert s.specs[0].defines["COLOUT"] == 1 and s.intermediates == {"tmp2": ((1, 512, 3136), "float32")}
    s = plan([0, 0, 0, 0], [0, 0, 0, 0])
    assert [x.kernel for x in s.specs] == ["zero_pad2d_f32", "im2col_nchw_f32", "igemm_f32", "col2img_nchw_f32"]
    assert s.specs[1].defines["CH"] == 58 and s.specs[1].defines["CPADH"] == 0      # reads the padded image
    assert s.specs[2].defines["MODE"] == 0 and [a[1] for a in s.specs[2].args] == ["in1", "tmp1", "tmp2"]
    s = plan([1, 0, 0, 0], [0, 0, 0, 0])
    assert s.specs[0].kernel == "im2col_nchw_f32" and s.specs[0].defines["CH"] == 56 and s.specs[0].defines["CPADH"] == 1
    s = plan([0, 1, 0, 0], [0, 0, 0, 1])
    assert [x.kernel for x in s.specs] == ["zero_pad2d_f32", "igemm_f32"]
    assert s.specs[1].defines["CPADH"] == 0 and s.specs[1].defines["CH"] == 58 and "COLOUT" not in s.specs[1].defines
    # one image: [groups][M][P*Q] is NCHW already, so the GEMM over stored columns writes the output itself
    s = plan([1, 0, 0, 0], [0, 0, 0, 1])
    assert [x.kernel for x in s.specs] == ["im2col_nchw_f32", "igemm_f32"] and s.specs[1].args[2] == ("buf", "out")
    # a batch interleaves the images: then the NCHW store belongs to the kernel that knows the geometry
    key8 = Task("gemm_conv2d", "yolo_b85", None, (8, 256, 56, 56, 512, 3, 1, 1, 1, 1), "rocm", 0).key
    g8 = {k: [] for k in ["fuse", "spatial", "reduce", "reorder", "inline", "unroll", "merge", "special"]}
    g8["inline"], g8["merge"] = [[1, 0, 0, 0]], [[0, 0, 0, 1]]
    with pytest.raises(gfx950.InvalidConfig):
        schedule_with_config(key8, Config([], g8))
    # searched like any other task (host cost: fewer kernels is cheaper)
    np.random.seed(3)
    s, _, configs = schedule(key, op_trial=2, graph_trial=3, parallel=2, warm_up=(1, 4), verbose=False,
                             trials=[1, 1, 2, 1],
                             evaluator=lambda k, c, p, n: 1.0 + len(schedule_with_config(k, c, op_pos=p)[0].specs))
    assert len(configs.op_config_lst) == 4 and [x.kernel for x in s.specs] == ["igemm_f32"]
    assert configs.graph_config["inline"][0] == [1, 1, 0, 0] and configs.graph_config["merge"][0] == [0, 0, 0, 1]


def test_batch_gemm_lowers_to_one_launch_over_all_matrices():
    from flextensor_amd.task import register, batch_gemm
    args = (6, 128, 96, 192)
    register(batch_gemm, "gemm", "batch_gemm", args, "rocm", 0)
    key = Task("gemm", "batch_gemm", None, args, "rocm", 0).key
    assert "lds_pad" in TASK_TABLE[key].special_space
    s, bufs = schedule_with_config(key, Config([], None))
    spec = s.specs[-1]
    d = spec.defines
    assert [x.kernel for x in s.specs] == ["igemm_f32"] and d["CG"] == 6 and d["MODE"] == 0
    assert (d["M"], d["N"], d["K"]) == (128, 192, 96)
    tiles = math.ceil(128 / (d["WAVES_M"] * d["REP_M"] * d["MFMA"])) * math.ceil(192 / (d["WAVES_N"] * d["REP_N"] * d["MFMA"]))
    assert spec.grid[0] == tiles * 6 and [b.shape for b in bufs] == [(6, 128, 96), (6, 96, 192), (6, 128, 192)]


def test_lds_budget_respected_over_whole_space():
    ops, _ = TASK_TABLE[I8].func(*TASK_TABLE[I8].args)
    op_lst, down = flatten_graph(ops)
    space = generate_space_intra_op(op_lst[0], down, target="rocm")
    wg = WalkerGroup("t", space)
    rng = np.random.default_rng(0)
    n_ok = 0
    for _ in range(300):
        idx = {name: int(rng.integers(0, len(sub))) for name, sub in space.items()}
        cfg = wg.to_config(idx)
        try:
            s, _ = schedule_with_config(I8, Config([cfg], None))
        except gfx950.InvalidConfig:
            continue
        n_ok += 1
        d = s.specs[-1].defines
        bm = d["WAVES_M"] * d["REP_M"] * d["MFMA"]
        bn = d["WAVES_N"] * d["REP_N"] * d["MFMA"]
        assert d["STAGES"] * (bm + bn) * (d["BK"] + d["PAD"]) <= 160 * 1024
        assert d["REP_M"] * d["REP_N"] * d["MFMA"] ** 2 // 64 <= 256
    assert n_ok > 20


def _synthetic_cost(task_key, cfg, op_pos, number):
    """Smooth host-side cost with a known optimum, defined on the lowered kernel."""
    s, _ = schedule_with_config(task_key, cfg, op_pos=op_pos)
    d = s.specs[-1].defines
    bm = d["WAVES_M"] * d["REP_M"] * d["MFMA"]
    bn = d["WAVES_N"] * d["REP_N"] * d["MFMA"]
    cost = abs(math.log2(bm) - 6) + abs(math.log2(bn) - 6) + abs(math.log2(d["BK"]) - 5)
    cost += 0.5 * (d["SPLITK"] - 1) + 0.25 * (d["STAGES"] != 2) + 0.1 * abs(d["GROUP_M"] - 4)
    cost += 0.3 * (d["MFMA"] != 32) + 0.2 * (d["WAVES_M"] * d["WAVES_N"] != 4)
    return 1.0 + cost


def test_schedule_searching_finds_known_optimum_and_roundtrips():
    np.random.seed(0)
    s, bufs, configs = schedule(GEMM, op_trial=30, op_stop=30, graph_trial=2, parallel=4,
                                evaluator=_synthetic_cost, warm_up=(3, 10), verbose=False)
    best = _synthetic_cost(GEMM, configs, None, 1)
    assert best <= 1.5, best
    assert isinstance(configs, Config) and len(configs.op_config_lst) == 1
    assert sorted(configs.op_config_lst[0]) == sorted(
        ["fuse", "spatial", "reduce", "reorder", "inline", "unroll", "merge", "special"])
    assert len(configs.graph_config["special"]) == len(TASK_TABLE[GEMM].special_space)
    # JSON log line round trip (the reference's `key:json` format)
    line = GEMM + ":" + json.dumps(configs)
    name, string = line.split(":", 1)
    obj = json.loads(string)
    s2, _ = schedule_with_config(name, Config(obj[0], obj[1]))
    assert s2.describe() == s.describe()


def test_warm_start_takes_an_entry_written_before_a_knob_existed():
    """The shipped entry of a 1x1 layer pinned to the gather has both knobs, most have lds_pad only:
    either way the operator search runs under the entry's graph config, missing knobs at their defaults."""
    seen = {}

    def cost(task_key, cfg, op_pos, number):
        s, _ = schedule_with_config(task_key, cfg, op_pos=op_pos)
        if op_pos is not None:
            seen.setdefault(task_key, set()).add(s.specs[-1].defines["MODE"])
        return 1.0 + 1e-4 * s.specs[-1].grid[0]

    gather = "conv2d_yolo8_(1, 512, 28, 28, 512, 1, 1, 0, 1, 1)_rocm(0)"      # special [[..], [0]]
    older = "conv2d_yolo10_(1, 1024, 14, 14, 512, 1, 1, 0, 1, 1)_rocm(0)"     # special [[..]]
    assert len(lookup(gather).graph_config["special"]) == 2 and len(lookup(older).graph_config["special"]) == 1
    for key in (gather, older):
        np.random.seed(2)
        schedule(key, op_trial=2, graph_trial=1, parallel=2, method="random", evaluator=cost, verbose=False)
    assert seen[gather] == {1} and seen[older] == {0}


def test_schedule_random_method_and_conv_graph():
    np.random.seed(1)
    calls = []

    def cost(task_key, cfg, op_pos, number):
        calls.append(op_pos)
        s, _ = schedule_with_config(task_key, cfg, op_pos=op_pos)
        return 1.0 + 0.01 * len(s.specs) + 1e-4 * s.specs[-1].grid[0]

    s, bufs, configs = schedule(CONV, op_trial=3, graph_trial=2, parallel=3, method="random",
                                evaluator=cost, verbose=False)
    assert len(configs.op_config_lst) == 2          # [Padding, conv]
    assert not any(configs.op_config_lst[0].values())  # padding has no knobs
    assert configs.graph_config["inline"][0] == [1, 0]  # fused padding is cheaper here
    assert 1 in calls and None in calls


def test_an_operator_schedulers_workers_are_closed_before_the_next_scheduler_starts(monkeypatch):
    """Compile workers load the HIP runtime; two pools alive at once doubled the number of
    processes holding the device (a machine may bound it)."""
    import flextensor_amd.scheduler as sch
    events = []
    real_close, real_init = sch.OpScheduler.close, sch.GraphScheduler.__init__
    monkeypatch.setattr(sch.OpScheduler, "close", lambda self: (events.append("op closed"), real_close(self))[1])

    def init(self, *a, **k):
        events.append("graph scheduler")
        real_init(self, *a, **k)
    monkeypatch.setattr(sch.GraphScheduler, "__init__", init)
    schedule(CONV, op_trial=2, graph_trial=1, parallel=2, method="random",
             evaluator=lambda k, c, p, n: 1.0, verbose=False)
    assert events.index("op closed") < events.index("graph scheduler")


def test_failing_candidates_become_inf_and_search_survives():
    np.random.seed(2)
    n = {"calls": 0}

    def flaky(task_key, cfg, op_pos, number):
        n["calls"] += 1
        if n["calls"] % 3 == 0:
            raise RuntimeError("candidate crashed")
        return _synthetic_cost(task_key, cfg, op_pos, number)

    s, bufs, configs = schedule(GEMM, op_trial=5, graph_trial=1, parallel=2, evaluator=flaky,
                                warm_up=(2, 6), verbose=False)
    assert configs.op_config_lst[0]["spatial"]


def test_all_invalid_warm_up_escalates_then_gives_up():
    def never(task_key, cfg, op_pos, number):
        raise RuntimeError("nothing builds")

    ops, _ = TASK_TABLE[GEMM].func(*TASK_TABLE[GEMM].args)
    op_lst, down = flatten_graph(ops)
    space = generate_space_intra_op(op_lst[0], down, target="rocm")
    o = sch.OpScheduler(GEMM, 0, space, parallel=2, timeout=1, evaluator=never)
    o.verbose = False
    o._warm_up(1, 4, Config([], None), ["fuse", "reorder", "spatial", "reduce", "unroll"], max_repeat=3)
    assert o.walker_group.top1() == {} and o.timeout == 1


def test_walker_group_heap_semantics():
    ops, _ = gemm(256, 256, 256)
    op_lst, down = flatten_graph(ops)
    space = generate_space_intra_op(op_lst[0], down, target="rocm")
    wg = WalkerGroup("g", space)
    pts = []
    np.random.seed(3)
    ret = wg.forward(5)
    for i in range(5):
        idx = {name: int(ret[name][1][i]) for name in ret}
        pts.append(idx)
        wg.record(idx, float(5 - i))
    assert wg.top1_value() == 1.0 and wg.top1() == pts[4]
    assert [v for _, v in wg.topk(3, with_value=True)] == [1.0, 2.0, 3.0] and wg.mem_size == 5
    assert wg.ever_met(pts[0]) and wg.pop_top().value == 1.0 and wg.mem_size == 4
    nxt, acts = wg.full_walk(pts[0], no_repeat=True)
    assert all(not wg.ever_met(n) for n in nxt) and len(nxt) == len(acts)
    for n_, (name, d) in zip(nxt, acts):
        diff = [k for k in n_ if n_[k] != pts[0][k]]
        assert diff == [name]
    cfg = wg.to_config(pts[0])
    assert len(cfg["spatial"]) == 2 and len(cfg["reduce"]) == 1 and cfg["inline"] == []
    # a hopeless value is (almost surely) rejected by the Boltzmann filter
    wg.record(nxt[0], 1e9, random_reject=True)
    assert wg.mem_size == 4 and wg.ever_met(nxt[0])


def test_seed_points_cover_the_decisive_knobs_and_belong_to_the_space():
    """The heuristic points measured before the random warm-up: inside the
    operator's space, bounded in number, with direct-to-LDS depths, whole 3x3
    windows, K streaming for few tiles, and grid-level K splits for layers
    whose weights stream past a small image."""
    def seeds_of(key):
        task = TASK_TABLE[key]
        ops, _ = task.func(*task.args)
        op_lst, down = flatten_graph(ops)
        op = [o for o in op_lst if o.kind in gfx950.GEMM_KINDS][0]
        return op, generate_space_intra_op(op, down, target="rocm"), gfx950.seed_configs(op)

    for key in (GEMM, CONV, CONV1x1, I8, "conv2d_yolo14_(1, 1024, 7, 7, 1024, 3, 1, 1, 1, 1)_rocm(0)"):
        op, space, seeds = seeds_of(key)
        assert 1 <= len(seeds) <= 24, key
        assert seeds[0] == gfx950.default_config(op)
        for cfg in seeds[1:]:
            # every knob value of the variations is an entity of its sub-space
            assert space.subspaces["split_m_0"].index_of(cfg["spatial"][0]) >= 0, (key, cfg["spatial"])
            assert space.subspaces["split_n_1"].index_of(cfg["spatial"][1]) >= 0, (key, cfg["spatial"])
            assert space.subspaces["split_k_0"].index_of(cfg["reduce"][0]) >= 0, (key, cfg["reduce"])
    _, _, seeds = seeds_of(CONV)
    assert any(c["unroll"][0][0] == 5 for c in seeds) and any(c["reduce"][0][2] in (72, 144) for c in seeds)
    # 16 x 1 tiles of 64 x 64 on 256 compute units: K is split across workgroups in a third of the points
    _, _, seeds = seeds_of("conv2d_yolo14_(1, 1024, 7, 7, 1024, 3, 1, 1, 1, 1)_rocm(0)")
    splits = [c["reduce"][0][0] for c in seeds]
    assert sum(1 for s in splits if s > 1) == 8 and max(splits) <= 16
    assert any(c["reorder"][0][2] > 0 for c in seeds)            # K streaming is among them as well
    # plenty of tiles: no K split
    _, _, seeds = seeds_of(I8)
    assert all(c["reduce"][0][0] == 1 for c in seeds)
    # 1x1 convolution on a 7x7 image, K = 832 = 52 tiles of 16: single-wavefront tiles whose 13
    # wavefront groups share K inside the workgroup (one launch), beside the splits across workgroups
    key = "conv2d_google38_(1, 832, 7, 7, 256, 1, 1, 0, 1, 1)_rocm(0)"
    op, space, seeds = seeds_of(key)
    groups = [c for c in seeds if c["reorder"] and c["reorder"][0][1] == 1]
    assert [c["reduce"][0] for c in groups] == [[13, 4, 16], [4, 13, 16], [4, 13, 16]]
    assert groups[0]["spatial"] == [[16, 1, 1, 16], [4, 1, 1, 16]] and len(seeds) <= 24
    for cfg in groups:
        assert space.subspaces["split_n_1"].index_of(cfg["spatial"][1]) >= 0
        spec = gfx950.lower(op, cfg, None, "out", ["x", "w"])[-1]
        assert spec.defines["WAVES_K"] == cfg["reduce"][0][0] and spec.defines["SPLITK"] == 1
    _, _, seeds = seeds_of(CONV)
    assert not any(c["reorder"][0][1] == 1 for c in seeds[1:])


def test_awkward_k_may_be_zero_padded_to_wider_lds_tiles():
    """K = 400 (16 channels x 5x5) divides into LDS tiles of 8 and 16 only; up to an eighth of zero
    padding admits tiles of 32 .. 144. A K with a tile of 32 or more keeps its single extent."""
    def view_of(key):
        task = TASK_TABLE[key]
        ops, _ = task.func(*task.args)
        op = [o for o in flatten_graph(ops)[0] if o.kind in gfx950.GEMM_KINDS][0]
        return op, gfx950.GemmView(op)
    op, v = view_of("conv2d_google18_(1, 16, 14, 14, 48, 5, 1, 2, 1, 1)_rocm(0)")
    assert (v.K, v.KP, v.KP_options) == (400, 400, [400, 416, 432, 448])
    cfg = gfx950.default_config(op)
    assert cfg["reduce"][0][0] * cfg["reduce"][0][1] * cfg["reduce"][0][2] == 400
    for red, kp in (([1, 7, 64], 448), ([1, 3, 144], 432), ([13, 1, 32], 416)):
        cfg["reduce"] = [red]
        cfg["reorder"] = [[1, 1 if red[0] > 1 else 0, 0]]
        spec = gfx950.lower(op, cfg, None, "out", ["x", "w"])[-1]
        assert spec.defines["KP"] == kp and spec.defines["K"] == 400
    cfg["reduce"], cfg["reorder"] = [[1, 4, 128]], [[1, 0, 0]]       # 512: more than an eighth of padding
    with pytest.raises(gfx950.InvalidConfig):
        gfx950.lower(op, cfg, None, "out", ["x", "w"])
    assert view_of("conv2d_overfeat0_(1, 3, 192, 192, 96, 11, 4, 5, 1, 1)_rocm(0)")[1].KP_options == [368, 384]
    assert view_of(CONV)[1].KP_options == [576] and view_of(GEMM)[1].KP_options == [1024]
    assert view_of("conv2d_google0_(1, 3, 224, 224, 64, 7, 2, 3, 1, 1)_rocm(0)")[1].KP_options == [160]


def test_pointwise_convolution_of_one_image_lowers_in_the_gemm_mode():
    """1x1 / stride 1 / unpadded / one image: the image is the B matrix as it lies in memory; the task
    carries the knob that chooses between that and the general gather, other convolutions do not."""
    key = "conv2d_yolo10_(1, 1024, 14, 14, 512, 1, 1, 0, 1, 1)_rocm(0)"
    assert list(TASK_TABLE[key].special_space) == ["lds_pad", "image_as_matrix"]
    s, _ = schedule_with_config(key, Config([], None))
    d = s.specs[-1].defines
    assert (d["MODE"], d["BV"], d["M"], d["N"], d["K"]) == (0, 4, 512, 196, 1024) and "CH" not in d
    assert [a[1] for a in s.specs[-1].args[:3]] == ["in1", "in0", "out"]  # A = weight, B = image
    cfg = lookup(key)
    g = dict(cfg.graph_config)
    g["special"] = [list((g.get("special") or [[-1, -1]])[0]), [0]]
    d = schedule_with_config(key, Config(cfg.op_config_lst, g))[0].specs[-1].defines
    assert d["MODE"] == 1 and d["BV"] == 1 and d["CH"] == 14
    for other in (CONV, CONV1x1, "conv2d_res5_(64, 256, 56, 56, 512, 1, 2, 0, 1, 1)_rocm(0)"):
        assert list(TASK_TABLE[other].special_space) == ["lds_pad"]       # 3x3; batch 8; stride 2
        assert schedule_with_config(other, Config([], None))[0].specs[-1].defines["MODE"] == 1
    # a bias runs in the convolution's epilogue, which the GEMM mode does not have
    from flextensor_amd.nn import conv2d_nchw
    from flextensor_amd.te import placeholder

    def with_bias():
        x, w, b = placeholder((1, 32, 14, 14), name="Img"), placeholder((48, 32, 1, 1), name="W"), placeholder((48,), name="b")
        out = conv2d_nchw(x, w, b)
        return [out.op], [x, w, b, out]
    t = Task("conv2d", "pw_bias", with_bias, (), "rocm", 0)
    register_task(t, override=True)
    kernels = schedule_with_config(t.key, Config([], None))[0].specs
    assert kernels[-1].defines["MODE"] == 1 and kernels[-1].defines.get("HAS_BIAS") == 1


def test_depthwise_lowering_with_several_kernels_per_channel():
    """kernel_fuse: lanes own patches of input planes and compute every output plane of the channel
    (a sixth of the lanes for MobileNet's x6 stages); conv2d with one channel per group is that operator."""
    key = "conv2d_depthwise_(8, 16, 112, 112, 6, 3, 2, 1, 1)_rocm(0)"
    task = TASK_TABLE[key]
    assert task.special_space["kernel_fuse"].static_entities == [[1], [0]]
    base = gfx950.default_config(flatten_graph(task.func(*task.args)[0])[0][1])
    def plan(fuse):
        g = {k: [] for k in base}
        g["inline"], g["special"] = [[1, 0]], [[0], [0], [0], [1], [0], [fuse]]
        s, _ = schedule_with_config(key, Config([{k: [] for k in base}, base], g))
        return s.specs[-1]
    fused, single = plan(1), plan(0)
    assert fused.defines["MFUSE"] == 1 and "MFUSE" not in single.defines and fused.defines["FACT"] == 6
    assert single.grid[0] == 6 * fused.grid[0]
    s, _ = schedule_with_config(key, Config([], None))              # the default fuses
    assert s.specs[-1].defines.get("MFUSE") == 1
    # one kernel per channel: the knob changes nothing
    one = "conv2d_depthwise_(8, 512, 28, 28, 1, 3, 1, 1, 1)_rocm(0)"
    assert "MFUSE" not in schedule_with_config(one, Config([], None))[0].specs[-1].defines
    # conv2d with groups = input channels builds the depthwise operator and carries its knobs
    mob = "conv2d_mobile_v21_(1, 16, 112, 112, 96, 3, 2, 1, 1, 16)_rocm(0)"
    ops, bufs = TASK_TABLE[mob].func(*TASK_TABLE[mob].args)
    assert ops[0].kind == "depthwise_conv2d_nchw" and ops[0].attrs["factor"] == 6 and bufs[1].shape == (96, 1, 3, 3)
    assert "row_exchange" in TASK_TABLE[mob].special_space and "lds_pad" not in TASK_TABLE[mob].special_space
    grp = "conv2d_grouped_(1, 1024, 14, 14, 512, 1, 1, 0, 1, 4)_rocm(0)"
    assert TASK_TABLE[grp].func(*TASK_TABLE[grp].args)[0][0].kind == "conv2d_nchw"


def test_schedule_ops_with_config_takes_a_flattened_op_list():
    """flextensor/scheduler.py:1189-1220: configs are matched to the operators of an already
    flattened list by position; the plan comes back (a plan passed in is refilled)."""
    from flextensor_amd.scheduler import schedule_ops_with_config
    key = "conv2d_baseline0_(1, 64, 56, 56, 64, 3, 1, 1, 1, 1)_rocm(0)"
    task = TASK_TABLE[key]
    ops, bufs = task.func(*task.args)
    op_lst, _ = flatten_graph(ops)
    assert [op.kind for op in op_lst] == ["zero_pad2d", "conv2d_nchw"]
    ref, _ = schedule_with_config(key, Config([], None))
    plan = schedule_ops_with_config(None, op_lst, Config([], None), "rocm")
    assert [sp.defines for sp in plan.specs] == [sp.defines for sp in ref.specs]
    assert [tuple(b.shape) for b in plan.bufs] == [tuple(b.shape) for b in bufs]
    # a graph config that materialises the padding gives two kernels; an existing plan is refilled
    g = {k: [] for k in gfx950.Space.valid_type_keys}
    g["inline"] = [[0, 0]]
    again = schedule_ops_with_config(plan, op_lst, Config([], g), "rocm")
    assert again is plan and [sp.kernel for sp in plan.specs] == ["zero_pad2d_f32", "igemm_f32"]
    with pytest.raises(ValueError):
        schedule_ops_with_config(None, list(reversed(op_lst)), Config([], None), "rocm")
    with pytest.raises(RuntimeError):
        schedule_ops_with_config(None, op_lst, Config([], None), "cuda")


def test_clock_probe_plan_is_a_copy_with_one_more_argument():
    """KernelPlan.with_clock_probe: the main kernel gets the FT_CLKPROBE define, a last argument
    and a [workgroups][2] int64 workspace; every other kernel and the plan itself stay untouched,
    and the instrumented source compiles for gfx950."""
    from flextensor_amd.tuned import lookup
    key = "conv2d_baseline1_(8, 256, 14, 14, 512, 3, 1, 1, 1, 1)_rocm(0)"     # K streaming: workspaces of its own
    s, _ = schedule_with_config(key, lookup(key))
    probe = s.with_clock_probe()
    assert "CLKPROBE" not in s.specs[-1].defines and probe.specs[-1].defines["CLKPROBE"] == 1
    assert probe.specs[-1].args[:-1] == s.specs[-1].args and probe.specs[-1].args[-1] == ("buf", "clk_probe")
    nwg = s.specs[-1].grid[0]
    assert probe.workspaces["clk_probe"] == ((nwg, 2), "int64")
    assert set(probe.workspaces) == set(s.workspaces) | {"clk_probe"}
    assert probe.specs[:-1] == s.specs[:-1]
    assert all(len(code) > 1000 for code in probe.compile())
    # a plan without a kernel that takes the probe says so
    from flextensor_amd.plan import KernelPlan
    with pytest.raises(ValueError):
        KernelPlan("x", s.bufs, [], {}, None).with_clock_probe()
