"""Learned search (method="q", use_model): host-side, with a synthetic cost."""
import math
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from flextensor_amd.model import WalkerGroup, rank_loss
from flextensor_amd.scheduler import schedule, schedule_with_config
from flextensor_amd.space import generate_space_intra_op
from flextensor_amd.task import TASK_TABLE
from flextensor_amd.utils import Config

GEMM = "gemm_gemm_(1024, 1024, 1024)_rocm(0)"


def _space():
    task = TASK_TABLE[GEMM]
    ops, _ = task.func(*task.args)
    return generate_space_intra_op(ops[0], {}, slevel=4, rlevel=3, target="rocm")


def _cost(task_key, cfg, op_pos, number):
    s, _ = schedule_with_config(task_key, cfg, op_pos=op_pos)
    d = s.specs[-1].defines
    bm = d["WAVES_M"] * d["REP_M"] * d["MFMA"]
    bn = d["WAVES_N"] * d["REP_N"] * d["MFMA"]
    cost = abs(math.log2(bm) - 6) + abs(math.log2(bn) - 6) + abs(math.log2(d["BK"]) - 5)
    cost += 0.5 * (d["SPLITK"] - 1) + 0.25 * (d["STAGES"] != 2) + 0.1 * abs(d["GROUP_M"] - 4)
    return 1.0 + cost


def test_flattened_points_have_the_space_dimension():
    space = _space()
    wg = WalkerGroup("t", space)
    batch = wg.forward(8)
    for i in range(8):
        indices = {name: int(batch[name][1][i]) for name in batch}
        assert len(wg.flatten(indices)) == space.dim


def test_walker_steps_are_neighbours_and_training_lowers_td_error():
    np.random.seed(0)
    torch.manual_seed(0)
    space = _space()
    wg = WalkerGroup("t", space)
    batch = wg.forward(4)
    starts = [({name: int(batch[name][1][i]) for name in batch}, 1.0) for i in range(4)]
    from_lst, nxt, actions = wg.walk(starts, trial=0)
    assert len(from_lst) == len(nxt) == len(actions) > 0
    for (frm, _), to, (name, choice) in zip(from_lst, nxt, actions):
        changed = [k for k in frm if frm[k] != to[k]]
        assert changed in ([], [name])                       # one sub-space moves, or the move was a no-op
        sub = space.subspaces[name]
        assert to[name] == sub.next_entity(frm[name], sub.get_direction(choice))
    # transitions with a reward only for direction 0 of one sub-space: Q(.,0) must rise above the rest
    name = "spatial_0" if "spatial_0" in wg.walkers else list(wg.walkers)[0]
    w = wg.walkers[name]
    for _ in range(200):
        i = {n: int(np.random.randint(0, s.size)) for n, s in space.subspaces.items()}
        a = int(np.random.randint(0, w.subspace.num_direction))
        w.add_data(wg.flatten(i), a, wg.flatten(i), 1.0 if a == 0 else 0.0)
    first = w.train(epochs=1)
    for _ in range(5):
        last = w.train(epochs=20)
    x = torch.tensor([wg.flatten(starts[0][0])], dtype=torch.float32)
    q = w.pre_judger(x)[0]
    assert int(torch.argmax(q)) == 0
    assert last < first or last < 1.0


def test_rank_loss_orders_pairs():
    t = torch.tensor([1.0, 2.0, 3.0])
    good = rank_loss(torch.tensor([0.0, 5.0, 10.0]), t)
    bad = rank_loss(torch.tensor([10.0, 5.0, 0.0]), t)
    flat = rank_loss(torch.zeros(3), t)
    assert float(good) < float(flat) < float(bad)
    # the closed form for two items: log(1+e^-d) + log(1+e^-d) + 2 log 2 on the diagonal
    y = torch.tensor([0.0, 2.0])
    expect = 2 * math.log(1 + math.exp(-2.0)) + 2 * math.log(2.0)
    assert abs(float(rank_loss(y, torch.tensor([1.0, 2.0]))) - expect) < 1e-6


def test_performance_model_learns_a_ranking(tmp_path):
    np.random.seed(1)
    torch.manual_seed(1)
    space = _space()
    wg = WalkerGroup("t", space, lr=1.0)
    wg.model_dir = str(tmp_path)

    def sample(n):
        pts = [{name: int(np.random.randint(0, s.size)) for name, s in space.subspaces.items()} for _ in range(n)]
        return pts, [float(sum(wg.flatten(p)[:4])) for p in pts]    # cost = a visible function of the point

    for _ in range(60):
        pts, vals = sample(8)
        wg.add_perf_data(pts, vals)
    wg.load_or_create_model()
    before = wg.train_on_perf(epochs=1)
    after = wg.train_on_perf(epochs=30)
    assert after < before
    pts, vals = sample(64)
    pred = wg.query_performance(pts)
    agree = np.mean([(pred[i] < pred[j]) == (vals[i] < vals[j])
                     for i in range(64) for j in range(64) if vals[i] != vals[j]])
    assert agree > 0.6, agree
    assert os.path.exists(os.path.join(str(tmp_path), wg.model_path))
    # dump / load of the samples, inf stored as null
    wg.add_perf_data(pts[:2], [1.0, float("inf")])
    path = os.path.join(str(tmp_path), "perf.txt")
    wg.dump_performance_data(path)
    wg2 = WalkerGroup("t", space)
    wg2.load_performance_data(path)
    assert len(wg2.perfromance_data) == len(wg.perfromance_data)
    assert wg2.perfromance_data[-1][1][1] == float("inf")


def test_schedule_method_q_improves_on_warm_up_and_returns_a_valid_plan(tmp_path):
    np.random.seed(3)
    torch.manual_seed(3)
    seen = []

    def cost(task_key, cfg, op_pos, number):
        c = _cost(task_key, cfg, op_pos, number)
        seen.append(c)
        return c

    s, bufs, configs = schedule(GEMM, op_trial=10, op_stop=10, graph_trial=2, parallel=4, method="q",
                                evaluator=cost, warm_up=(2, 8), verbose=False, perf_path=str(tmp_path))
    final = _cost(GEMM, configs, None, 1)
    assert final <= min(seen) + 1e-9 or final <= 2.0
    assert final < np.median(seen[:16])
    assert s.specs[-1].kernel == "igemm_f32"
    assert any(f.startswith("walker_judger_model_") for f in os.listdir(str(tmp_path)))


def test_schedule_use_model_measures_the_models_choice(tmp_path):
    np.random.seed(4)
    torch.manual_seed(4)
    measured = []

    def cost(task_key, cfg, op_pos, number):
        measured.append(1)
        return _cost(task_key, cfg, op_pos, number)

    s, bufs, configs = schedule(GEMM, op_trial=4, op_stop=4, graph_trial=1, parallel=4, method="searching",
                                evaluator=cost, warm_up=(2, 8), verbose=False, use_model=True,
                                perf_path=str(tmp_path))
    # the device (here: the cost function) is only asked for seeds and for the model's final candidates
    assert 0 < len(measured) <= 2 * (24 + 10)      # per level: heuristic seeds + the model's final ten
    assert math.isfinite(_cost(GEMM, configs, None, 1))


def test_schedule_method_q_on_the_four_operator_im2col_graph(tmp_path):
    """method="q" over [Padding, Img2Col, ComputeGemm, Col2Img]: only the GEMM
    has knobs, the graph level decides which stages exist as kernels (host
    cost: one unit per kernel plus the GEMM's synthetic cost)."""
    from flextensor_amd.scheduler import schedule_with_config
    np.random.seed(7)
    torch.manual_seed(7)
    key = "gemm_conv2d_yolo7_(1, 256, 28, 28, 512, 3, 1, 1, 1, 1)_rocm(0)"

    def cost(task_key, cfg, op_pos, number):
        plan = schedule_with_config(task_key, cfg, op_pos=op_pos)[0]
        d = [sp for sp in plan.specs if sp.kernel == "igemm_f32"][0].defines
        tile = d["WAVES_M"] * d["REP_M"] * d["WAVES_N"] * d["REP_N"] * d["MFMA"] ** 2
        return len(plan.specs) + abs(np.log2(tile / 8192.0)) + (0.0 if d["BK"] in (72, 144) else 0.5)

    s, bufs, configs = schedule(key, op_trial=6, op_stop=6, graph_trial=3, parallel=4, method="q", evaluator=cost,
                                warm_up=(1, 6), verbose=False, perf_path=str(tmp_path), trials=[1, 1, 6, 1],
                                warm_start=False)
    assert len(configs.op_config_lst) == 4 and configs.op_config_lst[2]["spatial"]
    assert [sp.kernel for sp in s.specs] == ["igemm_f32"]            # folded: fewest kernels wins
    assert configs.graph_config["inline"][0][:2] == [1, 1] and configs.graph_config["merge"][0][3] == 1
