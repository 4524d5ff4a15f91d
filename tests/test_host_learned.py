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


def _dump_random_batches(path, space, nbatch, per_batch, seed):
    """A performance-data file as a search leaves it: batches of flattened points with their costs."""
    rng = np.random.RandomState(seed)
    wg = WalkerGroup("gemm_op0", space)
    for _ in range(nbatch):
        pts, costs = [], []
        while len(pts) < per_batch:
            indices = {name: int(rng.randint(sub.size)) for name, sub in space.items()}
            cfg = wg.to_config(indices)
            try:
                cost = _cost(GEMM, Config([cfg], None), 0, 1)
            except Exception:  # noqa: BLE001  (a point the templates refuse: redrawn, as the warm-up does)
                if rng.rand() < 0.02:
                    cost = float("inf")         # a few failed candidates stay in, as in a real dump
                else:
                    continue
            costs.append(cost)
            pts.append(indices)
        wg.add_perf_data(pts, costs)
    wg.dump_performance_data(path)
    return wg


def test_offline_trainer_ranks_a_held_out_dump_better_than_chance(tmp_path):
    """flextensor/train.py:123-295: a model trained on one dump of measured batches orders the
    points of another dump of the same task (other random points) clearly better than chance."""
    from flextensor_amd import train
    np.random.seed(11)
    torch.manual_seed(11)
    space = _space()
    train_file, held_out = str(tmp_path / "train.txt"), str(tmp_path / "held_out.txt")
    _dump_random_batches(train_file, space, nbatch=60, per_batch=8, seed=1)
    _dump_random_batches(held_out, space, nbatch=25, per_batch=8, seed=2)
    data = train.load_perf_data(train_file)
    assert len(data) == 60 and train.query_perf_data_info(data) == space.dim
    flat = train.normalize_perf_data(data)
    assert len(flat) == 480 and all(c == train.INF_COST or c < 100 for _, c in flat)
    model_path = str(tmp_path / "perf.pkl")
    res = train.train_performance_model(train_file, model_path, epoch=12, lr=0.5, override=True)
    assert os.path.exists(model_path) and res["input_len"] == space.dim
    with pytest.raises(RuntimeError):
        train.train_performance_model(train_file, model_path, epoch=1)          # no silent overwrite
    from flextensor_amd.model import make_performance_model
    model = make_performance_model(space.dim)
    model.load_state_dict(torch.load(model_path, weights_only=True))
    acc = train.pairwise_accuracy(model, train.load_perf_data(held_out))
    untrained = train.pairwise_accuracy(make_performance_model(space.dim), train.load_perf_data(held_out))
    assert acc > 0.62 and acc > untrained + 0.05, (acc, untrained)
    # the reference's active loss (regression of single points) trains as well
    res = train.train_performance_model(train_file, model_path, epoch=2, lr=0.5, override=True, loss="mse", batch_size=16)
    assert 0.0 <= res["test_accuracy"] <= 1.0


def test_search_dumps_its_measurements_and_train_for_schedule_reads_them(tmp_path):
    """schedule(perf_path=dir) leaves the measured batches and the walkers' transitions in dir;
    train_for_schedule (flextensor/train.py:27-62) trains every group from them; a later search
    with use_model=True picks the trained ranking network up."""
    from flextensor_amd import train
    np.random.seed(5)
    torch.manual_seed(5)
    d = str(tmp_path)
    schedule(GEMM, op_trial=6, op_stop=6, graph_trial=2, parallel=4, method="q", evaluator=_cost,
             warm_up=(2, 8), verbose=False, perf_path=d, warm_start=False)
    files = os.listdir(d)
    assert "performance_judger_data_gemm_op0.txt" in files and any(f.startswith("walker_judger_data_") for f in files)
    batches = train.load_perf_data(os.path.join(d, "performance_judger_data_gemm_op0.txt"))
    assert sum(len(t) for _, t in batches) >= 16
    losses = train.train_for_schedule(GEMM, q=True, perf=True, perf_path=d)
    assert "gemm_op0" in losses and math.isfinite(losses["gemm_op0"])
    assert "performance_judger_model_gemm_op0.pkl" in os.listdir(d)
    before = os.path.getmtime(os.path.join(d, "performance_judger_model_gemm_op0.pkl"))
    s, bufs, configs = schedule(GEMM, op_trial=3, op_stop=3, graph_trial=1, parallel=4, method="searching",
                                evaluator=_cost, warm_up=(1, 8), verbose=False, use_model=True, perf_path=d)
    assert os.path.getmtime(os.path.join(d, "performance_judger_model_gemm_op0.pkl")) == before    # loaded, not recreated
    assert math.isfinite(_cost(GEMM, configs, None, 1))
    with pytest.raises(ValueError):
        train.train_for_schedule(GEMM, perf=True)
