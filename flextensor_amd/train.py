"""Offline training of the learned search aids from dumped search data.

Counterpart of the reference's flextensor/train.py: ``train_for_schedule``
(:27-62) rebuilds a task's spaces and trains the per-sub-space Q networks
(``train_q``) and the performance model (``train_perf``) from the files a
search with ``perf_path=<dir>`` left behind; ``train_performance_model``
(:123-295) fits the ranking network to a file of (points, costs) batches and
reports how well it orders held-out batches. The networks are small MLPs on
the CPU; nothing here touches the GPU.
"""
import copy
import json
import os

import numpy as np

from .model import WalkerGroup, make_performance_model, rank_loss, _torch
from .scheduler import flatten_graph, SUPPORTED_TARGETS
from .space import generate_space_inter_op, generate_space_intra_op
from .task import TASK_TABLE

INF_COST = 1000.0      # what a failed candidate counts as (train.py:115-116)


def train_perf(name, space, model_dir, epochs=20):
    """Train one group's performance model from its dumped batches (train.py:14-17)."""
    walker_group = WalkerGroup(name, space)
    walker_group.model_dir = model_dir
    walker_group.prepare_performance_data()
    return walker_group.train_on_perf(epochs=epochs)


def train_q(name, space, model_dir):
    """Train one group's Q networks from its dumped transitions (train.py:20-23)."""
    walker_group = WalkerGroup(name, space)
    walker_group.model_dir = model_dir
    walker_group.load_walker_data()
    walker_group.train_walkers()


def train_for_schedule(task_key, q=False, perf=False, perf_path=None, slevel=4, rlevel=3):
    """Train the search aids of every operator level and of the graph level of
    a task (train.py:27-62); group names are the ones ``schedule`` uses."""
    task = TASK_TABLE[task_key]
    if task.target not in SUPPORTED_TARGETS:
        raise RuntimeError("Currently no support for target %s" % task.target)
    if perf_path is None:
        raise ValueError("perf_path: the directory a search with perf_path=... wrote to")
    ops, _ = task.func(*task.args)
    op_lst, down_graph = flatten_graph(ops)
    out = {}
    for pos, op in enumerate(op_lst):
        space = generate_space_intra_op(op, down_graph, slevel=slevel, rlevel=rlevel, target=task.target)
        if space.dim == 0:
            continue                      # an operator without knobs (padding, layout stages)
        name = task.category + "_op" + str(pos)
        if q:
            train_q(name, space, perf_path)
        if perf:
            out[name] = train_perf(name, space, perf_path)
    graph_space = generate_space_inter_op(op_lst, down_graph, special_space=task.special_space)
    name = task.category + "_graph"
    if graph_space.dim > 0:
        if q:
            train_q(name, graph_space, perf_path)
        if perf:
            out[name] = train_perf(name, graph_space, perf_path)
    return out


def load_perf_data(data_path):
    """Batches ``(points, costs)`` of a dumped file; a failed candidate (null) is ``inf``."""
    dataset = []
    with open(data_path, "r") as fin:
        for line in fin:
            line = line.strip()
            if line:
                x, t = json.loads(line)
                dataset.append((x, [float("inf") if v is None else float(v) for v in t]))
    return dataset


def query_perf_data_info(dataset):
    """Length of a flattened point (train.py:80-88)."""
    for x, _ in dataset:
        if len(x) > 0:
            return len(x[0])
    raise RuntimeError("Dataset size <= 0")


def normalize_perf_data(dataset):
    """Flatten the batches to ``[point, cost]`` samples; failed candidates count
    as a large constant (train.py:91-120)."""
    data_lst = []
    for x, t in dataset:
        for point, cost in zip(x, t):
            data_lst.append([copy.deepcopy(point), INF_COST if cost == float("inf") else float(cost)])
    return data_lst


def pairwise_accuracy(model, dataset):
    """Fraction of pairs inside a batch that the model orders as the measured
    costs do (ties and failed candidates left out); 0.5 is chance."""
    torch = _torch()
    model.eval()
    good = total = 0
    with torch.no_grad():
        for x, t in dataset:
            keep = [i for i, v in enumerate(t) if v < float("inf")]
            if len(keep) < 2:
                continue
            y = model(torch.tensor([x[i] for i in keep], dtype=torch.float32)).reshape(-1).numpy()
            tt = np.array([t[i] for i in keep])
            dy = np.sign(y[:, None] - y[None, :])
            dt = np.sign(tt[:, None] - tt[None, :])
            mask = np.triu(dt != 0, 1)
            good += int(np.sum((dy == dt) & mask))
            total += int(np.sum(mask))
    model.train()
    return good / total if total else float("nan")


def train_performance_model(data_path, model_path, epoch=10, batch_size=1, lr=0.02, override=False,
                            train_ratio=0.8, loss="rank", verbose=False):
    """Fit the ranking network to a dumped file and test it on the held-out
    part (train.py:123-295). ``loss="mse"`` regresses the cost of single points
    as the reference's active code does; ``loss="rank"`` uses the pairwise
    ranking loss the search itself trains with (model.py:181-189), over the
    points of one measured batch. Returns the pairwise accuracies.
    """
    torch = _torch()
    if loss not in ("rank", "mse"):
        raise ValueError("loss is 'rank' or 'mse'")
    if os.path.exists(model_path) and not override and epoch > 0:
        raise RuntimeError("Existing model file %s" % model_path)
    batches = [b for b in load_perf_data(data_path) if len(b[0]) > 0]
    if not batches:
        raise RuntimeError("Dataset size <= 0")
    input_len = query_perf_data_info(batches)
    order = np.random.permutation(len(batches))
    n_train = max(1, int(train_ratio * len(batches)))
    train_b = [batches[i] for i in order[:n_train]]
    test_b = [batches[i] for i in order[n_train:]]
    model = make_performance_model(input_len)
    optimizer = torch.optim.Adadelta(model.parameters(), lr=lr)
    samples = normalize_perf_data(train_b)
    for ep in range(epoch):
        acc_loss = 0.0
        if loss == "mse":
            np.random.shuffle(samples)
            for i in range(0, len(samples), max(batch_size, 1)):
                chunk = samples[i:i + max(batch_size, 1)]
                ys = model(torch.tensor([c[0] for c in chunk], dtype=torch.float32)).reshape(-1)
                step = torch.nn.functional.mse_loss(ys, torch.tensor([c[1] for c in chunk], dtype=torch.float32))
                optimizer.zero_grad()
                step.backward()
                optimizer.step()
                acc_loss += float(step.detach())
        else:
            np.random.shuffle(train_b)
            for x, t in train_b:
                keep = [i for i, v in enumerate(t) if v < float("inf")]
                if len(keep) < 2:
                    continue
                ys = model(torch.tensor([x[i] for i in keep], dtype=torch.float32)).reshape(-1)
                step = rank_loss(ys, torch.tensor([t[i] for i in keep], dtype=torch.float32))
                optimizer.zero_grad()
                step.backward()
                optimizer.step()
                acc_loss += float(step.detach())
        if verbose:
            print("Epoch %d accumulated loss %f" % (ep + 1, acc_loss))
        torch.save(model.state_dict(), model_path)
    result = {"input_len": input_len, "train_batches": len(train_b), "test_batches": len(test_b),
              "train_accuracy": pairwise_accuracy(model, train_b),
              "test_accuracy": pairwise_accuracy(model, test_b) if test_b else float("nan")}
    if verbose:
        print("Pairwise accuracy: train %.3f, test %.3f" % (result["train_accuracy"], result["test_accuracy"]))
    return result


def main(argv=None):
    import argparse
    ap = argparse.ArgumentParser(description="train the learned search aids from a search's dumped data")
    ap.add_argument("--key", help="task key: train every group of this task from --perf_path")
    ap.add_argument("--perf_path", help="directory a search with perf_path / --perf_path wrote to")
    ap.add_argument("--q", action="store_true", help="train the Q networks of the walkers")
    ap.add_argument("--perf", action="store_true", help="train the performance models")
    ap.add_argument("--data", help="instead: one performance-data file to fit a ranking network to")
    ap.add_argument("--model", help="where --data's network is saved")
    ap.add_argument("--epoch", type=int, default=10)
    ap.add_argument("--lr", type=float, default=0.02)
    ap.add_argument("--loss", choices=["rank", "mse"], default="rank")
    ap.add_argument("--override", action="store_true")
    args = ap.parse_args(argv)
    if args.data:
        if not args.model:
            ap.error("--data needs --model")
        print(json.dumps(train_performance_model(args.data, args.model, epoch=args.epoch, lr=args.lr,
                                                 override=args.override, loss=args.loss, verbose=True)))
    elif args.key:
        print(json.dumps(train_for_schedule(args.key, q=args.q, perf=args.perf or not args.q,
                                            perf_path=args.perf_path)))
    else:
        ap.error("give --key (with --perf_path) or --data (with --model)")


if __name__ == "__main__":
    main()
