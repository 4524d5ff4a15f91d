"""Search memory: measured points, visited set, neighbour generation.

This is the part of the reference's flextensor/model.py that
``method="searching"`` and ``method="random"`` use (WalkerGroup :235-509):
a min-heap of (indices, value), the set of visited points, random batches
for warm-up (:251-260), ``record`` with Boltzmann random-reject (:265-276),
``top1 / topk / top_random / pop_top`` (:278-353), ``to_config`` (:293-300)
and ``full_walk`` (:375-390).

``method="q"`` adds the learned part (model.py:20-190, 355-373, 392-456): one
Q network per sub-space that picks the direction of the next step
(epsilon-greedy, trained on (state, action, next state, reward) transitions
with a target network), and a ranking network over flattened points that can
stand in for the device (``use_model=True``). These are small host-side MLPs
on the CPU; torch is imported only when they are used, so the plain search
methods do not load it.
"""
import copy
import heapq
import json
import os

import numpy as np

from .utils import assert_print


class MemEntity(object):
    """Heap item: a point (sub-space name -> entity index) and its cost in ms."""

    def __init__(self, indices, value):
        self.indices = indices
        self.value = value

    def __lt__(self, b):
        return self.value < b.value


WALKER_MODEL_PREFIX = "walker_judger_model_"
WALKER_DATA_PREFIX = "walker_judger_data_"
PERF_MODEL_PREFIX = "performance_judger_model_"
PERF_DATA_PREFIX = "performance_judger_data_"


def _torch():
    import torch
    return torch


def make_judger(input_len, width, depth, output_len):
    """MLP input_len -> width x (depth-1) -> output_len with ReLU between
    (the reference's Judger, model.py:20-36)."""
    nn = _torch().nn
    assert_print(isinstance(width, int) and width > 0, "bad width")
    assert_print(isinstance(depth, int) and depth > 1, "bad depth")
    layers = [nn.Linear(input_len, width), nn.ReLU()]
    for _ in range(depth - 2):
        layers += [nn.Linear(width, width), nn.ReLU()]
    layers.append(nn.Linear(width, output_len))
    return nn.Sequential(*layers)


def make_performance_model(input_len):
    """Ranking network over flattened points (model.py:192-232):
    input -> 32 -> 64 -> 128 -> 64 -> 16 -> 1, ReLU everywhere, light dropout."""
    nn = _torch().nn
    return nn.Sequential(
        nn.Linear(input_len, 32), nn.Dropout(p=0.01), nn.ReLU(),
        nn.Linear(32, 64), nn.Dropout(p=0.01), nn.ReLU(),
        nn.Linear(64, 128), nn.Dropout(p=0.01), nn.ReLU(),
        nn.Linear(128, 64), nn.Dropout(p=0.01), nn.ReLU(),
        nn.Linear(64, 16), nn.ReLU(),
        nn.Linear(16, 1), nn.ReLU())


def rank_loss(y, t):
    """Pairwise logistic ranking loss (model.py:181-189), vectorised."""
    torch = _torch()
    dy = y.reshape(-1, 1) - y.reshape(1, -1)
    dt = torch.sign(t.reshape(-1, 1) - t.reshape(1, -1))
    return torch.log1p(torch.exp(-dt * dy)).sum()


class Walker(object):
    """Moves inside one sub-space; with ``enable_learning`` also a Q network
    over the flattened point that scores the sub-space's directions."""

    def __init__(self, name, subspace, input_len):
        self.name = name
        self.subspace = subspace
        self.input_len = input_len
        self.memory = []  # (pre_state, action, post_state, reward)
        self.mem_size = 0
        self.pre_judger = None
        self.post_judger = None
        self.model_path = WALKER_MODEL_PREFIX + name + ".pkl"
        self.data_path = WALKER_DATA_PREFIX + name + ".txt"

    # ---- learned direction choice ---------------------------------------
    def enable_learning(self):
        if self.pre_judger is None:
            self.pre_judger = make_judger(self.input_len, 64, 4, self.subspace.num_direction)
            self.post_judger = make_judger(self.input_len, 64, 4, self.subspace.num_direction)
            self.post_judger.load_state_dict(self.pre_judger.state_dict())

    def walk(self, inputs, index_lst, trial, epsilon, gamma):
        """One epsilon-greedy step per start point (model.py:73-90): with
        probability max(epsilon*exp(-trial*gamma), 0.1) a random direction,
        otherwise the direction with the largest Q value."""
        torch = _torch()
        self.enable_learning()
        with torch.no_grad():
            q_values_lst = self.pre_judger(torch.tensor(inputs, dtype=torch.float32).reshape(len(inputs), -1))
        ret_index_lst, ret_choice_lst = [], []
        for i, q_values in enumerate(q_values_lst):
            t = max(epsilon * np.exp(-trial * gamma), 0.1)
            if np.random.random() <= t:
                choice = np.random.randint(0, self.subspace.num_direction)
            else:
                choice = int(torch.argmax(q_values))
            direction = self.subspace.get_direction(choice)
            ret_index_lst.append(self.subspace.next_entity(index_lst[i], direction))
            ret_choice_lst.append(int(choice))
        return ret_index_lst, ret_choice_lst

    def train(self, lr=0.02, decay=0.9, epochs=20, batch=32, save_dir=None, verbose=False):
        """Q-learning on the stored transitions (model.py:104-129): target =
        reward + decay * max_a Q_target(next state), squared error, Adadelta;
        the target network is refreshed after every epoch."""
        torch = _torch()
        self.enable_learning()
        data_size = min(self.mem_size, 1000)
        if data_size == 0:
            return 0.0
        np.random.shuffle(self.memory)
        data = self.memory[:data_size]
        pre = torch.tensor([d[0] for d in data], dtype=torch.float32)
        act = torch.tensor([d[1] for d in data], dtype=torch.int64)
        post = torch.tensor([d[2] for d in data], dtype=torch.float32)
        rew = torch.tensor([d[3] for d in data], dtype=torch.float32)
        optimizer = torch.optim.Adadelta(self.pre_judger.parameters(), lr=lr)
        last = 0.0
        for ep in range(epochs):
            for lo in range(0, data_size, batch):
                sl = slice(lo, lo + batch)
                y = self.pre_judger(pre[sl]).gather(1, act[sl].reshape(-1, 1)).reshape(-1)
                with torch.no_grad():
                    target = self.post_judger(post[sl]).max(dim=-1)[0] * decay + rew[sl]
                loss = torch.pow(y - target, 2).sum()
                optimizer.zero_grad()
                loss.backward()
                optimizer.step()
                last = float(loss.detach())
            self.post_judger.load_state_dict(self.pre_judger.state_dict())
            if save_dir is not None:
                self.save_model(save_dir)
            if verbose:
                print("[cur/total]=[%d/%d] | loss=%f" % (ep + 1, epochs, last))
        return last

    def save_model(self, save_dir):
        torch = _torch()
        self.enable_learning()
        self.post_judger.load_state_dict(self.pre_judger.state_dict())
        torch.save(self.pre_judger.state_dict(), os.path.join(save_dir, self.model_path))

    def load_model(self, save_dir):
        torch = _torch()
        self.enable_learning()
        state = torch.load(os.path.join(save_dir, self.model_path), weights_only=True)
        self.pre_judger.load_state_dict(state)
        self.post_judger.load_state_dict(state)

    def load_or_create_model(self, save_dir):
        if os.path.exists(os.path.join(save_dir, self.model_path)):
            self.load_model(save_dir)
        else:
            self.save_model(save_dir)

    def dump_data(self, save_dir):
        with open(os.path.join(save_dir, self.data_path), "a") as fout:
            for data in self.memory:
                fout.write(json.dumps(data, default=float) + "\n")

    def load_data(self, save_dir):
        with open(os.path.join(save_dir, self.data_path), "r") as fin:
            for line in fin:
                self.memory.append(tuple(json.loads(line)))
                self.mem_size += 1

    def random_batch(self, batch_size):
        batch_indices = np.random.randint(0, self.subspace.size, batch_size)
        return [self.subspace.get_entity(i) for i in batch_indices], batch_indices

    def full_walk(self, index):
        """One step from ``index`` in every direction of the sub-space."""
        new_index_lst = [self.subspace.next_entity(index, d) for d in self.subspace.directions]
        return new_index_lst, copy.deepcopy(self.subspace.directions)

    def walk_random(self, index):
        choice = np.random.randint(0, self.subspace.num_direction)
        d = self.subspace.get_direction(choice)
        return self.subspace.next_entity(index, d), int(choice)

    def add_data(self, pre_state, action, post_state, reward):
        self.memory.append((pre_state, action, post_state, reward))
        self.mem_size += 1

    def clear_data(self):
        self.memory.clear()
        self.mem_size = 0


class WalkerGroup(object):
    def __init__(self, group_name, space, lr=0.02):
        self.group_name = group_name
        self.space = space
        self.lr = lr
        self.walkers = {}
        for name, subspace in self.space.items():
            self.walkers[name] = Walker(group_name + "_" + name, subspace, self.space.dim)
        self.memory = []
        self.mem_size = 0
        self.visit = set()
        self.perfromance_data = []
        self.performance_judger = None
        self.model_path = PERF_MODEL_PREFIX + group_name + ".pkl"
        self.data_path = PERF_DATA_PREFIX + group_name + ".txt"
        # directory for walker / performance model files; None = keep everything in memory
        self.model_dir = None

    # ---- sampling ------------------------------------------------------
    def forward(self, batch_size, policy="random"):
        assert_print(policy in ["random"], "only the random policy is available")
        ret = dict()
        for name, walker in self.walkers.items():
            ret[name] = walker.random_batch(batch_size)
        return ret

    # ---- memory --------------------------------------------------------
    def ever_met(self, indices):
        return str(indices) in self.visit

    def record(self, indices, value, random_reject=False, gamma=0.5):
        self.visit.add(str(indices))
        if random_reject:
            top = self.top1_value()
            if top < float("inf") and value < float("inf"):
                t = np.exp(-gamma * (value - top) / max(abs(top), 1e-12))
            elif value < float("inf"):
                t = 1.0
            else:
                t = 0.0
            if np.random.random() > t:
                return
        heapq.heappush(self.memory, MemEntity(indices, value))
        self.mem_size += 1

    def has_more(self):
        return self.mem_size > 0

    def flatten(self, indices):
        ret = []
        for name, index in indices.items():
            ret.extend(self.walkers[name].subspace.get_entity(index))
        return ret

    def to_config(self, indices):
        """Point -> config dict with every type key, entities in sub-space order."""
        ret = dict()
        for type_key, name_lst in self.space.types.items():
            ret[type_key] = []
            for name in name_lst:
                if name in indices:
                    ret[type_key].append(self.walkers[name].subspace.get_entity(indices[name]))
        return ret

    def top_random(self, gamma=0.5, with_value=False):
        e = self.memory[np.random.randint(0, len(self.memory))]
        top = self.top1_value()
        if e.value < float("inf") and top < float("inf"):
            t = np.exp(-gamma * (e.value - top) / max(abs(top), 1e-12))
        else:
            t = 0.0
        if np.random.random() <= t:
            return (e.indices, e.value) if with_value else e.indices
        return (self.top1(), self.top1_value()) if with_value else self.top1()

    def topk(self, k, modify=False, with_value=False):
        k = min(k, self.mem_size)
        ret = [heapq.heappop(self.memory) for _ in range(k)]
        self.mem_size -= k
        if not modify:
            for tmp in ret:
                heapq.heappush(self.memory, tmp)
            self.mem_size += k
        if with_value:
            return [(x.indices, x.value) for x in ret]
        return [x.indices for x in ret]

    def top1(self):
        return self.memory[0].indices if self.mem_size > 0 else {}

    def top1_value(self):
        return self.memory[0].value if self.mem_size > 0 else float("inf")

    def pop_top(self):
        if self.mem_size > 0:
            self.mem_size -= 1
            return heapq.heappop(self.memory)
        return MemEntity({}, float("inf"))

    # ---- neighbourhood -------------------------------------------------
    def full_walk(self, indices, no_repeat=True):
        next_indices_lst, action_lst = [], []
        for name, index in indices.items():
            next_index_lst, actions = self.walkers[name].full_walk(index)
            for next_index, action in zip(next_index_lst, actions):
                next_indices = copy.deepcopy(indices)
                next_indices[name] = next_index
                if no_repeat and self.ever_met(next_indices):
                    continue
                if no_repeat and any(str(next_indices) == str(x) for x in next_indices_lst):
                    continue
                next_indices_lst.append(next_indices)
                action_lst.append((name, action))
        return next_indices_lst, action_lst

    # ---- learned walk (method "q") ---------------------------------------
    def walk(self, indices_value_lst, trial, epsilon=0.8, gamma=0.01):
        """One learned step in every sub-space from every start point
        (model.py:355-373); returns (from, next, action) for the unvisited ones."""
        indices_lst = [x[0] for x in indices_value_lst]
        value_lst = [x[1] for x in indices_value_lst]
        flattened_lst = [self.flatten(indices) for indices in indices_lst]
        ret_from_lst, ret_indices_lst, ret_action_lst = [], [], []
        if not indices_lst:
            return ret_from_lst, ret_indices_lst, ret_action_lst
        for name in self.walkers.keys():
            index_lst = [indices[name] for indices in indices_lst]
            next_index_lst, direction_lst = self.walkers[name].walk(flattened_lst, index_lst, trial,
                                                                    epsilon, gamma)
            for i, indices in enumerate(indices_lst):
                next_indices = copy.deepcopy(indices)
                next_indices[name] = next_index_lst[i]
                if self.ever_met(next_indices) or any(str(next_indices) == str(x) for x in ret_indices_lst):
                    continue
                ret_from_lst.append((indices, value_lst[i]))
                ret_indices_lst.append(next_indices)
                ret_action_lst.append((name, direction_lst[i]))
        return ret_from_lst, ret_indices_lst, ret_action_lst

    def train_walkers(self, verbose=False):
        for walker in self.walkers.values():
            walker.train(lr=self.lr, save_dir=self.model_dir, verbose=verbose)

    def load_walker_model(self):
        for walker in self.walkers.values():
            walker.enable_learning()
            if self.model_dir is not None:
                walker.load_or_create_model(self.model_dir)

    def dump_data(self):
        """Append what the search measured to the files of ``model_dir``: the
        (points, costs) batches for the performance model and every walker's
        transitions (model.py:469-474); the offline trainer reads them back."""
        if self.model_dir is not None:
            self.dump_performance_data(os.path.join(self.model_dir, self.data_path))
            for walker in self.walkers.values():
                walker.dump_data(self.model_dir)

    def prepare_performance_data(self):
        """Load the dumped (points, costs) batches of this group (model.py:458-467)."""
        if self.model_dir is None:
            raise RuntimeError("no model directory to read performance data from")
        path = os.path.join(self.model_dir, self.data_path)
        if os.path.exists(path):
            self.load_performance_data(path)

    def load_walker_data(self):
        for walker in self.walkers.values():
            walker.enable_learning()
            if self.model_dir is not None and os.path.exists(os.path.join(self.model_dir, walker.data_path)):
                walker.load_data(self.model_dir)

    # ---- performance model (use_model=True) ------------------------------
    def _perf_model(self):
        if self.performance_judger is None:
            self.performance_judger = make_performance_model(self.space.dim)
        return self.performance_judger

    def load_or_create_model(self):
        torch = _torch()
        model = self._perf_model()
        if self.model_dir is None:
            return
        path = os.path.join(self.model_dir, self.model_path)
        if os.path.exists(path):
            model.load_state_dict(torch.load(path, weights_only=True))
        else:
            torch.save(model.state_dict(), path)

    def train_on_perf(self, epochs=20, batch=32, verbose=False):
        """Fit the ranking network to the measured batches (model.py:402-431)."""
        torch = _torch()
        model = self._perf_model()
        finite = []
        for x, t in self.perfromance_data:
            keep = [i for i, v in enumerate(t) if v < float("inf")]
            if len(keep) >= 2:
                finite.append(([x[i] for i in keep], [t[i] for i in keep]))
        data_size = min(len(finite), 1000)
        if data_size == 0:
            return 0.0
        np.random.shuffle(finite)
        optimizer = torch.optim.Adadelta(model.parameters(), lr=self.lr)
        full_loss = 0.0
        for ep in range(epochs):
            loss, full_loss = 0.0, 0.0
            for p_data in range(data_size):
                x, t = finite[p_data]
                y = model(torch.tensor(x, dtype=torch.float32)).reshape(-1)
                tmp_loss = rank_loss(y, torch.tensor(t, dtype=torch.float32))
                loss = loss + tmp_loss
                full_loss += float(tmp_loss.detach())
                if (p_data + 1) % batch == 0:
                    optimizer.zero_grad()
                    loss.backward()
                    optimizer.step()
                    loss = 0.0
            if not isinstance(loss, float):
                optimizer.zero_grad()
                loss.backward()
                optimizer.step()
            if verbose:
                print("[cur/total]=[%d/%d] | loss=%f" % (ep + 1, epochs, full_loss))
        if self.model_dir is not None:
            torch.save(model.state_dict(), os.path.join(self.model_dir, self.model_path))
        return full_loss / data_size

    def query_performance(self, indices_lst):
        """Predicted cost (a ranking score, not ms) per point (model.py:448-456)."""
        if not indices_lst:
            return []
        torch = _torch()
        model = self._perf_model()
        model.eval()
        with torch.no_grad():
            out = model(torch.tensor([self.flatten(i) for i in indices_lst], dtype=torch.float32))
        model.train()
        return out.reshape(-1).tolist()

    def load_performance_data(self, data_path):
        with open(data_path, "r") as fin:
            for line in fin:
                x, t = json.loads(line)
                self.perfromance_data.append((x, [float("inf") if v is None else v for v in t]))

    # ---- data collected for learned methods ----------------------------
    def add_data(self, name, pre_state, action, post_state, reward):
        self.walkers[name].add_data(self.flatten(pre_state), action, self.flatten(post_state), reward)

    def add_perf_data(self, indices_lst, performance_lst):
        self.perfromance_data.append(([self.flatten(i) for i in indices_lst], list(performance_lst)))

    def dump_performance_data(self, data_path):
        with open(data_path, "a") as fout:
            for data in self.perfromance_data:
                x, t = data
                t = [None if v == float("inf") else float(v) for v in t]
                fout.write(json.dumps((x, t), default=int) + "\n")

    def clear_data(self):
        self.perfromance_data.clear()
        for walker in self.walkers.values():
            walker.clear_data()
