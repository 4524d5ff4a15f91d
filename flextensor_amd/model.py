"""Search memory: measured points, visited set, neighbour generation.

This is the part of the reference's flextensor/model.py that
``method="searching"`` and ``method="random"`` use (WalkerGroup :235-509):
a min-heap of (indices, value), the set of visited points, random batches
for warm-up (:251-260), ``record`` with Boltzmann random-reject (:265-276),
``top1 / topk / top_random / pop_top`` (:278-353), ``to_config`` (:293-300)
and ``full_walk`` (:375-390). The learned walkers (per-sub-space Q networks)
and the ranking network are not needed by those methods; transitions and
performance samples are still collected so that they can be dumped.
"""
import copy
import heapq
import json

import numpy as np

from .utils import assert_print


class MemEntity(object):
    """Heap item: a point (sub-space name -> entity index) and its cost in ms."""

    def __init__(self, indices, value):
        self.indices = indices
        self.value = value

    def __lt__(self, b):
        return self.value < b.value


class Walker(object):
    """Moves inside one sub-space."""

    def __init__(self, name, subspace, input_len):
        self.name = name
        self.subspace = subspace
        self.input_len = input_len
        self.memory = []  # (pre_state, action, post_state, reward)
        self.mem_size = 0

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
                t = np.exp(-gamma * (value - top) / top)
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
            t = np.exp(-gamma * (e.value - top) / top)
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

    # ---- data collected for learned methods ----------------------------
    def add_data(self, name, pre_state, action, post_state, reward):
        self.walkers[name].add_data(self.flatten(pre_state), action, self.flatten(post_state), reward)

    def add_perf_data(self, indices_lst, performance_lst):
        self.perfromance_data.append(([self.flatten(i) for i in indices_lst], list(performance_lst)))

    def dump_performance_data(self, data_path):
        with open(data_path, "a") as fout:
            for data in self.perfromance_data:
                fout.write(json.dumps(data, default=int) + "\n")

    def clear_data(self):
        self.perfromance_data.clear()
        for walker in self.walkers.values():
            walker.clear_data()
