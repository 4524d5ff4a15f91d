"""Search driver and config replay.

Keeps the reference's entry points and their signatures
(flextensor/scheduler.py): ``schedule`` (:969-1111), ``schedule_with_config``
(:1114-1130), ``schedule_with_config_ops`` (:1133-1186), ``Scheduler`` with
``_warm_up`` (:222-280), ``_random_schedule`` (:282-291) and
``_searching_schedule`` (:293-442), ``OpScheduler`` (:767-822),
``GraphScheduler`` (:863-920), ``flatten_graph`` (:36-55).

What differs underneath: a config is lowered to hand-written gfx950 kernels
(templates/gfx950.py) instead of TVM schedule primitives; candidates are
compiled by a pool of ``parallel`` host workers (hiprtc, no device) and then
checked and timed one at a time on the GPU in this process (measure.py).
"""
import math
import multiprocessing as mp
import time
from collections import deque
from concurrent.futures import ProcessPoolExecutor

import numpy as np

from .model import WalkerGroup
from .plan import KernelPlan
from .space import Space, generate_space_inter_op, generate_space_intra_op
from .task import TASK_TABLE
from .te import ComputeOp
from .templates import gfx950
from .utils import Config, assert_print

SUPPORTED_TARGETS = ("rocm",)


def flatten_graph(ops):
    """Compute ops in producer->consumer order plus tensor -> consumers map."""
    bfs_order = []
    down_graph = {}
    visited = set()
    q = deque()
    for op in ops:
        q.append(op)
        visited.add(op)
    while q:
        cur = q.popleft()
        if isinstance(cur, ComputeOp):
            bfs_order.append(cur)
        for t in cur.input_tensors:
            if t.op not in visited:
                visited.add(t.op)
                q.append(t.op)
            down_graph.setdefault(t, []).append(cur)
    return list(reversed(bfs_order)), down_graph


class OpState(object):
    def __init__(self):
        self.inline = False
        self.loop_lst = []
        self.loop_idx = []
        self.compute_at = False
        self.consumer_lst = []


def _empty_config():
    return {k: [] for k in Space.valid_type_keys}


# --------------------------------------------------------------------------
# parallel compilation of candidates (host only)
# --------------------------------------------------------------------------

def _compile_job(template, options, arch):
    """Worker: compile one kernel into the on-disk cache. Returns an error
    string or None. Runs in a spawned process that never touches the GPU."""
    try:
        from . import runtime as rt
        rt.compile_to_code(gfx950.template_source(template), options, arch)
        return None
    except Exception as e:  # noqa: BLE001
        return str(e)


class CompilePool(object):
    def __init__(self, workers):
        self.workers = max(int(workers), 1)
        self._pool = None

    def _ensure(self):
        if self._pool is None and self.workers > 1:
            self._pool = ProcessPoolExecutor(max_workers=self.workers,
                                             mp_context=mp.get_context("spawn"))

    def compile_plans(self, plans, timeout):
        """Compile all kernels of ``plans`` (None entries skipped). Returns one
        error string or None per plan."""
        from . import runtime as rt
        errors = [None] * len(plans)
        jobs = {}
        for i, plan in enumerate(plans):
            if plan is None:
                continue
            for spec in plan.specs:
                key = (spec.template, tuple(spec.options()))
                jobs.setdefault(key, []).append(i)
        if not jobs:
            return errors
        self._ensure()
        if self._pool is None:
            for key, owners in jobs.items():
                err = _compile_job(key[0], list(key[1]), rt.DEFAULT_ARCH)
                if err:
                    for i in owners:
                        errors[i] = err
            return errors
        futs = {}
        try:
            for key in jobs:
                futs[key] = self._pool.submit(_compile_job, key[0], list(key[1]), rt.DEFAULT_ARCH)
            deadline = time.time() + max(float(timeout), 1.0) * max(1, math.ceil(len(jobs) / self.workers))
            for key, fut in futs.items():
                try:
                    err = fut.result(timeout=max(deadline - time.time(), 0.5))
                except Exception as e:  # noqa: BLE001  (timeout or broken pool)
                    err = "compile failed: %r" % (e,)
                    if not fut.done():
                        self.close(kill=True)
                if err:
                    for i in jobs[key]:
                        errors[i] = err
        except Exception as e:  # noqa: BLE001
            self.close(kill=True)
            for key, owners in jobs.items():
                for i in owners:
                    errors[i] = errors[i] or "compile pool failed: %r" % (e,)
        return errors

    def close(self, kill=False):
        if self._pool is not None:
            try:
                if kill:
                    for p in list(getattr(self._pool, "_processes", {}).values()):
                        p.terminate()
                self._pool.shutdown(wait=not kill, cancel_futures=True)
            except Exception:  # noqa: BLE001
                pass
            self._pool = None


def build_and_eval_wrapper(lib, task_key, config, op_pos=None, rpc_info=None, rewrite=False,
                           number=1):
    from .measure import build_and_eval
    task = TASK_TABLE[task_key]
    s, bufs = schedule_with_config(task_key, config, op_pos=op_pos, rewrite=rewrite)
    return build_and_eval(lib, s, bufs, task.target, task.dev_id, rpc_info, number)


class _Plateau(object):
    """The searches' stopping rule: the best value has moved by less than 2 % for ``patience``
    looks in a row."""

    def __init__(self, value, patience):
        self.value, self.patience, self.count = value, patience, 0

    def stalled(self, value):
        if self.value < float("inf") and math.fabs(value - self.value) < 0.02 * self.value:
            self.count += 1
        else:
            self.value, self.count = value, 0
        return self.count >= self.patience


class _Shelf(object):
    """Points taken off a WalkerGroup's heap (local minima the walk should leave): the best of
    them is kept apart from the rest, as the reference's ``minimal`` / ``retired_indices`` pair."""

    def __init__(self):
        self.best, self.best_value, self.rest = {}, float("inf"), []

    def put(self, indices, value):
        if value < self.best_value:
            if self.best_value < float("inf"):
                self.rest.append((self.best, self.best_value))
            self.best, self.best_value = indices, value
        else:
            self.rest.append((indices, value))

    def best_with(self, group):
        """(indices, value) of the better of the heap's top and the shelf's best."""
        if group.top1_value() < self.best_value:
            return group.top1(), group.top1_value()
        return self.best, self.best_value

    def pour_into(self, group):
        """Everything goes back on the heap; the shelf is empty afterwards."""
        if self.best_value < float("inf"):
            group.record(self.best, self.best_value, random_reject=False)
        for indices, value in self.rest:
            group.record(indices, value, random_reject=False)
        self.__init__()


class Scheduler(object):
    def __init__(self, name, task_key, space, parallel=2, timeout=4.0, trial=100, number=1,
                 early_stop=30, rpc_info=None, rewrite=False, evaluator=None):
        self.task_key = task_key
        self.space = space
        self.parallel = max(parallel, 1)
        self.timeout = timeout
        self.trial = trial
        self.number = number
        self.early_stop = early_stop
        self.task = TASK_TABLE[self.task_key]
        self.walker_group = WalkerGroup(self.task.category + "_" + name, self.space)
        self.rpc_info = rpc_info
        self.rewrite = rewrite
        # evaluator(task_key, Config, op_pos, number) -> ms; None = measure on the GPU
        self.evaluator = evaluator

        self.warm_start = True      # seed the search with the shipped log's entry for the task
        self.resample_rounds = 8    # redraws of random points that the templates refuse
        self.seed_limit = 24        # heuristic points measured before the random warm-up
        self.re_evalutate_number = 10
        self.warm_up_epoch = 10     # x warm_up_number valid points (refused draws are redrawn)
        self.warm_up_number = 20
        self.verbose = True
        self._pool = None
        self.op_pos = None

    def _log(self, *args):
        if self.verbose:
            print(*args, flush=True)

    # ---- cost of a list of points: the device, or the ranking model -----
    def _cost(self, configs, indices_lst, use_model=False):
        """ms per point measured on the device, or (``use_model``) the ranking
        network's scores, which order points but are not times
        (flextensor/scheduler.py:239-243, 466-471)."""
        if use_model:
            return self.walker_group.query_performance(indices_lst)
        next_configs = [self.walker_group.to_config(indices) for indices in indices_lst]
        results = self.parallel_evaluate(configs, next_configs, number=self.number)
        self.walker_group.add_perf_data(indices_lst, results)
        return results

    def _finish_with_model(self, configs, use_model):
        """After a search driven by the ranking model, measure its best points
        on the device and keep the measured order, so that what is returned is
        a checked, timed kernel."""
        if not use_model:
            return
        indices_lst = self.walker_group.topk(self.re_evalutate_number, modify=True)
        self.walker_group.memory, self.walker_group.mem_size = [], 0
        results = self._cost(configs, indices_lst, use_model=False)
        self._log("measured after model search [ %s]" % "".join("%.6f " % r for r in results))
        for indices, result in zip(indices_lst, results):
            if result < float("inf"):
                self.walker_group.record(indices, result, random_reject=False)

    # ---- warm-up: random points ---------------------------------------
    def _warm_up(self, warm_up_epoches, warm_up_trials, configs, type_keys, max_repeat=20,
                 use_model=False):
        warm_up_enough = False
        count_repeat = 0
        old_timeout = self.timeout
        while not warm_up_enough:
            for ep in range(warm_up_epoches):
                warm_up_configs, warm_up_indices = [], []
                # Random points of the product space are mostly combinations the
                # templates refuse (the sub-spaces are independent, the constraints
                # are not): lowering is host-only and cheap, so refused points are
                # redrawn instead of spending a measurement slot on a certain inf.
                for attempt in range(self.resample_rounds):
                    need = warm_up_trials - len(warm_up_configs)
                    if need <= 0:
                        break
                    ret = self.walker_group.forward(need, policy="random")
                    last_round = attempt == self.resample_rounds - 1
                    for count in range(need):
                        config, indices = {}, {}
                        for type_key in type_keys:
                            config[type_key] = []
                            for name in self.space.types[type_key]:
                                indices[name] = int(ret[name][1][count])
                                config[type_key].append(ret[name][0][count])
                        if last_round or self._lowers(configs, config):
                            warm_up_configs.append(config)
                            warm_up_indices.append(indices)
                        else:
                            self.walker_group.visit.add(str(indices))
                warm_up_trials_now = len(warm_up_configs)
                # points already measured are not measured again
                fresh = [i for i in range(warm_up_trials_now)
                         if not self.walker_group.ever_met(warm_up_indices[i])]
                seen = set()
                uniq = []
                for i in fresh:
                    k = str(warm_up_indices[i])
                    if k not in seen:
                        seen.add(k)
                        uniq.append(i)
                results = self._cost(configs, [warm_up_indices[i] for i in uniq], use_model)
                self._log("warm up [%.6f] [ %s]" % (time.time(), "".join("%.6f " % r for r in results)))
                for i, res in zip(uniq, results):
                    if res < float("inf"):
                        self.walker_group.record(warm_up_indices[i], res)
                    else:
                        self.walker_group.visit.add(str(warm_up_indices[i]))
            if not self.walker_group.top1():
                self._log("Warning: No valid schedule found in warm up process, please use more trials")
                self._log("Now automatically use more trials, increase %d" % warm_up_trials)
                warm_up_epoches = 1
                count_repeat += 1
                self.timeout = min(2 * self.timeout, 40)
                if count_repeat >= max_repeat:
                    self._log("Fail to find valid schedule, too many errors")
                    warm_up_enough = True
            else:
                warm_up_enough = True
        self.timeout = old_timeout

    def _seed(self, configs, type_keys):
        """Measure known-good points first so that the walk starts from them:
        the template's default config and, when the task has one, the entry of
        the shipped tuned log (points that are not in the space are skipped)."""
        if self.op_pos is None:
            return
        ops, _ = self.task.func(*self.task.args)
        op = flatten_graph(ops)[0][self.op_pos]
        candidates = []
        # an operator the templates cannot seed (no admissible tile, a variant that is not built)
        # simply starts from random points; any other error is a bug in the templates and surfaces
        try:
            candidates.extend(gfx950.seed_configs(op, limit=self.seed_limit))
        except (gfx950.InvalidConfig, NotImplementedError):
            pass
        from .tuned import lookup
        shipped = lookup(self.task_key, similar=True) if self.warm_start else None
        if shipped is not None and self.op_pos < len(shipped.op_config_lst):
            candidates.append(shipped.op_config_lst[self.op_pos])
        points = []
        for cfg in candidates:
            indices = {}
            ok = True
            for type_key in type_keys:
                names = self.space.types[type_key]
                ents = cfg.get(type_key, []) if cfg else []
                if len(names) != len(ents):
                    ok = False
                    break
                for name, ent in zip(names, ents):
                    try:
                        indices[name] = self.space.subspaces[name].static_entities.index(list(ent))
                    except ValueError:
                        ok = False
                        break
                if not ok:
                    break
            if not ok or not indices or self.walker_group.ever_met(indices) \
                    or any(str(indices) == str(p) for p in points):
                continue
            if not self._lowers(configs, self.walker_group.to_config(indices)):
                self.walker_group.visit.add(str(indices))
                continue
            points.append(indices)
        if not points:
            return
        # one batch: the candidates compile side by side
        results = self.parallel_evaluate(configs, [self.walker_group.to_config(p) for p in points],
                                         number=self.number)
        self.walker_group.add_perf_data(points, results)
        self._log("seed [%.6f] [ %s]" % (time.time(), "".join("%.6f " % r for r in results)))
        for indices, res in zip(points, results):
            if res < float("inf"):
                self.walker_group.record(indices, res)
            else:
                self.walker_group.visit.add(str(indices))

    def _random_schedule(self, configs, type_keys, use_model=False):
        if use_model:
            self.walker_group.load_or_create_model()
        for trial in range(self.trial):
            self._warm_up(1, self.parallel, configs, type_keys, use_model=use_model)
        self._finish_with_model(configs, use_model)
        self.walker_group.dump_data()
        self.walker_group.clear_data()
        return self.walker_group.to_config(self.walker_group.top1())

    # ---- learned walk ---------------------------------------------------
    def _q_schedule(self, configs, type_keys, use_model=False):
        """Walk the space with one Q network per sub-space choosing directions
        (flextensor/scheduler.py:444-540): warm up with random points, then per
        trial take the best ``parallel`` points, step each of them once in every
        sub-space, measure, store the transitions with reward
        tanh(max(from - to, 0)), and train the walkers every trial/5 trials."""
        self.walker_group.load_walker_model()
        if use_model:
            self.walker_group.load_or_create_model()
        self._seed(configs, type_keys)
        self._warm_up(min(self.warm_up_epoch, 10), self.warm_up_number, configs, type_keys,
                      use_model=use_model)
        best = self.walker_group.top1()
        best_value = self.walker_group.top1_value()
        retired_indices = []
        plateau = _Plateau(best_value, self.early_stop)
        cur_lst = self.walker_group.topk(self.parallel, modify=True, with_value=True)
        part = math.ceil(self.trial / 5)
        for trial in range(self.trial):
            from_lst, next_points, action_lst = self.walker_group.walk(cur_lst, trial)
            results = self._cost(configs, next_points, use_model)
            self._log("walk [%.6f] [ %s]" % (time.time(), "".join("%.6f " % r for r in results)))
            for indices, action, (from_indices, from_value), result in zip(next_points, action_lst,
                                                                           from_lst, results):
                gain = from_value - result if result < float("inf") else 0.0
                if not use_model and from_value < float("inf"):
                    gain = gain / from_value * 10.0      # kernels run for microseconds: scale to the start point
                reward = float(np.tanh(max(gain, 0.0)))
                self.walker_group.add_data(action[0], from_indices, action[1], indices, reward)
                if result < float("inf"):
                    self.walker_group.record(indices, result, random_reject=True)
                else:
                    self.walker_group.visit.add(str(indices))
            if self.walker_group.top1_value() < best_value:
                best_value = self.walker_group.top1_value()
                best = self.walker_group.top1()
            for indices, value in cur_lst:
                if value < best_value:
                    best, best_value = indices, value
            self._log("No. %d | [%.6f] The best currently %.6f" % (trial, time.time(), best_value), best)
            if plateau.stalled(best_value):
                self._log("Early stop with value %f repeats %d times" % (plateau.value, plateau.count))
                break
            retired_indices.extend(cur_lst)
            if not self.walker_group.has_more():
                self._warm_up(1, self.parallel, configs, type_keys, use_model=use_model)
                if not self.walker_group.has_more():
                    self._log("No more points, end of scheduling")
                    break
            cur_lst = self.walker_group.topk(self.parallel, modify=True, with_value=True)
            if (trial + 1) % part == 0:
                self.walker_group.train_walkers()
                if not use_model:
                    # re-measure the leaders one after another
                    for indices, value in retired_indices[-self.parallel:] + cur_lst:
                        self.walker_group.record(indices, value, random_reject=False)
                    indices_lst = self.walker_group.topk(self.parallel, modify=True)
                    results = self._cost(configs, indices_lst, use_model=False)
                    self._log("re-evaluate [%.6f] [ %s]" % (time.time(), "".join("%.6f " % r for r in results)))
                    for indices, result in zip(indices_lst, results):
                        if result < float("inf"):
                            self.walker_group.record(indices, result, random_reject=False)
                    if indices_lst:
                        best, best_value = {}, float("inf")
                self._warm_up(1, self.parallel, configs, type_keys, use_model=use_model)
                if self.walker_group.top1_value() < best_value:
                    best_value = self.walker_group.top1_value()
                    best = self.walker_group.top1()
                cur_lst = self.walker_group.topk(self.parallel, modify=True, with_value=True)
        # everything still held outside the heap goes back before the final pick
        for indices, value in retired_indices + cur_lst:
            if value < float("inf"):
                self.walker_group.record(indices, value, random_reject=False)
        if best and best_value < float("inf"):
            self.walker_group.record(best, best_value, random_reject=False)
        self._finish_with_model(configs, use_model)
        self.walker_group.dump_data()
        self.walker_group.clear_data()
        return self.walker_group.to_config(self.walker_group.top1())

    # ---- neighbourhood search -----------------------------------------
    def _searching_schedule(self, configs, type_keys, use_model=False):
        """The reference's walk (flextensor/scheduler.py:321-442): start from a good point chosen
        at random, measure all its neighbours, take a point that none of them beats off the heap,
        re-measure the leaders every trial/20 trials, one random warm-up batch per trial; stop on
        a plateau of the best value or when no point has unvisited neighbours left."""
        group = self.walker_group
        if use_model:
            group.load_or_create_model()
        self._seed(configs, type_keys)
        self._warm_up(self.warm_up_epoch, self.warm_up_number, configs, type_keys, use_model=use_model)

        shelf = _Shelf()                       # local minima, off the heap so the walk leaves them
        plateau = _Plateau(group.top1_value(), self.early_stop)
        remeasure_every = math.ceil(self.trial / 20)
        barren = 0                             # trials in a row whose start point had no new neighbour
        for trial in range(self.trial):
            if not group.has_more():
                self._warm_up(1, self.parallel, configs, type_keys, use_model=use_model)
                continue
            start, start_value = group.top_random(with_value=True)
            neighbours, moves = group.full_walk(start, no_repeat=True)
            barren = barren + 1 if not neighbours else 0
            costs = self._cost(configs, neighbours, use_model)
            self._log("tune [%.6f] [ %s]" % (time.time(), "".join("%.6f " % c for c in costs)))
            beaten = False
            for point, (name, direction), cost in zip(neighbours, moves, costs):
                reward = np.tanh(max(start_value - cost, 0.0))
                group.add_data(name, start, direction, point, reward)
                group.record(point, cost, random_reject=True)
                beaten = beaten or cost < group.top1_value()
            if not beaten or barren:
                top = group.pop_top()
                shelf.put(top.indices, top.value)
            leader, leader_value = shelf.best_with(group)
            self._log("No. %d | [%.6f] The best currently %.6f" % (trial, time.time(), leader_value), leader)
            if barren >= self.early_stop:
                self._log("Early stop after continuous no trials %d times" % barren)
                break
            # "no progress" = the best moved by less than 2 % (the reference uses
            # an absolute 0.02 ms, which every microsecond-scale kernel satisfies)
            if plateau.stalled(leader_value):
                self._log("Early stop with value %f repeats %d times" % (plateau.value, plateau.count))
                break
            if (trial + 1) % remeasure_every == 0:
                # everything goes back on the heap, and its top points are measured again
                shelf.pour_into(group)
                again = group.topk(self.re_evalutate_number, modify=True)
                costs = self._cost(configs, again, use_model)
                self._log("re-evaluate [%.6f] [ %s]" % (time.time(), "".join("%.6f " % c for c in costs)))
                for point, cost in zip(again, costs):
                    if cost < float("inf"):
                        group.record(point, cost, random_reject=False)
                group.dump_data()             # keep what was measured for the offline trainer
                group.clear_data()
            self._warm_up(1, self.parallel, configs, type_keys, use_model=use_model)
        group.dump_data()
        group.clear_data()
        if use_model:
            shelf.pour_into(group)
            self._finish_with_model(configs, use_model)
            return group.to_config(group.top1())
        return group.to_config(shelf.best_with(group)[0])

    def _lowers(self, old_configs, config):
        """True when the templates accept ``config`` in the context of ``old_configs``."""
        mode = "op" if self.op_pos is not None else "graph"
        try:
            cfg, op_pos = self._fetch_config(old_configs, config, mode)
            schedule_with_config(self.task_key, cfg, op_pos=op_pos, rewrite=self.rewrite)
            return True
        except (gfx950.InvalidConfig, NotImplementedError):
            return False          # a point the templates refuse; anything else is a template bug and surfaces

    # ---- evaluation ----------------------------------------------------
    def _fetch_config(self, old_configs, config, mode):
        if mode == "op":
            return Config(old_configs.op_config_lst + [config], old_configs.graph_config), self.op_pos
        if mode == "graph":
            return Config(old_configs.op_config_lst, config), None
        raise RuntimeError("Unknown mode %s" % mode)

    def _parallel_evaluate(self, old_configs, new_configs, mode="op", number=1):
        """One cost in ms per new config; any failure is ``inf``."""
        if not new_configs:
            return []
        built = [self._fetch_config(old_configs, c, mode) for c in new_configs]
        if self.evaluator is not None:
            res = []
            for cfg, op_pos in built:
                try:
                    res.append(float(self.evaluator(self.task_key, cfg, op_pos, number)))
                except Exception:  # noqa: BLE001
                    res.append(float("inf"))
            return res
        from .measure import get_measurer
        plans = []
        for cfg, op_pos in built:
            try:
                s, _ = schedule_with_config(self.task_key, cfg, op_pos=op_pos, rewrite=self.rewrite)
                plans.append(s)
            except (gfx950.InvalidConfig, NotImplementedError):
                plans.append(None)        # a point the templates refuse costs inf, as a failed build does
        if self._pool is None or self._pool.workers != self.parallel:
            if self._pool is not None:
                self._pool.close()
            self._pool = CompilePool(self.parallel)
        errors = self._pool.compile_plans(plans, self.timeout)
        res = []
        measurer = None
        for plan, err in zip(plans, errors):
            if plan is None or err is not None:
                res.append(float("inf"))
                continue
            try:
                if measurer is None:
                    measurer = get_measurer(self.task_key)
                # the per-candidate time limit of the reference (timeout -> inf, scheduler.py:742-748):
                # the device wait has a deadline; nothing is killed and no process is re-executed
                res.append(float(measurer.evaluate(plan, number=number, timeout=self.timeout)))
            except Exception:  # noqa: BLE001  (a failing candidate never propagates)
                res.append(float("inf"))
        return res

    def close(self):
        if self._pool is not None:
            self._pool.close()
            self._pool = None


class OpScheduler(Scheduler):
    def __init__(self, task_key, op_pos, space, decay=0.7, parallel=1, timeout=4.0, trial=100,
                 number=1, early_stop=30, rpc_info=None, rewrite=False, evaluator=None):
        super(OpScheduler, self).__init__("op" + str(op_pos), task_key, space, parallel, timeout,
                                          trial, number, early_stop, rpc_info, rewrite=rewrite,
                                          evaluator=evaluator)
        self.op_pos = op_pos

    def schedule(self, configs, method="searching", use_model=False, perf_path=None):
        wanted_types = ["fuse", "reorder", "spatial", "reduce", "unroll"]
        if perf_path is not None:
            self.walker_group.model_dir = perf_path
        if method == "searching":
            return self._searching_schedule(configs, wanted_types, use_model=use_model)
        elif method == "random":
            return self._random_schedule(configs, wanted_types, use_model=use_model)
        elif method == "q":
            return self._q_schedule(configs, wanted_types, use_model=use_model)
        else:
            raise RuntimeError("Currently no support for method %s" % method)

    def parallel_evaluate(self, configs, next_op_configs, number=1, rpc_info=None):
        return self._parallel_evaluate(configs, next_op_configs, mode="op", number=number)

    @staticmethod
    def generate_op_schedule(target, config):
        """Return ``template(op, special, out_name, in_names, materialized_pad)``
        -> list of KernelSpec for this target."""
        if target == "rocm":
            def template(op, special, out_name, in_names, materialized_pad=False, bias_name=None,
                         through=(), merged_out=None):
                return gfx950.lower(op, config, special, out_name, in_names, materialized_pad, bias_name,
                                    through=through, merged_out=merged_out)
            return template
        raise RuntimeError("Currently no support for target %s" % target)


class GraphScheduler(Scheduler):
    def __init__(self, task_key, space, decay=0.7, parallel=10, timeout=4.0, trial=100, number=1,
                 early_stop=30, rpc_info=None, rewrite=False, evaluator=None):
        super(GraphScheduler, self).__init__("graph", task_key, space, parallel, timeout, trial,
                                             number, early_stop, rpc_info, rewrite=rewrite,
                                             evaluator=evaluator)

    def schedule(self, configs, method="searching", use_model=False, perf_path=None):
        types = ["inline", "merge", "special"]
        if perf_path is not None:
            self.walker_group.model_dir = perf_path
        if method == "searching":
            return self._searching_schedule(configs, types, use_model=use_model)
        elif method == "random":
            return self._random_schedule(configs, types, use_model=use_model)
        elif method == "q":
            return self._q_schedule(configs, types, use_model=use_model)
        else:
            raise RuntimeError("Currently no support for method %s" % method)

    def parallel_evaluate(self, configs, graph_configs, number=1):
        return self._parallel_evaluate(configs, graph_configs, mode="graph", number=number)


# --------------------------------------------------------------------------
# entry points
# --------------------------------------------------------------------------

def _op_states(op_lst, down_graph):
    states = [OpState() for _ in op_lst]
    for i, op in enumerate(op_lst):
        consumers = []
        for k in range(op.num_outputs):
            if op.output(k) in down_graph:
                consumers.extend(down_graph[op.output(k)])
        states[i].consumer_lst = list(set(consumers))
    return states


def schedule(task_key, slevel=4, rlevel=3, op_trial=50, graph_trial=10, op_stop=15, graph_stop=5,
             number=1, timeout=5, parallel=8, method="searching", **kwargs):
    """Tune a registered task; returns ``(s, bufs, configs)``.

    Keyword extras understood (flextensor/scheduler.py:990-1014): ``trials``
    (per-op trial counts), ``force_inline``, ``rpc_info`` (must not request a
    remote session), ``use_model`` (rank candidates with the learned
    performance model instead of the device; the model's best points are
    measured at the end), ``perf_path`` (directory of the walker / performance
    model files; nothing is written without it). Additional: ``evaluator``
    (a cost function used instead of the GPU, for host-only tests),
    ``warm_up`` = (epochs, points per epoch), ``verbose``, ``warm_start``
    (default true: start from the shipped log's entry for this task, if any).
    ``method``: "searching", "random" or "q" (learned walkers).
    """
    task = TASK_TABLE[task_key]
    if task.target not in SUPPORTED_TARGETS:
        raise RuntimeError("Currently no support for target %s" % task.target)
    if method not in ("searching", "random", "q"):
        raise RuntimeError("Currently no support for method %s" % method)
    ops, bufs = task.func(*task.args)
    op_lst, down_graph = flatten_graph(ops)
    _op_states(op_lst, down_graph)

    if "trials" in kwargs:
        assert_print(len(kwargs["trials"]) == len(op_lst), str(len(op_lst)))
        force_trials = kwargs["trials"]
    else:
        force_trials = [op_trial for _ in op_lst]
    use_model = bool(kwargs.get("use_model", False))
    perf_path = kwargs.get("perf_path")
    force_inline = bool(kwargs.get("force_inline", False))
    rpc_info = kwargs.get("rpc_info")
    if rpc_info is not None and getattr(rpc_info, "use_rpc", None):
        raise RuntimeError("remote measurement is not supported by the gfx950 backend")
    evaluator = kwargs.get("evaluator")
    warm_up = kwargs.get("warm_up")
    verbose = kwargs.get("verbose", True)

    graph_space = generate_space_inter_op(op_lst, down_graph, force_inline=force_inline,
                                          special_space=task.special_space)
    if verbose:
        print("graph space size", len(graph_space))
    total_size = len(graph_space)

    if force_inline:
        configs = Config([], {"inline": [graph_space.subspaces["inline"].static_entities[0]]})
    else:
        configs = Config([], None)
        # Operators are searched before the graph level, i.e. under the graph
        # level's defaults. When the shipped log knows this task, its graph
        # config (inline flags, special knobs) is the context instead, so that
        # the shipped point keeps its measured cost when it seeds the search.
        if kwargs.get("warm_start", True):
            from .tuned import lookup
            shipped = lookup(task_key, similar=True)
            if shipped is not None and shipped.graph_config:
                # an entry written before a knob existed leaves it out: it takes the knob's default
                graph = dict(shipped.graph_config)
                have = list(graph.get("special") or [])
                names = list(task.special_space)
                if len(have) <= len(names) and all(n in gfx950.SPECIAL_DEFAULTS for n in names[len(have):]):
                    graph["special"] = have + [list(gfx950.SPECIAL_DEFAULTS[n]) for n in names[len(have):]]
                    configs = Config([], graph)

    schedulers = []
    try:
        for pos, op in enumerate(op_lst):
            space = generate_space_intra_op(op, down_graph, slevel=slevel, rlevel=rlevel,
                                            target=task.target)
            total_size *= max(len(space), 1)
            if verbose:
                print("op", pos, "space size:", len(space))
            if len(space.subspaces) == 0 or \
                    (force_inline and graph_space.subspaces["inline"].able_inline(pos)):
                # nothing to decide for this op (e.g. padding, which has no knobs)
                configs.op_config_lst.append(_empty_config() if len(space.subspaces) == 0 else {})
                continue
            op_scheduler = OpScheduler(task_key, pos, space, parallel=parallel, timeout=timeout,
                                       trial=force_trials[pos], number=number, early_stop=op_stop,
                                       rpc_info=rpc_info, evaluator=evaluator)
            op_scheduler.verbose = verbose
            op_scheduler.warm_start = bool(kwargs.get("warm_start", True))
            if warm_up:
                op_scheduler.warm_up_epoch, op_scheduler.warm_up_number = warm_up
            schedulers.append(op_scheduler)
            op_config = op_scheduler.schedule(configs, method=method, use_model=use_model,
                                              perf_path=perf_path)
            configs.op_config_lst.append(op_config)
            # its compile workers go before the next scheduler starts its own: the workers load the
            # HIP runtime, and a machine may bound the number of processes that do
            op_scheduler.close()

        if verbose:
            print("space size", total_size)

        graph_scheduler = GraphScheduler(task_key, graph_space, parallel=parallel, timeout=timeout,
                                         trial=graph_trial, number=number, early_stop=graph_stop,
                                         rpc_info=rpc_info, evaluator=evaluator)
        graph_scheduler.verbose = verbose
        if warm_up:
            graph_scheduler.warm_up_epoch, graph_scheduler.warm_up_number = warm_up
        else:
            # the graph space is tiny (inline flags x a few enumerated knobs)
            graph_scheduler.warm_up_epoch = 2
            graph_scheduler.warm_up_number = min(20, max(len(graph_space), 1))
        schedulers.append(graph_scheduler)
        graph_config = graph_scheduler.schedule(configs, method=method, use_model=use_model,
                                                perf_path=perf_path)
        configs = Config(configs.op_config_lst, graph_config)
    finally:
        for sch in schedulers:
            sch.close()

    s, bufs = schedule_with_config(task_key, configs)
    return s, bufs, configs


def schedule_with_config(task_key, configs, op_pos=None, rewrite=False):
    """Replay ``configs`` for a registered task; returns ``(s, bufs)`` where
    ``s`` is a KernelPlan (``s.build()`` gives the callable)."""
    task = TASK_TABLE[task_key]
    if rewrite:
        raise RuntimeError("the NCHWc rewrite is a CPU-only path of the reference")
    if task.target not in SUPPORTED_TARGETS:
        raise RuntimeError("Currently no support for target %s" % task.target)
    ops, bufs = task.func(*task.args)
    s, bufs = schedule_with_config_ops(ops, bufs, configs, op_pos=op_pos, target=task.target,
                                       task_key=task_key, special_names=list(task.special_space))
    return s, bufs


def schedule_with_config_ops(ops, bufs, configs, op_pos=None, target="rocm", task_key=None,
                             special_names=None):
    """Lower an operator graph with given configs to a KernelPlan."""
    if target not in SUPPORTED_TARGETS:
        raise RuntimeError("Currently no support for target %s" % target)
    if not isinstance(configs, Config):
        configs = Config(configs[0], configs[1])
    op_lst, down_graph = flatten_graph(ops)
    op_states = _op_states(op_lst, down_graph)
    op_config_lst = list(configs.op_config_lst)
    if op_pos is not None:
        assert_print(isinstance(op_pos, int), "op_pos should be int")
        assert_print(op_pos < len(op_lst) and op_pos < len(op_config_lst), "op_pos too big")
    else:
        assert_print(len(op_config_lst) <= len(op_lst), "config length exceed op_lst")

    # ---- graph level: which ops are folded into their consumer ----------
    graph_config = configs.graph_config
    inline_flags = None
    if graph_config is not None and graph_config.get("inline"):
        inline_flags = list(graph_config["inline"][0])
    from .space import able_inline
    for i, op in enumerate(op_lst):
        if inline_flags is not None:
            op_states[i].inline = bool(inline_flags[i]) if i < len(inline_flags) else False
        else:
            op_states[i].inline = able_inline(op, down_graph)  # default: fold padding in
        if op_states[i].inline and not able_inline(op, down_graph):
            raise gfx950.InvalidConfig("op %d cannot be inlined" % i)
    special = None
    if graph_config is not None and graph_config.get("special") and special_names:
        special = dict(zip(special_names, graph_config["special"]))
    # ---- graph level: bias stages merged into the producing convolution ---
    from .space import able_merge
    merge_flags = None
    if graph_config is not None and graph_config.get("merge"):
        merge_flags = list(graph_config["merge"][0])
    merged = set()            # stages that run inside their producer's kernel
    for i, op in enumerate(op_lst):
        can = able_merge(op, down_graph)
        want = can if merge_flags is None else (bool(merge_flags[i]) if i < len(merge_flags) else False)
        if want and not can:
            raise gfx950.InvalidConfig("op %d cannot be merged into its producer" % i)
        if want:
            merged.add(i)
    for i in merged:
        # a stage merges into a kernel: a merged stage behind an unmerged one has none
        src = op_lst.index(op_lst[i].input_tensors[0].op)
        if op_lst[src].kind in ("bias_add_nchw", "bias_add_ghw") and src not in merged:
            raise gfx950.InvalidConfig("op %d follows a stage that is not merged" % i)

    # ---- name the buffers ------------------------------------------------
    names = {}
    for i, t in enumerate(bufs[:-1]):
        names[t] = "in%d" % i
    names[bufs[-1]] = "out"
    intermediates = {}
    specs = []
    for i, op in enumerate(op_lst):
        if op_states[i].inline or i in merged:
            continue
        out_t = op.output(0)
        bias_name = None
        merged_out = None
        while True:
            # follow the chain of merged stages: the kernel writes the last one's output
            users = list(down_graph.get(out_t, []))
            if len(users) != 1 or op_lst.index(users[0]) not in merged:
                break
            stage = users[0]
            if stage.kind in ("bias_add_nchw", "bias_add_ghw"):
                bias_name = names[stage.input_tensors[1]]
            else:
                merged_out = stage.kind
            out_t = stage.output(0)
        if out_t not in names:
            names[out_t] = "tmp%d" % i
            intermediates[names[out_t]] = (out_t.shape, out_t.dtype)
        in_names = []
        materialized_pad = False
        through = []
        for t in op.input_tensors:
            src = t
            # an inlined producer is read through: the consumer sees its input
            while isinstance(src.op, ComputeOp) and op_states[op_lst.index(src.op)].inline:
                through.append(src.op.kind)
                src = src.op.input_tensors[0]
            if isinstance(src.op, ComputeOp) and src.op.kind == "zero_pad2d":
                materialized_pad = True
            in_names.append(names[src])
        config = op_config_lst[i] if i < len(op_config_lst) and op_config_lst[i] else None
        if config is None or not any(config.get(k) for k in ("spatial", "reduce", "fuse")):
            config = gfx950.default_config(op)
        template = OpScheduler.generate_op_schedule(target, config)
        specs.extend(template(op, special, names[out_t], in_names, materialized_pad, bias_name,
                              through=tuple(through), merged_out=merged_out))
    return KernelPlan(task_key, bufs, specs, intermediates, configs), bufs


def schedule_ops_with_config(s, op_lst, configs, target):
    """Schedule an already flattened operator list with given configs
    (flextensor/scheduler.py:1189-1220): ``op_lst`` is in producer -> consumer
    order and ``configs.op_config_lst[i]`` belongs to ``op_lst[i]``. The
    reference mutates the TVM schedule ``s`` and returns it; here ``s`` is a
    KernelPlan to refill (or None) and the lowered plan is returned. The
    plan's buffers are the graph's placeholders in order of first use, then
    the output of the last operator."""
    if target not in SUPPORTED_TARGETS:
        raise RuntimeError("Currently no support for target %s" % target)
    op_lst = list(op_lst)
    if not op_lst:
        raise ValueError("empty operator list")
    consumed = set()
    for op in op_lst:
        for t in op.input_tensors:
            consumed.add(t.op)
    outputs = [op for op in op_lst if op not in consumed]
    if len(outputs) != 1:
        raise ValueError("expected one output operator, found %d" % len(outputs))
    order, _ = flatten_graph(outputs)
    if order != op_lst:
        raise ValueError("op_lst is not the flattened graph of its output operator "
                         "(configs are matched to operators by position)")
    inputs = []
    for op in op_lst:
        for t in op.input_tensors:
            if not isinstance(t.op, ComputeOp) and t not in inputs:
                inputs.append(t)
    bufs = inputs + [outputs[0].output(0)]
    plan, _ = schedule_with_config_ops(outputs, bufs, configs, target=target,
                                       task_key=getattr(s, "task_key", None))
    if isinstance(s, KernelPlan):
        s.__dict__.update(plan.__dict__)
        return s
    return plan
