"""Refine the entries of a tuned log one knob at a time, on the device.

    python -m flextensor_amd.optimize.polish --log tuned.log --out refined.log

A search ends at a point of a large space after a bounded number of trials; kernels change
afterwards (a cheaper set-up shifts the balance between LDS layouts, for one). This pass takes
every ``key:json`` line of a log, measures it, and tries the neighbours along the knobs that
cost nothing to enumerate: the task's enumerated knobs (the LDS layout `lds_pad`, the int8 store
forms, the depthwise variants), the number of k blocks the next tile's loads are spread over
(depth 8), the traversal group height and the XCD renumbering, for depthwise the wavefronts per
workgroup. A
neighbour replaces the entry when it is faster by more than ``--threshold`` (default 1 %) in a
first measurement and then in every one of four rounds that alternate between it and the
then-current entry (kernels near the launch floor time bimodally; a single pair of
measurements lets noise through); every
measurement passes the on-device correctness gate. Lines of tasks that are not registered are
copied as they are.
"""
import argparse
import json
import sys

from ..measure import get_measurer
from ..scheduler import schedule_with_config
from ..task import TASK_TABLE
from ..templates import gfx950
from ..utils import Config


ROUNDS = 4          # alternating confirmations a neighbour has to win, all of them


def _time(measurer, plan, number):
    return min(measurer.evaluate(plan, number=number) for _ in range(2))


def neighbours(key, cfg):
    """[(what, Config)] one knob away from ``cfg``."""
    out = []
    task = TASK_TABLE[key]
    # the task's enumerated knobs (LDS layout, store forms, the depthwise variants): every other value
    names = list(task.special_space)
    special = [list(x) for x in (cfg.graph_config.get("special") or [])]
    while len(special) < len(names):
        special.append(list(gfx950.SPECIAL_DEFAULTS[names[len(special)]]))
    for at, name in enumerate(names):
        for value in task.special_space[name].static_entities:
            if list(value) != special[at]:
                s2 = [list(x) for x in special]
                s2[at] = list(value)
                out.append(("%s %s" % (name, list(value)), Config(cfg.op_config_lst, dict(cfg.graph_config, special=s2))))
    pos = [i for i, c in enumerate(cfg.op_config_lst) if c.get("spatial")]
    if not pos:
        return out
    pos = pos[0]
    op = cfg.op_config_lst[pos]
    if len(op["spatial"]) == 4:          # depthwise: wavefronts per workgroup
        waves = (op.get("fuse") or [[4]])[0][0]
        for x in (1, 2, 4, 8):
            if x != waves:
                ops = [dict(c) for c in cfg.op_config_lst]
                ops[pos]["fuse"] = [[x]]
                out.append(("wavefronts %d" % x, Config(ops, dict(cfg.graph_config))))
        return out

    def with_op(knob, value):
        ops = [dict(c) for c in cfg.op_config_lst]
        ops[pos][knob] = value
        return Config(ops, dict(cfg.graph_config))

    depth, spread = (list((op.get("unroll") or [[2, 1]])[0]) + [1])[:2]
    if depth == 8:
        out += [("load spread %d" % x, with_op("unroll", [[8, x]])) for x in (1, 2, 4, 6, 7, 8) if x != spread]
    group = (op.get("fuse") or [[4]])[0][0]
    out += [("group %d" % x, with_op("fuse", [[x]])) for x in (1, 2, 4, 8, 16) if x != group]
    order = (list((op.get("reorder") or [[1, 0, 0]])[0]) + [0, 0])[:3]
    out.append(("xcd %d" % (1 - order[0]), with_op("reorder", [[1 - order[0], order[1], order[2]]])))
    return out


def polish_entry(key, cfg, threshold=0.01, number=1000, longest_ms=0.2):
    """(Config, ms before, ms after, [accepted moves]); the entry itself when nothing is faster."""
    plan, _ = schedule_with_config(key, cfg)
    if plan.specs[-1].kernel not in ("igemm_f32", "gemm_i8", "depthwise_f32"):
        return cfg, None, None, []
    m = get_measurer(key)
    base = _time(m, plan, number)
    if base > longest_ms:                 # long kernels: none of these knobs moves them by a percent
        return cfg, base, base, []
    best_cfg, best, moves = cfg, base, []
    tried = set()
    improved = True
    while improved:
        improved = False
        for what, cand in neighbours(key, best_cfg):
            sig = json.dumps(cand, sort_keys=True)
            if sig in tried:
                continue
            tried.add(sig)
            try:
                p1, _ = schedule_with_config(key, cand)
                t = _time(m, p1, number)
            except Exception:  # noqa: BLE001  (refused on the host, failed to build, wrong result)
                continue
            if t < best * (1.0 - threshold):
                # kernels near the launch floor time bimodally from one build to the next: the candidate
                # has to win every one of several rounds that alternate with the current entry
                p0, _ = schedule_with_config(key, best_cfg)
                rounds = [(m.evaluate(p0, number=number), m.evaluate(p1, number=number)) for _ in range(ROUNDS)]
                if all(c < b * (1.0 - threshold) for b, c in rounds):
                    best_cfg, best, improved = cand, min(c for _, c in rounds), True
                    moves.append(what)
    return best_cfg, base, best, moves


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--log", required=True, help="key:json lines to refine")
    ap.add_argument("--out", required=True, help="where the refined lines go (every line of --log, refined or not)")
    ap.add_argument("--threshold", type=float, default=0.01)
    ap.add_argument("--number", type=int, default=1000, help="launches per timing")
    ap.add_argument("-f", "--from_", type=int, default=0)
    ap.add_argument("-t", "--to", type=int, default=-1)
    args = ap.parse_args(argv)
    lines = [l for l in open(args.log).read().split("\n") if l.strip()]
    end = len(lines) if args.to < 0 else args.to
    changed = 0
    with open(args.out, "w") as out:
        for i, line in enumerate(lines):
            key, text = line.split(":", 1)
            if not (args.from_ <= i < end) or key not in TASK_TABLE:
                print(line, file=out, flush=True)
                continue
            obj = json.loads(text)
            cfg = Config(obj[0], obj[1])
            try:
                new, before, after, moves = polish_entry(key, cfg, args.threshold, args.number)
            except Exception as e:  # noqa: BLE001
                print("%s: kept (%s)" % (key, str(e)[:100]))
                new, before, after, moves = cfg, None, None, []
            print(key + ":" + json.dumps(new), file=out, flush=True)
            if moves:
                changed += 1
                print("%s: %.3f -> %.3f us (%.1f %%): %s" % (key, before * 1e3, after * 1e3,
                                                             (1 - after / before) * 100, ", ".join(moves)), flush=True)
            elif before is not None:
                print("%s: %.3f us, kept" % (key, before * 1e3), flush=True)
    print("%d of %d entries refined" % (changed, len(lines)))
    return 0


if __name__ == "__main__":
    sys.exit(main())
