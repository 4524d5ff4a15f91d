"""Refine the entries of a tuned log one knob at a time, on the device.

    python -m flextensor_amd.optimize.polish --log tuned.log --out refined.log

A search ends at a point of a large space after a bounded number of trials; kernels change
afterwards (a cheaper set-up shifts the balance between LDS layouts, for one). This pass takes
every ``key:json`` line of a log, measures it, and tries the neighbours along the knobs that
cost nothing to enumerate: the LDS layout (`lds_pad`), the number of k blocks the next tile's
loads are spread over (depth 8), the traversal group height and the XCD renumbering. A
neighbour replaces the entry when it is faster by more than ``--threshold`` (default 1.2 %)
in two measurements and again in a second pair against the then-current entry; every
measurement passes the on-device correctness gate. Lines of tasks that are not registered, or
whose last kernel is not the fp32 contraction template, are copied as they are.
"""
import argparse
import json
import sys

from ..measure import get_measurer
from ..scheduler import schedule_with_config
from ..task import TASK_TABLE
from ..templates import gfx950
from ..utils import Config


def _time(measurer, plan, number):
    return min(measurer.evaluate(plan, number=number) for _ in range(2))


def neighbours(key, cfg):
    """[(what, Config)] one knob away from ``cfg``."""
    out = []
    task = TASK_TABLE[key]
    names = list(task.special_space)
    if "lds_pad" in names:
        at = names.index("lds_pad")
        special = [list(x) for x in (cfg.graph_config.get("special") or [])]
        while len(special) <= at:
            special.append(list(gfx950.SPECIAL_DEFAULTS[names[len(special)]]))
        for pad in task.special_space["lds_pad"].static_entities:
            if list(pad) != special[at]:
                s2 = [list(x) for x in special]
                s2[at] = list(pad)
                out.append(("lds_pad %s" % list(pad), Config(cfg.op_config_lst, dict(cfg.graph_config, special=s2))))
    pos = [i for i, c in enumerate(cfg.op_config_lst) if c.get("spatial")]
    if not pos:
        return out
    pos = pos[0]
    op = cfg.op_config_lst[pos]

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


def polish_entry(key, cfg, threshold=0.012, number=400, longest_ms=0.2):
    """(Config, ms before, ms after, [accepted moves]); the entry itself when nothing is faster."""
    plan, _ = schedule_with_config(key, cfg)
    if plan.specs[-1].kernel != "igemm_f32":
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
                again_best = min(_time(m, schedule_with_config(key, best_cfg)[0], number), best)
                again = min(_time(m, p1, number), t)
                if again < again_best * (1.0 - threshold):
                    best_cfg, best, improved = cand, again, True
                    moves.append(what)
    return best_cfg, base, best, moves


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--log", required=True, help="key:json lines to refine")
    ap.add_argument("--out", required=True, help="where the refined lines go (every line of --log, refined or not)")
    ap.add_argument("--threshold", type=float, default=0.012)
    ap.add_argument("--number", type=int, default=400, help="launches per timing")
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
