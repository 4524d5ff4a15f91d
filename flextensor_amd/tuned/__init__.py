"""Tuned configs shipped with the package.

``mi355x.log`` holds one ``key:json`` line per tuned task, the format the
reference's drivers append to their logs
(flextensor/optimize/optimize_gemm.py:62-64). ``lookup(key)`` returns the
``Config`` of a task, or None when the task has not been tuned.
"""
import json
import os

from ..utils import Config

LOG = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mi355x.log")
_cache = None


def load(path=LOG):
    out = {}
    if not os.path.exists(path):
        return out
    with open(path, "r") as f:
        for line in f:
            line = line.strip()
            if not line or line.startswith("#"):
                continue
            name, string = line.split(":", 1)
            obj = json.loads(string)
            out[name] = Config(obj[0], obj[1])  # later lines win
    return out


def _from_direct_convolution(key, table):
    """A convolution written as im2col, GEMM, col2img folds into the very
    kernel of the direct convolution with the same arguments, so that task's
    tuned point carries over: the GEMM stage takes the convolution's config,
    the column matrix is inlined and the col2img merged."""
    prefix = "gemm_conv2d_"
    if not key.startswith(prefix):
        return None
    direct = table.get("conv2d_" + key[len(prefix):])
    if direct is None or len(direct.op_config_lst) != 2:
        return None
    pad_cfg, conv_cfg = direct.op_config_lst
    if len(conv_cfg.get("spatial") or []) != 2:
        return None      # one channel per group: the direct task is tuned for the depthwise kernel
    empty = {k: [] for k in conv_cfg}
    graph = dict(direct.graph_config or {})
    pad_inline = (graph.get("inline") or [[1, 0]])[0][0]
    graph["inline"] = [[pad_inline, 1, 0, 0]]
    graph["merge"] = [[0, 0, 0, 1]]
    return Config([dict(pad_cfg), dict(empty), dict(conv_cfg), dict(empty)], graph)


def _parse_key(key):
    """'cat_name_(args)_target(dev)' -> (category_and_name_prefix, args tuple, tail) or None."""
    import ast
    import re
    m = re.match(r"^(.*)_(\([^()]*\))_([a-z]+\(\d+\))$", key)
    if not m:
        return None
    try:
        args = tuple(ast.literal_eval(m.group(2)))
    except (ValueError, SyntaxError):
        return None
    return m.group(1), args, m.group(3)


def _from_other_batch(key, table):
    """A convolution layer that is tuned at another batch size lends its point:
    the batch only stretches the N axis (batch * out_h * out_w) of the
    implicit GEMM, so the workgroup tile, the K division and every other knob
    carry over and the N grid level is recomputed. A starting point for the
    search, not a tuned entry: the key it comes from is a different task."""
    parsed = _parse_key(key)
    if parsed is None or not parsed[0].startswith("conv2d_") or len(parsed[1]) != 10:
        return None
    _, args, tail = parsed
    for other, cfg in table.items():
        q = _parse_key(other)
        if q is None or not q[0].startswith("conv2d_") or len(q[1]) != 10:
            continue
        if q[1][1:] != args[1:] or q[1][0] == args[0] or q[2] != tail or len(cfg.op_config_lst) != 2:
            continue
        conv_cfg = cfg.op_config_lst[1]
        if len(conv_cfg.get("spatial") or []) != 2:
            continue          # a depthwise entry: its lanes own whole batch entries
        batch, _, h, w, _, k, stride, pad, dil, _ = args
        out_h = (h + 2 * pad - dil * (k - 1) - 1) // stride + 1
        out_w = (w + 2 * pad - dil * (k - 1) - 1) // stride + 1
        n_ext = batch * out_h * out_w
        new_cfg = {name: [list(e) if isinstance(e, list) else e for e in v] for name, v in conv_cfg.items()}
        _, waves, reps, mfma = new_cfg["spatial"][1]
        tile = waves * reps * mfma
        new_cfg["spatial"][1] = [(n_ext + tile - 1) // tile, waves, reps, mfma]
        return Config([dict(cfg.op_config_lst[0]), new_cfg], dict(cfg.graph_config or {}))
    return None


def lookup(key, similar=False):
    """The shipped entry of a task, or None. A ``gemm_conv2d`` task without an
    entry replays the direct convolution's (the same kernel). With
    ``similar=True`` a convolution without an entry also accepts the point of
    the same layer tuned at another batch size, as a seed for the search."""
    global _cache
    if _cache is None:
        _cache = load()
    found = _cache.get(key)
    if found is None:
        found = _from_direct_convolution(key, _cache)
    if found is None and similar:
        found = _from_other_batch(key, _cache)
    return found
