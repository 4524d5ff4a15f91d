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
    empty = {k: [] for k in conv_cfg}
    graph = dict(direct.graph_config or {})
    pad_inline = (graph.get("inline") or [[1, 0]])[0][0]
    graph["inline"] = [[pad_inline, 1, 0, 0]]
    graph["merge"] = [[0, 0, 0, 1]]
    return Config([dict(pad_cfg), dict(empty), dict(conv_cfg), dict(empty)], graph)


def lookup(key):
    global _cache
    if _cache is None:
        _cache = load()
    found = _cache.get(key)
    if found is None:
        found = _from_direct_convolution(key, _cache)
    return found
