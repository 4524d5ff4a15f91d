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


def lookup(key):
    global _cache
    if _cache is None:
        _cache = load()
    return _cache.get(key)
