"""Host-side helpers shared by the space, the search and the drivers.

Counterparts in the reference: flextensor/utils.py (Config :11-12,
get_factor_lst :82-93, any_factor_split :106-128, gen_enum :218-221,
gen_group :235-242, is_power_of_x :257-259, test_allclose :267-277).
The Android/RPC helper (RpcInfo) is accepted for call compatibility only.
"""
from collections import namedtuple

import numpy as np


class Config(namedtuple("Config", ("op_config_lst", "graph_config"))):
    """(list of per-op config dicts, graph config dict); JSON-serialisable as
    ``[op_config_lst, graph_config]`` (flextensor/optimize/optimize_gemm.py:62-64)."""
    pass


class RpcInfo(object):
    """Kept so that drivers written for the reference still construct; the
    gfx950 backend measures on the local device and never opens a session."""

    def __init__(self, host=None, port=None, target_host=None, device_key="", use_rpc=None,
                 fcompile=None, sess_timeout=0):
        self.host = host
        self.port = port
        self.target_host = target_host
        self.device_key = device_key
        self.use_rpc = use_rpc
        self.fcompile = None
        self.sess_timeout = sess_timeout

    def get_remote(self):
        if self.use_rpc:
            raise RuntimeError("remote measurement is not supported by the gfx950 backend")
        return None


def assert_print(bool_stmt, false_str=""):
    if not bool_stmt:
        raise AssertionError(false_str)


def to_int(expr):
    try:
        return int(expr)
    except Exception as e:
        raise RuntimeError("fail to convert to int: %s" % str(e))


def to_tuple(expr_tuple):
    return tuple(to_int(x) for x in expr_tuple)


def get_factor_lst(value):
    """All divisors of ``value``, ascending."""
    assert isinstance(value, int) and value > 0
    small, large = [], []
    i = 1
    while i * i <= value:
        if value % i == 0:
            small.append(i)
            if i != value // i:
                large.append(value // i)
        i += 1
    return small + large[::-1]


def powerx_lst(x, left, right):
    """Powers of x in [left, right)."""
    ret = []
    beg = 1
    while beg < left:
        beg *= x
    while beg < right:
        ret.append(beg)
        beg *= x
    return ret


def any_factor_split(value, number, allow_non_divisible="off"):
    """Every ordered way to write ``value`` as a product of ``number`` factors.

    ``off``: exact divisors only, enumerated with each level's candidates in
    ascending order (so any_factor_split(8, 2) is [[1,8],[2,4],[4,2],[8,1]]).
    ``power2``: divisors plus powers of two below the remainder, remainder
    taken with floor division. ``continuous``: every integer 1..remainder.
    """
    assert allow_non_divisible in ("off", "power2", "continuous")
    assert isinstance(number, int) and number >= 1
    ret = []

    def rec(left, cur, n):
        if n == 1:
            ret.append(cur + [left])
            return
        if allow_non_divisible == "power2":
            cands = sorted(set(get_factor_lst(left)) | set(powerx_lst(2, 1, left)))
        elif allow_non_divisible == "continuous":
            cands = list(range(1, left + 1))
        else:
            cands = get_factor_lst(left)
        for f in cands:
            rec(left // f, cur + [f], n - 1)

    rec(int(value), [], number)
    return ret


def gen_enum(elements, length):
    """All sequences of ``length`` items drawn from ``elements`` (first index slowest)."""
    res = [[]]
    for _ in range(length):
        res = [r + [e] for r in res for e in elements]
    return res


def gen_group(elements, most_groups=3):
    """Ways to cut ``elements`` into min(len, most_groups) consecutive groups.

    Each result lists the exclusive end index of every group; when there are
    fewer elements than ``most_groups`` the last end index is repeated so that
    every result has ``most_groups`` entries.
    """
    length = len(elements)
    groups = min(length, most_groups)
    padding = most_groups - groups
    res = []

    def rec(cur, p, left):
        if left == 1:
            res.append(cur + [length] * (1 + padding))
            return
        for i in range(p + 1, length):
            rec(cur + [i], i, left - 1)

    if groups < 1:
        raise RuntimeError("At least 1 group")
    rec([], 0, groups)
    return res


def is_power_of_x(x, val):
    assert isinstance(val, int) and val > 0
    while val % x == 0:
        val //= x
    return val == 1


def nearest_power_of_two(val):
    assert isinstance(val, int) and val > 0
    return 1 << (val.bit_length() - 1)


def ceil_div(a, b):
    return -(-a // b)


def test_allclose(value, target, rtol=1e-5, print_diff=False):
    """1 if ``value`` matches ``target`` to ``rtol`` (numpy.testing semantics), else 0."""
    try:
        np.testing.assert_allclose(value, target, rtol)
        return 1
    except AssertionError:
        if print_diff:
            print(target - value)
            print("Max diff:", np.max(np.fabs(target - value)))
        return 0


test_allclose.__test__ = False  # not a pytest test


def max_rel_err(value, target):
    """max|value - target| / max|target| — the fp32 acceptance metric."""
    value = np.asarray(value, dtype=np.float64)
    target = np.asarray(target, dtype=np.float64)
    denom = float(np.max(np.abs(target))) if target.size else 0.0
    if denom == 0.0:
        return float(np.max(np.abs(value))) if value.size else 0.0
    return float(np.max(np.abs(value - target))) / denom
