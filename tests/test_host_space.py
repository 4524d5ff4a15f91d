"""Host logic: factor splits, sub-spaces, neighbour moves, config format."""
import json
import os
from functools import reduce

import numpy as np
import pytest

from flextensor_amd import space as sp
from flextensor_amd.utils import (Config, any_factor_split, gen_enum, gen_group, get_factor_lst,
                                  is_power_of_x, test_allclose as allclose, max_rel_err)

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def n_ordered_factorizations(n, parts):
    """Brute force: tuples of `parts` positive ints with product n."""
    if parts == 1:
        return 1
    return sum(n_ordered_factorizations(n // d, parts - 1) for d in range(1, n + 1) if n % d == 0)


def test_factor_lists():
    assert get_factor_lst(1) == [1]
    assert get_factor_lst(12) == [1, 2, 3, 4, 6, 12]
    assert get_factor_lst(49) == [1, 7, 49]
    for n in range(1, 200):
        assert get_factor_lst(n) == [d for d in range(1, n + 1) if n % d == 0]


def test_any_factor_split_known_answer_and_invariants():
    # by inspection of the enumeration order (ascending candidates per level)
    assert any_factor_split(8, 2) == [[1, 8], [2, 4], [4, 2], [8, 1]]
    assert any_factor_split(6, 3)[0] == [1, 1, 6] and any_factor_split(6, 3)[-1] == [6, 1, 1]
    for n in (1, 7, 12, 56, 64, 1024):
        for parts in (1, 2, 3, 4):
            ents = any_factor_split(n, parts)
            assert len(ents) == n_ordered_factorizations(n, parts)
            assert len(set(map(tuple, ents))) == len(ents)
            for e in ents:
                assert len(e) == parts and reduce(lambda a, b: a * b, e) == n
    assert len(any_factor_split(1024, 4)) == 286  # C(13, 3)
    cont = any_factor_split(5, 2, "continuous")
    assert cont == [[1, 5], [2, 2], [3, 1], [4, 1], [5, 1]]
    p2 = any_factor_split(6, 2, "power2")
    assert [2, 3] in p2 and [4, 1] in p2


def test_gen_enum_group():
    assert gen_enum([1, 0], 2) == [[1, 1], [1, 0], [0, 1], [0, 0]]
    assert gen_enum([1, 0], 0) == [[]]
    assert gen_group(list("bchw"), 3) == [[1, 2, 4], [1, 3, 4], [2, 3, 4]]
    assert gen_group(list("ij"), 3) == [[1, 2, 2]]
    assert gen_group(list("i"), 3) == [[1, 1, 1]]
    assert is_power_of_x(2, 1024) and not is_power_of_x(2, 48) and is_power_of_x(3, 27)


def test_allclose_and_rel_err():
    a = np.array([1.0, 2.0, 3.0])
    assert allclose(a, a * (1 + 1e-7)) == 1
    assert allclose(a, a * 1.1) == 0
    assert max_rel_err(a, a) == 0.0
    assert abs(max_rel_err(a + np.array([0, 0, 3e-5]), a) - 1e-5) < 1e-12


def test_split_space_moves_preserve_product():
    s = sp.SplitSpace(4, 1024)
    assert len(s) == 286 and s.num_direction == 12 and len(s.directions) == 12
    rng = np.random.default_rng(0)
    for _ in range(200):
        pos = int(rng.integers(0, s.size))
        d = s.get_direction(int(rng.integers(0, 100)))
        nxt = s.next_entity(pos, d)
        cur, new = s.get_entity(pos), s.get_entity(nxt)
        assert reduce(lambda a, b: a * b, new) == 1024
        asc, dec = d
        if nxt != pos:
            assert new[asc] > cur[asc] and new[dec] < cur[dec]
            assert new[asc] * new[dec] == cur[asc] * cur[dec]
            # the next admissible value: no divisor in between
            assert not [v for v in range(cur[asc] + 1, new[asc]) if (cur[asc] * cur[dec]) % v == 0]
            for l in range(4):
                if l not in d:
                    assert new[l] == cur[l]
        else:
            assert cur[dec] == 1
    # ring move
    assert s.next_entity(0, (-1,)) == s.size - 1


def test_split_space_with_pruning_never_hangs():
    s = sp.SplitSpace(3, 576, keep=lambda e: e[2] in (8, 16, 32, 64) and e[0] <= 16)
    assert s.size > 0
    for pos in range(s.size):
        for d in s.directions:
            nxt = s.next_entity(pos, d)
            assert 0 <= nxt < s.size
            assert s.get_entity(nxt)[2] in (8, 16, 32, 64)


def test_ring_spaces():
    u = sp.UnrollSpace([0, 1, 512, 1500])
    assert u.static_entities[:3] == [[0, 0], [0, 1], [1, 0]] and len(u) == 8
    assert len(sp.UnrollSpace([0, 1, 512, 1500], explicit=True)) == 4
    r = sp.ReorderSpace(3)
    assert r.static_entities == [[0], [1], [2]] and r.next_entity(2, (1,)) == 0
    e = sp.EnumSpace([[4, 8], [0, 0]])
    assert e.next_entity(0, (-1,)) == 1
    with pytest.raises(RuntimeError):
        e.next_entity(0, (0, 1))
    i = sp.InlineSpace([0], 2)
    assert i.static_entities == [[1, 0], [0, 0]] and i.able_inline(0) and not i.able_inline(1)
    assert sp.InlineSpace([0], 2, force_inline=True).static_entities == [[1, 0]]
    p = sp.PosSpace(2, 3)
    assert len(p) == 6


def test_tile_split_space():
    s = sp.TileSplitSpace(392)  # 8*7*7 pixels: never a multiple of 16
    assert s.size > 0
    for g, w, r, m in s.static_entities:
        tile = w * r * m
        assert m in (16, 32) and g == -(-392 // tile)
        assert g * tile >= 392 and (g * tile - 392) <= 0.25 * 392 or g == 1
    for pos in range(s.size):
        for d in s.directions:
            nxt = s.next_entity(pos, d)
            cur, new = s.get_entity(pos), s.get_entity(nxt)
            if nxt != pos:
                assert new[d[0]] > cur[d[0]] and new[d[1]] < cur[d[1]]
    small = sp.TileSplitSpace(64)
    assert max(w * r * m for _, w, r, m in small.static_entities) <= 64
    # 49 = a 7x7 image: four blocks of 16 pad 15 columns, more than a quarter of 49 but less than one
    # block, which is what the single 64-wide tile pads as well; five blocks would pad a whole one
    tiny = sp.TileSplitSpace(49, reps=(1, 2, 3, 4, 5, 6, 7, 8))
    assert [4, 1, 1, 16] in tiny.static_entities and [1, 4, 1, 16] in tiny.static_entities
    assert [2, 1, 1, 32] in tiny.static_entities and [3, 1, 1, 32] not in tiny.static_entities
    assert all(g * w * r * m - 49 < m for g, w, r, m in tiny.static_entities)


def test_space_container_and_generic_intra_op_space():
    from flextensor_amd.task import gemm, conv2d
    from flextensor_amd.scheduler import flatten_graph
    ops, bufs = gemm(1024, 1024, 1024)
    op_lst, down = flatten_graph(ops)
    s = sp.generate_space_intra_op(op_lst[0], down, slevel=4, rlevel=4, unroll_policy="off",
                                   fuse_policy="off", reorder_policy="off")
    # the reference's llvm space for GEMM 1024^3: three 286-entry splits x 8 unroll entries
    assert len(s) == 286 ** 3 * 8
    assert s.types["spatial"] == ["split_i_0", "split_j_1"] and s.types["reduce"] == ["split_k_0"]
    s = sp.generate_space_intra_op(op_lst[0], down)
    assert "fuse_spatial" in s.subspaces and "reorder" in s.subspaces
    with pytest.raises(RuntimeError):
        s.add_subspace("reorder", sp.ReorderSpace(2), "reorder")
    ops, bufs = conv2d(1, 64, 56, 56, 64, 3, 1, 1, 1, 1)
    op_lst, down = flatten_graph(ops)
    assert [o.kind for o in op_lst] == ["zero_pad2d", "conv2d_nchw"]
    g = sp.generate_space_inter_op(op_lst, down)
    assert g.subspaces["inline"].static_entities == [[1, 0], [0, 0]]
    assert [a.name for a in op_lst[1].reduce_axis] == ["rc", "rw", "rh"]


def test_reference_config_lines_parse_and_roundtrip():
    """`key:json` lines written by the reference's drivers are data this
    package must read: [[op configs...], graph config] with all eight keys."""
    keys = ["fuse", "spatial", "reduce", "reorder", "inline", "unroll", "merge", "special"]
    n = 0
    with open(os.path.join(GOLD, "reference_config_lines.txt")) as f:
        for line in f:
            if not line.strip():
                continue
            name, string = line.split(":", 1)
            obj = json.loads(string)
            cfg = Config(obj[0], obj[1])
            assert name.endswith("_opencl(0)")
            for oc in cfg.op_config_lst:
                assert sorted(oc) == sorted(keys)
                for lst in oc["spatial"]:
                    assert len(lst) == 4
            assert sorted(cfg.graph_config) == sorted(keys)
            assert json.loads(json.dumps(cfg)) == obj
            n += 1
    assert n == 6
