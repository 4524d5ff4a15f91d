"""Model check of the balanced K-streaming hand-off of igemm_f32.hip, on the CPU.

The kernel cuts the work into (output tile, k-tile) units; workgroup w takes
units [w * PER, (w + 1) * PER). A tile that several workgroups cover is
exchanged through workspace slots and a per-tile arrival counter; nobody
waits: whoever finds all other sharers arrived sums the slots and stores the
tile. Special rules: the arrival of a workgroup's first segment is counted in
the prologue of its next segment and looked at when the workgroup ends; the
workgroup that holds a tile's lowest K range looks at the counter first and,
when everybody else has arrived, adds their slots to its registers; the
counter is reset by whoever sums.

This file restates those rules as a small transition system (one atomic step
per access to shared state, plus an environment event for "the stores of a
slot have landed in memory") and explores EVERY interleaving of 2-5
workgroups over a set of (tiles, k-tiles per tile, units per workgroup)
shapes, two launches in a row, asserting

  * a slot is only ever read after all its stores landed, and it holds the
    partial sum of the reader's tile written in the current launch,
  * every tile is stored exactly once, from every k-tile exactly once,
    with the partial sums added in sharer order (so the result cannot depend
    on timing),
  * every counter is back at zero when the launch ends.

The same checker runs over the rules of the first version of the exchange
(every sharer counts its arrival right after its slot stores, the last arrival
sums; slot stores followed by a workgroup-scope fence, which on gfx950 does not
wait for vector stores): its interleavings are fine when stores land at once,
and it reads a slot whose stores are still in flight as soon as they may land
late, which is the failure the explicit wait removed.
"""
import itertools
import os
import random
import re

import pytest

TEMPLATE = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                        "flextensor_amd", "templates", "igemm_f32.hip")


# ---- the kernel's arithmetic, restated ----------------------------------------------------

def sharers(tile, KT, PER):
    return (tile * KT) // PER, (tile * KT + KT - 1) // PER


def slot_index(w, tile, KT, PER):
    return 2 * w + (0 if w * PER >= tile * KT else 1)


def segments(w, KT, PER, units):
    """(tile, first k-tile, k-tiles) runs of workgroup w, in order."""
    unit, end = w * PER, min(w * PER + PER, units)
    out = []
    while unit < end:
        tile = unit // KT
        lo = unit - tile * KT
        nk = min(KT - lo, end - unit)
        unit += nk
        out.append((tile, lo, nk))
    return out


def test_restated_arithmetic_is_the_template_s():
    src = open(TEMPLATE).read()
    for text in ("first_ = (tile_ * KT) / SK_PER;",
                 "last_ = (tile_ * KT + KT - 1) / SK_PER;",
                 "(2 * w + ((w * SK_PER >= tile_ * KT) ? 0 : 1))",
                 "const int nk = (KT - kt_lo < unit_end - unit) ? KT - kt_lo : unit_end - unit;",
                 "if (kt_lo == 0) {",
                 "if (unit < unit_end) {\n            arrive_tile = tile;"):
        assert text in src, text
    # the order of the hand-off in the source: slot stores, wait, barrier, arrival
    tail = src[src.index("float* mine = slot_of(wg, tile);"):]
    order = [tail.index(t) for t in ("__hip_atomic_store(&mine", "SK_DRAIN_STORES();", "__syncthreads();",
                                     "__hip_atomic_fetch_add(&sk_cnt[tile]")]
    assert order == sorted(order)
    pro = src[src.index("if (arrive_tile >= 0) SK_DRAIN_STORES();"):]
    assert pro.index("__syncthreads();") < pro.index("__hip_atomic_fetch_add(&sk_cnt[arrive_tile]")
    assert re.search(r"#define SK_DRAIN_STORES\(\) __builtin_amdgcn_s_waitcnt\(0x0F70\)", src)


# ---- the transition system ------------------------------------------------------------------

class Violation(AssertionError):
    pass


class Model(object):
    """rules = "shipped" or "first"; wait_for_stores: the arrival is only counted once the
    workgroup's slot stores have landed (the explicit vmcnt(0) wait)."""

    def __init__(self, tiles, KT, PER, rules="shipped", wait_for_stores=True, stores_land_at_once=False,
                 mutate=None):
        self.mutate = mutate                # a deliberate mistake, to show that the checker sees it
        self.tiles, self.KT, self.PER = tiles, KT, PER
        self.units = tiles * KT
        self.nwg = -(-self.units // PER)
        self.rules, self.wait, self.instant = rules, wait_for_stores, stores_land_at_once
        self.segs = [segments(w, KT, PER, self.units) for w in range(self.nwg)]
        self.programs = [self._program(w) for w in range(self.nwg)]

    def slot(self, w, tile):
        if self.mutate == "one_slot":
            return 2 * w
        return slot_index(w, tile, self.KT, self.PER)

    # a program is a list of ops; the interpreter keeps (pc, check_before) per workgroup
    def _program(self, w):
        ops = []
        segs = self.segs[w]
        pending = None                      # tile whose arrival is still to be counted
        deferred = None
        for si, (tile, lo, nk) in enumerate(segs):
            last = si == len(segs) - 1
            if pending is not None:
                ops.append(("drain", self.slot(w, pending)))
                ops.append(("arrive_deferred", pending))
                deferred, pending = pending, None
            if nk == self.KT:
                ops.append(("store_whole", tile))
                continue
            first, lastw = sharers(tile, self.KT, self.PER)
            others = lastw - first
            mine = frozenset(range(lo, lo + nk))
            if self.rules == "shipped" and lo == 0:
                # [look, sum-from-registers path ..., skip target]
                ops.append(("look", tile, others, w, mine))
            ops.append(("write_slot", self.slot(w, tile), tile, mine))
            if self.rules == "shipped" and not last:
                pending = tile
                continue
            ops.append(("drain", self.slot(w, tile)))
            ops.append(("arrive", tile, others))
        if deferred is not None:
            first, lastw = sharers(deferred, self.KT, self.PER)
            ops.append(("check_deferred", deferred, lastw - first))
        return ops

    def initial(self, launch, slots=None):
        nslots = 2 * self.nwg
        slots = slots if slots is not None else tuple([None] * nslots)
        wgs = tuple((0, -1) for _ in range(self.nwg))          # (pc, check_before)
        return (wgs, tuple([0] * self.tiles), slots, tuple([0] * self.tiles), launch)

    def _sum(self, state_slots, tile, launch, from_registers=None):
        """Partial sums of ``tile`` in sharer order; from_registers = (w, k-tiles) of a reducer that
        keeps its own share in registers."""
        first, lastw = sharers(tile, self.KT, self.PER)
        order, got = [], []
        for w in range(first, lastw + 1):
            if from_registers is not None and w == from_registers[0]:
                order.append(w)
                got.append(from_registers[1])
                continue
            s = state_slots[self.slot(w, tile)]
            if s is None:
                raise Violation("tile %d: slot of workgroup %d read before it was written" % (tile, w))
            s_launch, s_tile, s_units, landed = s
            if s_launch != launch or s_tile != tile:
                raise Violation("tile %d: slot of workgroup %d holds launch %d tile %d" % (tile, w, s_launch, s_tile))
            if not landed:
                raise Violation("tile %d: slot of workgroup %d read with its stores in flight" % (tile, w))
            order.append(w)
            got.append(s_units)
        if order != list(range(first, lastw + 1)):
            raise Violation("tile %d summed out of sharer order" % tile)
        allk = sorted(k for g in got for k in g)
        if allk != list(range(self.KT)):
            raise Violation("tile %d summed from k-tiles %s" % (tile, allk))

    def successors(self, state):
        wgs, cnt, slots, stored, launch = state
        out = []
        # environment: the stores of a written slot land
        for i, s in enumerate(slots):
            if s is not None and s[0] == launch and not s[3]:
                ns = list(slots)
                ns[i] = (s[0], s[1], s[2], True)
                out.append((wgs, cnt, tuple(ns), stored, launch))
        for w in range(self.nwg):
            n = self.step(state, w)
            if n is not None:
                out.append(n)
        return out

    def step(self, state, w):
        """The state after workgroup w's next access to shared memory; None when it has ended or waits."""
        wgs, cnt, slots, stored, launch = state
        pc, before = wgs[w]
        prog = self.programs[w]
        if pc >= len(prog):
            return None
        op = prog[pc]
        cnt2, slots2, stored2 = list(cnt), list(slots), list(stored)
        npc, nbefore = pc + 1, before

        def store(tile):
            if stored2[tile]:
                raise Violation("tile %d stored twice" % tile)
            stored2[tile] = 1

        kind = op[0]
        if kind == "store_whole":
            store(op[1])
        elif kind == "look":
            _, tile, others, me, mine = op
            if cnt[tile] == others - (1 if self.mutate == "look_early" and others > 1 else 0):
                self._sum(slots, tile, launch, from_registers=(me, mine))
                cnt2[tile] = 0
                store(tile)
                npc = pc + 4            # past write_slot, drain, arrive (the lowest range ends the run)
                assert prog[pc + 1][0] == "write_slot" and prog[pc + 3][0] == "arrive"
        elif kind == "write_slot":
            _, idx, tile, mine = op
            slots2[idx] = (launch, tile, mine, self.instant)
        elif kind == "drain":
            s = slots[op[1]]
            if self.wait and not (s is not None and s[0] == launch and s[3]):
                return None             # the wavefronts are still waiting for their stores
        elif kind == "arrive":
            _, tile, others = op
            b = cnt[tile]
            cnt2[tile] = b + 1
            if b == others:
                if self.mutate != "no_reset":
                    cnt2[tile] = 0
                self._sum(slots, tile, launch)
                store(tile)
        elif kind == "arrive_deferred":
            nbefore = cnt[op[1]]
            cnt2[op[1]] = nbefore + 1
        elif kind == "check_deferred":
            _, tile, others = op
            if before == others:
                cnt2[tile] = 0
                self._sum(slots, tile, launch)
                store(tile)
        else:
            raise AssertionError(kind)
        nw = list(wgs)
        nw[w] = (npc, nbefore)
        return (tuple(nw), tuple(cnt2), tuple(slots2), tuple(stored2), launch)

    def finished(self, state):
        return all(pc >= len(self.programs[w]) for w, (pc, _) in enumerate(state[0]))

    def check_end(self, state):
        _, cnt, _, stored, _ = state
        if any(cnt):
            raise Violation("counters at the end of the launch: %s" % (cnt,))
        if not all(stored):
            raise Violation("tiles never stored: %s" % [t for t, s in enumerate(stored) if not s])

    def explore(self, launches=2):
        """Every interleaving of ``launches`` launches in a row; returns the number of states."""
        total = 0
        starts = {self.initial(1)}
        for launch in range(1, launches + 1):
            seen, stack, ends = set(starts), list(starts), set()
            while stack:
                st = stack.pop()
                nxt = self.successors(st)
                if self.finished(st):
                    self.check_end(st)
                    # at the end of a kernel every store has landed
                    slots = tuple(None if s is None else (s[0], s[1], s[2], True) for s in st[2])
                    ends.add(slots)
                for n in nxt:
                    if n not in seen:
                        seen.add(n)
                        stack.append(n)
            total += len(seen)
            starts = {self.initial(launch + 1, slots) for slots in ends}
        return total

    def random_run(self, rng, launches=2):
        slots = None
        for launch in range(1, launches + 1):
            st = self.initial(launch, slots)
            live = list(range(self.nwg))
            while live:
                w = rng.choice(live)
                n = self.step(st, w)
                if n is None:
                    if st[0][w][0] >= len(self.programs[w]):
                        live.remove(w)
                        continue
                    # waiting for its stores: let one of its slots land
                    wgs, cnt, sl, stored, la = st
                    sl = list(sl)
                    for i in (2 * w, 2 * w + 1):
                        if sl[i] is not None and sl[i][0] == la and not sl[i][3]:
                            sl[i] = sl[i][:3] + (True,)
                    n = (wgs, cnt, tuple(sl), stored, la)
                st = n
            assert self.finished(st)
            self.check_end(st)
            slots = tuple(None if s is None else (s[0], s[1], s[2], True) for s in st[2])


# shapes: (tiles, k-tiles per tile, units per workgroup); 2-5 workgroups, 2-4 sharers per tile,
# workgroups that end one tile and begin the next, whole tiles between shared ones, ranges inside
# one tile, a last workgroup with fewer units
SMALL = [
    (1, 4, 2), (1, 4, 3), (1, 6, 2), (1, 8, 2), (1, 7, 2),
    (2, 3, 2), (2, 4, 3), (2, 5, 3), (2, 5, 4), (2, 6, 4), (2, 3, 4), (2, 2, 3),
    (3, 2, 3), (3, 3, 2), (3, 4, 3), (3, 3, 4), (3, 4, 5), (3, 5, 4),
    (4, 3, 4), (4, 2, 3), (4, 3, 5), (5, 2, 3), (3, 4, 6), (4, 3, 7), (5, 3, 4),
]


@pytest.mark.parametrize("tiles,KT,PER", SMALL)
def test_every_interleaving_of_the_shipped_protocol(tiles, KT, PER):
    m = Model(tiles, KT, PER)
    assert 2 <= m.nwg <= 6
    n = m.explore(launches=2)
    assert n > 0


def test_the_shapes_cover_the_cases_the_rules_distinguish():
    kinds = set()
    for tiles, KT, PER in SMALL:
        m = Model(tiles, KT, PER)
        for w, segs in enumerate(m.segs):
            for si, (tile, lo, nk) in enumerate(segs):
                if nk == KT:
                    kinds.add("whole tile between shared ones" if 0 < si < len(segs) - 1 else "whole tile")
                elif lo == 0:
                    kinds.add("lowest range")
                elif lo + nk == KT and si < len(segs) - 1:
                    kinds.add("ends a tile, goes on (deferred arrival)")
                elif lo + nk == KT:
                    kinds.add("ends a tile, stops")
                else:
                    kinds.add("inside a tile")
        for t in range(tiles):
            a, b = sharers(t, KT, PER)
            kinds.add("%d sharers" % (b - a + 1))
    for want in ("whole tile between shared ones", "lowest range", "ends a tile, goes on (deferred arrival)",
                 "ends a tile, stops", "inside a tile", "2 sharers", "3 sharers", "4 sharers"):
        assert want in kinds, want


def test_shipped_rules_on_the_benchmark_layer_s_real_shape_random_schedules():
    """conv 8x256x14x14 -> 512 as shipped (64x64 tiles of 1568 x 512, K 2304 in tiles of 144: 200 tiles
    of 16 k-tiles, 13 units per workgroup) and the shape of the one wrong result ever seen
    (98 tiles of 36 k-tiles, 14 units per workgroup): seeded random schedules."""
    rng = random.Random(11)
    for tiles, KT, PER in ((200, 16, 13), (98, 36, 14), (196, 4, 4), (25, 16, 2)):
        m = Model(tiles, KT, PER)
        for _ in range(3):
            m.random_run(rng)


def test_slots_are_never_shared_between_two_partial_sums():
    for tiles, KT, PER in itertools.product(range(1, 7), range(1, 10), range(1, 12)):
        m = Model(tiles, KT, PER)
        used = {}
        for w, segs in enumerate(m.segs):
            assert len([s for s in segs if s[2] != KT]) <= 2          # a range begins and ends in at most two shared tiles
            for tile, lo, nk in segs:
                if nk != KT:
                    idx = slot_index(w, tile, KT, PER)
                    assert idx not in used, (tiles, KT, PER, w, tile)
                    used[idx] = (w, tile)
                    first, last = sharers(tile, KT, PER)
                    assert first <= w <= last
        for t in range(tiles):
            first, last = sharers(t, KT, PER)
            for w in range(first, last + 1):
                assert any(seg[0] == t for seg in m.segs[w])


def test_the_first_version_s_interleavings_are_fine_but_not_its_unwaited_stores():
    """First version: every sharer counts its arrival behind its slot stores, the last arrival sums.
    With stores that land at once every interleaving is right; with stores that may land late and
    no wait before the arrival (a workgroup-scope fence does not wait for vector stores on gfx950)
    a reader finds a slot in flight. A share of a 36-k-tile tile is 14 k-tiles: one late cache line
    of one sharer is an error of 14/36 = 0.39 of an element, the size of the wrong result seen."""
    for tiles, KT, PER in SMALL[:12]:
        Model(tiles, KT, PER, rules="first", stores_land_at_once=True).explore()
        Model(tiles, KT, PER, rules="first", wait_for_stores=True).explore()
        with pytest.raises(Violation, match="stores in flight"):
            Model(tiles, KT, PER, rules="first", wait_for_stores=False).explore()
        # and the shipped rules need the wait just as much
        with pytest.raises(Violation, match="stores in flight"):
            Model(tiles, KT, PER, rules="shipped", wait_for_stores=False).explore()


def test_the_checker_has_teeth():
    """Rule changes a plausible mistake would make are caught."""
    with pytest.raises(Violation, match="counters at the end"):
        Model(2, 4, 3, mutate="no_reset").explore(launches=1)          # a reducer that forgets the reset
    with pytest.raises(Violation):
        Model(3, 3, 2, mutate="one_slot").explore(launches=1)          # one slot per workgroup instead of two
    with pytest.raises(Violation):
        Model(1, 6, 2, mutate="look_early").explore(launches=1)        # the lowest range sums one sharer early
    with pytest.raises(Violation, match="stored twice|never stored|k-tiles|counters at the end"):
        m = Model(2, 4, 3)
        # a workgroup whose program lost the check of its deferred arrival
        m.programs = [[o for o in prog if o[0] != "check_deferred"] for prog in m.programs]
        m.explore(launches=1)
