"""Schedule space: typed sub-spaces of knob values and neighbour moves.

The container (`Space`), the sub-space protocol (`static_entities`,
`get_entity`, `next_entity(pos, direction)`, `directions`) and the type keys
are those of the reference (flextensor/space.py:46-452), so the search in
scheduler.py / model.py and the JSON `Config` format are unchanged.

What the knobs *mean* is re-expressed for gfx950 (`generate_space_intra_op`
with a "rocm" target):

  spatial   one 4-level list per GEMM-view axis  [grid, waves, reps, mfma]
            workgroup tile = waves*reps*mfma, wavefront tile = reps*mfma,
            mfma = edge of the matrix-core instruction (16 or 32); for the
            direct depthwise lowering  [grid, 1, 1, outputs per lane]
  reduce    [split-K factor, sequential K iterations, K extent of an LDS tile]
  unroll    [[LDS stages, 1]]   1 = single buffer, 2 = double buffer
  fuse      [[GROUP_M]] tile-traversal group height (depthwise: [[wavefronts
            per workgroup]])
  reorder   [[0|1]]   1 = remap workgroup ids so that neighbouring tiles run
            on the same XCD (shared L2)
  special   enumerated knobs attached to a task (LDS padding, load width,
            non-temporal stores, ...)
"""
import numpy as np

from .utils import (assert_print, any_factor_split, gen_enum, gen_group, is_power_of_x, ceil_div)


def able_inline(op, down_graph):
    """An op can be folded into its consumer when it has no reduction and is
    not a graph output (flextensor/space.py:10-19)."""
    from .te import ComputeOp
    is_compute = isinstance(op, ComputeOp)
    has_reduce = bool(getattr(op, "reduce_axis", None))
    is_output = False
    for i in range(op.num_outputs):
        if op.output(i) not in down_graph:
            is_output = True
            break
    return is_compute and (not has_reduce) and (not is_output)


# stage kind -> producer kinds whose kernel can take the stage over
MERGE_RULES = {
    "bias_add_nchw": ("conv2d_nchw", "depthwise_conv2d_nchw"),   # bias in the convolution's epilogue
    "bias_add_ghw": ("col_gemm",),                # the same for the GEMM of an im2col convolution
    "col2img_nchw": ("col_gemm", "bias_add_ghw"),  # the GEMM stores NCHW itself
}


def able_merge(op, down_graph):
    """An elementwise stage (per-channel bias, col2img) can be merged into the
    stores of the kernel that feeds it, when nothing else reads that kernel's
    output."""
    from .te import ComputeOp
    if not isinstance(op, ComputeOp) or op.kind not in MERGE_RULES:
        return False
    src = op.input_tensors[0]
    if not isinstance(src.op, ComputeOp) or src.op.kind not in MERGE_RULES[op.kind]:
        return False
    return list(down_graph.get(src, [])) == [op]


class Space(object):
    valid_type_keys = ["fuse", "spatial", "reduce", "reorder", "inline", "unroll", "merge", "special"]

    def __init__(self):
        self.subspaces = {}
        self.types = {k: [] for k in self.valid_type_keys}
        self.dim = 0

    def add_subspace(self, name, subspace, type_key, override=False):
        if name in self.subspaces and not override:
            raise RuntimeError("Same subspace name")
        assert_print(type_key in self.valid_type_keys, "unknown type key %s" % type_key)
        self.subspaces[name] = subspace
        if name not in self.types[type_key]:
            self.types[type_key].append(name)
        self.dim += subspace.dim

    def items(self):
        return self.subspaces.items()

    def __len__(self):
        ret = 1
        for _, subspace in self.subspaces.items():
            ret *= len(subspace)
        return ret

    def length(self):
        ret = {}
        total, added = 1, 0
        for name, subspace in self.subspaces.items():
            ret[name] = len(subspace)
            total *= ret[name]
            added += ret[name]
        ret["total"] = total
        ret["added"] = added
        return ret


DirectedSubSpaceTypeKeys = ["spatial", "reduce"]
UndirectedSubSpaceTypeKeys = ["fuse", "reorder", "unroll", "inline", "merge", "special"]


class SubSpace(object):
    def __init__(self):
        self.dim = 0
        self.static_entities = []
        self.size = 0
        self.num_direction = 0
        self.directions = []

    def random_entity(self):
        return self.static_entities[np.random.randint(0, self.size)]

    def next_entity(self, *args, **kwargs):
        raise NotImplementedError()

    def get_entity(self, p):
        return self.static_entities[p]

    def get_direction(self, num):
        return self.directions[num % self.num_direction]

    def __len__(self):
        return self.size


class _RingSpace(SubSpace):
    """Sub-space whose only moves are one step left or right, cyclically."""

    def _finish(self):
        self.size = len(self.static_entities)
        self.num_direction = 2
        self.directions = [(-1,), (1,)]

    def next_entity(self, pos, d):
        if len(d) == 1:
            return (pos + d[0]) % self.size
        raise RuntimeError("Not support for direction more than one dim: {}".format(d))


class SplitSpace(SubSpace):
    """All ordered factorizations of ``total`` into ``dim`` factors.

    A direction (i, j) moves weight from factor j to factor i: factor i grows
    to its next admissible value and factor j becomes what is left of their
    product (flextensor/space.py:112-167). An optional ``keep`` predicate
    prunes entities; moves skip pruned points and stay put when nothing
    further exists in that direction.
    """

    def __init__(self, dim, total, allow_non_divisible="off", keep=None):
        super(SplitSpace, self).__init__()
        self.total = total
        self.allow_non_divisible = allow_non_divisible
        self.dim = dim
        ents = any_factor_split(total, dim, allow_non_divisible=allow_non_divisible)
        if keep is not None:
            ents = [e for e in ents if keep(e)]
        self.static_entities = ents
        self._index = {tuple(e): i for i, e in enumerate(ents)}
        self.size = len(ents)
        self.num_direction = dim * (dim - 1)
        self.directions = [(i, j) for i in range(dim) for j in range(dim) if i != j]
        self.type_key = "split"

    def index_of(self, entity):
        return self._index.get(tuple(entity), -1)

    def _admissible(self, tmp, left):
        if self.allow_non_divisible == "continuous":
            return True
        if self.allow_non_divisible == "power2" and is_power_of_x(2, tmp):
            return True
        return left % tmp == 0

    def next_entity(self, pos, d):
        if len(d) == 1:
            return (pos + d[0]) % self.size
        if len(d) != 2:
            raise RuntimeError("Not support for direction more than two dims: {}".format(d))
        asc, dec = d
        assert_print(0 <= asc < self.dim and 0 <= dec < self.dim and asc != dec, "bad direction")
        cur = self.static_entities[pos]
        left = cur[asc] * cur[dec]
        tmp = cur[asc]
        while tmp < left:
            tmp += 1
            while tmp < left and not self._admissible(tmp, left):
                tmp += 1
            cand = list(cur)
            cand[asc] = tmp
            cand[dec] = ceil_div(left, tmp)
            idx = self.index_of(cand)
            if idx >= 0:
                return idx
        return pos


class FuseSpace(_RingSpace):
    def __init__(self, dim, elements):
        super(FuseSpace, self).__init__()
        self.dim = dim
        self.static_entities = gen_group(elements, most_groups=self.dim)
        self.type_key = "fuse"
        self._finish()


class ReorderSpace(_RingSpace):
    def __init__(self, num_spatial_axis):
        super(ReorderSpace, self).__init__()
        self.dim = 1
        self.static_entities = [[i] for i in range(num_spatial_axis)]
        self.type_key = "reorder"
        self._finish()


class UnrollSpace(_RingSpace):
    def __init__(self, steps, explicit=False, extra=()):
        super(UnrollSpace, self).__init__()
        self.dim = 2
        self.steps = steps
        explicits = [1] if explicit else [0, 1]
        self.static_entities = [[step, e] for step in steps for e in explicits] + [list(e) for e in extra]
        self.type_key = "unroll"
        self._finish()


class PosSpace(_RingSpace):
    def __init__(self, parts, num_axis):
        super(PosSpace, self).__init__()
        self.dim = 2
        self.parts = parts
        self.num_axis = num_axis
        self.static_entities = [[i, j] for i in range(parts) for j in range(num_axis)]
        self.type_key = "local"
        self._finish()


def _flag_entities(positions, op_num, force):
    if force:
        entity = [0] * op_num
        for pos in positions:
            entity[pos] = 1
        return [entity]
    out = []
    for enum in gen_enum([1, 0], len(positions)):
        entity = [0] * op_num
        for i, pos in enumerate(positions):
            entity[pos] = enum[i]
        out.append(entity)
    return out


class InlineSpace(_RingSpace):
    def __init__(self, inline_op_pos, op_num, force_inline=False):
        super(InlineSpace, self).__init__()
        self.dim = op_num
        self.able_inline_list = list(inline_op_pos)
        self.static_entities = _flag_entities(self.able_inline_list, op_num, force_inline)
        self.type_key = "inline"
        self._finish()

    def able_inline(self, pos):
        return pos in self.able_inline_list


class MergeSpce(_RingSpace):
    def __init__(self, merge_op_pos, op_num, force_merge=False):
        super(MergeSpce, self).__init__()
        self.dim = op_num
        self.able_merge_list = list(merge_op_pos)
        self.static_entities = _flag_entities(self.able_merge_list, op_num, force_merge)
        self.type_key = "merge"
        self._finish()

    def able_merge(self, pos):
        return pos in self.able_merge_list


class EnumSpace(_RingSpace):
    """Free-form enumerated knob; each entity is a list of numbers
    (flextensor/space.py:347-365)."""

    def __init__(self, knobs):
        super(EnumSpace, self).__init__()
        self.dim = 2
        self.static_entities = [list(k) for k in knobs]
        if self.static_entities:
            self.dim = len(self.static_entities[0])
        self.type_key = "enum"
        self._finish()


# --------------------------------------------------------------------------
# gfx950 sub-spaces
# --------------------------------------------------------------------------

class TileSplitSpace(SubSpace):
    """[grid, waves, reps, mfma] tilings of one GEMM-view axis of ``extent``.

    waves*reps*mfma is the workgroup tile; grid = ceil(extent / tile), so an
    extent that is not a multiple of the tile is covered by a predicated edge
    tile. Entities whose padding wastes more than ``max_waste`` of the work
    are dropped. Directions are the (grow, shrink) level pairs of SplitSpace:
    level ``grow`` moves to its next larger admissible value while level
    ``shrink`` moves to a smaller one and the two other levels stay (the grid
    level is derived, so it always follows).
    """

    def __init__(self, extent, mfma_dims=(16, 32), waves=(1, 2, 4), reps=(1, 2, 3, 4, 6, 8),
                 max_tile=512, max_waste=0.25):
        super(TileSplitSpace, self).__init__()
        self.total = extent
        self.dim = 4
        ents = []
        for mf in mfma_dims:
            for w in waves:
                for r in reps:
                    tile = w * r * mf
                    if tile > max_tile:
                        continue
                    grid = ceil_div(extent, tile)
                    padded = grid * tile
                    if grid > 1 and (padded - extent) > max_waste * extent and padded - extent >= mf:
                        continue      # (less than one MFMA block of padding is what any tiling of the axis has)
                    if grid == 1 and tile - extent >= mf:
                        continue  # a smaller tile covers the axis as well
                    ents.append([grid, w, r, mf])
        ents.sort(key=lambda e: (e[1] * e[2] * e[3], e[3], e[1]))
        self.static_entities = ents
        self._index = {tuple(e): i for i, e in enumerate(ents)}
        self.size = len(ents)
        self.directions = [(i, j) for i in range(4) for j in range(4) if i != j]
        self.num_direction = len(self.directions)
        self.type_key = "split"

    def index_of(self, entity):
        return self._index.get(tuple(entity), -1)

    def next_entity(self, pos, d):
        if len(d) == 1:
            return (pos + d[0]) % self.size
        grow, shrink = d
        cur = self.static_entities[pos]
        best, best_key = pos, None
        for idx, e in enumerate(self.static_entities):
            if idx == pos or e[grow] <= cur[grow] or e[shrink] >= cur[shrink]:
                continue
            if any(e[l] != cur[l] for l in (1, 2, 3) if l not in (grow, shrink)):
                continue
            key = (e[grow], -e[shrink])
            if best_key is None or key < best_key:
                best, best_key = idx, key
        return best


class LaneTileSpace(SubSpace):
    """[grid, 1, 1, t] — t outputs per lane along one axis of a direct
    (non matrix-core) lowering; grid = ceil(extent / t)."""

    def __init__(self, extent, choices):
        super(LaneTileSpace, self).__init__()
        self.total = extent
        self.dim = 4
        ts = sorted(set(t for t in choices if 1 <= t <= extent))
        self.static_entities = [[ceil_div(extent, t), 1, 1, t] for t in ts] or [[extent, 1, 1, 1]]
        self.size = len(self.static_entities)
        self.directions = [(0, 3), (3, 0)]
        self.num_direction = 2
        self.type_key = "split"

    def next_entity(self, pos, d):
        if len(d) == 1:
            return (pos + d[0]) % self.size
        grow, _ = d
        step = 1 if grow == 3 else -1
        return min(max(pos + step, 0), self.size - 1)


def generate_inline_space(op_lst, down_graph, force_inline=False):
    inline_op_pos = [i for i, op in enumerate(op_lst) if able_inline(op, down_graph)]
    return InlineSpace(inline_op_pos, len(op_lst), force_inline=force_inline)


def generate_merge_space(op_lst, down_graph, force_merge=False):
    return MergeSpce(list(range(len(op_lst))), len(op_lst), force_merge=force_merge)


def generate_fuse_space(loops, groups):
    return FuseSpace(groups, loops)


def generate_split_space(extent, nparts, allow_non_divisible="off"):
    return SplitSpace(nparts, extent, allow_non_divisible=allow_non_divisible)


def generate_reorder_space(num_spatial_axis):
    return ReorderSpace(num_spatial_axis)


def generate_unroll_space(explicit=False):
    return UnrollSpace([0, 1, 512, 1500], explicit=explicit)


def _generic_space_intra_op(op, slevel, rlevel, groups, split_policy, unroll_policy, fuse_policy,
                            reorder_policy):
    """The target-independent space of flextensor/space.py:397-432."""
    space = Space()
    snames = [x.name for x in op.axis]
    sext = [x.extent for x in op.axis]
    rnames = [x.name for x in op.reduce_axis]
    rext = [x.extent for x in op.reduce_axis]
    if fuse_policy == "fuse_spatial":
        space.add_subspace("fuse_spatial", generate_fuse_space(snames, groups), "fuse")
    for i, (name, extent) in enumerate(zip(snames, sext)):
        space.add_subspace("split_{}_{}".format(name, i),
                           generate_split_space(extent, slevel, split_policy), "spatial")
    for i, (name, extent) in enumerate(zip(rnames, rext)):
        space.add_subspace("split_{}_{}".format(name, i),
                           generate_split_space(extent, rlevel, split_policy), "reduce")
    if reorder_policy == "last":
        space.add_subspace("reorder", generate_reorder_space(groups), "reorder")
    space.add_subspace("unroll", generate_unroll_space(explicit=(unroll_policy == "explicit")),
                       "unroll")
    return space


def generate_space_intra_op(op, down_graph, slevel=4, rlevel=3, groups=3, split_policy="off",
                            unroll_policy="off", fuse_policy="fuse_spatial",
                            reorder_policy="last", target=None):
    """Per-operator schedule space.

    With ``target="rocm"`` the gfx950 template owning ``op.kind`` defines the
    sub-spaces (see the module docstring); otherwise the reference's generic
    split/fuse/reorder/unroll space is produced.
    """
    if target == "rocm":
        from .templates import gfx950
        assert_print(slevel == 4 and rlevel == 3,
                     "the gfx950 templates use 4 spatial and 3 reduce levels")
        return gfx950.generate_space(op)
    return _generic_space_intra_op(op, slevel, rlevel, groups, split_policy, unroll_policy,
                                   fuse_policy, reorder_policy)


def generate_space_inter_op(op_lst, down_graph, force_inline=False, force_merge=False,
                            special_space=None):
    """Graph-level space: the inline flags plus any task-specific enumerated
    knobs (flextensor/space.py:435-452)."""
    space = Space()
    space.add_subspace("inline", generate_inline_space(op_lst, down_graph, force_inline), "inline")
    # the reference declares a "merge" key and leaves it unused (space.py:443-445); here it
    # decides whether a bias stage runs in the epilogue of the convolution before it
    mergeable = [i for i, op in enumerate(op_lst) if able_merge(op, down_graph)]
    if mergeable:
        space.add_subspace("merge", MergeSpce(mergeable, len(op_lst), force_merge=force_merge), "merge")
    for key, sspace in (special_space or {}).items():
        space.add_subspace(key, sspace, "special")
    return space
