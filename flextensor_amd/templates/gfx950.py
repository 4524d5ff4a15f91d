"""gfx950 (MI355X) kernel templates: schedule space and config -> kernel.

Where the reference turns a config dict into TVM schedule primitives
(flextensor/templates/cuda.py:390-661 for GPUs, templates/cpu.py:316-518 for
CPUs), this module turns the same dict into the ``-D`` constants of a
hand-written HIP kernel template plus launch geometry. Nothing here touches a
device: lowering is pure Python and can be unit-tested on a CPU.

Operator kinds and the template each one lowers to:

  gemm                   igemm_f32.hip  MODE 0 (MODE 2 for transposeB)
  conv2d_nchw            igemm_f32.hip  MODE 1 (implicit GEMM, padding folded
                                         into the gather; or PAD=0 over a
                                         materialised padded tensor)
  gemm_int8              gemm_i8.hip
  depthwise_conv2d_nchw  depthwise_f32.hip (direct; also what conv2d_nchw builds
                                         for one input channel per group)
  zero_pad2d             elementwise.hip   (only when not inlined)

Meaning of the config keys: see flextensor_amd/space.py.
"""
import json
import os

from ..space import (Space, SplitSpace, TileSplitSpace, LaneTileSpace, UnrollSpace, EnumSpace)
from ..utils import ceil_div

_HERE = os.path.dirname(os.path.abspath(__file__))

LDS_BYTES = 160 * 1024        # per workgroup on gfx950
MAX_ACC_REGS = 256            # accumulation VGPRs per lane
MAX_THREADS = 1024
NUM_XCD = 8
NUM_CUS = 256                 # compute units of one MI355X


class InvalidConfig(ValueError):
    """The config does not describe a kernel this template can build."""


_SOURCES = {}


def template_source(name):
    if name not in _SOURCES:
        with open(os.path.join(_HERE, name), "r") as f:
            _SOURCES[name] = f.read()
    return _SOURCES[name]


class KernelSpec(object):
    """One kernel of a plan, fully determined on the host.

    template     file name of the HIP source
    kernel       extern "C" symbol
    defines      dict of -D constants
    grid, block  launch geometry
    args         list of argument descriptors: ("buf", name) for a device
                 buffer bound by the plan, ("i32", value) / ("i64", value) /
                 ("u32", value) for scalars
    """

    def __init__(self, template, kernel, defines, grid, block, args, lds_bytes=0, note="",
                 workspace=None):
        # name -> (shape, dtype) of zero-initialised device buffers the plan
        # owns and the kernel leaves zeroed where it relies on zeros
        self.workspace = dict(workspace or {})
        self.template = template
        self.kernel = kernel
        self.defines = dict(defines)
        self.grid = tuple(grid)
        self.block = tuple(block)
        self.args = list(args)
        self.lds_bytes = lds_bytes
        self.note = note

    def options(self):
        return ["-DFT_%s=%s" % (k, v) for k, v in sorted(self.defines.items())]

    def source(self):
        return template_source(self.template)

    def __repr__(self):
        return "KernelSpec(%s %s grid=%s block=%s)" % (self.kernel, self.defines, self.grid, self.block)


# --------------------------------------------------------------------------
# GEMM view of an operator
# --------------------------------------------------------------------------

def _conv_steps(attrs):
    """Stride, padding and dilation constants of a convolution, rows (H) and columns (W)
    apart: the operator definitions take pairs (flextensor/nn/ops.py:448-459)."""
    return dict(CSTRH=attrs["stride"][0], CSTRW=attrs["stride"][1], CPADH=attrs["padding"][0],
                CPADW=attrs["padding"][1], CDILH=attrs["dilation"][0], CDILW=attrs["dilation"][1])


class GemmView(object):
    """M, N, K and addressing mode of a contraction-shaped operator."""

    def __init__(self, op, col_inlined=False):
        kind = op.kind
        self.kind = kind
        self.conv = None
        self.groups = 1
        self.trans_a = False
        if kind == "gemm":
            self.trans_a = bool(op.attrs.get("transposeA"))     # A stored [K][M] (ops.py:1093-1100)
            self.M, self.N = op.axis[0].extent, op.axis[1].extent
            self.K = op.reduce_axis[0].extent
            self.mode = 2 if op.attrs.get("transposeB") else 0
            self.dtype = "float32"
        elif kind == "batch_gemm":
            # one GEMM per batch entry: the batch index is the group index of the kernel
            self.groups = op.axis[0].extent
            self.trans_a = bool(op.attrs.get("transposeA"))
            self.M, self.N = op.axis[1].extent, op.axis[2].extent
            self.K = op.reduce_axis[0].extent
            self.mode = 2 if op.attrs.get("transposeB") else 0
            self.dtype = "float32"
        elif kind == "gemm_int8":
            self.M, self.N = op.axis[0].extent, op.axis[1].extent
            self.K = op.reduce_axis[0].extent
            self.mode = 0
            self.dtype = "int8"
        elif kind == "conv2d_nchw":
            a = op.attrs
            b, kout, p, q = [x.extent for x in op.axis]
            c = op.reduce_axis[0].extent
            s = op.reduce_axis[1].extent  # rw
            r = op.reduce_axis[2].extent  # rh
            _, _, h, w = a["in_shape"]
            groups = a["groups"]
            # one GEMM per group: c is already the per-group channel count
            self.M, self.N, self.K = kout // groups, b * p * q, c * r * s
            self.mode = 1
            self.dtype = "float32"
            self.groups = groups
            self.conv = dict(CB=b, CG=groups, CC=c * groups, CH=h, CW=w, CR=r, CS=s, CP=p, CQ=q,
                             **_conv_steps(a))
            # one image, 1x1 kernel, stride 1, no padding: O [K][H*W] = W [K][C] x X [C][H*W] in the
            # tensors' own layouts, a plain GEMM whose B rows load as 16-byte vectors
            self.pointwise = (b == 1 and groups == 1 and r == 1 and s == 1 and tuple(a["stride"]) == (1, 1)
                              and tuple(a["padding"]) == (0, 0))
        elif kind == "col_gemm":
            # the GEMM stage of an im2col convolution: one [Mg,K] x [K,N] product per group.
            # With the column matrix read through (inlined) it is the implicit GEMM over the
            # image; otherwise a batch of plain GEMMs over the stored columns.
            a = op.attrs
            groups = op.axis[0].extent
            self.M, self.N = op.axis[1].extent, op.axis[2].extent
            self.K = op.reduce_axis[0].extent
            self.groups = groups
            self.dtype = "float32"
            b, cin, h, w = a["in_shape"]
            r, sw = a["kernel"]
            p, q = a["out_hw"]
            self.conv = dict(CB=b, CG=groups, CC=cin, CH=h, CW=w, CR=r, CS=sw, CP=p, CQ=q, **_conv_steps(a))
            self.mode = 1 if col_inlined else 0
        else:
            raise InvalidConfig("operator kind %s has no GEMM view" % kind)
        # K as the kernels iterate it: fp32 pads the tail up to a multiple of
        # 16 (int8: 64) with zero-filling loads unless it already is a multiple
        # of 8.
        if min(self.M, self.N, self.K) < 1:
            raise InvalidConfig("empty operator: M, N, K = %d, %d, %d" % (self.M, self.N, self.K))
        if self.dtype == "int8":
            self.KP_options = [ceil_div(self.K, 64) * 64]
        else:
            self.KP = ceil_div(self.K, 16) * 16
            self.KP_options = [self.KP]
            if self.K % 8 == 0 and self.K % 16 != 0:
                # e.g. K = 72: unpadded for 32x32x2 tiles of 8 or 72, padded to 80 for 16x16x4
                self.KP_options.insert(0, self.K)
            if not any(kp % 32 == 0 or kp % 48 == 0 or kp % 72 == 0 for kp in self.KP_options):
                # an awkward K (400 = 16 channels x 5x5) only divides into LDS tiles of 8 or 16: every
                # tile is a round trip to memory, 25 in a row. Up to an eighth of zero padding (the load
                # predicates supply it) buys tiles of 32 .. 144: 416, 432, 448 for K = 400
                wider = {ceil_div(self.K, bk) * bk for bk in (32, 48, 64, 72, 144)}
                self.KP_options += sorted(kp for kp in wider if kp > self.KP and kp * 8 <= self.K * 9)
            return
        self.KP = self.KP_options[-1]


GEMM_KINDS = ("gemm", "gemm_int8", "conv2d_nchw", "batch_gemm", "col_gemm")

F32_BK = (8, 16, 32, 48, 64, 72, 128, 144)   # 72/144: whole 3x3 windows per LDS tile
I8_BK = (64, 128, 256)


def _gemm_space(view):
    space = Space()
    i8 = view.dtype == "int8"
    reps = (1, 2, 3, 4, 5, 6, 7, 8)
    space.add_subspace("split_m_0", TileSplitSpace(view.M, reps=reps), "spatial")
    space.add_subspace("split_n_1", TileSplitSpace(view.N, reps=reps), "spatial")
    bks = I8_BK if i8 else F32_BK
    max_split = 16

    def keep(e):
        return e[2] in bks and e[0] <= max_split

    rs = SplitSpace(3, view.KP_options[0], keep=keep)
    for other in view.KP_options[1:]:
        extra = SplitSpace(3, other, keep=keep)
        rs.static_entities = rs.static_entities + extra.static_entities
        rs._index = {tuple(e): i for i, e in enumerate(rs.static_entities)}
        rs.size = len(rs.static_entities)
    if rs.size == 0:
        raise InvalidConfig("K=%d has no admissible LDS tile extent" % view.K)
    space.add_subspace("split_k_0", rs, "reduce")
    space.add_subspace("unroll", UnrollSpace([1, 2, 3, 4, 5, 6, 7, 8], explicit=True,
                                               extra=() if i8 else [[8, 2], [8, 4], [8, 6], [8, 8]]),
                       "unroll")
    space.add_subspace("group_m", EnumSpace([[1], [2], [4], [8], [16]]), "fuse")
    # [xcd remap, K partitions inside the workgroup (1) or across workgroups (0)]
    # the third number: balanced K streaming with that many workgroups per compute unit (fp32 only)
    space.add_subspace("xcd_remap", EnumSpace([[1, 0, 0], [0, 0, 0], [1, 1, 0], [0, 1, 0]] if i8 else
                                            [[1, 0, 0], [0, 0, 0], [1, 1, 0], [0, 1, 0], [1, 0, 1], [1, 0, 2]]),
                       "reorder")
    return space


def _depthwise_space(op):
    space = Space()
    b, c, p, q = [x.extent for x in op.axis]
    space.add_subspace("split_b_0", LaneTileSpace(b, [1]), "spatial")
    space.add_subspace("split_c_1", LaneTileSpace(c, [1]), "spatial")
    space.add_subspace("split_h_2", LaneTileSpace(p, [1, 2, 4, 7, 8, 14]), "spatial")
    space.add_subspace("split_w_3", LaneTileSpace(q, [1, 2, 4]), "spatial")
    space.add_subspace("waves", EnumSpace([[1], [2], [4], [8]]), "fuse")
    return space


def generate_space(op):
    """Schedule space of one operator for gfx950."""
    if op.kind in GEMM_KINDS:
        return _gemm_space(GemmView(op))
    if op.kind == "depthwise_conv2d_nchw":
        return _depthwise_space(op)
    if op.kind in ("zero_pad2d", "bias_add_nchw", "bias_add_ghw", "im2col_nchw", "col2img_nchw"):
        return Space()
    raise InvalidConfig("no gfx950 template for operator kind %s" % op.kind)


# --------------------------------------------------------------------------
# special (task-level enumerated) knobs
# --------------------------------------------------------------------------

SPECIAL_DEFAULTS = {
    # fp32: [APAD, BPAD] in floats; APAD -1 = unpadded, XOR-swizzled A tile;
    # BPAD -1 = the padding that spreads the k-groups of one MFMA operand read
    # over disjoint banks (4 floats for 16x16x4, 8 for 32x32x2).
    # int8: [PAD bytes / 4, unused]
    # the default admits every pipeline depth (tiles straight into LDS need unpadded A rows), so
    # that an operator search under the graph level's defaults can reach them
    "lds_pad": [-1, -1],
    "nt_store": [0],
    "halo_shfl": [0],
    "lds_planes": [0],
    "lane_items": [1],
    "row_exchange": [0],
    # depthwise with several kernels per input channel: 1 = a lane computes its patch for all of them
    "kernel_fuse": [1],
    # 1x1 convolution, stride 1, no padding, one image: 1 = the GEMM addressing mode (the image is
    # the B matrix as it lies in memory, rows load as 16-byte vectors), 0 = the gather of the general case
    "image_as_matrix": [1],
    # K streaming: 1 = the arrival count and the look at the counter are a device-scope
    # release / acquire (what the memory model asks for; costs an L2 write-back and invalidate per
    # hand-off, +4.5 % on the 8x256x14x14 benchmark layer), 0 = relaxed device-scope atomics behind
    # an explicit wait for the slot stores (the measured trade-off the shipped entries use). Not in
    # the searched knobs: a task opts in with set_specific_space("sk_fenced", "enum", [[1]])
    "sk_fenced": [0],
}

# unroll entity [[depth, 1]] -> (LDS stages, prefetch distance in tiles);
# depth 5 = two stages with the fragment-prefetch pipeline (int8 GEMM)
# depth -> (LDS buffers, global prefetch distance); 5 = int8: MFMA fragment prefetch, fp32: tiles
# loaded straight into LDS; int8 only:
# 6 = tiles loaded straight into LDS (no staging registers), 7 = 6 with MFMA fragment prefetch,
# 8 = 7 with the main loop's instruction order written out (fragment reads and tile loads issued
# one at a time between the MFMAs);
# fp32: 6 and 7 = 5 with three and four LDS buffers (two and three tiles requested ahead)
PIPELINE = {1: (1, 1), 2: (2, 1), 3: (2, 2), 4: (2, 3), 5: (2, 1), 6: (2, 1), 7: (2, 1), 8: (2, 1)}


def special_knobs(kind):
    """Enumerated knobs a task of this operator kind carries by default; they
    are attached with Task.set_specific_space and searched at graph level."""
    if kind == "pointwise_conv2d_nchw":
        # a 1x1 / stride 1 / unpadded convolution over one image (the task tells: the operator kind
        # is conv2d_nchw like any other convolution's)
        return {"lds_pad": [[-1, -1], [4, -1], [4, 8], [4, 4], [0, 0], [8, -1], [-1, 0]],
                "image_as_matrix": [[1], [0]]}
    if kind in ("gemm", "conv2d_nchw", "batch_gemm", "col_gemm"):
        return {"lds_pad": [[-1, -1], [4, -1], [4, 8], [4, 4], [0, 0], [8, -1], [-1, 0]]}
    if kind == "gemm_int8":
        return {"lds_pad": [[-1, 0], [4, 0], [0, 0], [8, 0]],
                "nt_store": [[0], [1], [2], [3], [4], [5], [6], [7]]}
    if kind == "depthwise_conv2d_nchw":
        return {"nt_store": [[0], [1], [2], [3]], "halo_shfl": [[0], [1]], "lds_planes": [[0], [1], [2], [4], [8]],
                "lane_items": [[1], [2], [3], [4], [6], [8]], "row_exchange": [[0], [1], [2], [3], [4]],
                "kernel_fuse": [[1], [0]]}
    return {}


def _special(graph_special, name):
    if graph_special and name in graph_special:
        return list(graph_special[name])
    return list(SPECIAL_DEFAULTS[name])


# --------------------------------------------------------------------------
# lowering
# --------------------------------------------------------------------------

def _one(config, key, n, what):
    lst = config.get(key) or []
    if len(lst) != n:
        raise InvalidConfig("%s: expected %d '%s' entries, got %d" % (what, n, key, len(lst)))
    return lst


def _lower_gemm(op, config, special, out_name, in_names, materialized_pad=False, bias_name=None,
                through=(), merged_out=None):
    view = GemmView(op, col_inlined="im2col_nchw" in through)
    if getattr(view, "pointwise", False) and int(_special(special, "image_as_matrix")[0]) \
            and bias_name is None and merged_out is None:
        view.mode = 0        # A = weight [K][C], B = image [C][H*W], C = output [K][H*W]
    if bias_name is not None and view.mode != 1 and op.kind != "col_gemm":
        raise InvalidConfig("only the convolution has a bias epilogue")
    if merged_out is not None and not (op.kind == "col_gemm" and merged_out == "col2img_nchw"):
        raise InvalidConfig("stage %s cannot run in the stores of %s" % (merged_out, op.kind))
    if merged_out is not None and view.mode != 1 and view.conv["CB"] != 1:
        # for one image [groups][M][P*Q] is NCHW already; a batch interleaves the images
        raise InvalidConfig("col2img merges into the GEMM that reads the image itself")
    sp = _one(config, "spatial", 2, op.kind)
    rd = _one(config, "reduce", 1, op.kind)
    (gm, wm, rm, mfm), (gn, wn, rn, mfn) = [list(map(int, x)) for x in sp]
    splitk, kiters, bk = [int(x) for x in rd[0]]
    depth = int((config.get("unroll") or [[2, 1]])[0][0])
    if depth not in PIPELINE:
        raise InvalidConfig("pipeline depth %d is not available" % depth)
    stages, pd = PIPELINE[depth]
    if view.dtype != "int8" and depth in (6, 7):
        stages = depth - 3        # fp32: 6 and 7 = tiles straight into LDS with three and four buffers
    # fp32 depth 8: as 5 (two buffers), and the first operands of the next tile are read from LDS
    # right behind the barrier, ahead of the last MFMAs of the current tile
    frag_prefetch = view.dtype != "int8" and depth == 8
    # with it, the second number of the unroll entry is the number of k blocks over which the
    # loads of the next tile are spread (1 = all in front of the tile's first MFMAs)
    load_spread = int((config.get("unroll") or [[2, 1]])[0][1]) if frag_prefetch else 1
    group_m = int((config.get("fuse") or [[4]])[0][0])
    ro = list((config.get("reorder") or [[1, 0]])[0]) + [0, 0]
    xcd, in_wg, stream_k = int(ro[0]), int(ro[1]), int(ro[2])
    i8 = view.dtype == "int8"
    waves_k = 1
    if in_wg and splitk > 1:
        waves_k, splitk = splitk, 1

    if mfm != mfn or mfm not in (16, 32):
        raise InvalidConfig("MFMA edge must be 16 or 32 and equal on both axes")
    if min(wm, rm, wn, rn, splitk, kiters, bk, group_m) < 1:
        raise InvalidConfig("non-positive factor")
    nwaves = wm * wn * waves_k
    if nwaves * 64 > MAX_THREADS:
        raise InvalidConfig("more than 16 wavefronts per workgroup")
    bm, bn = wm * rm * mfm, wn * rn * mfn
    if gm != ceil_div(view.M, bm) or gn != ceil_div(view.N, bn):
        raise InvalidConfig("grid level does not match ceil(extent / tile)")
    nacc = rm * rn * (mfm * mfm // 64)
    if nacc > MAX_ACC_REGS:
        raise InvalidConfig("accumulators need %d registers per lane" % nacc)
    kp = splitk * waves_k * kiters * bk
    if kp not in view.KP_options:
        raise InvalidConfig("reduce split does not multiply to K")
    nt = wm * wn * 64          # threads of one k-group
    D = dict(M=view.M, N=view.N, K=view.K, KP=kp, MFMA=mfm, WAVES_M=wm, WAVES_N=wn, REP_M=rm,
             REP_N=rn, BK=bk, STAGES=stages, GROUP_M=group_m, XCD_REMAP=xcd)

    if i8:
        if stream_k:
            # the grid-level split (integer atomics: exact, any order) and the in-workgroup split
            # cover the int8 operator; the balanced K streaming protocol is an fp32 path
            raise InvalidConfig("int8 GEMM splits K across workgroups or wavefront groups, not by K streaming")
        mfma_k = 32 if mfm == 32 else 64
        if bk % mfma_k != 0:
            raise InvalidConfig("BK must be a multiple of the MFMA K extent")
        if view.K % 16 != 0 and depth >= 6:
            # rows that are not 16-byte aligned: chunks are put together from dword or byte loads in
            # registers, which the loads that write LDS directly cannot do
            raise InvalidConfig("int8 tiles straight into LDS need K to be a multiple of 16")
        pad = int(_special(special, "lds_pad")[0])
        pad = -1 if pad < 0 else pad * 4
        if pad >= 0 and pad % 16 != 0:
            raise InvalidConfig("int8 LDS padding must be a multiple of 16 bytes")
        if view.M * view.K >= 2 ** 31 or view.N * view.K >= 2 ** 31:
            raise InvalidConfig("operands of 2 GiB or more are not addressable by the buffer loads")
        if depth >= 6:
            if pad > 0 or (bm * bk // 16) % nt or (bn * bk // 16) % nt:
                raise InvalidConfig("direct-to-LDS tiles need unpadded rows and whole rounds of 16-byte chunks")
            if depth == 8:
                nm, nr, loads = rm * rn, rm + rn, (bm + bn) * bk // 16 // nt
                if (bk // mfma_k) % 2 or nm // 4 + nr > nm or nm // 4 + loads > nm:
                    raise InvalidConfig("the written-out schedule needs an even number of k-steps per tile "
                                        "and enough MFMAs per k-step to interleave with")
        elif (ceil_div(bm * bk // 16, nt) + ceil_div(bn * bk // 16, nt)) * 4 * pd > 160:
            raise InvalidConfig("global->LDS staging needs too many registers")
        lds = max(waves_k * stages * (bm + bn) * (bk + max(pad, 0)), (waves_k - 1) * nt * nacc * 4)
        if lds > LDS_BYTES:
            raise InvalidConfig("LDS tile needs %d bytes" % lds)
        # nt_store: bit 0 = non-temporal stores, bit 1 = transposed MFMA so that lanes store 128-bit rows,
        # bit 2 = the last tile multiplied block by block, every block stored as soon as it is complete
        store_mode = int(_special(special, "nt_store")[0])
        if store_mode & 2 and view.N % 4 != 0:
            raise InvalidConfig("128-bit C stores need N to be a multiple of 4")
        if store_mode & 4 and (depth != 7 or bk != 2 * mfma_k or kp // bk < 2 or splitk * waves_k != 1):
            raise InvalidConfig("early stores come with pipeline depth 7, two k-steps per tile, two tiles or more, "
                                "and an undivided K")
        D.update(PAD=pad, PD=pd, FRAGPF=1 if depth == 5 else 0, NT_STORE=store_mode & 1)
        if depth >= 6:
            D.update(DTL=depth - 5)
        if store_mode & 2:
            D.update(CVEC=1)
        if store_mode & 4:
            D.update(EARLYST=1)
        specs = []
        if splitk > 1:
            # partial sums meet in C: zero it first (the fill writes zero bit patterns, whatever the type)
            D.update(SPLITK=splitk)
            nout = view.M * view.N
            specs.append(KernelSpec("elementwise.hip", "fill_zero_f32", {},
                                    (min(ceil_div(ceil_div(nout, 4), 256), 2048), 1, 1), (256, 1, 1),
                                    [("buf", out_name), ("i32", nout)], note="split-K zero fill"))
        if waves_k > 1:
            D.update(WAVES_K=waves_k)
        grid = (gm * gn * splitk, 1, 1)
        specs.append(KernelSpec("gemm_i8.hip", "gemm_i8", D, grid, (nt * waves_k, 1, 1),
                                [("buf", in_names[0]), ("buf", in_names[1]), ("buf", out_name)]))
        return specs

    kblk = 4 * (64 // mfm)
    if bk % kblk != 0:
        raise InvalidConfig("BK must be a multiple of %d for this MFMA shape" % kblk)
    apad, bpad = [int(x) for x in _special(special, "lds_pad")[:2]]
    bpad_auto = bpad < 0
    if bpad < 0:
        bpad = 4 if mfm == 16 else 8
    if apad < -1 or (apad >= 0 and apad % 4 != 0) or bpad % 4 != 0:
        raise InvalidConfig("fp32 LDS padding must keep 16-byte alignment")
    av = 4 if view.K % 4 == 0 else 1
    if view.trans_a:
        av = 4 if view.M % 4 == 0 else 1      # vectors run along M, the contiguous axis of a [K][M] operand
    if view.mode == 0:
        bv = 4 if view.N % 4 == 0 else 1
    elif view.mode == 2:
        bv = av
    else:
        bv = 1
    dtl = depth >= 5          # fp32: tiles loaded straight into LDS
    if dtl and view.trans_a and (bm % 64 or av != 4):
        raise InvalidConfig("direct-to-LDS tiles of a transposed A operand need tile rows of a multiple of 64 "
                            "and M a multiple of 4")
    if dtl:
        if view.mode == 0 and view.N % 4 == 0 and bn % 64 == 0 and (bpad_auto or bpad == 0):
            bv, bpad = 4, 0   # B in 16-byte chunks too: unpadded rows, columns swizzled by k
        elif view.mode != 2:
            bv = 1            # B goes one float per lane
        if av != 4 or apad > 0 or (bm * bk // 4) % 64:
            raise InvalidConfig("direct-to-LDS tiles need 16-byte A chunks in whole wavefronts and unpadded A rows")
        if view.mode == 2 and (bv != 4 or (bn * bk // 4) % 64):
            raise InvalidConfig("direct-to-LDS tiles need 16-byte B chunks in whole wavefronts")
        if view.mode != 2 and bv == 1 and bn % 64:
            # B one float per lane: a wavefront writes 64 consecutive floats, so rows that are
            # not multiples of 64 floats land unpadded, in whole wavefronts per tile
            if bpad_auto:
                bpad = 0
            if bpad != 0 or (bn * bk) % 64:
                raise InvalidConfig("direct-to-LDS tiles with rows that are not multiples of 64 floats need "
                                    "unpadded B rows and whole wavefronts of floats per tile")
    sa = bk + max(apad, 0)
    if view.mode == 2:
        lds_b = bn * sa
    else:
        lds_b = bk * (bn + bpad)
    lds = max(waves_k * stages * 4 * (bm * sa + lds_b), (waves_k - 1) * nt * nacc * 4)
    if stream_k:
        lds += 16             # the arrival word of the K-streaming exchange
    if lds > LDS_BYTES:
        raise InvalidConfig("LDS tile needs %d bytes" % lds)
    # staging registers for the global->LDS copy must stay reasonable
    ea = ceil_div(bm * bk // av, nt)
    eb = ceil_div((bn * bk) // bv, nt)
    if not dtl and (ea * av + eb * bv) * pd > 160:
        raise InvalidConfig("global->LDS staging needs too many registers")
    if dtl and stages > 2 and ((bm * bk // av) % nt or ((bn * bk) // bv) % nt or (stages - 2) * (ea + eb) > 63):
        raise InvalidConfig("more than two direct-to-LDS buffers need whole rounds of loads per tile, "
                            "at most 63 of them in flight")
    # bytes behind the two buffer descriptors (A_BYTES / B_BYTES of the template) and of C: in MODE 1
    # B is the image itself, larger than K x N when the stride exceeds the kernel, and larger
    # still once the padding is materialised
    a_bytes = view.groups * view.M * view.K * 4
    if view.mode == 1:
        cv = view.conv
        grow_h, grow_w = (2 * cv["CPADH"], 2 * cv["CPADW"]) if materialized_pad else (0, 0)
        b_bytes = cv["CB"] * cv["CC"] * (cv["CH"] + grow_h) * (cv["CW"] + grow_w) * 4
    else:
        b_bytes = view.groups * view.K * view.N * 4
    if max(a_bytes, b_bytes, view.groups * view.M * view.N * 4) >= 2 ** 31:
        raise InvalidConfig("operands of 2 GiB or more are not addressable by the buffer loads")
    D.update(MODE=view.mode, SPLITK=splitk, WAVES_K=waves_k, APAD=apad, BPAD=bpad, AV=av, BV=bv, PD=pd)
    if view.trans_a:
        D.update(TA=1)
    if dtl:
        D.update(DTL=1)
    if frag_prefetch:
        D.update(FPF=1)
        if load_spread < 1 or (load_spread > 1 and load_spread > bk // kblk - 1):
            raise InvalidConfig("the loads of the next tile spread over at most all but the last k block")
        if load_spread > 1:
            D.update(LSPREAD=load_spread)
    specs = []
    if view.mode == 1:
        conv = dict(view.conv)
        if materialized_pad:
            conv["CH"] += 2 * conv["CPADH"]
            conv["CW"] += 2 * conv["CPADW"]
            conv["CPADH"] = conv["CPADW"] = 0
        D.update(conv)
        if op.kind == "col_gemm" and merged_out is None:
            D.update(COLOUT=1)            # C stays [groups][M][N] for the col2img stage
        # A = weight, B = image
        a_name, b_name = in_names[1], in_names[0]
    else:
        a_name, b_name = in_names[0], in_names[1]
        if op.kind in ("col_gemm", "conv2d_nchw"):
            a_name, b_name = in_names[1], in_names[0]      # A = weight, B = stored columns / the image
        if view.groups > 1:
            D.update(CG=view.groups)      # batched GEMM
    if splitk > 1:
        nout = view.M * view.N * view.groups
        specs.append(KernelSpec("elementwise.hip", "fill_zero_f32", {},
                                (min(ceil_div(ceil_div(nout, 4), 256), 2048), 1, 1), (256, 1, 1),
                                [("buf", out_name), ("i32", nout)], note="split-K zero fill"))
    args = [("buf", a_name), ("buf", b_name), ("buf", out_name)]
    if bias_name is not None:
        D.update(HAS_BIAS=1)       # C = A*B + bias[row], added once whatever the K division
    workspace = {}
    if stream_k:
        # balanced K streaming: stream_k workgroups per compute unit share the
        # (tile, k-tile) units evenly; see the template for the protocol
        if stream_k < 0 or splitk != 1 or waves_k != 1:
            raise InvalidConfig("K streaming excludes the other K splits")
        units = gm * gn * view.groups * (kp // bk)
        per = ceil_div(units, NUM_CUS * stream_k)
        ngrid = ceil_div(units, per)
        if xcd:
            ngrid = ceil_div(ngrid, NUM_XCD) * NUM_XCD   # renumbering by XCD needs whole rounds
        D.update(SK_PER=per)
        if int(_special(special, "sk_fenced")[0]):
            D.update(SK_FENCED=1)
        grid = (ngrid, 1, 1)
        workspace = {out_name + "_parts": ((ngrid * 2 * nt * nacc,), "float32"),
                     out_name + "_count": ((gm * gn * view.groups,), "int32")}
        args += [("buf", out_name + "_parts"), ("buf", out_name + "_count")]
    else:
        grid = (gm * gn * splitk * view.groups, 1, 1)
    if bias_name is not None:
        args.append(("buf", bias_name))
    specs.append(KernelSpec("igemm_f32.hip", "igemm_f32", D, grid, (nt * waves_k, 1, 1), args,
                            workspace=workspace))
    return specs


def _lower_depthwise(op, config, special, out_name, in_names, materialized_pad=False, bias_name=None):
    sp = _one(config, "spatial", 4, op.kind)
    th, tw = int(sp[2][3]), int(sp[3][3])
    if int(sp[0][3]) != 1 or int(sp[1][3]) != 1:
        raise InvalidConfig("depthwise lanes own one batch entry and one channel")
    waves = int((config.get("fuse") or [[4]])[0][0])
    if waves < 1 or waves * 64 > MAX_THREADS:
        raise InvalidConfig("bad wavefront count")
    a = op.attrs
    b, cout, p, q = [x.extent for x in op.axis]
    s_ext = op.reduce_axis[0].extent  # rw
    r_ext = op.reduce_axis[1].extent  # rh
    _, c, h, w = a["in_shape"]
    if th < 1 or tw < 1 or th > p or tw > q:
        raise InvalidConfig("lane patch larger than the output plane")
    if int(sp[2][0]) != ceil_div(p, th) or int(sp[3][0]) != ceil_div(q, tw):
        raise InvalidConfig("grid level does not match ceil(extent / patch)")
    (st_h, st_w), (pad_h, pad_w), (dl_h, dl_w) = a["stride"], a["padding"], a["dilation"]   # rows, columns
    if materialized_pad:
        h, w, pad_h, pad_w = h + 2 * pad_h, w + 2 * pad_w, 0, 0
    ih_t = (th - 1) * st_h + (r_ext - 1) * dl_h + 1
    iw_t = (tw - 1) * st_w + (s_ext - 1) * dl_w + 1
    # the 128-bit input path requests every row of the patch before the first is used
    vec_rows = (tw == 4 and st_w <= 2 and w % 4 == 0 and q * st_w == w and pad_w + 4 * st_w <= iw_t)
    # kernel_fuse: with several kernels per input channel a lane computes its patch for all of them
    fm = a["factor"] if int(_special(special, "kernel_fuse")[0]) else 1
    # lane_items: patches per lane, all requested before the first is computed
    ipl = int(_special(special, "lane_items")[0])
    if ipl < 1 or ipl > 16:
        raise InvalidConfig("lane_items is 1 .. 16")
    if th * tw + ipl * (ih_t * iw_t + fm * r_ext * s_ext) > 220:
        raise InvalidConfig("lane patches need too many registers")
    if max(b * c * h * w, b * cout * p * q) * 4 >= 2 ** 31:
        raise InvalidConfig("tensors of 2 GiB or more are not addressable by the buffer accesses")
    nt = waves * 64
    items = b * (cout // fm) * ceil_div(p, th) * ceil_div(q, tw)
    ldsp = int(_special(special, "lds_planes")[0])
    nt_mode = int(_special(special, "nt_store")[0])     # bit 0: non-temporal stores, bit 1: non-temporal loads
    steps = dict(STRH=st_h, STRW=st_w, PADH=pad_h, PADW=pad_w, DILH=dl_h, DILW=dl_w)
    args = [("buf", in_names[0]), ("buf", in_names[1]), ("buf", out_name)]
    if bias_name is not None:
        # the bias stage merged into the kernel: added to every result in the store (ops.py:673-677)
        steps["HAS_BIAS"] = 1
        args.append(("buf", bias_name))
    if ldsp:
        # plane-staged variant: whole planes through LDS in copy order; the lane patch knobs do not apply
        if not (st_h == st_w == 1 and dl_h == dl_w == 1 and r_ext == 3 and s_ext == 3 and pad_h == pad_w == 1
                and p == h and q == w and w % 4 == 0 and a["factor"] == 1):
            raise InvalidConfig("plane staging needs a same-size 3x3 stride-1 pad-1 layer with rows of whole vectors")
        if ldsp < 0 or (ldsp * (h + 2) * (w + 8) + ldsp * 12) * 4 > LDS_BYTES:
            raise InvalidConfig("staged planes do not fit the LDS")
        D = dict(NT=nt, TH=th, TW=tw, NT_STORE=nt_mode & 1, NT_LOAD=nt_mode >> 1, SHFL=0, LDSP=ldsp,
                 CB=b, CC=c, CH=h, CW=w, CR=r_ext, CS=s_ext, FACT=1, CP=p, CQ=q, **steps)
        return [KernelSpec("depthwise_f32.hip", "depthwise_f32", D, (ceil_div(b * cout, ldsp), 1, 1),
                           (nt, 1, 1), args)]
    wx = int(_special(special, "row_exchange")[0])
    if wx:
        # row-exchange variant: a wavefront owns rpi * wx rows of one plane (rpi whole rows per load
        # instruction), loads each 16-byte chunk once and passes rows between lanes through its own
        # LDS window; the lane patch knobs do not apply
        if not (st_h == st_w == 1 and dl_h == dl_w == 1 and r_ext == 3 and s_ext == 3 and pad_h == pad_w == 1
                and p == h and q == w and w % 4 == 0 and a["factor"] == 1):
            raise InvalidConfig("row exchange needs a same-size 3x3 stride-1 pad-1 layer with rows of whole vectors")
        q4 = w // 4
        if wx < 1 or wx > 8 or 2 * q4 > 64:
            raise InvalidConfig("row exchange: 1 .. 8 chunks per lane, rows of at most 128 floats")
        # rows per instruction: as many as fit 64 lanes, fewer when that makes the spans tile the plane
        rpi_max = min(64 // q4, h)
        rpi = max([r for r in range(1, rpi_max + 1) if h % (r * wx) == 0] or [0])
        if rpi * 4 < rpi_max * 3:
            rpi = rpi_max         # too few lanes would carry work: ragged last span instead
        rows = rpi * wx
        if (waves * (rows + 2) * q4 + 64) * 16 > LDS_BYTES:      # 64 chunks of slack for the idle lanes' reads
            raise InvalidConfig("row-exchange windows do not fit the LDS")
        D = dict(NT=nt, TH=th, TW=tw, NT_STORE=nt_mode & 1, NT_LOAD=nt_mode >> 1, SHFL=0, WX=wx, WXR=rpi,
                 CB=b, CC=c, CH=h, CW=w, CR=r_ext, CS=s_ext, FACT=1, CP=p, CQ=q, **steps)
        return [KernelSpec("depthwise_f32.hip", "depthwise_f32", D,
                           (ceil_div(b * cout * ceil_div(h, rows), waves), 1, 1), (nt, 1, 1), args)]
    shfl = int(_special(special, "halo_shfl")[0])
    tiles_w = ceil_div(q, tw)
    if shfl:
        if not (vec_rows and st_w == 1 and s_ext == 3 and dl_w == 1 and pad_w == 1 and tiles_w <= 64):
            raise InvalidConfig("the shuffled halo needs the 128-bit input path of a 3-wide pad-1 layer")
        lanes = (64 // tiles_w) * tiles_w
        grid_x = ceil_div(ceil_div(items, lanes), waves * ipl)
    else:
        grid_x = ceil_div(items, nt * ipl)
    D = dict(NT=nt, TH=th, TW=tw, NT_STORE=nt_mode & 1, NT_LOAD=nt_mode >> 1, SHFL=shfl,
             CB=b, CC=c, CH=h, CW=w, CR=r_ext, CS=s_ext, FACT=a["factor"], CP=p, CQ=q, **steps)
    if ipl > 1:
        D.update(IPL=ipl)
    if fm > 1:
        D.update(MFUSE=1)
    return [KernelSpec("depthwise_f32.hip", "depthwise_f32", D, (grid_x, 1, 1), (nt, 1, 1), args)]


def _lower_pad(op, out_name, in_names):
    b, c, ph, pw = [x.extent for x in op.axis]
    pt, pb, pl, pr = op.attrs["padding"]          # rows above / below, columns left / right
    h, w = ph - pt - pb, pw - pl - pr
    D = dict(PADK=1, PB=b * c, CH=h, CW=w, PT=pt, PBOT=pb, PL=pl, PR=pr)
    n = b * c * ph * pw
    return [KernelSpec("elementwise.hip", "zero_pad2d_f32", D, (ceil_div(n, 256), 1, 1),
                       (256, 1, 1), [("buf", in_names[0]), ("buf", out_name)])]


def _lower_bias(op, out_name, in_names):
    if op.kind == "bias_add_ghw":
        # [groups][Mg][N] is one image of groups*Mg channels with N elements each
        g, mg, hw = [x.extent for x in op.axis]
        b, c, h, w = 1, g * mg, 1, hw
    else:
        b, c, h, w = [x.extent for x in op.axis]
    n = b * c * h * w
    return [KernelSpec("elementwise.hip", "bias_add_nchw_f32", {},
                       (min(ceil_div(n, 256), 4096), 1, 1), (256, 1, 1),
                       [("buf", in_names[0]), ("buf", in_names[1]), ("buf", out_name),
                        ("i32", n), ("i32", h * w), ("i32", c)])]


def _conv_defines(attrs, materialized_pad):
    b, cin, h, w = attrs["in_shape"]
    steps = _conv_steps(attrs)
    if materialized_pad:
        h, w = h + 2 * steps["CPADH"], w + 2 * steps["CPADW"]
        steps["CPADH"] = steps["CPADW"] = 0
    groups = attrs["groups"]
    return dict(COLK=1, CB=b, CG=groups, CC=cin, CH=h, CW=w, CR=attrs["kernel"][0], CS=attrs["kernel"][1],
                CP=attrs["out_hw"][0], CQ=attrs["out_hw"][1], MG=attrs["out_channel"] // groups, **steps)


def _lower_im2col(op, out_name, in_names, materialized_pad):
    g, k, n = [x.extent for x in op.axis]
    total = g * k * n
    return [KernelSpec("elementwise.hip", "im2col_nchw_f32", _conv_defines(op.attrs, materialized_pad),
                       (min(ceil_div(total, 256), 16384), 1, 1), (256, 1, 1),
                       [("buf", in_names[0]), ("buf", out_name)])]


def _lower_col2img(op, out_name, in_names):
    b, c, p, q = [x.extent for x in op.axis]
    g, mg, _ = op.input_tensors[0].shape
    # only the output geometry matters to this kernel; the image constants are placeholders
    D = dict(COLK=1, CB=b, CG=g, CC=g, CH=1, CW=1, CR=1, CS=1, CSTRH=1, CSTRW=1, CPADH=0, CPADW=0,
             CDILH=1, CDILW=1, CP=p, CQ=q, MG=mg)
    total = b * c * p * q
    return [KernelSpec("elementwise.hip", "col2img_nchw_f32", D,
                       (min(ceil_div(total, 256), 16384), 1, 1), (256, 1, 1),
                       [("buf", in_names[0]), ("buf", out_name)])]


def lower(op, config, special, out_name, in_names, materialized_pad=False, bias_name=None,
          through=(), merged_out=None):
    """Config of one operator -> list of KernelSpec (raises InvalidConfig).
    ``bias_name``: buffer of a per-channel bias merged into the epilogue;
    ``through``: kinds of the inlined producers the operator reads through;
    ``merged_out``: kind of a layout stage merged into the operator's stores."""
    if op.kind in GEMM_KINDS:
        return _lower_gemm(op, config, special, out_name, in_names, materialized_pad, bias_name,
                           through, merged_out)
    if merged_out is not None:
        raise InvalidConfig("operator kind %s takes no merged stage" % op.kind)
    if op.kind == "depthwise_conv2d_nchw":
        return _lower_depthwise(op, config, special, out_name, in_names, materialized_pad, bias_name)
    if bias_name is not None:
        raise InvalidConfig("operator kind %s has no bias epilogue" % op.kind)
    if op.kind == "im2col_nchw":
        return _lower_im2col(op, out_name, in_names, materialized_pad)
    if op.kind == "col2img_nchw":
        return _lower_col2img(op, out_name, in_names)
    if op.kind in ("bias_add_nchw", "bias_add_ghw"):
        return _lower_bias(op, out_name, in_names)
    if op.kind == "zero_pad2d":
        return _lower_pad(op, out_name, in_names)
    raise InvalidConfig("no gfx950 template for operator kind %s" % op.kind)


# --------------------------------------------------------------------------
# default (untuned) configs
# --------------------------------------------------------------------------

def _empty_config():
    return {k: [] for k in Space.valid_type_keys}


def default_config(op):
    """A reasonable untuned config: what schedule_with_config falls back to
    when a task has no tuned entry, and the seed point of the search."""
    cfg = _empty_config()
    if op.kind in GEMM_KINDS:
        view = GemmView(op)
        i8 = view.dtype == "int8"

        def tile(extent, want, mf):
            """[grid, waves, reps, mfma] with a tile close to ``want``."""
            w, r = 1, 1
            while w * r * mf * 2 <= want and w * r * mf * 2 <= max(extent, mf):
                if w < 2:
                    w *= 2
                else:
                    r *= 2
            return [ceil_div(extent, w * r * mf), w, r, mf]

        mf = 32 if min(view.M, view.N) >= 64 else 16
        # the largest square-ish tile that still yields one workgroup per CU
        want = 256 if i8 else 128
        while True:
            tm, tn = tile(view.M, want, mf), tile(view.N, want, mf)
            if tm[0] * tn[0] >= 256 or want <= mf:
                break
            want //= 2
        cfg["spatial"] = [tm, tn]
        bks = I8_BK if i8 else F32_BK
        kblk = (32 if mf == 32 else 64) if i8 else 4 * (64 // mf)
        bk = None
        for cand in sorted(bks, reverse=True):
            if view.KP % cand == 0 and cand % kblk == 0 and cand <= (64 if i8 else 32):
                bk = cand
                break
        if bk is None:
            for cand in sorted(bks):
                if view.KP % cand == 0 and cand % kblk == 0:
                    bk = cand
                    break
        if bk is None:
            raise InvalidConfig("K=%d has no admissible LDS tile extent" % view.K)
        cfg["reduce"] = [[1, view.KP // bk, bk]]
        cfg["unroll"] = [[2, 1]] if i8 else [[3, 1]]
        cfg["fuse"] = [[4]]
        cfg["reorder"] = [[1, 0, 0]]
    elif op.kind == "depthwise_conv2d_nchw":
        b, c, p, q = [x.extent for x in op.axis]
        th = 4 if p >= 4 else 1
        tw = 4 if q >= 4 else 1
        cfg["spatial"] = [[b, 1, 1, 1], [c, 1, 1, 1], [ceil_div(p, th), 1, 1, th],
                          [ceil_div(q, tw), 1, 1, tw]]
        cfg["fuse"] = [[4]]
    return cfg


def seed_configs(op, limit=24):
    """Points worth measuring before the random warm-up: the default config
    and variations of it along the knobs that decided the hand-tuned shapes
    (tile aspect and MFMA edge, LDS tile extent incl. whole 3x3 windows,
    pipeline depth incl. tiles straight into LDS, K streaming when the tiles
    are fewer than the compute units, and for layers with few tiles and a
    long K a grid-level K split sized to fill the compute units, or with
    small tiles wavefront groups that share K inside the workgroup; a third
    of the points is kept for those). The variations are entities of the op's
    space (the default config itself need not be: it may waste more of an
    edge tile than the space admits); points the templates refuse are
    dropped by the caller."""
    base = default_config(op)
    if op.kind not in GEMM_KINDS:
        return [base]
    view = GemmView(op)
    i8 = view.dtype == "int8"
    out = [base]

    def tile(extent, w, r, mf):
        return [ceil_div(extent, w * r * mf), w, r, mf]

    if i8:
        shapes = [((4, 4, 16), (2, 8, 16)), ((4, 4, 16), (4, 4, 16)), ((4, 2, 32), (4, 2, 32))]
        bks, depths, streams = [128, 64], [7, 6, 2], [0]
    else:
        shapes = [((4, 1, 16), (4, 1, 16)), ((4, 1, 32), (2, 1, 32)), ((2, 1, 32), (2, 1, 32)),
                  ((4, 1, 16), (1, 1, 16)), ((4, 1, 16), (2, 1, 16)), ((2, 2, 16), (4, 1, 16)),
                  ((2, 1, 16), (4, 1, 16))]
        bks = [b for b in (144, 72, 64, 48, 32) if b in F32_BK]
        depths, streams = [8, 5, 3, 2, 1], [0, 1]
    def in_space(extent, t):
        # the tile space's own rules: no tile a smaller one covers as well, bounded edge waste
        size = t[1] * t[2] * t[3]
        if t[0] == 1:
            return size - extent < t[3]
        return t[0] * size - extent <= 0.25 * extent or t[0] * size - extent < t[3]

    split_seeds = []
    for (m_w, m_r, mf), (n_w, n_r, _) in shapes:
        tm, tn = tile(view.M, m_w, m_r, mf), tile(view.N, n_w, n_r, mf)
        if not (in_space(view.M, tm) and in_space(view.N, tn)):
            continue
        tiles = tm[0] * tn[0] * view.groups
        for bk in bks:
            kps = [kp for kp in view.KP_options if kp % bk == 0]
            if not kps:
                continue
            # K streaming first where the tiles alone cannot fill the compute units
            order = [(d, st) for st in (streams[::-1] if tiles < NUM_CUS else streams) for d in depths]
            for depth, stream in order:
                if not (stream and (i8 or tiles >= 2 * NUM_CUS)):
                    cfg = _empty_config()
                    cfg["spatial"] = [tm, tn]
                    cfg["reduce"] = [[1, kps[0] // bk, bk]]
                    cfg["unroll"] = [[depth, 1]]
                    cfg["fuse"] = [[8]]
                    cfg["reorder"] = [[1, 0, stream]]
                    out.append(cfg)
                if depth == depths[0] and stream == 0 and tiles * 2 <= NUM_CUS:
                    # few tiles and a long K (weights streamed past a small image): K parts across
                    # workgroups, as many as fill the compute units
                    split = 1
                    while split * 2 * tiles <= NUM_CUS and split < 16 and (kps[0] // bk) % (split * 2) == 0:
                        split *= 2
                    if split > 1:
                        cfg = _empty_config()
                        cfg["spatial"] = [tm, tn]
                        cfg["reduce"] = [[split, kps[0] // (bk * split), bk]]
                        cfg["unroll"] = [[depth, 1]]
                        cfg["fuse"] = [[8]]
                        cfg["reorder"] = [[1, 0, 0]]
                        split_seeds.append(cfg)
    group_seeds = []
    if not i8:
        # a few small tiles and a long K (1x1 layers on a 7x7 image): one launch whose wavefront
        # groups share K inside the workgroup and add up in LDS, with single-wavefront tiles
        for (m_w, n_w) in ((1, 1), (2, 1), (1, 2)):
            tm, tn = tile(view.M, m_w, 1, 16), tile(view.N, n_w, 1, 16)
            if not (in_space(view.M, tm) and in_space(view.N, tn)) or tm[0] * tn[0] * view.groups * 2 > NUM_CUS:
                continue
            kps = [kp for kp in view.KP_options if kp % 16 == 0]
            for groups in range(16 // (m_w * n_w), 1, -1):
                if kps and (kps[0] // 16) % groups == 0:
                    cfg = _empty_config()
                    cfg["spatial"] = [tm, tn]
                    cfg["reduce"] = [[groups, kps[0] // (16 * groups), 16]]
                    cfg["unroll"] = [[3, 1]]
                    cfg["fuse"] = [[8]]
                    cfg["reorder"] = [[1, 1, 0]]
                    group_seeds.append(cfg)
                    break

    # spread over the variations instead of exhausting the first tile shape
    def spread(lst, n):
        if len(lst) <= n:
            return lst
        step = (len(lst) - 1) / float(max(n - 1, 1))
        return [lst[int(round(i * step))] for i in range(n)]

    def spread_groups(first, lst, n):
        """``first`` and n - 1 of ``lst``: the (tile, BK) groups are visited in turn, and each visit
        of a group takes its next (depth, streaming) variant, starting at a variant that moves
        with the group, so that every tile shape and every pipeline depth gets measured."""
        if len(lst) + 1 <= n:
            return [first] + lst
        groups, index = [], {}
        for c in lst:
            gkey = json.dumps([c["spatial"], c["reduce"]])
            if gkey not in index:
                index[gkey] = len(groups)
                groups.append([])
            groups[index[gkey]].append(c)
        picked, taken, k = [first], [0] * len(groups), 0
        while len(picked) < n:
            gi = k % len(groups)
            g = groups[gi]
            if taken[gi] < len(g):
                # the start moves through the depths with the group; the streaming choice listed
                # first for the group stays first
                picked.append(g[(taken[gi] + gi % len(depths)) % len(g)])
                taken[gi] += 1
            k += 1
        return picked

    group_seeds = group_seeds[:max(limit // 3, 0)]
    nsplit = max(0, min(len(split_seeds), limit // 3 - len(group_seeds)))
    return (spread_groups(out[0], out[1:], max(limit - nsplit - len(group_seeds), 1)) + group_seeds +
            spread(split_seeds, nsplit))[:max(limit, 1)]
