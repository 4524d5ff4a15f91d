"""The 128-bit input path of the direct depthwise kernel, emulated on the CPU.

With four outputs per lane along W and rows of whole 16-byte vectors the kernel
reads the 4 * stride centre columns of a patch row as vectors from the flat
tensor (depthwise_f32.hip, VEC_IN). In a ragged last patch of a row those
vectors run into the next row of the plane. This test replays that addressing
in numpy, element for element, for every (kernel width, stride, padding,
dilation, row length) the path admits, and compares the stored outputs with the
operator's definition (flextensor/nn/ops.py:622-678). Which shapes take the
path and which get the clip of the right padding is read from the template's
own preprocessor conditions, so the emulation cannot drift from the kernel.
"""
import itertools
import os
import re
import subprocess

import numpy as np
import pytest

from oracle import oracle  # checker

HERE = os.path.dirname(os.path.abspath(__file__))
TEMPLATE = os.path.join(os.path.dirname(HERE), "flextensor_amd", "templates", "depthwise_f32.hip")


def template_flags(defs):
    """VEC_IN and VEC_CLIP of the template for the given shape constants, by running the C
    preprocessor over the template's macro block."""
    src = open(TEMPLATE).read()
    head = src[:src.index("typedef float f32x4")]
    tail = src[src.index("#define PLANES"):src.index("#if SHFL")]
    text = head + tail + "\nFLAGS VEC_IN ; VEC_CLIP\n"
    cmd = ["gcc", "-E", "-P", "-x", "c", "-"] + ["-DFT_%s=%d" % kv for kv in defs.items()]
    out = subprocess.run(cmd, input=text, capture_output=True, text=True, check=True).stdout
    line = [l for l in out.splitlines() if l.startswith("FLAGS")][0][len("FLAGS"):]
    vec_in, vec_clip = line.split(";")
    to_py = lambda e: eval(re.sub(r"&&", " and ", re.sub(r"\|\|", " or ", e)).replace("!=", " != "))  # noqa: E731
    return bool(to_py(vec_in)), bool(to_py(vec_clip))


def emulate(x, wt, cs, stride, pad, dil, clip):
    """One plane pair through the patch addressing of the vector path: TH = 1, TW = 4."""
    planes, ch, cw = x.shape
    cr = wt.shape[1]
    cp = (ch + 2 * pad - dil * (cr - 1) - 1) // stride + 1
    cq = (cw + 2 * pad - dil * (cs - 1) - 1) // stride + 1
    assert cq * stride == cw
    flat = np.concatenate([x.reshape(-1), np.zeros(64, x.dtype)])     # beyond the buffer: zeros
    nbytes = x.size
    iw_t = 3 * stride + (cs - 1) * dil + 1
    nvec = stride
    out = np.zeros((planes, cp, cq), np.float64)
    for pl in range(planes):
        xplane = pl * ch * cw
        for oh in range(cp):
            for tw in range((cq + 3) // 4):
                ow0 = tw * 4
                iw0 = ow0 * stride - pad
                acc = np.zeros(4, np.float64)
                for r in range(cr):
                    ih = oh * stride - pad + r * dil
                    row_ok = 0 <= ih < ch
                    inp = np.zeros(iw_t, np.float64)
                    for j in range(iw_t):
                        if pad <= j < pad + 4 * nvec:
                            # centre: element j - pad of the row's vectors, straight from the flat tensor
                            off = xplane + ih * cw + ow0 * stride + (j - pad)
                            v = flat[off] if (row_ok and off < nbytes) else 0.0
                            if clip and tw * 4 * stride + (j - pad) >= cw:
                                v = 0.0
                        else:
                            iw = iw0 + j
                            v = x[pl, ih, iw] if (row_ok and 0 <= iw < cw) else 0.0
                        inp[j] = v
                    for j in range(4):
                        for s in range(cs):
                            acc[j] += inp[j * stride + s * dil] * wt[pl, r, s]
                for j in range(4):
                    if ow0 + j < cq:
                        out[pl, oh, ow0 + j] = acc[j]
    return out


CASES = [c for c in itertools.product((3, 5, 7), (1, 2), (0, 1, 2, 3), (1, 2), (8, 12, 16, 20, 24, 28))]


def test_vector_path_matches_the_definition_for_every_admitted_shape():
    rng = np.random.default_rng(5)
    admitted = clipped = broken_without_clip = 0
    for cs, stride, pad, dil, cw in CASES:
        ch = 6
        cq = (cw + 2 * pad - dil * (cs - 1) - 1) // stride + 1
        cp = (ch + 2 * pad - dil * (cs - 1) - 1) // stride + 1
        if cq < 4 or cp < 1:
            continue
        defs = dict(NT=64, TH=1, TW=4, NT_STORE=0, SHFL=0, CB=1, CC=2, CH=ch, CW=cw, CR=cs, CS=cs,
                    STRH=stride, STRW=stride, PADH=pad, PADW=pad, DILH=dil, DILW=dil, FACT=1, CP=cp, CQ=cq)
        vec_in, vec_clip = template_flags(defs)
        if not vec_in:
            continue
        admitted += 1
        clipped += vec_clip
        x = rng.uniform(-1, 1, (2, ch, cw))
        wt = rng.uniform(-1, 1, (2, cs, cs))
        ref = oracle.depthwise_nchw_np(x[None], wt[:, None], stride, pad, dil)[0]
        got = emulate(x, wt, cs, stride, pad, dil, vec_clip)
        assert np.max(np.abs(got - ref)) < 1e-12, (cs, stride, pad, dil, cw, vec_clip)
        if vec_clip:
            # the clip is what makes these right: without it the next row's data would be summed
            bad = emulate(x, wt, cs, stride, pad, dil, False)
            broken_without_clip += np.max(np.abs(bad - ref)) > 1e-3
    assert admitted >= 40 and clipped >= 6
    assert broken_without_clip == clipped


@pytest.mark.parametrize("args", [
    (28, 5, 2, 2, 1),      # 5x5, stride 2, padding 2 over 28 columns: 14 outputs per row
    (12, 3, 2, 2, 2),      # 3x3, stride 2, dilation 2, padding 2
    (20, 7, 2, 3, 1),      # 7x7, stride 2, padding 3
])
def test_shapes_that_once_summed_the_next_row_are_clipped(args):
    cw, cs, stride, pad, dil = args
    cq = (cw + 2 * pad - dil * (cs - 1) - 1) // stride + 1
    defs = dict(NT=64, TH=1, TW=4, NT_STORE=0, SHFL=0, CB=1, CC=2, CH=cw, CW=cw, CR=cs, CS=cs,
                STRH=stride, STRW=stride, PADH=pad, PADW=pad, DILH=dil, DILW=dil, FACT=1, CP=cq, CQ=cq)
    assert template_flags(defs) == (True, True)


def test_full_rows_and_narrow_kernels_need_no_clip():
    for cw, cs, stride, pad, dil in ((32, 5, 2, 2, 1), (28, 3, 2, 1, 1), (28, 3, 1, 1, 1)):
        cq = (cw + 2 * pad - dil * (cs - 1) - 1) // stride + 1
        defs = dict(NT=64, TH=1, TW=4, NT_STORE=0, SHFL=0, CB=1, CC=2, CH=cw, CW=cw, CR=cs, CS=cs,
                    STRH=stride, STRW=stride, PADH=pad, PADW=pad, DILH=dil, DILW=dil, FACT=1, CP=cq, CQ=cq)
        assert template_flags(defs) == (True, False)
