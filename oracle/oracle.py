"""Python face of the CPU oracle. TEST INFRASTRUCTURE ONLY.

Two layers, both restating the reference's operator definitions:

* ``*_c``  — ctypes calls into liboracle.so (oracle.c): the loop nests of the
  reference's te.compute definitions in fp32, in the reference's loop order.
* ``*_np`` — independent numpy formulations (float64 accumulation / exact
  integers) used to pin the C functions and as the high-precision
  adjudicator for fp32 results.

plus ``*_loops``: brute-force pure-Python loops for tiny shapes, written from
the index expressions alone (flextensor/nn/ops.py:83-117, 419-479, 622-678,
1074-1108; flextensor/test/test_tvm/legacy/gemm_int8.py:15-21).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_BASE = None

_f32p = ctypes.POINTER(ctypes.c_float)
_i8p = ctypes.POINTER(ctypes.c_int8)
_i32p = ctypes.POINTER(ctypes.c_int32)


def build(force=False):
    """Compile liboracle.so and libcpubaseline.so with the host compiler."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE, "all"], stdout=subprocess.DEVNULL)


def _load(name):
    path = os.path.join(_HERE, name)
    if not os.path.exists(path):
        build()
    return ctypes.CDLL(path)


def lib():
    global _LIB
    if _LIB is None:
        L = _load("liboracle.so")
        L.ft_conv_out_size.restype = ctypes.c_int
        L.ft_conv2d_nchw.restype = ctypes.c_int
        L.ft_depthwise_nchw.restype = ctypes.c_int
        _LIB = L
    return _LIB


def baseline_lib():
    global _BASE
    if _BASE is None:
        L = _load("libcpubaseline.so")
        L.ftb_num_threads.restype = ctypes.c_int
        _BASE = L
    return _BASE


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_f32p)


def conv_out_size(n, pad, dil, k, stride):
    """(in + 2p - d(k-1) - 1)//s + 1 (flextensor/nn/ops.py:458-459)."""
    return (n + 2 * pad - dil * (k - 1) - 1) // stride + 1


# ---------------------------------------------------------------- C layer --

def zero_pad2d_c(x, padding):
    pt, pb, pl, pr = padding
    x, xp = _f32(x)
    b, c, h, w = x.shape
    out = np.empty((b, c, h + pt + pb, w + pl + pr), dtype=np.float32)
    lib().ft_zero_pad2d(xp, out.ctypes.data_as(_f32p), b * c, h, w, pt, pb, pl, pr)
    return out


def _hw(v):
    """int or (rows, columns) pair, as flextensor/nn/ops.py:448-456 accepts."""
    return (int(v), int(v)) if isinstance(v, (int, np.integer)) else (int(v[0]), int(v[1]))


def conv2d_nchw_c(x, wt, stride=1, padding=0, dilation=1, groups=1, fma=True):
    x, xp = _f32(x)
    wt, wp = _f32(wt)
    nb, c, h, w = x.shape
    ko, cg, r, s = wt.shape
    assert cg * groups == c
    (sh, sw), (ph, pw), (dh, dw) = _hw(stride), _hw(padding), _hw(dilation)
    p = conv_out_size(h, ph, dh, r, sh)
    q = conv_out_size(w, pw, dw, s, sw)
    out = np.empty((nb, ko, p, q), dtype=np.float32)
    rc = lib().ft_conv2d_nchw(xp, wp, out.ctypes.data_as(_f32p), nb, c, h, w, ko, r, s, sh,
                              sw, ph, pw, dh, dw, groups, int(fma))
    if rc != 0:
        raise MemoryError("oracle conv2d scratch")
    return out


def depthwise_nchw_c(x, wt, stride=1, padding=0, dilation=1, fma=True):
    x, xp = _f32(x)
    wt, wp = _f32(wt)
    nb, c, h, w = x.shape
    c2, f, r, s = wt.shape
    assert c2 == c
    (sh, sw), (ph, pw), (dh, dw) = _hw(stride), _hw(padding), _hw(dilation)
    p = conv_out_size(h, ph, dh, r, sh)
    q = conv_out_size(w, pw, dw, s, sw)
    out = np.empty((nb, c * f, p, q), dtype=np.float32)
    rc = lib().ft_depthwise_nchw(xp, wp, out.ctypes.data_as(_f32p), nb, c, h, w, f, r, s, sh,
                                 sw, ph, pw, dh, dw, int(fma))
    if rc != 0:
        raise MemoryError("oracle depthwise scratch")
    return out


def gemm_f32_c(a, b, transB=False, fma=True, transA=False):
    a, ap = _f32(a)
    b, bp = _f32(b)
    k, m = a.shape if transA else a.shape[::-1]
    n = b.shape[0] if transB else b.shape[1]
    assert (b.shape[1] if transB else b.shape[0]) == k
    out = np.empty((m, n), dtype=np.float32)
    lib().ft_gemm_f32(ap, bp, out.ctypes.data_as(_f32p), m, n, k, int(bool(transB)), int(fma),
                      int(bool(transA)))
    return out


def gemm_i8_c(a, b, row0=0, row1=None):
    """Rows [row0, row1) of A·Bᵀ in int32 (other rows are left zero)."""
    a = np.ascontiguousarray(a, dtype=np.int8)
    b = np.ascontiguousarray(b, dtype=np.int8)
    m, k = a.shape
    n, k2 = b.shape
    assert k == k2
    row1 = m if row1 is None else row1
    out = np.zeros((m, n), dtype=np.int32)
    lib().ft_gemm_i8(a.ctypes.data_as(_i8p), b.ctypes.data_as(_i8p), out.ctypes.data_as(_i32p),
                     m, n, k, row0, row1)
    return out


# ------------------------------------------------------------ numpy layer --

def zero_pad2d_np(x, padding):
    pt, pb, pl, pr = padding
    return np.pad(x, ((0, 0), (0, 0), (pt, pb), (pl, pr)))


def gemm_np(a, b, transB=False):
    """float64 matmul, the adjudicator for fp32 GEMM."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return a @ (b.T if transB else b)


def gemm_i8_np(a, b):
    """Exact A·Bᵀ: products are < 2^14 and sums < 2^53, so float64 BLAS is exact."""
    c = np.asarray(a, dtype=np.float64) @ np.asarray(b, dtype=np.float64).T
    return np.rint(c).astype(np.int64).astype(np.int32)


def conv2d_nchw_np(x, wt, stride=1, padding=0, dilation=1, groups=1):
    """float64 im2col formulation (independent of the loop nest in oracle.c)."""
    x = np.asarray(x, dtype=np.float64)
    wt = np.asarray(wt, dtype=np.float64)
    nb, c, h, w = x.shape
    ko, cg, r, s = wt.shape
    p = conv_out_size(h, padding, dilation, r, stride)
    q = conv_out_size(w, padding, dilation, s, stride)
    xp = np.pad(x, ((0, 0), (0, 0), (padding, padding), (padding, padding)))
    kg = ko // groups
    out = np.zeros((nb, ko, p, q), dtype=np.float64)
    for g in range(groups):
        cols = np.empty((nb, cg, r, s, p, q), dtype=np.float64)
        for rh in range(r):
            for rw in range(s):
                cols[:, :, rh, rw] = xp[:, g * cg:(g + 1) * cg,
                                        rh * dilation: rh * dilation + (p - 1) * stride + 1: stride,
                                        rw * dilation: rw * dilation + (q - 1) * stride + 1: stride]
        wg = wt[g * kg:(g + 1) * kg].reshape(kg, cg * r * s)
        out[:, g * kg:(g + 1) * kg] = np.einsum("kc,bcn->bkn", wg,
                                                cols.reshape(nb, cg * r * s, p * q)).reshape(nb, kg, p, q)
    return out


def bias_add_nchw_np(y, bias):
    """O[b,c,h,w] = I[b,c,h,w] + bias[c] in fp32 (flextensor/nn/ops.py:474-478)."""
    return (np.asarray(y, np.float32) + np.asarray(bias, np.float32)[None, :, None, None]).astype(np.float32)


def im2col_nchw_np(x, kernel_shape, stride=1, padding=0, dilation=1, groups=1):
    """col[g, h, w] gathered with the index expression of flextensor/nn/ops.py:943-949
    (index arrays built from the formula itself; fp32 values are copied, not computed)."""
    x = np.asarray(x, np.float32)
    nb, c, h, w = x.shape
    _, cg, r, s = [int(v) for v in kernel_shape]
    p = conv_out_size(h, padding, dilation, r, stride)
    q = conv_out_size(w, padding, dilation, s, stride)
    xp = np.pad(x, ((0, 0), (0, 0), (padding, padding), (padding, padding)))
    gi = np.arange(groups)[:, None, None]
    hi = np.arange(cg * r * s)[None, :, None]
    wi = np.arange(nb * p * q)[None, None, :]
    return xp[wi // (p * q),
              gi * cg + hi // (r * s),
              wi % (p * q) // q * stride + hi % (r * s) // s * dilation,
              wi % q * stride + hi % s * dilation]


def col2img_nchw_np(y, p, q):
    """O[b, c, h, w] = I[c // Mg, c % Mg, b*(P*Q) + h*Q + w] (flextensor/nn/ops.py:972-978)."""
    y = np.asarray(y)
    g, mg, width = y.shape
    nb = width // (p * q)
    bi = np.arange(nb)[:, None, None, None]
    ci = np.arange(g * mg)[None, :, None, None]
    hi = np.arange(p)[None, None, :, None]
    wi = np.arange(q)[None, None, None, :]
    return y[ci // mg, ci % mg, bi * (p * q) + hi * q + wi]


def gemm_conv2d_nchw_np(x, wt, bias=None, stride=1, padding=0, dilation=1, groups=1):
    """im2col, one float64 GEMM per group, optional bias, col2img
    (flextensor/nn/ops.py:982-1044). Returns (output, col, gemm stage)."""
    wt = np.asarray(wt, np.float32)
    ko, cg, r, s = wt.shape
    mg = ko // groups
    col = im2col_nchw_np(x, wt.shape, stride, padding, dilation, groups)
    ki = np.arange(cg * r * s)
    # W[g*Mg + h, k // (kh*kw), k % (kh*kw) // kw, k % kw]
    wmat = wt[:, ki // (r * s), ki % (r * s) // s, ki % s].reshape(groups, mg, cg * r * s)
    gemm = np.einsum("ghk,gkw->ghw", wmat.astype(np.float64), col.astype(np.float64))
    if bias is not None:
        gemm = gemm + np.asarray(bias, np.float64).reshape(groups, mg, 1)
    h, w = np.asarray(x).shape[2:]
    p = conv_out_size(h, padding, dilation, r, stride)
    q = conv_out_size(w, padding, dilation, s, stride)
    return col2img_nchw_np(gemm, p, q), col, gemm


def depthwise_nchw_np(x, wt, stride=1, padding=0, dilation=1):
    x = np.asarray(x, dtype=np.float64)
    wt = np.asarray(wt, dtype=np.float64)
    nb, c, h, w = x.shape
    _, f, r, s = wt.shape
    p = conv_out_size(h, padding, dilation, r, stride)
    q = conv_out_size(w, padding, dilation, s, stride)
    xp = np.pad(x, ((0, 0), (0, 0), (padding, padding), (padding, padding)))
    out = np.zeros((nb, c, f, p, q), dtype=np.float64)
    for rh in range(r):
        for rw in range(s):
            patch = xp[:, :, rh * dilation: rh * dilation + (p - 1) * stride + 1: stride,
                       rw * dilation: rw * dilation + (q - 1) * stride + 1: stride]
            out += patch[:, :, None] * wt[None, :, :, rh, rw, None, None]
    return out.reshape(nb, c * f, p, q)


# ------------------------------------------------------- brute-force loops --

def conv2d_nchw_loops(x, wt, stride, padding, dilation, groups):
    nb, c, h, w = x.shape
    ko, cg, r, s = wt.shape
    p = conv_out_size(h, padding, dilation, r, stride)
    q = conv_out_size(w, padding, dilation, s, stride)
    kg = ko // groups
    out = np.zeros((nb, ko, p, q), dtype=np.float64)
    for b in range(nb):
        for k in range(ko):
            for oh in range(p):
                for ow in range(q):
                    acc = 0.0
                    for rc in range(cg):
                        for rh in range(r):
                            for rw in range(s):
                                ih = oh * stride + rh * dilation - padding
                                iw = ow * stride + rw * dilation - padding
                                if 0 <= ih < h and 0 <= iw < w:
                                    acc += float(x[b, (k // kg) * cg + rc, ih, iw]) * float(wt[k, rc, rh, rw])
                    out[b, k, oh, ow] = acc
    return out


def depthwise_nchw_loops(x, wt, stride, padding, dilation):
    nb, c, h, w = x.shape
    _, f, r, s = wt.shape
    p = conv_out_size(h, padding, dilation, r, stride)
    q = conv_out_size(w, padding, dilation, s, stride)
    out = np.zeros((nb, c * f, p, q), dtype=np.float64)
    for b in range(nb):
        for co in range(c * f):
            for oh in range(p):
                for ow in range(q):
                    acc = 0.0
                    for rh in range(r):
                        for rw in range(s):
                            ih = oh * stride + rh * dilation - padding
                            iw = ow * stride + rw * dilation - padding
                            if 0 <= ih < h and 0 <= iw < w:
                                acc += float(x[b, co // f, ih, iw]) * float(wt[co // f, co % f, rh, rw])
                    out[b, co, oh, ow] = acc
    return out


# ------------------------------------------------- multi-threaded baseline --

def baseline_threads():
    return baseline_lib().ftb_num_threads()


def baseline_gemm_f32(a, b, out, tk=256):
    baseline_lib().ftb_gemm_f32(a.ctypes.data_as(_f32p), b.ctypes.data_as(_f32p),
                                out.ctypes.data_as(_f32p), a.shape[0], b.shape[1], a.shape[1], tk)


def baseline_gemm_f32_tiles():
    """(rows, columns) of the register tiles the port was built with; the index is the variant."""
    L = baseline_lib()
    out = []
    for v in range(L.ftb_gemm_f32_variants()):
        ti, tj = ctypes.c_int(), ctypes.c_int()
        L.ftb_gemm_f32_variant_tile(v, ctypes.byref(ti), ctypes.byref(tj))
        out.append((ti.value, tj.value))
    return out


def baseline_gemm_f32_v(a, b, out, tk, variant):
    baseline_lib().ftb_gemm_f32_v(a.ctypes.data_as(_f32p), b.ctypes.data_as(_f32p),
                                  out.ctypes.data_as(_f32p), a.shape[0], b.shape[1], a.shape[1], tk,
                                  int(variant))


def baseline_conv2d_tiles():
    """(output channels, output columns) of the convolution's register tiles, by variant index."""
    L = baseline_lib()
    out = []
    for v in range(L.ftb_conv2d_variants()):
        a, b = ctypes.c_int(), ctypes.c_int()
        L.ftb_conv2d_variant_tile(v, ctypes.byref(a), ctypes.byref(b))
        out.append((a.value, b.value))
    return out


def baseline_conv2d_v(x, wt, out, scratch, stride, padding, dilation, variant):
    nb, c, h, w = x.shape
    ko, _, r, s = wt.shape
    baseline_lib().ftb_conv2d_nchw_v(x.ctypes.data_as(_f32p), wt.ctypes.data_as(_f32p),
                                     out.ctypes.data_as(_f32p), scratch.ctypes.data_as(_f32p),
                                     nb, c, h, w, ko, r, s, stride, padding, dilation, int(variant))


def baseline_gemm_i8(a, b, out, row0=0, row1=None):
    row1 = a.shape[0] if row1 is None else row1
    baseline_lib().ftb_gemm_i8(a.ctypes.data_as(_i8p), b.ctypes.data_as(_i8p),
                               out.ctypes.data_as(_i32p), a.shape[0], b.shape[0], a.shape[1],
                               row0, row1)


def baseline_conv2d(x, wt, out, scratch, stride, padding, dilation):
    nb, c, h, w = x.shape
    ko, _, r, s = wt.shape
    baseline_lib().ftb_conv2d_nchw(x.ctypes.data_as(_f32p), wt.ctypes.data_as(_f32p),
                                   out.ctypes.data_as(_f32p), scratch.ctypes.data_as(_f32p),
                                   nb, c, h, w, ko, r, s, stride, padding, dilation)


def baseline_depthwise(x, wt, out, scratch, stride, padding, dilation):
    nb, c, h, w = x.shape
    _, f, r, s = wt.shape
    baseline_lib().ftb_depthwise_nchw(x.ctypes.data_as(_f32p), wt.ctypes.data_as(_f32p),
                                      out.ctypes.data_as(_f32p), scratch.ctypes.data_as(_f32p),
                                      nb, c, h, w, f, r, s, stride, padding, dilation)
