"""Operator definitions: the numerics contract of the tuned kernels.

Each function mirrors the signature and the index expression of its
counterpart in the reference's flextensor/nn/ops.py and returns the output
``Tensor`` of a ``ComputeOp`` that the gfx950 templates know how to lower.
The CPU restatement of the same expressions lives in oracle/.
"""
from ..te import ComputeOp, IterVar


def _pair(v, what):
    if isinstance(v, int):
        return (v, v)
    v = tuple(int(x) for x in v)
    if len(v) != 2:
        raise ValueError("%s must be an int or a pair, got %r" % (what, v))
    return v


def zero_pad2d(inputs, padding=0):
    """P[b,c,h,w] = X[b,c,h-pt,w-pl] inside the image, 0 outside.

    Follows flextensor/nn/ops.py:83-117 (padding is an int, (ph, pw) or
    (top, bottom, left, right)).
    """
    if isinstance(padding, int):
        padding = (padding,) * 4
    padding = tuple(int(p) for p in padding)
    if len(padding) == 2:
        padding = (padding[0], padding[0], padding[1], padding[1])
    if len(padding) != 4:
        raise ValueError("padding must have 1, 2 or 4 entries")
    b, c, h, w = inputs.shape
    out_shape = (b, c, h + padding[0] + padding[1], w + padding[2] + padding[3])
    axis = [IterVar(n, e) for n, e in zip("bchw", out_shape)]
    op = ComputeOp("Padding", "zero_pad2d", out_shape, inputs.dtype, axis, [], [inputs],
                   {"padding": padding})
    return op.output(0)


def bias_add_nchw(inputs, bias):
    """O[b,c,h,w] = I[b,c,h,w] + bias[c]: the stage the reference appends to a
    convolution that has a bias (flextensor/nn/ops.py:474-478, 673-677)."""
    if len(bias.shape) != 1 or bias.shape[0] != inputs.shape[1]:
        raise ValueError("bias must have one entry per output channel")
    axis = [IterVar(n, e) for n, e in zip("bchw", inputs.shape)]
    op = ComputeOp("bias", "bias_add_nchw", inputs.shape, inputs.dtype, axis, [], [inputs, bias], {})
    return op.output(0)


def conv2d_nchw(inputs, weight, bias=None, stride=1, padding=0, dilation=1, groups=1):
    """O[b,k,h,w] = sum_{rc,rw,rh} P[b, (k//Kg)*Cg+rc, h*s+rh*d, w*s+rw*d] * W[k,rc,rh,rw].

    Follows flextensor/nn/ops.py:419-479: the padded input is its own operator
    (so the graph is [Padding, conv]); reduce axes are declared [rc, rw, rh];
    out = (in + 2p - d(k-1) - 1)//s + 1.
    """
    batch, in_c, in_h, in_w = inputs.shape
    out_c, c_per_group, k_h, k_w = weight.shape
    if c_per_group * groups != in_c:
        raise ValueError("weight channels %d * groups %d != input channels %d"
                         % (c_per_group, groups, in_c))
    if out_c % groups != 0:
        raise ValueError("output channels not divisible by groups")
    stride = _pair(stride, "stride")
    padding = _pair(padding, "padding")
    dilation = _pair(dilation, "dilation")
    out_h = (in_h + 2 * padding[0] - dilation[0] * (k_h - 1) - 1) // stride[0] + 1
    out_w = (in_w + 2 * padding[1] - dilation[1] * (k_w - 1) - 1) // stride[1] + 1
    padded = zero_pad2d(inputs, padding=padding)
    out_shape = (batch, out_c, out_h, out_w)
    axis = [IterVar(n, e) for n, e in zip("bchw", out_shape)]
    if c_per_group == 1 and groups > 1:
        # one input channel per group (MobileNet's stages in flextensor/configs/conv2d_config.py:58-78):
        # rc has a single value, output channel k reads input channel k // (out_c / groups) and the
        # weight [out_c, 1, kh, kw] is the depthwise weight [C, factor, kh, kw] in memory, so this is
        # the depthwise operator (ops.py:622-678), with the same reduce order rw, rh, and takes its kernel
        raxis = [IterVar("rw", k_w, "reduce"), IterVar("rh", k_h, "reduce")]
        op = ComputeOp("compute", "depthwise_conv2d_nchw", out_shape, inputs.dtype, axis, raxis,
                       [padded, weight],
                       {"stride": stride, "padding": padding, "dilation": dilation,
                        "factor": out_c // groups, "in_shape": inputs.shape})
    else:
        raxis = [IterVar("rc", c_per_group, "reduce"), IterVar("rw", k_w, "reduce"),
                 IterVar("rh", k_h, "reduce")]
        op = ComputeOp("compute", "conv2d_nchw", out_shape, inputs.dtype, axis, raxis,
                       [padded, weight],
                       {"stride": stride, "padding": padding, "dilation": dilation,
                        "groups": int(groups), "in_shape": inputs.shape})
    if bias is not None:
        return bias_add_nchw(op.output(0), bias)
    return op.output(0)


def depthwise_conv2d_nchw(inputs, weight, bias=None, stride=1, padding=0, dilation=1):
    """O[b,c,h,w] = sum_{rw,rh} P[b, c//f, h*s+rh*d, w*s+rw*d] * W[c//f, c%f, rh, rw].

    Follows flextensor/nn/ops.py:622-678; weight layout [C, factor, kh, kw];
    a bias (one entry per output channel) is its own stage behind it (ops.py:673-677).
    """
    batch, in_c, in_h, in_w = inputs.shape
    w_c, factor, k_h, k_w = weight.shape
    if w_c != in_c:
        raise ValueError("weight channels %d != input channels %d" % (w_c, in_c))
    stride = _pair(stride, "stride")
    padding = _pair(padding, "padding")
    dilation = _pair(dilation, "dilation")
    out_h = (in_h + 2 * padding[0] - dilation[0] * (k_h - 1) - 1) // stride[0] + 1
    out_w = (in_w + 2 * padding[1] - dilation[1] * (k_w - 1) - 1) // stride[1] + 1
    padded = zero_pad2d(inputs, padding=padding)
    out_shape = (batch, in_c * factor, out_h, out_w)
    axis = [IterVar(n, e) for n, e in zip("bchw", out_shape)]
    raxis = [IterVar("rw", k_w, "reduce"), IterVar("rh", k_h, "reduce")]
    op = ComputeOp("compute", "depthwise_conv2d_nchw", out_shape, inputs.dtype, axis, raxis,
                   [padded, weight],
                   {"stride": stride, "padding": padding, "dilation": dilation,
                    "factor": int(factor), "in_shape": inputs.shape})
    if bias is not None:
        return bias_add_nchw(op.output(0), bias)
    return op.output(0)


def im2col_nchw_naive(inputs, kernel_size, stride=1, padding=0, dilation=1, groups=1):
    """col[g, h, w] = P[w // (P*Q), g*Cg + h // (kh*kw),
                        (w % (P*Q)) // Q * s + (h % (kh*kw)) // kw * d,  w % Q * s + h % kw * d]

    Follows flextensor/nn/ops.py:896-950: the padded image is its own operator;
    rows are (channel, kh, kw), columns are (batch, out_h, out_w).
    """
    batch, in_c, in_h, in_w = inputs.shape
    out_c, c_per_group, k_h, k_w = [int(x) for x in kernel_size]
    if c_per_group * groups != in_c:
        raise ValueError("kernel channels %d * groups %d != input channels %d" % (c_per_group, groups, in_c))
    if out_c % groups != 0:
        raise ValueError("output channels not divisible by groups")
    stride = _pair(stride, "stride")
    padding = _pair(padding, "padding")
    dilation = _pair(dilation, "dilation")
    out_h = (in_h + 2 * padding[0] - dilation[0] * (k_h - 1) - 1) // stride[0] + 1
    out_w = (in_w + 2 * padding[1] - dilation[1] * (k_w - 1) - 1) // stride[1] + 1
    padded = zero_pad2d(inputs, padding=padding)
    out_shape = (groups, k_h * k_w * c_per_group, batch * out_h * out_w)
    axis = [IterVar(n, e) for n, e in zip("ghw", out_shape)]
    op = ComputeOp("Img2Col", "im2col_nchw", out_shape, inputs.dtype, axis, [], [padded],
                   {"stride": stride, "padding": padding, "dilation": dilation, "groups": int(groups),
                    "in_shape": inputs.shape, "kernel": (k_h, k_w), "out_hw": (out_h, out_w),
                    "out_channel": out_c})
    return op.output(0)


def col2img_nchw(inputs, P, Q):
    """O[b, c, h, w] = I[c // Mg, c % Mg, b*(P*Q) + h*Q + w] (flextensor/nn/ops.py:953-979)."""
    groups, m_per_group, width = inputs.shape
    if width % (P * Q) != 0:
        raise ValueError("column count %d is not a multiple of P*Q = %d" % (width, P * Q))
    out_shape = (width // (P * Q), m_per_group * groups, int(P), int(Q))
    axis = [IterVar(n, e) for n, e in zip("bchw", out_shape)]
    op = ComputeOp("Col2Img", "col2img_nchw", out_shape, inputs.dtype, axis, [], [inputs], {})
    return op.output(0)


def gemm_conv2d_nchw(inputs, weight, bias=None, stride=1, padding=0, dilation=1, groups=1):
    """Convolution as an explicit im2col, one GEMM per group and a col2img
    (flextensor/nn/ops.py:982-1044):

        gemm[g, h, w] = sum_k col[g, k, w] * W[g*Mg + h, k // (kh*kw), (k % (kh*kw)) // kw, k % kw]

    The graph is [Padding, Img2Col, ComputeGemm, (ComputeBias,) Col2Img]; the
    result equals conv2d_nchw's.
    """
    out_c, c_per_group, k_h, k_w = weight.shape
    if out_c % groups != 0:
        raise ValueError("output channels not divisible by groups")
    m_per_group = out_c // groups
    col = im2col_nchw_naive(inputs, weight.shape, stride, padding, dilation, groups)
    out_h, out_w = col.op.attrs["out_hw"]
    _, k_ext, n_ext = col.shape
    axis = [IterVar("g", groups), IterVar("h", m_per_group), IterVar("w", n_ext)]
    raxis = [IterVar("k", k_ext, "reduce")]
    op = ComputeOp("ComputeGemm", "col_gemm", (groups, m_per_group, n_ext), inputs.dtype, axis, raxis,
                   [col, weight], dict(col.op.attrs))
    out = op.output(0)
    if bias is not None:
        if len(bias.shape) != 1 or bias.shape[0] != out_c:
            raise ValueError("bias must have one entry per output channel")
        baxis = [IterVar(n, e) for n, e in zip("ghw", out.shape)]
        bop = ComputeOp("ComputeBias", "bias_add_ghw", out.shape, out.dtype, baxis, [], [out, bias], {})
        out = bop.output(0)
    return col2img_nchw(out, out_h, out_w)


def gemm(A, B, transposeA=False, transposeB=False):
    """C[i,j] = sum_k A[i,k] * B[k,j] (operands optionally stored transposed).

    Follows flextensor/nn/ops.py:1074-1108.
    """
    if transposeA:
        k_a, m = A.shape
    else:
        m, k_a = A.shape
    if transposeB:
        n, k_b = B.shape
    else:
        k_b, n = B.shape
    if k_a != k_b:
        raise ValueError("reduce extents differ: %d vs %d" % (k_a, k_b))
    axis = [IterVar("i", m), IterVar("j", n)]
    raxis = [IterVar("k", k_a, "reduce")]
    op = ComputeOp("compute", "gemm", (m, n), A.dtype, axis, raxis, [A, B],
                   {"transposeA": bool(transposeA), "transposeB": bool(transposeB)})
    return op.output(0)


def batch_gemm(A, B, transposeA=False, transposeB=False):
    """C[b,i,j] = sum_k A[b,i,k] * B[b,k,j] (A optionally stored [b,k,i], B [b,j,k]).

    Follows flextensor/nn/ops.py:1111-1158.
    """
    if A.shape[0] != B.shape[0]:
        raise ValueError("batch extents differ: %d vs %d" % (A.shape[0], B.shape[0]))
    if transposeA:
        batch, k_a, m = A.shape
    else:
        batch, m, k_a = A.shape
    if transposeB:
        _, n, k_b = B.shape
    else:
        _, k_b, n = B.shape
    if k_a != k_b:
        raise ValueError("reduce extents differ: %d vs %d" % (k_a, k_b))
    axis = [IterVar("b", batch), IterVar("i", m), IterVar("j", n)]
    raxis = [IterVar("k", k_a, "reduce")]
    op = ComputeOp("compute", "batch_gemm", (batch, m, n), A.dtype, axis, raxis, [A, B],
                   {"transposeA": bool(transposeA), "transposeB": bool(transposeB)})
    return op.output(0)


def gemm_int8(A, B):
    """C[i,j] = sum_k int32(A[i,k]) * int32(B[j,k]); A [n,l], B [m,l] int8, C int32.

    Follows flextensor/test/test_tvm/legacy/gemm_int8.py:15-21 (B is K-major).
    """
    if A.dtype != "int8" or B.dtype != "int8":
        raise ValueError("gemm_int8 takes int8 operands")
    m, k_a = A.shape
    n, k_b = B.shape
    if k_a != k_b:
        raise ValueError("reduce extents differ: %d vs %d" % (k_a, k_b))
    axis = [IterVar("i", m), IterVar("j", n)]
    raxis = [IterVar("k", k_a, "reduce")]
    op = ComputeOp("C", "gemm_int8", (m, n), "int32", axis, raxis, [A, B], {})
    return op.output(0)
