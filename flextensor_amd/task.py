"""Tasks: named, registered operator instances to tune.

Same contract as the reference's flextensor/task.py:29-57: ``Task`` builds
its key as ``"{category}_{name}_{args}_{target}({dev_id})"``, keeps
``func(*args) -> (ops, bufs)`` with bufs ordered inputs..., output, and can
carry enumerated "special" knobs; ``register_task`` fills ``TASK_TABLE``.
Drivers create a ``func=None`` task only to compute a key and then look the
real one up (flextensor/optimize/optimize_gemm.py:26-35), so every shape that
should be tunable is registered at import time, here for target ``"rocm"``.
"""
from .nn import conv2d_nchw, depthwise_conv2d_nchw, gemm as op_gemm, gemm_int8 as op_gemm_int8
from .space import EnumSpace
from .te import placeholder
from .configs.shapes import (gemm_shapes, yolo_shapes, yolo_shapes_b8, grouped_shapes, dilation_shapes,
                             depthwise_shapes, depthwise_shapes_b8, depthwise_shapes_b16,
                             baseline_conv_shapes, baseline_depthwise_shapes, baseline_gemm_shapes,
                             baseline_gemm_int8_shapes, gemm_int8_shapes, google_shapes, res_shapes, squeeze_shapes,
                             vgg_16_shapes, test_conv_shapes, mobilev2_shapes, overfeat_shapes)

# table name -> conv2d shapes, the names of flextensor/task.py:274-284 plus this backend's benchmark shapes
conv2d_shape_dict = {
    "yolo": yolo_shapes, "google": google_shapes, "res": res_shapes, "squeeze": squeeze_shapes,
    "vgg-16": vgg_16_shapes, "test": test_conv_shapes, "yolo_b8": yolo_shapes_b8,
    "mobile_v2": mobilev2_shapes, "overfeat": overfeat_shapes, "baseline": baseline_conv_shapes,
}

TASK_TABLE = {}

ROCM_TARGET = "rocm"


class Task(object):
    def __init__(self, category, name, func, args, target, dev_id=0):
        self.key = "{}_{}_{}_{}({})".format(category, name, args, target, dev_id)
        self.func = func
        self.args = args
        self.target = target
        self.dev_id = dev_id
        self.category = category
        self.special_space = {}

    def set_specific_space(self, key, type, knobs):
        if type == "enum":
            self.special_space[key] = EnumSpace(knobs)
        else:
            raise RuntimeError("Not supported space type: %s" % type)


def register_task(task, override=False):
    if task.key in TASK_TABLE and not override:
        return
    TASK_TABLE[task.key] = task


def register(func, category, name, args, target, dev_id=0, override=False):
    task = Task(category, name, func, args, target, dev_id)
    _attach_default_knobs(task)
    register_task(task, override=override)


# ---- operator wrappers: shapes -> (ops, bufs) ------------------------------

def conv2d(N, C, H, W, K, kernel_size, stride=1, padding=0, dilation=1, groups=1):
    """flextensor/task.py:74-78; bufs = [Img, W, Output], fp32, no bias."""
    Img = placeholder((N, C, H, W), name="Img")
    Wt = placeholder((K, C // groups, kernel_size, kernel_size), name="W")
    Output = conv2d_nchw(Img, Wt, stride=stride, padding=padding, dilation=dilation, groups=groups)
    return [Output.op], [Img, Wt, Output]


def depthwise_conv2d(N, C, H, W, factor, kernel_size, stride=1, padding=0, dilation=1):
    """flextensor/task.py:96-100; weight [C, factor, k, k]."""
    Img = placeholder((N, C, H, W), name="Img")
    Wt = placeholder((C, factor, kernel_size, kernel_size), name="W")
    Output = depthwise_conv2d_nchw(Img, Wt, stride=stride, padding=padding, dilation=dilation)
    return [Output.op], [Img, Wt, Output]


def gemm_conv2d(N, C, H, W, K, kernel_size, stride=1, padding=0, dilation=1, groups=1):
    """flextensor/task.py:131-135: the convolution as im2col, GEMM, col2img;
    bufs = [Img, W, Output]. The weight holds C // groups channels per filter
    (the reference declares all C, which its GEMM stage never reads beyond
    C // groups and which only agrees with the image for groups = 1)."""
    from .nn import gemm_conv2d_nchw
    Img = placeholder((N, C, H, W), name="Img")
    Wt = placeholder((K, C // groups, kernel_size, kernel_size), name="W")
    Output = gemm_conv2d_nchw(Img, Wt, stride=stride, padding=padding, dilation=dilation, groups=groups)
    return [Output.op], [Img, Wt, Output]


def gemm(N, K, M):
    """flextensor/task.py:145-149; A [N,K] · B [K,M] -> [N,M], fp32."""
    A = placeholder((N, K), name="A")
    B = placeholder((K, M), name="B")
    Output = op_gemm(A, B)
    return [Output.op], [A, B, Output]


def gemm_int8(N, K, M):
    """int8 A [N,K], int8 B [M,K] (K-major) -> int32 [N,M]
    (flextensor/test/test_tvm/legacy/gemm_int8.py:15-21)."""
    A = placeholder((N, K), dtype="int8", name="A")
    B = placeholder((M, K), dtype="int8", name="B")
    Output = op_gemm_int8(A, B)
    return [Output.op], [A, B, Output]


def batch_gemm(B, N, K, M):
    """A batch of B products [N,K] x [K,M] (flextensor/nn/ops.py:1111-1158); bufs = [A, B, C]."""
    from .nn import batch_gemm as op_batch_gemm
    A = placeholder((B, N, K), name="A")
    Bm = placeholder((B, K, M), name="B")
    C = op_batch_gemm(A, Bm)
    return [C.op], [A, Bm, C]


def _attach_default_knobs(task):
    """Give a rocm task the enumerated knobs of its operator family."""
    if task.target != ROCM_TARGET or task.func is None:
        return
    from .templates.gfx950 import special_knobs
    kind = {gemm: "gemm", batch_gemm: "batch_gemm", gemm_int8: "gemm_int8", conv2d: "conv2d_nchw",
            gemm_conv2d: "col_gemm", depthwise_conv2d: "depthwise_conv2d_nchw"}.get(task.func)
    if kind is None:
        return
    if kind == "conv2d_nchw" and len(task.args) > 9 and task.args[9] > 1 and task.args[1] == task.args[9]:
        kind = "depthwise_conv2d_nchw"        # one input channel per group: nn.conv2d_nchw builds that operator
    elif kind == "conv2d_nchw" and len(task.args) > 9 and \
            (task.args[0], task.args[5], task.args[6], task.args[7], task.args[9]) == (1, 1, 1, 0, 1):
        kind = "pointwise_conv2d_nchw"        # one image, 1x1, stride 1, no padding, one group
    for key, knobs in special_knobs(kind).items():
        if key not in task.special_space:
            task.set_specific_space(key, "enum", knobs)


# ---- registration ----------------------------------------------------------

NUM_DEVICES = 4  # the reference registers every task for dev_id 0..3


def _register_all():
    for j in range(NUM_DEVICES):
        for shape in gemm_shapes + baseline_gemm_shapes:
            N, K, M = shape
            register(gemm, "gemm", "gemm", (N, K, M), ROCM_TARGET, j)
        for shape in baseline_gemm_int8_shapes + gemm_int8_shapes:
            N, K, M = shape
            register(gemm_int8, "gemm", "gemm_int8", (N, K, M), ROCM_TARGET, j)
        for name, shapes in conv2d_shape_dict.items():
            for i, shape in enumerate(shapes):
                batch, in_c, h, w, out_c, _, k_h, k_w, _, stride, pad, dil, groups = shape
                register(conv2d, "conv2d", name + str(i),
                         (batch, in_c, h, w, out_c, k_h, stride, pad, dil, groups),
                         ROCM_TARGET, j)
                # flextensor/task.py:349-366
                register(gemm_conv2d, "gemm_conv2d", name + str(i),
                         (batch, in_c, h, w, out_c, k_h, stride, pad, dil, groups), ROCM_TARGET, j)
        # flextensor/task.py:436-478
        for name, shapes in (("grouped", grouped_shapes), ("dilation", dilation_shapes)):
            for shape in shapes:
                batch, in_c, h, w, out_c, k, _, stride, pad, dil, groups = shape
                register(conv2d, "conv2d", name, (batch, in_c, h, w, out_c, k, stride, pad, dil, groups),
                         ROCM_TARGET, j)
        for shape in depthwise_shapes + depthwise_shapes_b8 + depthwise_shapes_b16 + \
                baseline_depthwise_shapes:
            batch, in_c, h, w, factor, k_h, k_w, stride, pad, dil = shape
            register(depthwise_conv2d, "conv2d", "depthwise",
                     (batch, in_c, h, w, factor, k_h, stride, pad, dil), ROCM_TARGET, j)


_register_all()
