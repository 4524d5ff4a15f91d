"""Tune convolutions written as im2col, GEMM, col2img — the reference's
flextensor/optimize/optimize_gemm_conv2d.py:27-75 for the gfx950 backend.

    python -m flextensor_amd.optimize.optimize_gemm_conv2d --shapes yolo --from 4 --to 5 --trials 40

The graph has four operators, [Padding, Img2Col, ComputeGemm, Col2Img]. The
graph level decides which of them exist as kernels: with the padding and the
column matrix inlined and the col2img merged into the GEMM's stores the whole
graph is one implicit-GEMM kernel; every other combination materialises the
intermediate tensors the flags name.
"""
import argparse

from ..configs.shapes import vgg_19_shapes
from ..task import Task, conv2d_shape_dict
from .common import init_arg_parser, run_driver

# flextensor/optimize/optimize_gemm_conv2d.py:17-24 plus the benchmark shapes
SHAPES = dict(conv2d_shape_dict)
SHAPES["vgg-19"] = vgg_19_shapes


def make_task_for(prefix):
    def make_task(index, shape, args):
        batch, in_c, h, w, out_c, _, k_h, k_w, _, stride, pad, dil, groups = shape
        task = Task("gemm_conv2d", prefix + str(index), None,
                    (batch, in_c, h, w, out_c, k_h, stride, pad, dil, groups), args.target, args.device)
        # the reference gives its four ops trials//10, trials//5, trials, trials//5
        # (optimize_gemm_conv2d.py:52); only the GEMM has knobs here
        return task, [max(args.trials // 10, 1), max(args.trials // 5, 1), args.trials,
                      max(args.trials // 5, 1)]
    return make_task


if __name__ == "__main__":
    parser = argparse.ArgumentParser()
    init_arg_parser(parser)
    args = parser.parse_args()
    run_driver(args, SHAPES[args.shapes], make_task_for(args.shapes), args.shapes + " im2col convolution layer")
