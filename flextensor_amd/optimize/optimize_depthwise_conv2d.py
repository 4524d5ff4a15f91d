"""Tune depthwise conv2d NCHW tasks — the reference's
flextensor/optimize/optimize_depthwise_conv2d.py:18-120 for the gfx950 backend.

    python -m flextensor_amd.optimize.optimize_depthwise_conv2d --log dw.log --trials 20
"""
import argparse

from ..configs.shapes import (baseline_depthwise_shapes, depthwise_shapes, depthwise_shapes_b8,
                              depthwise_shapes_b16)
from ..task import Task
from .common import init_arg_parser, run_driver

SHAPES = {"baseline": baseline_depthwise_shapes, "mobile": depthwise_shapes,
          "mobile_b8": depthwise_shapes_b8, "mobile_b16": depthwise_shapes_b16}


def make_task(index, shape, args):
    batch, in_c, h, w, factor, k, _, stride, pad, dil = shape
    task = Task("conv2d", "depthwise", None, (batch, in_c, h, w, factor, k, stride, pad, dil),
                args.target, args.device)
    return task, [max(args.trials // 10, 1), args.trials]


if __name__ == "__main__":
    parser = argparse.ArgumentParser()
    init_arg_parser(parser)
    args = parser.parse_args()
    run_driver(args, SHAPES[args.shapes], make_task, "depthwise conv2d")
