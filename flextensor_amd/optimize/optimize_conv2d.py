"""Tune conv2d NCHW tasks — the reference's
flextensor/optimize/optimize_conv2d.py:29-140 for the gfx950 backend.

    python -m flextensor_amd.optimize.optimize_conv2d --shapes baseline --log conv2d.log --trials 40
"""
import argparse

from ..configs.shapes import (baseline_conv_shapes, yolo_shapes, yolo_shapes_b8, grouped_shapes,
                              dilation_shapes)
from ..task import Task
from .common import init_arg_parser, run_driver

SHAPES = {"baseline": baseline_conv_shapes, "yolo": yolo_shapes, "yolo_b8": yolo_shapes_b8,
          "grouped": grouped_shapes, "dilation": dilation_shapes}


def make_task_for(prefix):
    def make_task(index, shape, args):
        if prefix in ("grouped", "dilation"):
            # these tables have 11 entries and their tasks carry no index (flextensor/task.py:436-478)
            batch, in_c, h, w, out_c, k_h, _, stride, pad, dil, groups = shape
            name = prefix
        else:
            batch, in_c, h, w, out_c, _, k_h, k_w, _, stride, pad, dil, groups = shape
            name = prefix + str(index)
        task = Task("conv2d", name, None,
                    (batch, in_c, h, w, out_c, k_h, stride, pad, dil, groups), args.target, args.device)
        # two ops: [Padding, conv]; the padding op has no knobs
        return task, [max(args.trials // 10, 1), args.trials]
    return make_task


if __name__ == "__main__":
    parser = argparse.ArgumentParser()
    init_arg_parser(parser)
    args = parser.parse_args()
    run_driver(args, SHAPES[args.shapes], make_task_for(args.shapes), args.shapes + " convolution layer")
