"""Tune conv2d NCHW tasks — the reference's
flextensor/optimize/optimize_conv2d.py:29-140 for the gfx950 backend.

    python -m flextensor_amd.optimize.optimize_conv2d --shapes baseline --log conv2d.log --trials 40
"""
import argparse

from ..configs.shapes import grouped_shapes, dilation_shapes, vgg_19_shapes
from ..task import Task, conv2d_shape_dict
from .common import init_arg_parser, run_driver

# the reference's tables (optimize_conv2d.py:17-26) plus the benchmark shapes and the two single-name tables
SHAPES = dict(conv2d_shape_dict)
SHAPES.update({"vgg-19": vgg_19_shapes, "grouped": grouped_shapes, "dilation": dilation_shapes})


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
