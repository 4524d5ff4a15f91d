"""Tune GEMM tasks (fp32 and int8) — the reference's
flextensor/optimize/optimize_gemm.py:18-116 for the gfx950 backend.

    python -m flextensor_amd.optimize.optimize_gemm --log gemm.log --trials 40 --parallel 16
    python -m flextensor_amd.optimize.optimize_gemm --test gemm.log --check
"""
import argparse

from ..configs.shapes import baseline_gemm_shapes, baseline_gemm_int8_shapes, gemm_int8_shapes, gemm_shapes
from ..task import Task
from .common import init_arg_parser, run_driver

SHAPES = {"baseline": [("gemm", s) for s in baseline_gemm_shapes],
          "int8": [("gemm_int8", s) for s in baseline_gemm_int8_shapes],
          "int8_more": [("gemm_int8", s) for s in gemm_int8_shapes],
          "pow2": [("gemm", tuple(s)) for s in gemm_shapes]}


def make_task(index, entry, args):
    name, (N, K, M) = entry
    # an empty task that only carries the key of the registered one
    return Task("gemm", name, None, (N, K, M), args.target, args.device), [args.trials]


if __name__ == "__main__":
    parser = argparse.ArgumentParser()
    init_arg_parser(parser)
    args = parser.parse_args()
    run_driver(args, SHAPES[args.shapes], make_task, "gemm")
