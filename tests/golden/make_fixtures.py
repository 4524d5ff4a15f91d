"""Writes tests/golden/small_cases.npz: seeded inputs and expected outputs of
small operator instances.

Expected outputs come from brute-force Python loops over the operators' index
expressions in float64 (oracle.oracle.*_loops) and from exact integer
arithmetic — not from the reference (which needs TVM and cannot run here) and
not from the C oracle they are used to pin. Shapes follow the cases the
reference's own op tests use (flextensor/test/test_ops.py:85-115, 152-184;
flextensor/test/test_tvm/legacy/gemm_int8.py:135-148), shrunk where needed.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as o  # noqa: E402


def main():
    rng = np.random.default_rng(20200316)
    out = {}
    # conv2d: the reference's test case — x [4,6,7,7], w [9,2,3,3], stride 2,
    # pad 1, dilation 2, groups 3
    x = rng.uniform(-1, 1, (4, 6, 7, 7)).astype(np.float32)
    w = rng.uniform(-1, 1, (9, 2, 3, 3)).astype(np.float32)
    out["conv_g3_x"], out["conv_g3_w"] = x, w
    out["conv_g3_y"] = o.conv2d_nchw_loops(x, w, 2, 1, 2, 3)
    # conv2d groups=1, 3x3 s1 p1 and 1x1 s1 p0, odd sizes
    x = rng.uniform(-1, 1, (2, 5, 9, 6)).astype(np.float32)
    w = rng.uniform(-1, 1, (7, 5, 3, 3)).astype(np.float32)
    out["conv_a_x"], out["conv_a_w"] = x, w
    out["conv_a_y"] = o.conv2d_nchw_loops(x, w, 1, 1, 1, 1)
    w = rng.uniform(-1, 1, (4, 5, 1, 1)).astype(np.float32)
    out["conv_b_w"] = w
    out["conv_b_y"] = o.conv2d_nchw_loops(x, w, 1, 0, 1, 1)
    # depthwise: the reference's test case — x [4,6,7,7], w [6,3,3,3], stride 2, pad 1, dil 2
    x = rng.uniform(-1, 1, (4, 6, 7, 7)).astype(np.float32)
    w = rng.uniform(-1, 1, (6, 3, 3, 3)).astype(np.float32)
    out["dw_x"], out["dw_w"] = x, w
    out["dw_y"] = o.depthwise_nchw_loops(x, w, 2, 1, 2)
    # depthwise factor 1, 3x3 s1 p1
    x = rng.uniform(-1, 1, (2, 5, 8, 12)).astype(np.float32)
    w = rng.uniform(-1, 1, (5, 1, 3, 3)).astype(np.float32)
    out["dw1_x"], out["dw1_w"] = x, w
    out["dw1_y"] = o.depthwise_nchw_loops(x, w, 1, 1, 1)
    # gemm fp32 (float64 expected) and int8 (exact)
    a = rng.uniform(-1, 1, (37, 64)).astype(np.float32)
    b = rng.uniform(-1, 1, (64, 29)).astype(np.float32)
    out["gemm_a"], out["gemm_b"] = a, b
    out["gemm_c"] = np.array([[sum(float(a[i, k]) * float(b[k, j]) for k in range(64))
                               for j in range(29)] for i in range(37)])
    ai = rng.integers(-128, 128, (19, 48), dtype=np.int8)
    bi = rng.integers(-128, 128, (23, 48), dtype=np.int8)
    ai[0, :] = -128
    bi[0, :] = -128  # the extreme product
    out["i8_a"], out["i8_b"] = ai, bi
    out["i8_c"] = np.array([[sum(int(ai[i, k]) * int(bi[j, k]) for k in range(48))
                             for j in range(23)] for i in range(19)], dtype=np.int32)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "small_cases.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
