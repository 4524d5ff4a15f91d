"""Pins the CPU oracle (oracle/oracle.c) against independent routines.

Each check is chosen so that a plausible mistake fails it: a transposed
operand (non-square GEMM), a swapped rh/rw (non-square kernels and images),
wrong group or factor indexing (groups=3, factor=3), a wrong padding or
dilation sign (stride 2, pad 1, dilation 2 — the reference's own test case,
flextensor/test/test_ops.py:85-115, 152-184), int8 sign handling (-128 * -128).
"""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden", "small_cases.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD)


def rel(a, b):
    return float(np.max(np.abs(np.asarray(a, np.float64) - b)) / np.max(np.abs(b)))


def test_out_size_closed_form(oracle):
    # (in + 2p - d(k-1) - 1)//s + 1, spot values worked by hand
    assert oracle.lib().ft_conv_out_size(56, 1, 1, 3, 1) == 56
    assert oracle.lib().ft_conv_out_size(7, 1, 2, 3, 2) == 3
    assert oracle.lib().ft_conv_out_size(448, 3, 1, 7, 2) == 224
    assert oracle.lib().ft_conv_out_size(7, 0, 1, 1, 1) == 7
    for n in range(1, 20):
        for k in (1, 3, 5):
            for s in (1, 2, 3):
                for p in (0, 1, 2):
                    for d in (1, 2):
                        if n + 2 * p - d * (k - 1) - 1 < 0:
                            continue
                        # count valid window positions by brute force
                        cnt = len([o for o in range(0, n + 2 * p) if o % s == 0
                                   and o + d * (k - 1) <= n + 2 * p - 1])
                        assert oracle.conv_out_size(n, p, d, k, s) == cnt
                        assert oracle.lib().ft_conv_out_size(n, p, d, k, s) == cnt


def test_zero_pad2d_closed_form(oracle):
    x = np.arange(2 * 3 * 4 * 5, dtype=np.float32).reshape(2, 3, 4, 5) + 1
    p = oracle.zero_pad2d_c(x, (1, 2, 3, 0))
    assert p.shape == (2, 3, 7, 8)
    assert np.array_equal(p, oracle.zero_pad2d_np(x, (1, 2, 3, 0)))
    assert np.array_equal(p[:, :, 1:5, 3:8], x)
    assert p.sum() == x.sum()
    assert np.all(p[:, :, 0, :] == 0) and np.all(p[:, :, 5:, :] == 0) and np.all(p[:, :, :, :3] == 0)


def test_conv2d_reference_case_golden(oracle, gold):
    y = oracle.conv2d_nchw_c(gold["conv_g3_x"], gold["conv_g3_w"], 2, 1, 2, 3)
    assert y.shape == (4, 9, 3, 3)
    assert rel(y, gold["conv_g3_y"]) < 1e-6
    y0 = oracle.conv2d_nchw_c(gold["conv_g3_x"], gold["conv_g3_w"], 2, 1, 2, 3, fma=False)
    assert rel(y0, gold["conv_g3_y"]) < 1e-6


def test_conv2d_golden_and_numpy(oracle, gold):
    x = gold["conv_a_x"]
    assert rel(oracle.conv2d_nchw_c(x, gold["conv_a_w"], 1, 1, 1, 1), gold["conv_a_y"]) < 1e-6
    assert rel(oracle.conv2d_nchw_c(x, gold["conv_b_w"], 1, 0, 1, 1), gold["conv_b_y"]) < 1e-6
    assert rel(oracle.conv2d_nchw_np(x, gold["conv_a_w"], 1, 1, 1, 1), gold["conv_a_y"]) < 1e-12
    assert rel(oracle.conv2d_nchw_np(gold["conv_g3_x"], gold["conv_g3_w"], 2, 1, 2, 3),
               gold["conv_g3_y"]) < 1e-12


def test_conv2d_vs_torch(oracle):
    torch = pytest.importorskip("torch")
    F = torch.nn.functional
    rng = np.random.default_rng(1)
    for (n, c, h, w, k, r, s_, st, p, d, g) in [
            (4, 6, 7, 7, 9, 3, 3, 2, 1, 2, 3),     # the reference's case
            (1, 8, 12, 10, 6, 3, 3, 1, 1, 1, 1),
            (2, 4, 9, 9, 8, 1, 1, 1, 0, 1, 1),
            (1, 3, 17, 13, 5, 5, 5, 2, 2, 1, 1),
            (2, 8, 8, 8, 8, 3, 3, 1, 1, 1, 4)]:
        x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
        wt = rng.uniform(-1, 1, (k, c // g, r, s_)).astype(np.float32)
        ref = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(wt).double(), None, st, p, d, g).numpy()
        assert rel(oracle.conv2d_nchw_c(x, wt, st, p, d, g), ref) < 1e-6
        assert rel(oracle.conv2d_nchw_np(x, wt, st, p, d, g), ref) < 1e-12


def test_conv2d_and_depthwise_with_row_column_pairs_vs_torch(oracle):
    """stride, padding and dilation given as (rows, columns) pairs (flextensor/nn/ops.py:448-459):
    each of the three differs between the axes, so a swapped or shared pair changes the output
    size or the values."""
    torch = pytest.importorskip("torch")
    F = torch.nn.functional
    rng = np.random.default_rng(8)
    for (n, c, h, w, k, r, s_, st, p, d, g) in [
            (2, 6, 11, 14, 8, 3, 3, (2, 1), (1, 2), (1, 2), 1),
            (1, 4, 13, 9, 6, 3, 5, (1, 2), (0, 2), (2, 1), 2),
            (3, 5, 8, 8, 5, 1, 3, (1, 1), (0, 1), (1, 1), 1)]:
        x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
        wt = rng.uniform(-1, 1, (k, c // g, r, s_)).astype(np.float32)
        ref = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(wt).double(), None, st, p, d, g).numpy()
        out = oracle.conv2d_nchw_c(x, wt, st, p, d, g)
        assert out.shape == ref.shape and rel(out, ref) < 1e-6
    for (n, c, h, w, f, r, s_, st, p, d) in [(2, 6, 11, 14, 2, 3, 3, (2, 1), (1, 2), (1, 2)),
                                             (1, 5, 9, 12, 1, 3, 3, (1, 2), (1, 0), (1, 1))]:
        x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
        wt = rng.uniform(-1, 1, (c, f, r, s_)).astype(np.float32)
        ref = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(wt.reshape(c * f, 1, r, s_)).double(),
                       None, st, p, d, c).numpy()
        out = oracle.depthwise_nchw_c(x, wt, st, p, d)
        assert out.shape == ref.shape and rel(out, ref) < 1e-6


def test_conv2d_bias_vs_torch(oracle):
    """conv + per-channel bias, as the reference's own test runs it
    (flextensor/test/test_ops.py:85-115 passes a bias to both sides)."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(5)
    x = rng.uniform(-1, 1, (4, 6, 7, 7)).astype(np.float32)
    w = rng.uniform(-1, 1, (9, 2, 3, 3)).astype(np.float32)
    bias = rng.uniform(-1, 1, (9,)).astype(np.float32)
    ref = torch.nn.functional.conv2d(torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(bias),
                                     stride=2, padding=1, dilation=2, groups=3).numpy()
    got = oracle.bias_add_nchw_np(oracle.conv2d_nchw_c(x, w, 2, 1, 2, 3), bias)
    assert np.max(np.abs(got - ref)) <= 1e-5 * np.max(np.abs(ref))
    # the bias alone: a zero image gives bias[c] everywhere
    z = oracle.bias_add_nchw_np(oracle.conv2d_nchw_c(np.zeros_like(x), w, 2, 1, 2, 3), bias)
    assert np.array_equal(z, np.broadcast_to(bias[None, :, None, None], z.shape))


def test_gemm_conv2d_vs_torch_and_direct(oracle):
    """im2col, GEMM, bias, col2img against torch's convolution, the check the
    reference runs (flextensor/test/test_ops.py:254-284, 1x1 case with bias),
    plus padded, strided, dilated and grouped cases and the intermediate
    tensors against forms that share no indexing with the restatement."""
    torch = pytest.importorskip("torch")
    F = torch.nn.functional
    rng = np.random.default_rng(11)
    for (n, c, h, w, k, r, st, p, d, g) in [
            (1, 384, 27, 27, 64, 1, 1, 0, 1, 1),   # the reference's case
            (2, 6, 9, 8, 4, 3, 1, 1, 1, 1),
            (2, 6, 11, 9, 9, 3, 2, 1, 2, 3),
            (1, 4, 7, 7, 6, 5, 1, 2, 1, 2)]:
        x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
        wt = rng.uniform(-1, 1, (k, c // g, r, r)).astype(np.float32)
        bias = rng.uniform(-1, 1, (k,)).astype(np.float32)
        ref = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(wt).double(),
                       torch.from_numpy(bias).double(), st, p, d, g).numpy()
        out, col, stage = oracle.gemm_conv2d_nchw_np(x, wt, bias, st, p, d, g)
        assert out.shape == ref.shape
        assert rel(out, ref) < 1e-12
        # without bias it is the direct convolution's own restatement
        assert rel(oracle.gemm_conv2d_nchw_np(x, wt, None, st, p, d, g)[0],
                   oracle.conv2d_nchw_c(x, wt, st, p, d, g)) < 1e-6
        # the column matrix is torch's unfold, group by group
        unf = F.unfold(torch.from_numpy(x), r, dilation=d, padding=p, stride=st).numpy()   # [n, c*r*r, P*Q]
        pq = unf.shape[2]
        cg = c // g
        for gi in range(g):
            want = unf[:, gi * cg * r * r:(gi + 1) * cg * r * r].transpose(1, 0, 2).reshape(cg * r * r, n * pq)
            assert np.array_equal(col[gi], want)
        # col2img is a pure permutation: [g, Mg, n, P*Q] -> [n, g*Mg, P, Q]
        mg = k // g
        want = stage.reshape(g * mg, n, pq).transpose(1, 0, 2).reshape(ref.shape)
        assert np.array_equal(out, want)


def test_conv2d_linearity_and_delta(oracle):
    rng = np.random.default_rng(2)
    x1 = rng.uniform(-1, 1, (1, 3, 6, 6)).astype(np.float32)
    x2 = rng.uniform(-1, 1, (1, 3, 6, 6)).astype(np.float32)
    w = rng.uniform(-1, 1, (4, 3, 3, 3)).astype(np.float32)
    y = oracle.conv2d_nchw_np(x1 + x2, w, 1, 1, 1, 1)
    assert np.allclose(y, oracle.conv2d_nchw_np(x1, w, 1, 1, 1, 1) + oracle.conv2d_nchw_np(x2, w, 1, 1, 1, 1))
    # a one-hot centre tap copies channel sums: identifies rh/rw/c indexing
    w = np.zeros((2, 3, 3, 3), np.float32)
    w[0, 1, 1, 1] = 1.0   # out 0 <- in channel 1, centre
    w[1, 2, 0, 2] = 1.0   # out 1 <- in channel 2, tap (rh=0, rw=2): shift up 1, left... right 1
    y = oracle.conv2d_nchw_c(x1, w, 1, 1, 1, 1)
    assert np.array_equal(y[0, 0], x1[0, 1])
    exp = np.zeros((6, 6), np.float32)
    exp[1:, :5] = x1[0, 2][:5, 1:]
    assert np.array_equal(y[0, 1], exp)


def test_depthwise_reference_case_golden(oracle, gold):
    y = oracle.depthwise_nchw_c(gold["dw_x"], gold["dw_w"], 2, 1, 2)
    assert y.shape == (4, 18, 3, 3)
    assert rel(y, gold["dw_y"]) < 1e-6
    assert rel(oracle.depthwise_nchw_np(gold["dw_x"], gold["dw_w"], 2, 1, 2), gold["dw_y"]) < 1e-12
    assert rel(oracle.depthwise_nchw_c(gold["dw1_x"], gold["dw1_w"], 1, 1, 1), gold["dw1_y"]) < 1e-6


def test_depthwise_vs_torch(oracle):
    torch = pytest.importorskip("torch")
    F = torch.nn.functional
    rng = np.random.default_rng(3)
    for (n, c, h, w, f, k, st, p, d) in [(4, 6, 7, 7, 3, 3, 2, 1, 2), (2, 8, 28, 28, 1, 3, 1, 1, 1),
                                         (1, 5, 9, 11, 2, 3, 1, 0, 1)]:
        x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
        wt = rng.uniform(-1, 1, (c, f, k, k)).astype(np.float32)
        # weight reshape of the reference's test: [C, f, k, k] -> [C*f, 1, k, k], groups=C
        ref = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(wt.reshape(c * f, 1, k, k)).double(),
                       None, st, p, d, c).numpy()
        assert rel(oracle.depthwise_nchw_c(x, wt, st, p, d), ref) < 1e-6
        assert rel(oracle.depthwise_nchw_np(x, wt, st, p, d), ref) < 1e-12


def test_identities_the_special_lowerings_rest_on(oracle):
    """A convolution with one input channel per group is the depthwise operator on the same weight
    bytes, term for term (so bit for bit); a 1x1 stride-1 unpadded convolution of one image is the
    product W [K][C] x X [C][H*W], summed over c in the same order."""
    rng = np.random.default_rng(11)
    for (n, c, h, w, f, k, st, p, d) in [(2, 6, 9, 11, 1, 3, 1, 1, 1), (1, 4, 12, 16, 6, 3, 2, 1, 1),
                                         (2, 5, 9, 11, 2, 3, 1, 1, 2)]:
        x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
        wt = rng.uniform(-1, 1, (c, f, k, k)).astype(np.float32)
        grouped = oracle.conv2d_nchw_c(x, wt.reshape(c * f, 1, k, k), st, p, d, c)
        assert np.array_equal(grouped, oracle.depthwise_nchw_c(x, wt, st, p, d))
    for (c, h, w, ko) in [(64, 14, 14, 96), (48, 7, 7, 40)]:
        x = rng.uniform(-1, 1, (1, c, h, w)).astype(np.float32)
        wt = rng.uniform(-1, 1, (ko, c, 1, 1)).astype(np.float32)
        conv = oracle.conv2d_nchw_c(x, wt, 1, 0, 1, 1)
        prod = oracle.gemm_f32_c(wt.reshape(ko, c), x.reshape(c, h * w))
        assert np.array_equal(conv.reshape(ko, h * w), prod)
        assert rel(conv.reshape(ko, h * w), wt.reshape(ko, c).astype(np.float64) @ x.reshape(c, h * w).astype(np.float64)) < 1e-6


def test_gemm_f32(oracle, gold):
    a, b = gold["gemm_a"], gold["gemm_b"]
    assert rel(oracle.gemm_f32_c(a, b), gold["gemm_c"]) < 1e-6
    assert rel(oracle.gemm_f32_c(a, b, fma=False), gold["gemm_c"]) < 1e-6
    assert rel(oracle.gemm_f32_c(a, np.ascontiguousarray(b.T), transB=True), gold["gemm_c"]) < 1e-6
    # the transposeA branches (flextensor/nn/ops.py:1093-1100): A stored [K][M]; a transposed
    # or mixed-up operand would not reproduce the same product from the same data
    at, bt = np.ascontiguousarray(a.T), np.ascontiguousarray(b.T)
    assert np.array_equal(oracle.gemm_f32_c(at, b, transA=True), oracle.gemm_f32_c(a, b))
    assert np.array_equal(oracle.gemm_f32_c(at, bt, transA=True, transB=True), oracle.gemm_f32_c(a, b))
    r = np.random.default_rng(5)
    x, y = r.uniform(-1, 1, (7, 5)).astype(np.float32), r.uniform(-1, 1, (7, 3)).astype(np.float32)
    assert rel(oracle.gemm_f32_c(x, y, transA=True), x.astype(np.float64).T @ y.astype(np.float64)) < 1e-6
    assert rel(oracle.gemm_np(a, b), gold["gemm_c"]) < 1e-13
    # identity and a permutation matrix: exact
    eye = np.eye(64, dtype=np.float32)
    assert np.array_equal(oracle.gemm_f32_c(a, eye), a)
    perm = eye[:, ::-1].copy()
    assert np.array_equal(oracle.gemm_f32_c(a, perm), a[:, ::-1])


def test_gemm_i8_exact(oracle, gold):
    a, b = gold["i8_a"], gold["i8_b"]
    c = oracle.gemm_i8_c(a, b)
    assert np.array_equal(c, gold["i8_c"])
    assert c[0, 0] == 48 * 128 * 128
    assert np.array_equal(oracle.gemm_i8_np(a, b), gold["i8_c"])
    # the reference's own check: np.dot(a.astype(int32), b.T.astype(int32))
    rng = np.random.default_rng(4)
    a = rng.integers(-128, 127, (40, 96), dtype=np.int8)
    b = rng.integers(-128, 127, (24, 96), dtype=np.int8)
    assert np.array_equal(oracle.gemm_i8_c(a, b), np.dot(a.astype("int32"), b.T.astype("int32")))
    part = oracle.gemm_i8_c(a, b, 8, 16)
    assert np.array_equal(part[8:16], np.dot(a.astype("int32"), b.T.astype("int32"))[8:16])
    assert not part[:8].any() and not part[16:].any()


def test_cpu_baseline_matches_oracle(oracle):
    rng = np.random.default_rng(5)
    a = rng.uniform(-1, 1, (70, 96)).astype(np.float32)
    b = rng.uniform(-1, 1, (96, 50)).astype(np.float32)
    c = np.empty((70, 50), np.float32)
    oracle.baseline_gemm_f32(a, b, c, 32)
    assert rel(c, oracle.gemm_np(a, b)) < 1e-6
    x = rng.uniform(-1, 1, (2, 6, 9, 20)).astype(np.float32)
    w = rng.uniform(-1, 1, (7, 6, 3, 3)).astype(np.float32)
    for st, p, d in [(1, 1, 1), (2, 1, 1), (1, 2, 2)]:
        ref = oracle.conv2d_nchw_np(x, w, st, p, d, 1)
        out = np.empty(ref.shape, np.float32)
        scratch = np.empty((2, 6, 9 + 2 * p, 20 + 2 * p), np.float32)
        oracle.baseline_conv2d(x, w, out, scratch, st, p, d)
        assert rel(out, ref) < 1e-6
    wd = rng.uniform(-1, 1, (6, 2, 3, 3)).astype(np.float32)
    for st, p, d in [(1, 1, 1), (2, 1, 2)]:
        ref = oracle.depthwise_nchw_np(x, wd, st, p, d)
        out = np.empty(ref.shape, np.float32)
        scratch = np.empty((2, 6, 9 + 2 * p, 20 + 2 * p), np.float32)
        oracle.baseline_depthwise(x, wd, out, scratch, st, p, d)
        assert rel(out, ref) < 1e-6
    ai = rng.integers(-128, 128, (20, 64), dtype=np.int8)
    bi = rng.integers(-128, 128, (12, 64), dtype=np.int8)
    ci = np.zeros((20, 12), np.int32)
    oracle.baseline_gemm_i8(ai, bi, ci)
    assert np.array_equal(ci, oracle.gemm_i8_np(ai, bi))
