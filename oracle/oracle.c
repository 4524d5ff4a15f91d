/*
 * oracle.c — CPU restatement of the operator arithmetic the tuned GPU kernels
 * must reproduce. TEST INFRASTRUCTURE ONLY: it is built into
 * oracle/liboracle.so and may be loaded by tests/, __graft_entry__.smoke()
 * and bench.py's cpu_baseline leg, never by the flextensor_amd package.
 *
 * What it restates. The reference defines its operators as TVM tensor
 * expressions and executes whatever TVM's LLVM backend emits for them; TVM
 * (fork KnowingNothing/tvm@mirror, README.md:46, unversioned and not
 * vendored) is not available, so the published semantics of a te.compute with
 * te.sum are restated directly: one output element per point of the spatial
 * axes taken in declaration order, an fp32 (int32) accumulator initialised to
 * zero, and the reduce axes iterated as nested loops in the order of the
 * axis=[...] list, outermost first. Each function names the expression it
 * follows:
 *
 *   ft_zero_pad2d        flextensor/nn/ops.py:83-117
 *   ft_conv2d_nchw       flextensor/nn/ops.py:419-479  (reduce order rc, rw, rh;
 *                        reads the materialised padded tensor, as the graph does)
 *   ft_depthwise_nchw    flextensor/nn/ops.py:622-678  (reduce order rw, rh)
 *   ft_gemm_f32          flextensor/nn/ops.py:1074-1108 (all four transposeA / transposeB branches)
 *   ft_gemm_i8           flextensor/test/test_tvm/legacy/gemm_int8.py:15-21
 *
 * Pinning (see tests/test_oracle.py): every function is checked against
 * independent routines — numpy matmul in float64 / exact integer dot, torch's
 * CPU conv2d (the call the reference's own tests compare with,
 * flextensor/test/test_ops.py:85-115, 152-184), brute-force Python loops on
 * tiny shapes, and closed forms (padding, output size). The one thing that
 * cannot be pinned without a live TVM is the last-bit fp32 rounding of its
 * LLVM build (FMA contraction); both roundings are provided (`fma` flag) and
 * the fp32 acceptance bound of 1e-5 * max|ref| covers either.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(__GNUC__)
#define FT_NOCONTRACT _Pragma("STDC FP_CONTRACT OFF")
#else
#define FT_NOCONTRACT
#endif

/* a*b + c with one rounding (fma=1) or two (fma=0). volatile-free: the file is
 * compiled with -ffp-contract=off so the two-rounding form stays two roundings. */
static inline float mac(float acc, float a, float b, int fma)
{
    if (fma) return fmaf(a, b, acc);
    float p = a * b;
    return acc + p;
}

/* out-size formula of ops.py:458-459 */
int ft_conv_out_size(int in, int pad, int dil, int k, int stride)
{
    return (in + 2 * pad - dil * (k - 1) - 1) / stride + 1;
}

/* P[b][c][h][w] = X[b][c][h-pt][w-pl] inside, 0 outside; P is
 * [planes][H+pt+pb][W+pl+pr]. */
void ft_zero_pad2d(const float *X, float *P, int planes, int H, int W, int pt, int pb, int pl,
                   int pr)
{
    const int PH = H + pt + pb, PW = W + pl + pr;
    for (int p = 0; p < planes; ++p)
        for (int h = 0; h < PH; ++h)
            for (int w = 0; w < PW; ++w) {
                const int ih = h - pt, iw = w - pl;
                const int inside = (h >= pt) && (h < H + pt) && (w >= pl) && (w < W + pl);
                P[((size_t)p * PH + h) * PW + w] =
                    inside ? X[((size_t)p * H + ih) * W + iw] : 0.0f;
            }
}

/* O[b][k][h][w] = sum_{rc,rw,rh} P[b][(k/Kg)*Cg+rc][h*sh+rh*dh][w*sw+rw*dw] * Wt[k][rc][rh][rw]
 * X [NB][C][H][W], Wt [KO][C/G][R][S], O [NB][KO][P][Q]. Returns 0, or -1 when
 * the scratch buffer for the padded tensor cannot be allocated. */
int ft_conv2d_nchw(const float *X, const float *Wt, float *O, int NB, int C, int H, int W, int KO,
                   int R, int S, int sh, int sw, int ph, int pw, int dh, int dw, int G, int fma)
{
    const int PH = H + 2 * ph, PW = W + 2 * pw;
    const int P = ft_conv_out_size(H, ph, dh, R, sh);
    const int Q = ft_conv_out_size(W, pw, dw, S, sw);
    const int cg = C / G, kg = KO / G;
    float *pad = (float *)malloc((size_t)NB * C * PH * PW * sizeof(float));
    if (!pad) return -1;
    ft_zero_pad2d(X, pad, NB * C, H, W, ph, ph, pw, pw);
    for (int b = 0; b < NB; ++b)
        for (int k = 0; k < KO; ++k)
            for (int h = 0; h < P; ++h)
                for (int w = 0; w < Q; ++w) {
                    float acc = 0.0f;
                    const int c0 = (k / kg) * cg;
                    for (int rc = 0; rc < cg; ++rc)
                        for (int rw = 0; rw < S; ++rw)
                            for (int rh = 0; rh < R; ++rh) {
                                const float x =
                                    pad[(((size_t)b * C + c0 + rc) * PH + h * sh + rh * dh) * PW +
                                        w * sw + rw * dw];
                                const float wt = Wt[(((size_t)k * cg + rc) * R + rh) * S + rw];
                                acc = mac(acc, x, wt, fma);
                            }
                    O[(((size_t)b * KO + k) * P + h) * Q + w] = acc;
                }
    free(pad);
    return 0;
}

/* O[b][c][h][w] = sum_{rw,rh} P[b][c/F][h*sh+rh*dh][w*sw+rw*dw] * Wt[c/F][c%F][rh][rw]
 * X [NB][C][H][W], Wt [C][F][R][S], O [NB][C*F][P][Q]. */
int ft_depthwise_nchw(const float *X, const float *Wt, float *O, int NB, int C, int H, int W,
                      int F, int R, int S, int sh, int sw, int ph, int pw, int dh, int dw, int fma)
{
    const int PH = H + 2 * ph, PW = W + 2 * pw;
    const int P = ft_conv_out_size(H, ph, dh, R, sh);
    const int Q = ft_conv_out_size(W, pw, dw, S, sw);
    const int CO = C * F;
    float *pad = (float *)malloc((size_t)NB * C * PH * PW * sizeof(float));
    if (!pad) return -1;
    ft_zero_pad2d(X, pad, NB * C, H, W, ph, ph, pw, pw);
    for (int b = 0; b < NB; ++b)
        for (int c = 0; c < CO; ++c)
            for (int h = 0; h < P; ++h)
                for (int w = 0; w < Q; ++w) {
                    float acc = 0.0f;
                    for (int rw = 0; rw < S; ++rw)
                        for (int rh = 0; rh < R; ++rh) {
                            const float x =
                                pad[(((size_t)b * C + c / F) * PH + h * sh + rh * dh) * PW +
                                    w * sw + rw * dw];
                            const float wt = Wt[(((size_t)(c / F) * F + c % F) * R + rh) * S + rw];
                            acc = mac(acc, x, wt, fma);
                        }
                    O[(((size_t)b * CO + c) * P + h) * Q + w] = acc;
                }
    free(pad);
    return 0;
}

/* C[i][j] = sum_k A[i][k] * B[k][j]  (transB: B stored [N][K], B[j][k]) */
void ft_gemm_f32(const float *A, const float *B, float *C, int M, int N, int K, int transB,
                 int fma, int transA)
{
    /* A is [M][K], or [K][M] when transA; B is [K][N], or [N][K] when transB (ops.py:1093-1108) */
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            float acc = 0.0f;
            for (int k = 0; k < K; ++k) {
                const float a = transA ? A[(size_t)k * M + i] : A[(size_t)i * K + k];
                const float b = transB ? B[(size_t)j * K + k] : B[(size_t)k * N + j];
                acc = mac(acc, a, b, fma);
            }
            C[(size_t)i * N + j] = acc;
        }
}

/* rows [row0, row1) of C[i][j] = sum_k int32(A[i][k]) * int32(B[j][k]);
 * A [M][K], B [N][K] (K-major), C [M][N]. */
void ft_gemm_i8(const int8_t *A, const int8_t *B, int32_t *C, int M, int N, int K, int row0,
                int row1)
{
    (void)M;
    for (int i = row0; i < row1; ++i)
        for (int j = 0; j < N; ++j) {
            int32_t acc = 0;
            const int8_t *a = A + (size_t)i * K;
            const int8_t *b = B + (size_t)j * K;
            for (int k = 0; k < K; ++k) acc += (int32_t)a[k] * (int32_t)b[k];
            C[(size_t)i * N + j] = acc;
        }
}
