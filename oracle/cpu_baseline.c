/*
 * cpu_baseline.c — multi-threaded CPU versions of the four operators with the
 * loop structure the reference's llvm template produces
 * (flextensor/templates/cpu.py:316-518, cpu_schedule_simple): the outermost
 * tiles of all spatial axes fused into one `parallel` loop (:387), a local
 * accumulation block ("cache_write") per inner tile (:320, :408), the
 * innermost reduce loop placed outside the innermost spatial loops
 * (:484-493), the innermost spatial axis vectorised (:505) and the remaining
 * inner spatial tile unrolled (:506-514).
 *
 * TEST/BENCH INFRASTRUCTURE ONLY (bench.py's cpu_baseline leg): this is the
 * reference's CPU path timed beside the GPU result, not a product path. Each
 * output element is still accumulated over k in ascending order with one fp32
 * accumulator, so results equal oracle.c's with fma=1 up to the compiler's
 * choice of FMA contraction.
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

int ftb_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* C[M][N] = A[M][K] * B[K][N]; register tile TI rows (unrolled) x TJ columns
 * (vectorised), tk = K tile kept in cache. One function per register tile of
 * the small sweep the benchmark runs (the reference's tuner would pick among
 * such splits, flextensor/templates/cpu.py:330-372). */
#define FTB_DEFINE_GEMM(TI, TJ)                                                                   \
    static void gemm_f32_##TI##x##TJ(const float *A, const float *B, float *C, int M, int N,      \
                                     int K, int tk)                                               \
    {                                                                                             \
        const int nio = (M + TI - 1) / TI, njo = (N + TJ - 1) / TJ;                               \
        if (tk < 1) tk = K;                                                                       \
        _Pragma("omp parallel for schedule(static)")                                              \
        for (int t = 0; t < nio * njo; ++t) {                                                     \
            const int i0 = (t / njo) * TI, j0 = (t % njo) * TJ;                                   \
            const int ni = (M - i0) < TI ? (M - i0) : TI;                                         \
            const int nj = (N - j0) < TJ ? (N - j0) : TJ;                                         \
            float acc[TI][TJ];                                                                    \
            memset(acc, 0, sizeof acc);                                                           \
            for (int k0 = 0; k0 < K; k0 += tk) {                                                  \
                const int k1 = (k0 + tk) < K ? (k0 + tk) : K;                                     \
                if (ni == TI && nj == TJ) {                                                       \
                    for (int k = k0; k < k1; ++k)                                                 \
                        for (int i = 0; i < TI; ++i) {                                            \
                            const float a = A[(size_t)(i0 + i) * K + k];                          \
                            _Pragma("omp simd")                                                   \
                            for (int j = 0; j < TJ; ++j)                                          \
                                acc[i][j] += a * B[(size_t)k * N + j0 + j];                       \
                        }                                                                         \
                } else {                                                                          \
                    for (int k = k0; k < k1; ++k)                                                 \
                        for (int i = 0; i < ni; ++i) {                                            \
                            const float a = A[(size_t)(i0 + i) * K + k];                          \
                            for (int j = 0; j < nj; ++j)                                          \
                                acc[i][j] += a * B[(size_t)k * N + j0 + j];                       \
                        }                                                                         \
                }                                                                                 \
            }                                                                                     \
            for (int i = 0; i < ni; ++i)                                                          \
                for (int j = 0; j < nj; ++j) C[(size_t)(i0 + i) * N + j0 + j] = acc[i][j];        \
        }                                                                                         \
    }
FTB_DEFINE_GEMM(6, 32)
FTB_DEFINE_GEMM(4, 32)
FTB_DEFINE_GEMM(8, 16)
FTB_DEFINE_GEMM(6, 16)
FTB_DEFINE_GEMM(4, 64)

/* number of register-tile variants, their (rows, columns), and the call by variant index */
int ftb_gemm_f32_variants(void) { return 5; }
void ftb_gemm_f32_variant_tile(int v, int *ti, int *tj)
{
    static const int t[5][2] = {{6, 32}, {4, 32}, {8, 16}, {6, 16}, {4, 64}};
    *ti = t[v][0];
    *tj = t[v][1];
}
void ftb_gemm_f32_v(const float *A, const float *B, float *C, int M, int N, int K, int tk, int v)
{
    switch (v) {
    case 1: gemm_f32_4x32(A, B, C, M, N, K, tk); break;
    case 2: gemm_f32_8x16(A, B, C, M, N, K, tk); break;
    case 3: gemm_f32_6x16(A, B, C, M, N, K, tk); break;
    case 4: gemm_f32_4x64(A, B, C, M, N, K, tk); break;
    default: gemm_f32_6x32(A, B, C, M, N, K, tk); break;
    }
}
void ftb_gemm_f32(const float *A, const float *B, float *C, int M, int N, int K, int tk)
{
    gemm_f32_6x32(A, B, C, M, N, K, tk);
}

/* C[M][N] int32 = A[M][K] int8 * B[N][K]^T int8 */
void ftb_gemm_i8(const int8_t *A, const int8_t *B, int32_t *C, int M, int N, int K, int row0,
                 int row1)
{
    (void)M;
#pragma omp parallel for schedule(static)
    for (int i = row0; i < row1; ++i) {
        const int8_t *a = A + (size_t)i * K;
        for (int j = 0; j < N; ++j) {
            const int8_t *b = B + (size_t)j * K;
            int32_t acc = 0;
#pragma omp simd reduction(+ : acc)
            for (int k = 0; k < K; ++k) acc += (int32_t)a[k] * (int32_t)b[k];
            C[(size_t)i * N + j] = acc;
        }
    }
}

static void pad2d(const float *X, float *P, int planes, int H, int W, int ph, int pw)
{
    const int PH = H + 2 * ph, PW = W + 2 * pw;
#pragma omp parallel for schedule(static)
    for (int p = 0; p < planes; ++p) {
        float *dst = P + (size_t)p * PH * PW;
        memset(dst, 0, (size_t)PH * PW * sizeof(float));
        for (int h = 0; h < H; ++h)
            memcpy(dst + (size_t)(h + ph) * PW + pw, X + ((size_t)p * H + h) * W,
                   (size_t)W * sizeof(float));
    }
}

/* conv2d NCHW, groups = 1; register tile TKO output channels (unrolled) x TW
 * output columns (vectorised). `scratch` holds the padded input
 * (NB*C*(H+2ph)*(W+2pw) floats) and is written inside the call, as the
 * reference's two-operator graph does. */
#define FTB_DEFINE_CONV(TKO, TW)                                                                  \
    static void conv2d_nchw_##TKO##x##TW(const float *X, const float *Wt, float *O,               \
                                         float *scratch, int NB, int C, int H, int W, int KO,     \
                                         int R, int S, int st, int pd, int dl)                    \
    {                                                                                             \
        const int PH = H + 2 * pd, PW = W + 2 * pd;                                               \
        const int P = (H + 2 * pd - dl * (R - 1) - 1) / st + 1;                                   \
        const int Q = (W + 2 * pd - dl * (S - 1) - 1) / st + 1;                                   \
        pad2d(X, scratch, NB * C, H, W, pd, pd);                                                  \
        const int nko = (KO + TKO - 1) / TKO;                                                     \
        _Pragma("omp parallel for schedule(static) collapse(3)")                                  \
        for (int b = 0; b < NB; ++b)                                                              \
            for (int kt = 0; kt < nko; ++kt)                                                      \
                for (int h = 0; h < P; ++h) {                                                     \
                    const int k0 = kt * TKO;                                                      \
                    const int nk = (KO - k0) < TKO ? (KO - k0) : TKO;                             \
                    for (int w0 = 0; w0 < Q; w0 += TW) {                                          \
                        const int nw = (Q - w0) < TW ? (Q - w0) : TW;                             \
                        float acc[TKO][TW];                                                       \
                        memset(acc, 0, sizeof acc);                                               \
                        for (int rc = 0; rc < C; ++rc)                                            \
                            for (int rw = 0; rw < S; ++rw)                                        \
                                for (int rh = 0; rh < R; ++rh) {                                  \
                                    const float *xr = scratch +                                   \
                                        (((size_t)b * C + rc) * PH + h * st + rh * dl) * PW +     \
                                        (size_t)w0 * st + rw * dl;                                \
                                    for (int kk = 0; kk < nk; ++kk) {                             \
                                        const float wv =                                          \
                                            Wt[(((size_t)(k0 + kk) * C + rc) * R + rh) * S + rw]; \
                                        if (st == 1) {                                            \
                                            _Pragma("omp simd")                                   \
                                            for (int ww = 0; ww < TW; ++ww)                       \
                                                if (ww < nw) acc[kk][ww] += xr[ww] * wv;          \
                                        } else {                                                  \
                                            for (int ww = 0; ww < nw; ++ww)                       \
                                                acc[kk][ww] += xr[(size_t)ww * st] * wv;          \
                                        }                                                         \
                                    }                                                             \
                                }                                                                 \
                        for (int kk = 0; kk < nk; ++kk)                                           \
                            for (int ww = 0; ww < nw; ++ww)                                       \
                                O[(((size_t)b * KO + k0 + kk) * P + h) * Q + w0 + ww] = acc[kk][ww]; \
                    }                                                                             \
                }                                                                                 \
    }
FTB_DEFINE_CONV(4, 16)
FTB_DEFINE_CONV(8, 16)
FTB_DEFINE_CONV(4, 32)
FTB_DEFINE_CONV(2, 16)
FTB_DEFINE_CONV(8, 8)

int ftb_conv2d_variants(void) { return 5; }
void ftb_conv2d_variant_tile(int v, int *tko, int *tw)
{
    static const int t[5][2] = {{4, 16}, {8, 16}, {4, 32}, {2, 16}, {8, 8}};
    *tko = t[v][0];
    *tw = t[v][1];
}
void ftb_conv2d_nchw_v(const float *X, const float *Wt, float *O, float *scratch, int NB, int C,
                       int H, int W, int KO, int R, int S, int st, int pd, int dl, int v)
{
    switch (v) {
    case 1: conv2d_nchw_8x16(X, Wt, O, scratch, NB, C, H, W, KO, R, S, st, pd, dl); break;
    case 2: conv2d_nchw_4x32(X, Wt, O, scratch, NB, C, H, W, KO, R, S, st, pd, dl); break;
    case 3: conv2d_nchw_2x16(X, Wt, O, scratch, NB, C, H, W, KO, R, S, st, pd, dl); break;
    case 4: conv2d_nchw_8x8(X, Wt, O, scratch, NB, C, H, W, KO, R, S, st, pd, dl); break;
    default: conv2d_nchw_4x16(X, Wt, O, scratch, NB, C, H, W, KO, R, S, st, pd, dl); break;
    }
}
void ftb_conv2d_nchw(const float *X, const float *Wt, float *O, float *scratch, int NB, int C,
                     int H, int W, int KO, int R, int S, int st, int pd, int dl)
{
    conv2d_nchw_4x16(X, Wt, O, scratch, NB, C, H, W, KO, R, S, st, pd, dl);
}

/* depthwise conv2d NCHW, weight [C][F][R][S] */
void ftb_depthwise_nchw(const float *X, const float *Wt, float *O, float *scratch, int NB, int C,
                        int H, int W, int F, int R, int S, int st, int pd, int dl)
{
    const int PH = H + 2 * pd, PW = W + 2 * pd;
    const int P = (H + 2 * pd - dl * (R - 1) - 1) / st + 1;
    const int Q = (W + 2 * pd - dl * (S - 1) - 1) / st + 1;
    const int CO = C * F;
    pad2d(X, scratch, NB * C, H, W, pd, pd);
#pragma omp parallel for schedule(static) collapse(2)
    for (int b = 0; b < NB; ++b)
        for (int c = 0; c < CO; ++c) {
            const float *xp = scratch + ((size_t)b * C + c / F) * PH * PW;
            const float *wp = Wt + (size_t)c * R * S;
            float *op = O + ((size_t)b * CO + c) * P * Q;
            for (int h = 0; h < P; ++h) {
                float *orow = op + (size_t)h * Q;
                for (int w = 0; w < Q; ++w) orow[w] = 0.0f;
                for (int rw = 0; rw < S; ++rw)
                    for (int rh = 0; rh < R; ++rh) {
                        const float wv = wp[rh * S + rw];
                        const float *xr = xp + (size_t)(h * st + rh * dl) * PW + rw * dl;
                        if (st == 1) {
#pragma omp simd
                            for (int w = 0; w < Q; ++w) orow[w] += xr[w] * wv;
                        } else {
                            for (int w = 0; w < Q; ++w) orow[w] += xr[(size_t)w * st] * wv;
                        }
                    }
            }
        }
}
