// Plain one-output-per-lane kernels for gfx950, hiprtc-compiled once.
//
// They play the role of the reference's *default schedule* build
// (te.create_schedule + tvm.build in flextensor/optimize/common.py:66-75):
// an untuned, obviously-structured lowering of each operator whose result
// every tuned candidate is compared against on the device before its timing
// is admitted. Loop order follows the operator definitions: spatial axes in
// declaration order (one lane each), then the reduce axes in the order the
// reference declares them ([rc, rw, rh] for conv2d, [rw, rh] for depthwise,
// k for GEMM), fp32 accumulation from zero.
//
// Shapes are run-time arguments so that one code object serves every task.

extern "C" __global__ __launch_bounds__(256)
void gemm_f32_naive(const float* __restrict__ A, const float* __restrict__ B,
                    float* __restrict__ C, int M, int N, int K, int transB, int transA)
{
    /* A is [M][K], or [K][M] when transA; B is [K][N], or [N][K] when transB */
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (long long)M * N) return;
    const int i = (int)(gid / N), j = (int)(gid % N);
    const size_t a0 = transA ? (size_t)i : (size_t)i * K, as = transA ? (size_t)M : 1;
    const size_t b0 = transB ? (size_t)j * K : (size_t)j, bs = transB ? 1 : (size_t)N;
    float acc = 0.0f;
    for (int k = 0; k < K; ++k) acc += A[a0 + k * as] * B[b0 + k * bs];
    C[gid] = acc;
}

extern "C" __global__ __launch_bounds__(256)
void gemm_i8_naive(const signed char* __restrict__ A, const signed char* __restrict__ B,
                   int* __restrict__ C, int M, int N, int K)
{
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (long long)M * N) return;
    const int i = (int)(gid / N), j = (int)(gid % N);
    int acc = 0;
    for (int k = 0; k < K; ++k)
        acc += (int)A[(size_t)i * K + k] * (int)B[(size_t)j * K + k];
    C[gid] = acc;
}

/* X [NB][C][H][W], Wt [KO][C/G][R][S], O [NB][KO][P][Q] */
extern "C" __global__ __launch_bounds__(256)
void conv2d_nchw_naive(const float* __restrict__ X, const float* __restrict__ Wt,
                       float* __restrict__ O, int NB, int C, int H, int W, int KO,
                       int R, int S, int sh, int sw, int ph, int pw, int dh, int dw,
                       int G, int P, int Q)
{
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (long long)NB * KO * P * Q) return;
    const int q = (int)(gid % Q);
    const int p = (int)((gid / Q) % P);
    const int ko = (int)((gid / ((long long)Q * P)) % KO);
    const int b = (int)(gid / ((long long)Q * P * KO));
    const int cg = C / G, kg = KO / G;
    const int c0 = (ko / kg) * cg;
    float acc = 0.0f;
    for (int rc = 0; rc < cg; ++rc)
        for (int rw = 0; rw < S; ++rw)
            for (int rh = 0; rh < R; ++rh) {
                const int ih = p * sh + rh * dh - ph;
                const int iw = q * sw + rw * dw - pw;
                if ((unsigned)ih < (unsigned)H && (unsigned)iw < (unsigned)W)
                    acc += X[(((size_t)b * C + c0 + rc) * H + ih) * W + iw] *
                           Wt[(((size_t)ko * cg + rc) * R + rh) * S + rw];
            }
    O[gid] = acc;
}

/* X [NB][C][H][W], Wt [C][F][R][S], O [NB][C*F][P][Q] */
extern "C" __global__ __launch_bounds__(256)
void depthwise_nchw_naive(const float* __restrict__ X, const float* __restrict__ Wt,
                          float* __restrict__ O, int NB, int C, int H, int W, int F,
                          int R, int S, int sh, int sw, int ph, int pw, int dh, int dw,
                          int P, int Q)
{
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (long long)NB * C * F * P * Q) return;
    const int q = (int)(gid % Q);
    const int p = (int)((gid / Q) % P);
    const int co = (int)((gid / ((long long)Q * P)) % (C * F));
    const int b = (int)(gid / ((long long)Q * P * C * F));
    const int ci = co / F;
    float acc = 0.0f;
    for (int rw = 0; rw < S; ++rw)
        for (int rh = 0; rh < R; ++rh) {
            const int ih = p * sh + rh * dh - ph;
            const int iw = q * sw + rw * dw - pw;
            if ((unsigned)ih < (unsigned)H && (unsigned)iw < (unsigned)W)
                acc += X[(((size_t)b * C + ci) * H + ih) * W + iw] *
                       Wt[((size_t)co * R + rh) * S + rw];
        }
    O[gid] = acc;
}

/* P [PL][H+pt+pb][W+pl+pr] from X [PL][H][W] */
extern "C" __global__ __launch_bounds__(256)
void zero_pad2d_naive(const float* __restrict__ X, float* __restrict__ P, int PL, int H, int W,
                      int pt, int pb, int pl, int pr)
{
    const int PH = H + pt + pb, PW = W + pl + pr;
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (long long)PL * PH * PW) return;
    const int w = (int)(gid % PW);
    const int h = (int)((gid / PW) % PH);
    const int pln = (int)(gid / ((long long)PW * PH));
    const int ih = h - pt, iw = w - pl;
    const bool ok = (unsigned)ih < (unsigned)H && (unsigned)iw < (unsigned)W;
    P[gid] = ok ? X[((size_t)pln * H + ih) * W + iw] : 0.0f;
}

/* res[0] = bits of max|out-ref| (+inf if out holds a NaN), res[1] = bits of
 * max|ref|. Non-negative floats order like their bit patterns, so an integer
 * atomic max suffices. The caller zero-fills res. */
extern "C" __global__ __launch_bounds__(256)
void check_f32(const float* __restrict__ out, const float* __restrict__ ref, long long n,
               unsigned* __restrict__ res)
{
    float md = 0.0f, mr = 0.0f;
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const float o = out[i], r = ref[i];
        float d = fabsf(o - r);
        if (!(d == d)) d = __builtin_inff();
        md = fmaxf(md, d);
        mr = fmaxf(mr, fabsf(r));
    }
    for (int off = 32; off > 0; off >>= 1) {
        md = fmaxf(md, __shfl_down(md, off, 64));
        mr = fmaxf(mr, __shfl_down(mr, off, 64));
    }
    if ((threadIdx.x & 63) == 0) {
        atomicMax(res + 0, __float_as_uint(md));
        atomicMax(res + 1, __float_as_uint(mr));
    }
}

/* res[0] += number of positions where out != ref. The caller zero-fills res. */
extern "C" __global__ __launch_bounds__(256)
void check_i32(const int* __restrict__ out, const int* __restrict__ ref, long long n,
               unsigned* __restrict__ res)
{
    unsigned bad = 0;
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        bad += (out[i] != ref[i]) ? 1u : 0u;
    for (int off = 32; off > 0; off >>= 1) bad += __shfl_down(bad, off, 64);
    if ((threadIdx.x & 63) == 0 && bad) atomicAdd(res, bad);
}

extern "C" __global__ __launch_bounds__(256)
void fill_u32(unsigned* __restrict__ p, unsigned v, long long n)
{
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) p[i] = v;
}
