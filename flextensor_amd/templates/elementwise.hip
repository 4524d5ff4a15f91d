// Small helper kernels for gfx950, hiprtc-compiled.
//
//   fill_zero_f32   zero-fill of a float buffer; precedes a split-K GEMM whose
//                   partial sums meet in C with atomics (a kernel rather than
//                   a memset call so that the launch sequence stays capturable)
//   copy_f32        streaming copy (bandwidth yardstick, counter calibration)
//   zero_pad2d_f32  P[b][c][h][w] = X[b][c][h-PT][w-PL] inside, 0 outside; PT / PB_ rows
//                   above / below, PL / PR columns left / right
//                   (flextensor/nn/ops.py:83-117), used when the graph config
//                   does not inline the padding into the convolution
//   bias_add_nchw_f32  O[b][c][h][w] = I[b][c][h][w] + bias[c] (ops.py:474-478),
//                   used when the graph config does not merge the bias into
//                   the convolution's epilogue
//   im2col_nchw_f32 col[g][k][n] = X[b][g*Cg + c][p*s + r*d - pad][q*s + t*d - pad],
//                   k = (c, r, t), n = (b, p, q), 0 outside the image
//                   (ops.py:896-950), used when the graph config does not
//                   inline the column matrix into the GEMM's loads
//   col2img_nchw_f32 O[b][c][p][q] = I[c][b*P*Q + p*Q + q] (ops.py:953-979), used
//                   when the graph config does not merge it into the GEMM's stores

typedef float f32x4 __attribute__((ext_vector_type(4)));

extern "C" __global__ __launch_bounds__(256)
void fill_zero_f32(float* __restrict__ p, int n)
{
    const int n4 = n >> 2;
    const int stride = gridDim.x * 256;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n4; i += stride)
        reinterpret_cast<f32x4*>(p)[i] = (f32x4)(0.0f);
    const int t = (n4 << 2) + blockIdx.x * 256 + threadIdx.x;
    if (t < n) p[t] = 0.0f;
}

/* plain streaming copy of n floats (n % 4 == 0): the yardstick for achievable
 * HBM bandwidth and for scaling the profiler's FETCH_SIZE / WRITE_SIZE */
extern "C" __global__ __launch_bounds__(256)
void copy_f32(const float* __restrict__ src, float* __restrict__ dst, long long n)
{
    const long long n4 = n >> 2;
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride)
        reinterpret_cast<f32x4*>(dst)[i] = reinterpret_cast<const f32x4*>(src)[i];
}

#ifdef FT_PADK
#define PB FT_PB
#define CH FT_CH
#define CW FT_CW
#define PT FT_PT
#define PBOT FT_PBOT
#define PL FT_PL
#define PR FT_PR
/* shape constants: PB planes (batch*channels), CH x CW input, padding rows above / below
 * and columns left / right (flextensor/nn/ops.py:83-117 takes all four) */
#define PH (CH + PT + PBOT)
#define PW (CW + PL + PR)
extern "C" __global__ __launch_bounds__(256)
void zero_pad2d_f32(const float* __restrict__ X, float* __restrict__ P)
{
    const int gid = blockIdx.x * 256 + threadIdx.x;
    if (gid >= PB * PH * PW) return;
    const int w = gid % PW;
    const int h = (gid / PW) % PH;
    const int pl = gid / (PW * PH);
    const int ih = h - PT, iw = w - PL;
    const bool ok = (unsigned)ih < (unsigned)CH && (unsigned)iw < (unsigned)CW;
    P[gid] = ok ? X[(size_t)pl * (CH * CW) + ih * CW + iw] : 0.0f;
}
#endif

/* n = total elements, hw = elements per plane, c = channels */
extern "C" __global__ __launch_bounds__(256)
void bias_add_nchw_f32(const float* __restrict__ I, const float* __restrict__ bias,
                       float* __restrict__ O, int n, int hw, int c)
{
    const int stride = gridDim.x * 256;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        O[i] = I[i] + bias[(i / hw) % c];
}

#ifdef FT_COLK
/* convolution geometry: CB batch, CG groups, CC input channels, CH x CW the
 * image as stored (already padded when CPADH/CPADW are 0 and the padding is its own
 * operator), CR x CS window, CP x CQ output plane, MG output channels per group */
#define CB FT_CB
#define CG FT_CG
#define CC FT_CC
#define CH FT_CH
#define CW FT_CW
#define CR FT_CR
#define CS FT_CS
#define CSTRH FT_CSTRH
#define CSTRW FT_CSTRW
#define CPADH FT_CPADH
#define CPADW FT_CPADW
#define CDILH FT_CDILH
#define CDILW FT_CDILW
#define CP FT_CP
#define CQ FT_CQ
#define MG FT_MG
#define COL_K ((CC / CG) * CR * CS)
#define COL_N (CB * CP * CQ)
extern "C" __global__ __launch_bounds__(256)
void im2col_nchw_f32(const float* __restrict__ X, float* __restrict__ col)
{
    const long long total = (long long)CG * COL_K * COL_N;
    const long long stride = (long long)gridDim.x * 256;
    for (long long gid = (long long)blockIdx.x * 256 + threadIdx.x; gid < total; gid += stride) {
        const int n = (int)(gid % COL_N);
        const int k = (int)((gid / COL_N) % COL_K);
        const int g = (int)(gid / ((long long)COL_N * COL_K));
        const int b = n / (CP * CQ);
        const int p = (n % (CP * CQ)) / CQ;
        const int q = n % CQ;
        const int c = g * (CC / CG) + k / (CR * CS);
        const int ih = p * CSTRH + ((k % (CR * CS)) / CS) * CDILH - CPADH;
        const int iw = q * CSTRW + (k % CS) * CDILW - CPADW;
        const bool ok = (unsigned)ih < (unsigned)CH && (unsigned)iw < (unsigned)CW;
        col[gid] = ok ? X[((size_t)b * CC + c) * (CH * CW) + ih * CW + iw] : 0.0f;
    }
}

extern "C" __global__ __launch_bounds__(256)
void col2img_nchw_f32(const float* __restrict__ I, float* __restrict__ O)
{
    const long long total = (long long)CG * MG * COL_N;
    const long long stride = (long long)gridDim.x * 256;
    for (long long gid = (long long)blockIdx.x * 256 + threadIdx.x; gid < total; gid += stride) {
        const int pq = (int)(gid % (CP * CQ));
        const int c = (int)((gid / (CP * CQ)) % (CG * MG));
        const int b = (int)(gid / ((long long)(CP * CQ) * (CG * MG)));
        O[gid] = I[(size_t)c * COL_N + (size_t)b * (CP * CQ) + pq];
    }
}
#endif
