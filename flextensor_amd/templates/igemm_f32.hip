// fp32 implicit-GEMM kernel template for gfx950 (CDNA4), compiled with hiprtc.
//
//   C[M][N] (+)= A[M][K] * B[K][N]        fp32 in, fp32 MFMA accumulate
//
// One source serves two operators; every shape and knob is a -D constant:
//   MODE 0  dense GEMM        A row-major [M][K], B row-major [K][N]
//                             (flextensor/nn/ops.py:1105-1108)
//   MODE 2  dense GEMM, B^T   A row-major [M][K], B stored [N][K]
//                             (the transposeB branch, ops.py:1101-1104)
//   MODE 1  conv2d NCHW       A = weight [Kout][C*R*S], B = im2col gather of
//                             the input with zero padding folded into the
//                             load predicate, N = batch*OH*OW
//                             (flextensor/nn/ops.py:83-117, 419-479)
//
// Knobs (set by the scheduler from a Config):
//   MFMA            32 -> v_mfma_f32_32x32x2_f32, 16 -> v_mfma_f32_16x16x4_f32
//   WAVES_M/N       wavefronts per workgroup along M / N
//   REP_M/N         MFMA tiles per wavefront along M / N
//   BK              K extent of one LDS tile
//   STAGES          1 or 2 LDS buffers (2 = global loads of tile t+1 overlap
//                   the MFMAs of tile t)
//   SPLITK          grid-level split of K; partial sums meet with float
//                   atomics in C, which the caller zero-fills first
//   GROUP_M         tile-traversal group height (L2 locality)
//   XCD_REMAP       1: consecutive logical tiles stay on one XCD
//   APAD / BPAD     LDS row padding in floats
//
// LDS layout: As[BM][BK+APAD] (k contiguous, read as one 128-bit load per
// lane per 4 k-steps), Bs[BK][BN+BPAD] (n contiguous, read as 32-bit loads).
// Within a k-block of 4*KL values, lane group g of an MFMA takes
// k = 4*g + s at step s for both operands, so the sum over k is unchanged.

/* Constants arrive as -DFT_<NAME>=value: single-letter macros on the command line
 * would be visible to (and break) the runtime-compilation built-in headers. */
#define MODE FT_MODE
#define M FT_M
#define N FT_N
#define K FT_K
#define KP FT_KP
#define MFMA FT_MFMA
#define WAVES_M FT_WAVES_M
#define WAVES_N FT_WAVES_N
#define REP_M FT_REP_M
#define REP_N FT_REP_N
#define BK FT_BK
#define STAGES FT_STAGES
#define SPLITK FT_SPLITK
#define GROUP_M FT_GROUP_M
#define XCD_REMAP FT_XCD_REMAP
#define APAD FT_APAD
#define BPAD FT_BPAD
#define AV FT_AV
#define BV FT_BV

#ifndef FT_MODE
#error "FT_MODE must be defined"
#endif

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#if MFMA == 32
typedef f32x16 acc_t;
#define NACC 16
#define MFMA_OP(a, b, c) __builtin_amdgcn_mfma_f32_32x32x2f32((a), (b), (c), 0, 0, 0)
#elif MFMA == 16
typedef f32x4 acc_t;
#define NACC 4
#define MFMA_OP(a, b, c) __builtin_amdgcn_mfma_f32_16x16x4f32((a), (b), (c), 0, 0, 0)
#else
#error "MFMA must be 16 or 32"
#endif

#define KL (64 / MFMA)            /* k values consumed per MFMA             */
#define KBLK (4 * KL)             /* k values per 128-bit A fragment round  */
#define BM (WAVES_M * REP_M * MFMA)
#define BN (WAVES_N * REP_N * MFMA)
#define NT (WAVES_M * WAVES_N * 64)
#define SA (BK + APAD)
#if MODE == 2
#define SB (BK + APAD)            /* Bs[BN][SB], k contiguous like As */
#define BS_FLOATS (BN * SB)
#else
#define SB (BN + BPAD)            /* Bs[BK][SB], n contiguous */
#define BS_FLOATS (BK * SB)
#endif
#define TILES_M ((M + BM - 1) / BM)
#define TILES_N ((N + BN - 1) / BN)
/* KP = K rounded up to a multiple of 16; the host checks KP % (SPLITK*BK) == 0.
 * When KP != K the tail is zero-filled by the load predicates. */
#define KSPLIT_LEN (KP / SPLITK)
#define KT (KSPLIT_LEN / BK)

#if BK % KBLK != 0
#error "BK must be a multiple of 4*(64/MFMA)"
#endif

/* ---- A tile: BM x BK, vectors of AV floats along K ---------------------- */
#define A_CHUNKS_ROW (BK / AV)
#define A_CHUNKS (BM * A_CHUNKS_ROW)
#define EA ((A_CHUNKS + NT - 1) / NT)
/* ---- B tile: BK x BN, vectors of BV floats along N (along K in MODE 2) --- */
#if MODE == 2
#define B_CHUNKS_ROW (BK / BV)
#define B_CHUNKS (BN * B_CHUNKS_ROW)
#else
#define B_CHUNKS_ROW (BN / BV)
#define B_CHUNKS (BK * B_CHUNKS_ROW)
#endif
#define EB ((B_CHUNKS + NT - 1) / NT)

#if AV == 4
typedef f32x4 avec_t;
#elif AV == 1
typedef float avec_t;
#else
#error "AV must be 1 or 4"
#endif
#if BV == 4
typedef f32x4 bvec_t;
#elif BV == 1
typedef float bvec_t;
#else
#error "BV must be 1 or 4"
#endif

#if MODE == 1
#define CB FT_CB
#define CC FT_CC
#define CH FT_CH
#define CW FT_CW
#define CR FT_CR
#define CS FT_CS
#define CSTR FT_CSTR
#define CPAD FT_CPAD
#define CDIL FT_CDIL
#define CP FT_CP
#define CQ FT_CQ
/* conv geometry, all compile-time: input [CB][CC][CH][CW], kernel CR x CS,
 * stride CSTR, padding CPAD, dilation CDIL, output CP x CQ. */
#define OHW (CP * CQ)
#if BV != 1
#error "conv mode gathers scalars: BV must be 1"
#endif
#endif

extern "C" __global__ __launch_bounds__(NT)
void igemm_f32(const float* __restrict__ A, const float* __restrict__ B,
               float* __restrict__ C)
{
    __shared__ __attribute__((aligned(16))) float As[STAGES][BM * SA];
    __shared__ __attribute__((aligned(16))) float Bs[STAGES][BS_FLOATS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N;
    const int wn = wave % WAVES_N;
    const int li = lane % MFMA;   /* row (A) / column (B, C) inside an MFMA tile */
    const int lg = lane / MFMA;   /* k group */

    /* ---- workgroup -> (split, tile_m, tile_n) ------------------------- */
    const int nblk = TILES_M * TILES_N * SPLITK;
    int bid = blockIdx.x;
#if XCD_REMAP
    if (nblk % 8 == 0) bid = (bid % 8) * (nblk / 8) + bid / 8;
#endif
    const int kz = bid / (TILES_M * TILES_N);
    const int r = bid % (TILES_M * TILES_N);
    const int grp = r / (GROUP_M * TILES_N);
    const int first_m = grp * GROUP_M;
    const int gsz = (TILES_M - first_m) < GROUP_M ? (TILES_M - first_m) : GROUP_M;
    const int rr = r % (GROUP_M * TILES_N);
    const int tile_m = first_m + rr % gsz;
    const int tile_n = rr / gsz;
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;
    const int kbase = kz * KSPLIT_LEN;

    /* ---- per-thread load coordinates ----------------------------------- */
    int a_row[EA], a_col[EA];
#pragma unroll
    for (int e = 0; e < EA; ++e) {
        const int q = tid + e * NT;
        a_row[e] = q / A_CHUNKS_ROW;
        a_col[e] = (q % A_CHUNKS_ROW) * AV;
    }
    int b_row[EB], b_col[EB];
#pragma unroll
    for (int e = 0; e < EB; ++e) {
        const int q = tid + e * NT;
        b_row[e] = q / B_CHUNKS_ROW;
        b_col[e] = (q % B_CHUNKS_ROW) * BV;
    }
#if MODE == 1
    /* pixel decomposition of each column this thread gathers */
    int px_off[EB], px_h[EB], px_w[EB];
    bool px_ok[EB];
#pragma unroll
    for (int e = 0; e < EB; ++e) {
        const int n = n0 + b_col[e];
        px_ok[e] = (n < N) && (tid + e * NT < B_CHUNKS);
        const int nn = px_ok[e] ? n : 0;
        const int b = nn / OHW;
        const int p = nn % OHW;
        px_h[e] = (p / CQ) * CSTR - CPAD;
        px_w[e] = (p % CQ) * CSTR - CPAD;
        px_off[e] = b * (CC * CH * CW);
    }
#endif

    avec_t areg[EA];
    bvec_t breg[EB];

    auto load_global = [&](int kt) {
        const int k0 = kbase + kt * BK;
#pragma unroll
        for (int e = 0; e < EA; ++e) {
            const int m = m0 + a_row[e];
            const int k = k0 + a_col[e];
            bool ok = (A_CHUNKS % NT == 0) || (tid + e * NT < A_CHUNKS);
            if (M % BM != 0) ok = ok && (m < M);
            if (KP != K) ok = ok && (k < K);
            if (ok) areg[e] = *reinterpret_cast<const avec_t*>(A + (size_t)m * K + k);
            else areg[e] = (avec_t)(0.0f);
        }
#pragma unroll
        for (int e = 0; e < EB; ++e) {
#if MODE == 2
            const int n = n0 + b_row[e];
            const int k = k0 + b_col[e];
            bool ok = (B_CHUNKS % NT == 0) || (tid + e * NT < B_CHUNKS);
            if (N % BN != 0) ok = ok && (n < N);
            if (KP != K) ok = ok && (k < K);
            if (ok) breg[e] = *reinterpret_cast<const bvec_t*>(B + (size_t)n * K + k);
            else breg[e] = (bvec_t)(0.0f);
#elif MODE == 0
            const int k = k0 + b_row[e];
            const int n = n0 + b_col[e];
            bool ok = (B_CHUNKS % NT == 0) || (tid + e * NT < B_CHUNKS);
            if (N % BN != 0) ok = ok && (n < N);
            if (KP != K) ok = ok && (k < K);
            if (ok) breg[e] = *reinterpret_cast<const bvec_t*>(B + (size_t)k * N + n);
            else breg[e] = (bvec_t)(0.0f);
#else
            const int k = k0 + b_row[e];
            const int c = k / (CR * CS);
            const int rs = k % (CR * CS);
            const int ih = px_h[e] + (rs / CS) * CDIL;
            const int iw = px_w[e] + (rs % CS) * CDIL;
            bool ok = px_ok[e] && (unsigned)ih < (unsigned)CH && (unsigned)iw < (unsigned)CW;
            if (KP != K) ok = ok && (k < K);
            breg[e] = ok ? B[px_off[e] + c * (CH * CW) + ih * CW + iw] : 0.0f;
#endif
        }
    };

    auto store_lds = [&](int buf) {
#pragma unroll
        for (int e = 0; e < EA; ++e) {
            if ((A_CHUNKS % NT == 0) || (tid + e * NT < A_CHUNKS))
                *reinterpret_cast<avec_t*>(&As[buf][a_row[e] * SA + a_col[e]]) = areg[e];
        }
#pragma unroll
        for (int e = 0; e < EB; ++e) {
            if ((B_CHUNKS % NT == 0) || (tid + e * NT < B_CHUNKS))
                *reinterpret_cast<bvec_t*>(&Bs[buf][b_row[e] * SB + b_col[e]]) = breg[e];
        }
    };

    acc_t acc[REP_M][REP_N];
#pragma unroll
    for (int i = 0; i < REP_M; ++i)
#pragma unroll
        for (int j = 0; j < REP_N; ++j)
            acc[i][j] = (acc_t)(0.0f);

    auto compute = [&](int buf) {
        const float* as = &As[buf][(wm * REP_M * MFMA + li) * SA + 4 * lg];
#if MODE == 2
        const float* bs = &Bs[buf][(wn * REP_N * MFMA + li) * SB + 4 * lg];
#else
        const float* bs = &Bs[buf][(4 * lg) * SB + wn * REP_N * MFMA + li];
#endif
#pragma unroll
        for (int kb = 0; kb < BK; kb += KBLK) {
            f32x4 a[REP_M];
#pragma unroll
            for (int i = 0; i < REP_M; ++i)
                a[i] = *reinterpret_cast<const f32x4*>(as + i * MFMA * SA + kb);
#if MODE == 2
            f32x4 b4[REP_N];
#pragma unroll
            for (int j = 0; j < REP_N; ++j)
                b4[j] = *reinterpret_cast<const f32x4*>(bs + j * MFMA * SB + kb);
#endif
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                float b[REP_N];
#pragma unroll
                for (int j = 0; j < REP_N; ++j)
#if MODE == 2
                    b[j] = b4[j][s];
#else
                    b[j] = bs[(kb + s) * SB + j * MFMA];
#endif
#pragma unroll
                for (int i = 0; i < REP_M; ++i)
#pragma unroll
                    for (int j = 0; j < REP_N; ++j)
                        acc[i][j] = MFMA_OP(a[i][s], b[j], acc[i][j]);
            }
        }
    };

    /* ---- main loop ------------------------------------------------------ */
    load_global(0);
    store_lds(0);
    __syncthreads();
#if STAGES == 2
    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) load_global(kt + 1);
        compute(cur);
        if (kt + 1 < KT) store_lds(cur ^ 1);
        __syncthreads();
    }
#else
    for (int kt = 0; kt < KT; ++kt) {
        if (kt + 1 < KT) load_global(kt + 1);
        compute(0);
        __syncthreads();
        if (kt + 1 < KT) {
            store_lds(0);
            __syncthreads();
        }
    }
#endif

    /* ---- epilogue: accumulators -> C ----------------------------------- */
#pragma unroll
    for (int i = 0; i < REP_M; ++i) {
#pragma unroll
        for (int j = 0; j < REP_N; ++j) {
            const int n = n0 + (wn * REP_N + j) * MFMA + li;
#if MODE == 1
            const int b = n / OHW;
            const int p = n % OHW;
            const size_t cbase = (size_t)b * M * OHW + p;
#endif
#pragma unroll
            for (int v = 0; v < NACC; ++v) {
#if MFMA == 32
                const int row = 8 * (v / 4) + 4 * lg + (v % 4);
#else
                const int row = 4 * lg + v;
#endif
                const int m = m0 + (wm * REP_M + i) * MFMA + row;
                bool ok = true;
                if (M % BM != 0) ok = ok && (m < M);
                if (N % BN != 0) ok = ok && (n < N);
                if (ok) {
#if MODE == 1
                    float* dst = C + cbase + (size_t)m * OHW;
#else
                    float* dst = C + (size_t)m * N + n;
#endif
#if SPLITK > 1
                    unsafeAtomicAdd(dst, acc[i][j][v]);
#else
                    *dst = acc[i][j][v];
#endif
                }
            }
        }
    }
}
