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
//   STAGES          1 or 2 LDS buffers (2 = the LDS stores of tile t+1 need no
//                   extra barrier against the reads of tile t)
//   PD              prefetch distance: global loads of tile t+PD are in
//                   flight (in PD register sets) while tile t is multiplied
//   SPLITK          grid-level split of K; partial sums meet with float
//                   atomics in C, which the caller zero-fills first
//   GROUP_M         tile-traversal group height (L2 locality)
//   XCD_REMAP       1: consecutive logical tiles stay on one XCD
//   APAD / BPAD     LDS row padding in floats; APAD = -1 selects an unpadded
//                   A tile whose 16-byte chunks are XOR-swizzled by row
//
// LDS layout: As[BM][BK+APAD] (k contiguous, read as one 128-bit load per
// lane per 4 k-steps), Bs[BK][BN+BPAD] (n contiguous, read as 32-bit loads).
// With the swizzle, chunk c of row r lives at chunk c ^ swz(r): 16 lanes that
// read (or write) the same logical chunk of 16 consecutive rows touch 16
// different groups of four banks.
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
#define PD FT_PD
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
#if APAD < 0
#define ASWZ 1
#define SA (BK)
#else
#define ASWZ 0
#define SA (BK + APAD)
#endif
/* chunk swizzle of a k-contiguous tile: CRW 16-byte chunks per row */
#define CRW (BK / 4)
#if ASWZ
#if CRW >= 16
#define SWZ(row) ((row) & 15)
#else
#define SWZ(row) (((row) / (16 / CRW)) & (CRW - 1))
#endif
#else
#define SWZ(row) 0
#endif
/* element column c of `row` -> physical column */
#define ACOL(row, c) (((((c) >> 2) ^ SWZ(row)) << 2) | ((c) & 3))
#if MODE == 2
#define SB (SA)                   /* Bs[BN][SB], k contiguous like As */
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

    avec_t areg[PD][EA];
    bvec_t breg[PD][EB];

    auto load_global = [&](int kt, int set) {
        const int k0 = kbase + kt * BK;
#pragma unroll
        for (int e = 0; e < EA; ++e) {
            const int m = m0 + a_row[e];
            const int k = k0 + a_col[e];
            bool ok = (A_CHUNKS % NT == 0) || (tid + e * NT < A_CHUNKS);
            if (M % BM != 0) ok = ok && (m < M);
            if (KP != K) ok = ok && (k < K);
            if (ok) areg[set][e] = *reinterpret_cast<const avec_t*>(A + (size_t)m * K + k);
            else areg[set][e] = (avec_t)(0.0f);
        }
#pragma unroll
        for (int e = 0; e < EB; ++e) {
#if MODE == 2
            const int n = n0 + b_row[e];
            const int k = k0 + b_col[e];
            bool ok = (B_CHUNKS % NT == 0) || (tid + e * NT < B_CHUNKS);
            if (N % BN != 0) ok = ok && (n < N);
            if (KP != K) ok = ok && (k < K);
            if (ok) breg[set][e] = *reinterpret_cast<const bvec_t*>(B + (size_t)n * K + k);
            else breg[set][e] = (bvec_t)(0.0f);
#elif MODE == 0
            const int k = k0 + b_row[e];
            const int n = n0 + b_col[e];
            bool ok = (B_CHUNKS % NT == 0) || (tid + e * NT < B_CHUNKS);
            if (N % BN != 0) ok = ok && (n < N);
            if (KP != K) ok = ok && (k < K);
            if (ok) breg[set][e] = *reinterpret_cast<const bvec_t*>(B + (size_t)k * N + n);
            else breg[set][e] = (bvec_t)(0.0f);
#else
            const int k = k0 + b_row[e];
            const int c = k / (CR * CS);
            const int rs = k % (CR * CS);
            const int ih = px_h[e] + (rs / CS) * CDIL;
            const int iw = px_w[e] + (rs % CS) * CDIL;
            bool ok = px_ok[e] && (unsigned)ih < (unsigned)CH && (unsigned)iw < (unsigned)CW;
            if (KP != K) ok = ok && (k < K);
            breg[set][e] = ok ? B[px_off[e] + c * (CH * CW) + ih * CW + iw] : 0.0f;
#endif
        }
    };

    auto store_lds = [&](int buf, int set) {
#pragma unroll
        for (int e = 0; e < EA; ++e) {
            if ((A_CHUNKS % NT == 0) || (tid + e * NT < A_CHUNKS))
                *reinterpret_cast<avec_t*>(&As[buf][a_row[e] * SA + ACOL(a_row[e], a_col[e])]) = areg[set][e];
        }
#pragma unroll
        for (int e = 0; e < EB; ++e) {
            if ((B_CHUNKS % NT == 0) || (tid + e * NT < B_CHUNKS))
#if MODE == 2
                *reinterpret_cast<bvec_t*>(&Bs[buf][b_row[e] * SB + ACOL(b_row[e], b_col[e])]) = breg[set][e];
#else
                *reinterpret_cast<bvec_t*>(&Bs[buf][b_row[e] * SB + b_col[e]]) = breg[set][e];
#endif
        }
    };

    acc_t acc[REP_M][REP_N];
#pragma unroll
    for (int i = 0; i < REP_M; ++i)
#pragma unroll
        for (int j = 0; j < REP_N; ++j)
            acc[i][j] = (acc_t)(0.0f);

    auto compute = [&](int buf) {
        const int arow = wm * REP_M * MFMA + li;   /* + i*MFMA: SWZ is the same when MFMA % 16 == 0 */
        const float* as = &As[buf][arow * SA];
#if MODE == 2
        const int brow = wn * REP_N * MFMA + li;
        const float* bs = &Bs[buf][brow * SB];
#else
        const float* bs = &Bs[buf][(4 * lg) * SB + wn * REP_N * MFMA + li];
#endif
#pragma unroll
        for (int kb = 0; kb < BK; kb += KBLK) {
            f32x4 a[REP_M];
#pragma unroll
            for (int i = 0; i < REP_M; ++i)
                a[i] = *reinterpret_cast<const f32x4*>(as + i * MFMA * SA + ACOL(arow + i * MFMA, kb + 4 * lg));
#if MODE == 2
            f32x4 b4[REP_N];
#pragma unroll
            for (int j = 0; j < REP_N; ++j)
                b4[j] = *reinterpret_cast<const f32x4*>(bs + j * MFMA * SB + ACOL(brow + j * MFMA, kb + 4 * lg));
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
    /* Tile t travels global -> register set t % PD -> LDS buffer -> MFMA.
     * While tile kt is multiplied, tiles kt+1 .. kt+PD are in registers or in
     * flight; tile kt+1 is written to LDS right after the MFMAs of tile kt. */
#pragma unroll
    for (int p = 0; p < PD; ++p)
        if (p < KT) load_global(p, p);
    store_lds(0, 0);
    __syncthreads();
    for (int kt0 = 0; kt0 < KT; kt0 += PD) {
#pragma unroll
        for (int u = 0; u < PD; ++u) {
            const int kt = kt0 + u;
            if (kt < KT) {
                const int cur = (STAGES == 2) ? (kt & 1) : 0;
                if (kt + PD < KT) load_global(kt + PD, u);
                compute(cur);
                if (STAGES == 1) __syncthreads();
                if (kt + 1 < KT) store_lds((STAGES == 2) ? (cur ^ 1) : 0, (u + 1) % PD);
                __syncthreads();
            }
        }
    }

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
