// fp32 implicit-GEMM kernel template for gfx950 (CDNA4), compiled with hiprtc.
//
//   C[M][N] (+)= A[M][K] * B[K][N]        fp32 in, fp32 MFMA accumulate
//
// One source serves two operators; every shape and knob is a -D constant:
//   MODE 0  dense GEMM        A row-major [M][K], B row-major [K][N]
//                             (flextensor/nn/ops.py:1105-1108)
//   MODE 2  dense GEMM, B^T   A row-major [M][K], B stored [N][K]
//                             (the transposeB branch, ops.py:1101-1104)
//           MODE 0 and 2 also run a batch of CG such GEMMs (ops.py:1111-1158)
//           TA 1 (MODE 0 and 2): A is stored [K][M] (the transposeA branches,
//           ops.py:1093-1100). On the register-staged pipelines its tile is
//           fetched in vectors along M and transposed on the way into LDS,
//           where it has the usual [BM][BK] layout; with DTL it lands as it
//           lies in memory, [BK][BM], and the fragments are read as scalars.
//   MODE 1  conv2d NCHW       A = weight [Kout][C*R*S], B = im2col gather of
//                             the input with zero padding folded into the
//                             load predicate, N = batch*OH*OW
//                             (flextensor/nn/ops.py:83-117, 419-479).
//                             Grouped convolution (CG groups) runs one GEMM
//                             per group: M = Kout/CG, K = (C/CG)*R*S, and the
//                             group index is one more grid factor.
//                             COLOUT 1 stores C as [CG][M][N], the layout of the
//                             GEMM stage of a convolution written as im2col,
//                             GEMM, col2img (ops.py:982-1044), instead of NCHW.
//
// Knobs (set by the scheduler from a Config):
//   MFMA            32 -> v_mfma_f32_32x32x2_f32, 16 -> v_mfma_f32_16x16x4_f32
//   WAVES_M/N       wavefronts per workgroup along M / N
//   REP_M/N         MFMA tiles per wavefront along M / N
//   BK              K extent of one LDS tile
//   STAGES          1 or 2 LDS buffers, 3 or 4 with DTL (2 = the LDS stores of tile t+1 need no
//                   extra barrier against the reads of tile t)
//   PD              prefetch distance: global loads of tile t+PD are in
//                   flight (in PD register sets) while tile t is multiplied
//   SPLITK          grid-level split of K; partial sums meet with float
//                   atomics in C, which the caller zero-fills first
//   WAVES_K         split of K inside the workgroup: WAVES_K groups of
//                   WAVES_M*WAVES_N wavefronts each multiply their own K slice
//                   through their own LDS tiles; the partial tiles are summed
//                   through LDS at the end (no atomics, no zero fill)
//   HAS_BIAS        1: C[m][n] = sum + bias[m] (the per-output-channel bias of a
//                   convolution, flextensor/nn/ops.py:474-478), added exactly
//                   once whichever way K is divided
//   DTL             1: tiles travel global -> LDS directly (buffer loads with
//                   the lds modifier): no staging registers and no LDS store
//                   instructions. A (and B^T) in 16-byte chunks, 64 per
//                   wavefront landing contiguously, so rows are unpadded and
//                   the swizzle is applied on the global side; B one float
//                   per lane: 64 consecutive columns of one k row per
//                   instruction (BN % 64 == 0, rows may be padded) or whole
//                   unpadded rows (BN < 64)
//   FPF             with DTL and two buffers: the MFMA operands are read from LDS one k
//                   block ahead of their use, and the first block of the next tile right
//                   behind the barrier, which stands before the last k block's MFMAs
//   LSPREAD         with FPF: the loads of the next tile are issued in LSPREAD parts in
//                   front of the first LSPREAD k blocks (1: all before the first)
//   SK_PER          > 0: balanced K streaming. The work is cut into units of
//                   one LDS tile step (output tile, k-tile); every workgroup
//                   takes SK_PER consecutive units, so a workgroup may
//                   finish one output tile, run whole tiles and begin a
//                   third. A partly covered tile is written to a workspace
//                   slot; the workgroup that arrives last at the tile's
//                   counter sums the slots in a fixed order and stores the
//                   tile (no waiting, no zero fill, deterministic)
//   GROUP_M         tile-traversal group height (L2 locality)
//   XCD_REMAP       1: consecutive logical tiles stay on one XCD
//   APAD / BPAD     LDS row padding in floats; APAD = -1 selects an unpadded
//                   A tile whose 16-byte chunks are XOR-swizzled by row
//
// LDS layout: As[BM][BK+APAD] (k contiguous, read as one 128-bit load per
// lane per 4 k-steps), Bs[BK][BN+BPAD] (n contiguous, read as 32-bit loads).
// With the swizzle, chunk c of row r lives at chunk c ^ swz(r): 16 lanes that
// read (or write) the same logical chunk of 16 consecutive rows touch 16
// different groups of four banks (the rows may hold any even number of chunks).
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
#define WAVES_K FT_WAVES_K
#define GROUP_M FT_GROUP_M
#define XCD_REMAP FT_XCD_REMAP
#define APAD FT_APAD
#define BPAD FT_BPAD
#define AV FT_AV
#define BV FT_BV
#ifdef FT_HAS_BIAS
#define HAS_BIAS FT_HAS_BIAS
#else
#define HAS_BIAS 0
#endif
#ifdef FT_DTL
#define DTL FT_DTL
#else
#define DTL 0
#endif
#ifdef FT_FPF
#define FPF FT_FPF          /* 1: first operands of the next tile read ahead of the last MFMAs of this one */
#else
#define FPF 0
#endif
#ifdef FT_LSPREAD
#define LSPREAD FT_LSPREAD  /* with FPF: k blocks over which the loads of the next tile are spread */
#else
#define LSPREAD 1
#endif
#ifdef FT_COLOUT
#define COLOUT FT_COLOUT
#else
#define COLOUT 0
#endif
#ifdef FT_TA
#define TA FT_TA
#else
#define TA 0
#endif
#ifdef FT_SK_PER
#define SK_PER FT_SK_PER
#else
#define SK_PER 0
#endif
/* SK_FENCED 1 makes the arrival count and the look at the counter a
 * device-scope release / acquire pair in the language's sense as well; see the
 * hand-off comment in the kernel for why the default does without. */
#ifdef FT_SK_FENCED
#define SK_FENCED FT_SK_FENCED
#else
#define SK_FENCED 0
#endif
#if SK_FENCED
#define SK_ARRIVE_ORDER __ATOMIC_ACQ_REL
#define SK_LOOK_ORDER __ATOMIC_ACQUIRE
#else
#define SK_ARRIVE_ORDER __ATOMIC_RELAXED
#define SK_LOOK_ORDER __ATOMIC_RELAXED
#endif

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
#define NT (WAVES_M * WAVES_N * 64)   /* threads of one k-group */
#define NTW (NT * WAVES_K)             /* threads of the workgroup */
#if APAD < 0
#define ASWZ 1
#define SA (BK)
#else
#define ASWZ 0
#define SA (BK + APAD)
#endif
/* chunk swizzle of a k-contiguous, unpadded tile: CRW 16-byte chunks per row.
 * A 128-bit LDS read is served 16 lanes at a time over 16 groups of four banks,
 * and the 16 lanes of a pass are not consecutive: lanes 0-3, 12-15, 20-23 and
 * 24-27 go together, then lanes 4-11, 16-19 and 28-31, then the same in the
 * upper half of the wavefront (SQ_LDS_BANK_CONFLICT reads zero exactly for the
 * patterns this predicts to be free, and the predicted count for the others).
 * Rows start SWZ_S = CRW mod 16 groups apart, so rows 16 / SWZ_G apart,
 * SWZ_G = gcd(SWZ_S, 16), would meet in one group; the chunk index of row r is
 * XOR-ed with (r / (16 / SWZ_G)) mod SWZ_G, which sends them to the SWZ_G groups
 * between. SWZ_G is a power of two that divides CRW, so the XOR stays inside the
 * row whatever its length (a power of two or not), and rows 16 apart get the
 * same XOR. One case needs another XOR: 16x16x4 fragments (a pass mixes rows
 * 0-3 and 12-15 of one k-group with rows 4-11 of the next) over rows of
 * 4 mod 8 chunks, where bit 1 of the chunk index is flipped by bit 2 of the row. */
#define CRW (BK / 4)
#if ASWZ
#define SWZ_S (CRW % 16)
#define SWZ_G (SWZ_S == 0 ? 16 : (SWZ_S % 2 ? 1 : (SWZ_S % 4 ? 2 : (SWZ_S % 8 ? 4 : 8))))
#if MFMA == 16 && CRW % 8 == 4
#define SWZ(row) ((((row) >> 2) & 1) << 1)
#define SWZ_X 4                   /* the XOR stays below this power of two */
#else
#define SWZ(row) (((row) / (16 / SWZ_G)) & (SWZ_G - 1))
#define SWZ_X SWZ_G
#endif
#else
#define SWZ(row) 0
#define SWZ_X KL
#endif
/* A fragment read takes chunk (kb/4 + lg) ^ SWZ(row). kb/4 is a multiple of KL,
 * lg < KL <= SWZ_X, so with kb/4 = hi + lo, lo = kb/4 mod SWZ_X, the chunk is
 * hi + ((lo + lg) ^ SWZ(row)): a compile-time part and one of SWZ_X / KL
 * lane-dependent values, which are computed once so that every read is a base
 * register plus an immediate offset. */
#define SWZ_CLASSES (SWZ_X / KL)
#define SWZ_HI(kb) ((((kb) >> 2) & ~(SWZ_X - 1)) << 2)       /* in floats */
#define SWZ_CLS(kb) ((((kb) >> 2) & (SWZ_X - 1)) / KL)
/* element column c of `row` -> physical column (the XOR is its own inverse) */
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
/* KP = K, or K rounded up to a multiple of 16 when K % 8 != 0; the host checks KP % (SPLITK*BK) == 0.
 * When KP != K the tail is zero-filled by the load predicates. */
#define KSPLIT_LEN (KP / SPLITK)
#define KGROUP_LEN (KSPLIT_LEN / WAVES_K)
#define KT (KGROUP_LEN / BK)

#if BK % KBLK != 0
#error "BK must be a multiple of 4*(64/MFMA)"
#endif

/* ---- A tile: BM x BK, vectors of AV floats along K (along M when A is stored [K][M]) */
#if TA
#if MODE == 1
#error "a transposed A operand: dense GEMM modes only"
#endif
#define A_CHUNKS_ROW (BM / AV)
#define A_CHUNKS (BK * A_CHUNKS_ROW)
#else
#define A_CHUNKS_ROW (BK / AV)
#define A_CHUNKS (BM * A_CHUNKS_ROW)
#endif
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
#if DTL
#if STAGES < 2 || STAGES > 4 || PD != 1 || AV != 4 || APAD > 0 || A_CHUNKS % 64 != 0 || B_CHUNKS % 64 != 0
#error "direct-to-LDS tiles: two to four buffers, 16-byte A chunks, unpadded A rows, whole wavefronts of chunks"
#endif
#if STAGES > 2 && (A_CHUNKS % NT != 0 || B_CHUNKS % NT != 0 || (STAGES - 2) * (EA + EB) > 63)
#error "more than two direct-to-LDS buffers: every wavefront must issue the same number of loads per tile"
#endif
/* loads one wavefront issues per tile, and a wait that lets the newest n loads stay in flight */
#define DMA_PER_TILE (EA + EB)
#define VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))
#if MODE == 2
#if BV != 4
#error "direct-to-LDS tiles: B^T needs 16-byte chunks"
#endif
#else
#if MODE == 0 && BV == 4
/* B in 16-byte chunks as well: rows land unpadded, so the four k rows that the
 * lane groups of an MFMA read together would hit the same banks; instead the
 * chunks of row k are XOR-ed (on the global side) by a function of k that moves
 * each lane group to its own banks. */
#if BPAD != 0 || BN % 64 != 0
#error "direct-to-LDS B in 16-byte chunks needs unpadded rows of a multiple of 64 floats"
#endif
#define BSWZ 1
#if MFMA == 16
#define BSWK(k) ((((k) >> 2) & 3) << 2)     /* chunk XOR of row k: 16 floats per lane group */
#else
#define BSWK(k) ((((k) >> 2) & 1) << 3)     /* 32 floats per lane group */
#endif
#elif BV != 1 || !(BN % 64 == 0 || BPAD == 0)
#error "direct-to-LDS tiles: B goes one float per lane; a wavefront covers part of one padded row, or 64 floats of the unpadded tile"
#endif
#if BV == 1 && BPAD == 0 && (BN % 64 == 0 || BN == 32 || BN == 16)
/* B one float per lane into unpadded rows: the four (two) k rows that the lane
 * groups of an MFMA read together would sit in the same banks. Every lane
 * computes its own global address, so any permutation of the tile is free on
 * the global side: the element of logical (k, n), k-group g = (k >> 2) & (KG-1),
 * lives at row (k & ~3) | ((k & 3) ^ BSW_R(g)), column n ^ BSW_C(g). Both only
 * move an element inside the 64 floats one wavefront writes, and they send the
 * lane groups of one MFMA operand read to disjoint banks:
 *   rows of 64 floats or more  columns XOR-ed by g * MFMA
 *   rows of 32 floats          16x16x4: column bit 4 by g's low bit, row parity
 *                              by g's high bit; 32x32x2: row parity by g
 *   rows of 16 floats          the row's low two bits by g */
#define BSWZ1 1
#define KG (64 / MFMA)
#if BN % 64 == 0
#define BSW_R(g) 0
#define BSW_C(g) ((g) * MFMA)
#elif BN == 32 && MFMA == 16
#define BSW_R(g) ((g) >> 1)
#define BSW_C(g) (((g) & 1) << 4)
#else
#define BSW_R(g) (g)
#define BSW_C(g) 0
#endif
#endif
#endif
#if TA
/* A stored [K][M]: its tile travels like the plain GEMM's B, in 16-byte chunks along M into
 * unpadded rows [BK][BM], the chunks of row k XOR-ed on the global side so that the lane groups
 * of an MFMA operand read (rows 4g + s) use different banks; the fragments are read as scalars. */
#if BM % 64 != 0
#error "direct-to-LDS tiles of a transposed A need rows of a multiple of 64 floats"
#endif
#if MFMA == 16
#define TSWK(k) ((((k) >> 2) & 3) << 2)
#else
#define TSWK(k) ((((k) >> 2) & 1) << 3)
#endif
#endif
typedef __attribute__((address_space(3))) void lds_void;
typedef int i32x4 __attribute__((ext_vector_type(4)));
#endif

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

/* byte sizes of the operands (the host checks that each is below 2 GiB) */
#define OOB 0x80000000u
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
static __device__ __forceinline__ float ld_f32(__amdgpu_buffer_rsrc_t r, unsigned vo, int so) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)vo, so, 0));
}
static __device__ __forceinline__ f32x4 ld_f32x4(__amdgpu_buffer_rsrc_t r, unsigned vo, int so) {
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)vo, so, 0));
}
#if AV == 4
#define LOAD_A ld_f32x4
#else
#define LOAD_A ld_f32
#endif
#if BV == 4
#define LOAD_B ld_f32x4
#else
#define LOAD_B ld_f32
#endif

#if MODE == 1
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
/* conv geometry, all compile-time: input [CB][CC][CH][CW], kernel CR x CS,
 * stride CSTRH x CSTRW, padding CPADH x CPADW, dilation CDILH x CDILW (rows x
 * columns, flextensor/nn/ops.py:448-459 takes pairs), output CP x CQ. */
#define OHW (CP * CQ)
#define A_BYTES (CG * M * K * 4)
#define B_BYTES (CB * CC * CH * CW * 4)
/* When an LDS tile spans whole kernel windows (BK % (CR*CS) == 0) every
 * gathered element keeps its tap (r, s) and its channel offset inside the
 * tile for the whole K loop: the index arithmetic and the padding predicate
 * are computed once and the loop only advances by a constant stride. */
#if BK % (CR * CS) == 0
#define KHOIST 1
#else
#define KHOIST 0
#endif
#if BV != 1
#error "conv mode gathers scalars: BV must be 1"
#endif
/* Element e of a thread is chunk tid + e * NT of the B tile. When NT is a whole number of
 * tile rows and that number is a multiple of the k block (the unit inside which the LDS
 * permutation moves rows), e only moves the element down by BROW_STEP rows: same pixel. */
#if (NT % BN == 0) && ((NT / BN) % KBLK == 0)
#define BROW_LINEAR 1
#define BROW_STEP (NT / BN)
#else
#define BROW_LINEAR 0
#endif
#else
/* a batch of independent GEMMs (flextensor/nn/ops.py:1111-1158) reuses the
 * group index: operand b of every matrix starts b*M*K, b*K*N, b*M*N floats in */
#ifdef FT_CG
#define CG FT_CG
#else
#define CG 1
#endif
#define A_BYTES (CG * M * K * 4)
#define B_BYTES (CG * K * N * 4)
#endif

#define A_FLOATS (BM * SA)
#define TILE_FLOATS (WAVES_K * STAGES * (A_FLOATS + BS_FLOATS))
#define RED_FLOATS ((WAVES_K - 1) * NT * REP_M * REP_N * NACC)
#define SMEM_FLOATS (TILE_FLOATS > RED_FLOATS ? TILE_FLOATS : RED_FLOATS)

/* FT_CLKPROBE: an instrumented build that measures the shader clock the kernel runs at. Every
 * workgroup writes, through one more argument, how many shader clocks (s_memtime) and how many ticks
 * of the constant 100 MHz counter (s_memrealtime) passed between its first instruction and the
 * completion of its first wavefront's last store. */
#ifdef FT_CLKPROBE
#define CLK_PARAM , unsigned long long* __restrict__ ft_clk
#if FT_CLKPROBE == 2
/* the two stamps of the 100 MHz counter themselves (it is common to the device): when the workgroup began and
 * when its first wavefront's stores had completed, to lay the workgroups of consecutive launches on one time axis */
#define CLK_BEGIN const unsigned long long ft_r0 = wall_clock64();
#define CLK_END do { __builtin_amdgcn_s_waitcnt(0x0F70); \
        if (threadIdx.x == 0) { ft_clk[2 * blockIdx.x] = ft_r0; ft_clk[2 * blockIdx.x + 1] = wall_clock64(); } } while (0)
#else
#define CLK_BEGIN const unsigned long long ft_t0 = __builtin_readcyclecounter(), ft_r0 = wall_clock64();
#define CLK_END do { __builtin_amdgcn_s_waitcnt(0x0F70); \
        if (threadIdx.x == 0) { ft_clk[2 * blockIdx.x] = __builtin_readcyclecounter() - ft_t0; \
                                ft_clk[2 * blockIdx.x + 1] = wall_clock64() - ft_r0; } } while (0)
#endif
#else
#define CLK_PARAM
#define CLK_BEGIN
#define CLK_END do { } while (0)
#endif

extern "C" __global__ __launch_bounds__(NTW)
void igemm_f32(const float* __restrict__ A, const float* __restrict__ B,
               float* __restrict__ C
#if SK_PER > 0
               , float* sk_part, unsigned* sk_cnt
#endif
#if HAS_BIAS
               , const float* __restrict__ bias
#endif
               CLK_PARAM)
{
    CLK_BEGIN
    __shared__ __attribute__((aligned(16))) float smem[SMEM_FLOATS];
    /* k-group of this wavefront (NT is a multiple of 64, so it is uniform
     * over a wavefront; readfirstlane tells the compiler so) */
#if WAVES_K > 1
    const int kg = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / NT));
    const int tid = threadIdx.x - kg * NT;      /* thread index inside the k-group */
#else
    const int kg = 0;
    const int tid = threadIdx.x;
#endif
    float (*As)[A_FLOATS] = reinterpret_cast<float (*)[A_FLOATS]>(smem + kg * STAGES * A_FLOATS);
    float (*Bs)[BS_FLOATS] = reinterpret_cast<float (*)[BS_FLOATS]>(
        smem + WAVES_K * STAGES * A_FLOATS + kg * STAGES * BS_FLOATS);

    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N;
    const int wn = wave % WAVES_N;
    const int li = lane % MFMA;   /* row (A) / column (B, C) inside an MFMA tile */
    const int lg = lane / MFMA;   /* k group */

    /* ---- per-thread load coordinates ----------------------------------- */
    int a_row[EA], a_col[EA];
#pragma unroll
    for (int e = 0; e < EA; ++e) {
        const int q = tid + e * NT;
        a_row[e] = q / A_CHUNKS_ROW;
#if DTL && TA
        a_col[e] = ((q % A_CHUNKS_ROW) ^ TSWK(a_row[e])) * AV;      /* a_row is k, a_col the first of four rows m */
#elif DTL
        /* chunk q lands at float 4*q of the tile, i.e. at physical chunk
         * q % A_CHUNKS_ROW of its row: fetch the logical chunk that belongs there */
        a_col[e] = ACOL(a_row[e], (q % A_CHUNKS_ROW) * AV);
#else
        a_col[e] = (q % A_CHUNKS_ROW) * AV;
#endif
    }
    int b_row[EB], b_col[EB];
#pragma unroll
    for (int e = 0; e < EB; ++e) {
        const int q = tid + e * NT;
        b_row[e] = q / B_CHUNKS_ROW;
#if DTL && MODE == 2
        b_col[e] = ACOL(b_row[e], (q % B_CHUNKS_ROW) * BV);
#elif defined(BSWZ)
        b_col[e] = ((q % B_CHUNKS_ROW) ^ BSWK(b_row[e])) * BV;
#elif defined(BSWZ1)
        {   /* float q of the tile is physical (row, column): fetch the logical element that lives there */
            const int pr = q / BN, g = (pr >> 2) & (KG - 1);
            b_row[e] = (pr & ~3) | ((pr & 3) ^ BSW_R(g));
            b_col[e] = (q % BN) ^ BSW_C(g);
        }
#else
        b_col[e] = (q % B_CHUNKS_ROW) * BV;
#endif
    }
    /* ---- workgroup -> (group, split, tile_m, tile_n) and K range -------- */
    /* tile index inside one group -> first row / column of the tile */
    auto tile_origin = [&](int r, int& m0_, int& n0_) {
        const int grp = r / (GROUP_M * TILES_N);
        const int first_m = grp * GROUP_M;
        const int gsz = (TILES_M - first_m) < GROUP_M ? (TILES_M - first_m) : GROUP_M;
        const int rr = r % (GROUP_M * TILES_N);
        m0_ = (first_m + rr % gsz) * BM;
        n0_ = (rr / gsz) * BN;
    };
    acc_t acc[REP_M][REP_N];
    /* accumulators -> C for the tile at (m0_, n0_) of group gi_ */
    auto store_c = [&](int m0_, int n0_, int gi_, bool first_k_part) {
#pragma unroll
        for (int i = 0; i < REP_M; ++i) {
#pragma unroll
            for (int j = 0; j < REP_N; ++j) {
                const int n = n0_ + (wn * REP_N + j) * MFMA + li;
#if MODE == 1 && !COLOUT
                const int b = n / OHW;
                const int p = n % OHW;
                const size_t cbase = ((size_t)b * (CG * M) + (size_t)gi_ * M) * OHW + p;
#endif
#pragma unroll
                for (int v = 0; v < NACC; ++v) {
#if MFMA == 32
                    const int row = 8 * (v / 4) + 4 * lg + (v % 4);
#else
                    const int row = 4 * lg + v;
#endif
                    const int m = m0_ + (wm * REP_M + i) * MFMA + row;
                    bool ok = true;
                    if (M % BM != 0) ok = ok && (m < M);
                    if (N % BN != 0) ok = ok && (n < N);
                    if (ok) {
#if MODE == 1 && !COLOUT
                        float* dst = C + cbase + (size_t)m * OHW;
#else
                        float* dst = C + ((size_t)gi_ * M + m) * N + n;
#endif
                        float val = acc[i][j][v];
#if HAS_BIAS
                        if (first_k_part) val += bias[gi_ * M + m];
#endif
#if SPLITK > 1
                        unsafeAtomicAdd(dst, val);
#else
                        *dst = val;
#endif
                    }
                }
            }
        }
    };
#if SK_PER > 0
#if SPLITK != 1 || WAVES_K != 1
#error "balanced K streaming excludes the other K splits"
#endif
#define SK_UNITS (TILES_M * TILES_N * CG * KT)
/* the grid is rounded up to a multiple of 8 when workgroups are renumbered by
 * XCD; the extra workgroups find no units */
#if XCD_REMAP
#define SK_GRID ((((SK_UNITS + SK_PER - 1) / SK_PER) + 7) / 8 * 8)
#else
#define SK_GRID ((SK_UNITS + SK_PER - 1) / SK_PER)
#endif
#define SK_SLOT (NT * REP_M * REP_N * NACC)
    /* A tile that several workgroups cover is exchanged through workspace
     * slots. The sharers of a tile are consecutive workgroups; each owns two
     * slots: slot 0 for the tile its range begins in, slot 1 for the tile it
     * ends in after beginning in an earlier one. Slots are written and read
     * with device-scope atomic accesses: these are coherent across the
     * per-XCD L2 caches by themselves, so no cache write-back or invalidation
     * is needed, only ordering, and the instruction stream supplies it:
     * every wavefront waits for its own slot stores (s_waitcnt vmcnt(0): a
     * barrier or a workgroup-scope fence does not wait for vector stores),
     * the barrier collects the wavefronts, then thread 0 counts the arrival;
     * a reader has the counter's value (a wait on that load) before the
     * branch that leads to its slot loads. A device-scope release / acquire
     * on the counter (SK_FENCED) adds an L2 write-back before and an L2
     * invalidate after each count, which these write-through, cache-bypassing
     * accesses do not need and which evicts the operands the other
     * workgroups of the XCD are reading (+4.5 % on an 8x256x14x14 -> 512
     * 3x3 layer). Nobody waits for anybody: whoever finds all other sharers
     * arrived sums the slots, always in sharer order, so the result does not
     * depend on the timing. */
#define SK_DRAIN_STORES() __builtin_amdgcn_s_waitcnt(0x0F70)   /* vmcnt(0) only */
    __shared__ unsigned sk_arrived;
    auto sharers = [&](int tile_, int& first_, int& last_) {
        first_ = (tile_ * KT) / SK_PER;
        last_ = (tile_ * KT + KT - 1) / SK_PER;
    };
    auto slot_of = [&](int w, int tile_) -> float* {
        return sk_part + (size_t)(2 * w + ((w * SK_PER >= tile_ * KT) ? 0 : 1)) * SK_SLOT;
    };
    auto add_slots = [&](int tile_, int from, int to) {
        for (int w = from; w <= to; ++w) {
            float* part = slot_of(w, tile_);
#pragma unroll
            for (int i = 0; i < REP_M; ++i)
#pragma unroll
                for (int j = 0; j < REP_N; ++j)
#pragma unroll
                    for (int v = 0; v < NACC; ++v)
                        acc[i][j][v] += __hip_atomic_load(&part[((i * REP_N + j) * NACC + v) * NT + tid],
                                                          __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };
    auto clear_acc = [&]() {
#pragma unroll
        for (int i = 0; i < REP_M; ++i)
#pragma unroll
            for (int j = 0; j < REP_N; ++j)
                acc[i][j] = (acc_t)(0.0f);
    };
    int wg = blockIdx.x;
#if XCD_REMAP
    wg = (wg % 8) * (SK_GRID / 8) + wg / 8;
#endif
    int unit = wg * SK_PER;
    const int unit_end = (unit + SK_PER < SK_UNITS) ? unit + SK_PER : SK_UNITS;
    int arrive_tile = -1;        /* slot written, arrival still to be counted */
    int check_tile = -1;         /* arrival counted, result still to be looked at */
    unsigned check_before = 0;   /* thread 0: sharers that had arrived before */
    while (unit < unit_end) {
    const int tile = unit / KT;
    const int kt_lo = unit - tile * KT;
    const int nk = (KT - kt_lo < unit_end - unit) ? KT - kt_lo : unit_end - unit;
    unit += nk;
    const int gi = tile / (TILES_M * TILES_N);
    const int kz = 0;
    const int r = tile % (TILES_M * TILES_N);
#else
    {
    const int nblk = TILES_M * TILES_N * SPLITK * CG;
    int bid = blockIdx.x;
#if XCD_REMAP
    if (nblk % 8 == 0) bid = (bid % 8) * (nblk / 8) + bid / 8;
#endif
    const int gi = bid / (TILES_M * TILES_N * SPLITK);   /* convolution group */
    bid = bid % (TILES_M * TILES_N * SPLITK);
    const int kz = bid / (TILES_M * TILES_N);
    const int r = bid % (TILES_M * TILES_N);
    const int kt_lo = 0;
    const int nk = KT;
#endif
    int m0, n0;
    tile_origin(r, m0, n0);
    const int kbase = kz * KSPLIT_LEN + kg * KGROUP_LEN + kt_lo * BK;

#if MODE == 1
    int px_off[EB], px_h[EB], px_w[EB];      /* pixel decomposition of each column this thread gathers */
    bool px_ok[EB];
#endif

    /* ---- global loads: raw buffer loads with hardware bounds checking --- */
    /* Every element gets a byte offset computed once; an element that must
     * read as zero (tile edge, zero padding, idle lane) gets an offset beyond
     * the buffer, for which the load returns 0 without a branch. The part of
     * the address that advances with the K loop is wave-uniform and goes into
     * the scalar offset operand. */
    const __amdgpu_buffer_rsrc_t rsrc_a =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(A), 0, A_BYTES, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(B), 0, B_BYTES, 0x00020000);
    unsigned a_voff[EA], b_voff[EB];
#if DTL
    /* The loads are written as instructions, not through the builtin: the
     * compiler makes every later LDS read wait for a direct-to-LDS load it
     * knows of (it cannot tell the two buffers apart), which would undo the
     * overlap. Completion is tracked by hand: vmcnt(0) before the barrier
     * that ends an iteration. */
    const int wv = __builtin_amdgcn_readfirstlane(wave);
    auto descriptor = [](const float* base, unsigned bytes) {
        const unsigned long long p = (unsigned long long)base;
        i32x4 d;                             /* raw buffer: base, stride 0, bytes, untyped dwords */
        d[0] = __builtin_amdgcn_readfirstlane((int)(unsigned)p);
        d[1] = __builtin_amdgcn_readfirstlane((int)((unsigned)(p >> 32) & 0xffffu));
        d[2] = (int)bytes;
        d[3] = 0x00020000;
        return d;
    };
    const i32x4 desc_a = descriptor(A, (unsigned)A_BYTES);
    const i32x4 desc_b = descriptor(B, (unsigned)B_BYTES);
    /* The descriptor, the LDS address and the scalar offset are wave-uniform by construction.
     * With more than two buffers the buffer index is carried around the tile loop as a variable,
     * and in some shapes of that loop (inside the K-streaming segment loop with its lane-dependent
     * exits; in a workgroup of one wavefront) the compiler keeps it in a vector register and would
     * hand the instruction vector operands, so there it is told. With one or two buffers the index
     * is a constant or a bit of the tile counter, the compiler knows, and telling it anyway costs
     * instructions in the main loop. */
#if STAGES > 2
#define DMA_UNIFORM(x) __builtin_amdgcn_readfirstlane((int)(x))
    auto uniform4 = [](const i32x4& v) {
        i32x4 r;
        r[0] = __builtin_amdgcn_readfirstlane(v[0]); r[1] = __builtin_amdgcn_readfirstlane(v[1]);
        r[2] = __builtin_amdgcn_readfirstlane(v[2]); r[3] = __builtin_amdgcn_readfirstlane(v[3]);
        return r;
    };
#else
#define DMA_UNIFORM(x) (x)
    auto uniform4 = [](const i32x4& v) -> const i32x4& { return v; };
#endif
    auto dma16 = [&](const i32x4& rsrc, const float* dst, unsigned vo, int so) {
        const unsigned lds_addr = (unsigned)DMA_UNIFORM((unsigned)(__UINTPTR_TYPE__)(lds_void*)dst);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     :: "s"(lds_addr), "v"(vo), "s"(uniform4(rsrc)), "s"(DMA_UNIFORM(so)) : "memory", "m0");
    };
    auto dma4 = [&](const i32x4& rsrc, const float* dst, unsigned vo, int so) {
        const unsigned lds_addr = (unsigned)DMA_UNIFORM((unsigned)(__UINTPTR_TYPE__)(lds_void*)dst);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                     :: "s"(lds_addr), "v"(vo), "s"(uniform4(rsrc)), "s"(DMA_UNIFORM(so)) : "memory", "m0");
    };
    /* part p of np: the loads e of the tile with e mod np == p (A first, then B) */
    auto dma_tile_a = [&](int kt, int buf, int part = 0, int nparts = 1) {
        const int k0 = kbase + kt * BK;
#pragma unroll
        for (int e = 0; e < EA; ++e) {
            if (e % nparts != part) continue;
            unsigned vo = a_voff[e];
#if TA
            if (KP != K) vo = (k0 + a_row[e] < K) ? vo : OOB;
            if ((A_CHUNKS % NT == 0) || (e * NT + wv * 64 < A_CHUNKS))
                dma16(desc_a, &As[buf][(e * NT + wv * 64) * 4], vo, k0 * (M * 4));
#else
            if (KP != K) vo = (k0 + a_col[e] < K) ? vo : OOB;
            if ((A_CHUNKS % NT == 0) || (e * NT + wv * 64 < A_CHUNKS))     /* whole wavefronts only */
                dma16(desc_a, &As[buf][(e * NT + wv * 64) * 4], vo, k0 * 4);
#endif
        }
    };
    auto dma_b_one = [&](int kt, int buf, int e) {
        const int k0 = kbase + kt * BK;
        {
            if (!((B_CHUNKS % NT == 0) || (e * NT + wv * 64 < B_CHUNKS))) return;
#if MODE == 2
            unsigned vo = b_voff[e];
            if (KP != K) vo = (k0 + b_col[e] < K) ? vo : OOB;
            dma16(desc_b, &Bs[buf][(e * NT + wv * 64) * 4], vo, k0 * 4);
#else
            /* the wavefront's 64 lanes are 64 consecutive columns of one k row */
            const int q0 = e * NT + wv * 64;
            const float* dst = &Bs[buf][(q0 / BN) * SB + (q0 % BN)];
#if MODE == 0 && defined(BSWZ)
            unsigned vo = b_voff[e];
            if (KP != K) vo = (k0 + b_row[e] < K) ? vo : OOB;
            dma16(desc_b, &Bs[buf][(e * NT + wv * 64) * 4], vo, k0 * (N * 4));
#elif MODE == 0
            unsigned vo = b_voff[e];
            if (KP != K) vo = (k0 + b_row[e] < K) ? vo : OOB;
            dma4(desc_b, dst, vo, k0 * (N * 4));
#elif KHOIST
            unsigned vo = b_voff[e];
            if (KP != K) vo = (k0 + b_row[e] < K) ? vo : OOB;
            dma4(desc_b, dst, vo, (k0 / (CR * CS)) * (CH * CW * 4));
#else
            const int k = k0 + b_row[e];
            const int c = k / (CR * CS);
            const int rs = k % (CR * CS);
            const int ih = px_h[e] + (rs / CS) * CDILH;
            const int iw = px_w[e] + (rs % CS) * CDILW;
            bool ok = px_ok[e] & ((unsigned)ih < (unsigned)CH) & ((unsigned)iw < (unsigned)CW);
            if (KP != K) ok = ok & (k < K);
            const unsigned off = (unsigned)(px_off[e] + c * (CH * CW) + ih * CW + iw) * 4u;
            const unsigned vo = ok ? off : OOB;      /* a select of two values, no branch (see a_voff) */
            dma4(desc_b, dst, vo, 0);
#endif
#endif
        }
    };
    auto dma_tile_b = [&](int kt, int buf, int part = 0, int nparts = 1) {
#pragma unroll
        for (int e = 0; e < EB; ++e)
            if ((EA + e) % nparts == part) dma_b_one(kt, buf, e);
    };
    auto dma_tile = [&](int kt, int buf, int part = 0, int nparts = 1) {
        dma_tile_a(kt, buf, part, nparts);
        dma_tile_b(kt, buf, part, nparts);
    };
#endif
    /* Every offset below is computed for all lanes and then chosen against the out-of-range
     * constant: a select of two values, never "compute it if in range". The second form becomes a
     * divergent branch around the arithmetic, and under register pressure the compiler has put its
     * own register-to-register copies of unrelated live values (live-range splits) into the join
     * block ahead of the instruction that restores the execution mask, so lanes that were out of
     * range kept stale registers and later tiles were gathered from wrong rows. */
#pragma unroll
    for (int e = 0; e < EA; ++e) {
#if TA
        /* a_row = k inside the tile, a_col = first of AV consecutive rows m (M % AV == 0) */
        const int m = m0 + a_col[e];
        bool ok = (A_CHUNKS % NT == 0) || (tid + e * NT < A_CHUNKS);
        if (M % BM != 0) ok = ok & (m < M);
        const unsigned off = (unsigned)((gi * K + a_row[e]) * M + m) * 4u;
        a_voff[e] = ok ? off : OOB;
#else
        const int m = m0 + a_row[e];
        bool ok = (A_CHUNKS % NT == 0) || (tid + e * NT < A_CHUNKS);
        if (M % BM != 0) ok = ok & (m < M);
        const unsigned off = (unsigned)((gi * M + m) * K + a_col[e]) * 4u;
        a_voff[e] = ok ? off : OOB;
#endif
    }
#if DTL
    /* tile 0 of A is requested before the index arithmetic of the gathered operand, which
     * its round trip then covers */
    dma_tile_a(0, 0);
#endif
#if MODE == 1
    /* pixel decomposition of each column this thread gathers */
#pragma unroll
    for (int e = 0; e < EB; ++e) {
        const int n = n0 + b_col[e];
        px_ok[e] = (n < N) & (tid + e * NT < B_CHUNKS);
        const int nn = px_ok[e] ? n : 0;
        const int b = nn / OHW;
        const int p = nn % OHW;
        px_h[e] = (p / CQ) * CSTRH - CPADH;
        px_w[e] = (p % CQ) * CSTRW - CPADW;
        px_off[e] = b * (CC * CH * CW) + gi * ((CC / CG) * CH * CW);
    }
#endif
#pragma unroll
    for (int e = 0; e < EB; ++e) {
        bool ok = (B_CHUNKS % NT == 0) || (tid + e * NT < B_CHUNKS);
#if MODE == 2
        const int n = n0 + b_row[e];
        if (N % BN != 0) ok = ok & (n < N);
        const unsigned off = (unsigned)((gi * N + n) * K + b_col[e]) * 4u;
        b_voff[e] = ok ? off : OOB;
#elif MODE == 0
        const int n = n0 + b_col[e];
        if (N % BN != 0) ok = ok & (n < N);
        const unsigned off = (unsigned)((gi * K + b_row[e]) * N + n) * 4u;
        b_voff[e] = ok ? off : OOB;
#elif KHOIST
#if BROW_LINEAR
        /* every element of this lane is the same pixel, BROW_STEP rows of the tile further down:
         * channel and tap follow from those of element 0 without another division */
        const int cl0 = b_row[0] / (CR * CS), rs0 = b_row[0] % (CR * CS);
        const int rsx = rs0 + (e * BROW_STEP) % (CR * CS);
        const int rs = rsx >= CR * CS ? rsx - CR * CS : rsx;
        const int cl = cl0 + (e * BROW_STEP) / (CR * CS) + (rsx >= CR * CS ? 1 : 0);
        const int ih = px_h[0] + (rs / CS) * CDILH;
        const int iw = px_w[0] + (rs % CS) * CDILW;
        ok = ok & px_ok[0] & ((unsigned)ih < (unsigned)CH) & ((unsigned)iw < (unsigned)CW);
        const unsigned off = (unsigned)(px_off[0] + cl * (CH * CW) + ih * CW + iw) * 4u;
        b_voff[e] = ok ? off : OOB;
#else
        const int cl = b_row[e] / (CR * CS);
        const int rs = b_row[e] % (CR * CS);
        const int ih = px_h[e] + (rs / CS) * CDILH;
        const int iw = px_w[e] + (rs % CS) * CDILW;
        ok = ok & px_ok[e] & ((unsigned)ih < (unsigned)CH) & ((unsigned)iw < (unsigned)CW);
        const unsigned off = (unsigned)(px_off[e] + cl * (CH * CW) + ih * CW + iw) * 4u;
        b_voff[e] = ok ? off : OOB;
#endif
#else
        b_voff[e] = OOB;  /* recomputed for every tile */
#endif
#if DTL
        dma_b_one(0, 0, e);       /* tile 0: each load leaves as soon as its address is known */
#endif
    }

    avec_t areg[PD][EA];
    bvec_t breg[PD][EB];

    auto load_global = [&](int kt, int set) {
        const int k0 = kbase + kt * BK;
#pragma unroll
        for (int e = 0; e < EA; ++e) {
            unsigned vo = a_voff[e];
#if TA
            if (KP != K) vo = (k0 + a_row[e] < K) ? vo : OOB;
            areg[set][e] = LOAD_A(rsrc_a, vo, k0 * (M * 4));
#else
            if (KP != K) vo = (k0 + a_col[e] < K) ? vo : OOB;
            areg[set][e] = LOAD_A(rsrc_a, vo, k0 * 4);
#endif
        }
#pragma unroll
        for (int e = 0; e < EB; ++e) {
#if MODE == 2
            unsigned vo = b_voff[e];
            if (KP != K) vo = (k0 + b_col[e] < K) ? vo : OOB;
            breg[set][e] = LOAD_B(rsrc_b, vo, k0 * 4);
#elif MODE == 0
            unsigned vo = b_voff[e];
            if (KP != K) vo = (k0 + b_row[e] < K) ? vo : OOB;
            breg[set][e] = LOAD_B(rsrc_b, vo, k0 * (N * 4));
#elif KHOIST
            unsigned vo = b_voff[e];
            if (KP != K) vo = (k0 + b_row[e] < K) ? vo : OOB;
            breg[set][e] = LOAD_B(rsrc_b, vo, (k0 / (CR * CS)) * (CH * CW * 4));
#else
            const int k = k0 + b_row[e];
            const int c = k / (CR * CS);
            const int rs = k % (CR * CS);
            const int ih = px_h[e] + (rs / CS) * CDILH;
            const int iw = px_w[e] + (rs % CS) * CDILW;
            bool ok = px_ok[e] & ((unsigned)ih < (unsigned)CH) & ((unsigned)iw < (unsigned)CW);
            if (KP != K) ok = ok & (k < K);
            const unsigned off = (unsigned)(px_off[e] + c * (CH * CW) + ih * CW + iw) * 4u;
            const unsigned vo = ok ? off : OOB;      /* a select of two values, no branch (see a_voff) */
            breg[set][e] = LOAD_B(rsrc_b, vo, 0);
#endif
        }
    };

    auto store_lds = [&](int buf, int set) {
#pragma unroll
        for (int e = 0; e < EA; ++e) {
            if ((A_CHUNKS % NT == 0) || (tid + e * NT < A_CHUNKS)) {
#if TA
                /* transpose: element i of the vector is row a_col + i, column k = a_row */
#if AV == 4
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    As[buf][(a_col[e] + i) * SA + ACOL(a_col[e] + i, a_row[e])] = areg[set][e][i];
#else
                As[buf][a_col[e] * SA + ACOL(a_col[e], a_row[e])] = areg[set][e];
#endif
#else
                *reinterpret_cast<avec_t*>(&As[buf][a_row[e] * SA + ACOL(a_row[e], a_col[e])]) = areg[set][e];
#endif
            }
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

#pragma unroll
    for (int i = 0; i < REP_M; ++i)
#pragma unroll
        for (int j = 0; j < REP_N; ++j)
            acc[i][j] = (acc_t)(0.0f);

    /* ---- MFMA operands: LDS -> registers -> matrix core ------------------ */
    /* lane constants of the fragment reads (the same for every tile and buffer) */
#if TA && DTL
    /* physical column of row m in tile row kb + 4*lg + s (see TSWK): m ^ (lane group part) */
    int acolx[REP_M];
#pragma unroll
    for (int i = 0; i < REP_M; ++i)
        acolx[i] = (wm * REP_M * MFMA + i * MFMA + li) ^ (MFMA == 16 ? (lg << 4) : (lg << 5));
#endif
    const int arow = wm * REP_M * MFMA + li;   /* + i*MFMA: SWZ is the same when MFMA % 16 == 0 */
    int acls[SWZ_CLASSES];
#pragma unroll
    for (int c = 0; c < SWZ_CLASSES; ++c)
        acls[c] = ((c * KL + lg) ^ SWZ(arow)) << 2;
#if MODE == 2
    const int brow = wn * REP_N * MFMA + li;
    int bcls[SWZ_CLASSES];
#pragma unroll
    for (int c = 0; c < SWZ_CLASSES; ++c)
        bcls[c] = ((c * KL + lg) ^ SWZ(brow)) << 2;
#elif defined(BSWZ)
    /* physical column of logical column n in row kb + 4*lg + s: n ^ (lane part) ^ (kb part) */
    int bcolx[REP_N];
#pragma unroll
    for (int j = 0; j < REP_N; ++j)
        bcolx[j] = (wn * REP_N * MFMA + j * MFMA + li) ^ (MFMA == 16 ? (lg << 4) : (lg << 5));
#elif defined(BSWZ1)
    /* logical (kb + 4*lg + s, n) sits at row kb + 4*lg + (s ^ BSW_R(lg)), column n ^ BSW_C(lg) */
    int bcolx[REP_N], browx[4];
#pragma unroll
    for (int j = 0; j < REP_N; ++j)
        bcolx[j] = (wn * REP_N * MFMA + j * MFMA + li) ^ BSW_C(lg);
#pragma unroll
    for (int s = 0; s < 4; ++s)
        browx[s] = (s ^ BSW_R(lg)) * SB;
#endif
    /* the operands of the k block [kb, kb + KBLK) of the tile in LDS buffer buf:
     * a[i] = four k values of row block i, b[s][j] = k value s of column block j */
    auto read_block = [&](int buf, int kb, f32x4 (&a)[REP_M], float (&b)[4][REP_N]) {
#if TA && DTL
        const float* at = &As[buf][(4 * lg) * BM];
#pragma unroll
        for (int i = 0; i < REP_M; ++i)
#pragma unroll
            for (int s = 0; s < 4; ++s)
                a[i][s] = at[(kb + s) * BM + acolx[i]];
#else
        const float* as = &As[buf][arow * SA];
#pragma unroll
        for (int i = 0; i < REP_M; ++i)
            a[i] = *reinterpret_cast<const f32x4*>(as + i * MFMA * SA + SWZ_HI(kb) + acls[SWZ_CLS(kb)]);
#endif
#if MODE == 2
        const float* bs = &Bs[buf][brow * SB];
#pragma unroll
        for (int j = 0; j < REP_N; ++j) {
            const f32x4 b4 = *reinterpret_cast<const f32x4*>(bs + j * MFMA * SB + SWZ_HI(kb) + bcls[SWZ_CLS(kb)]);
#pragma unroll
            for (int s = 0; s < 4; ++s)
                b[s][j] = b4[s];
        }
#else
#if defined(BSWZ) || defined(BSWZ1)
        const float* bs = &Bs[buf][(4 * lg) * SB];
#else
        const float* bs = &Bs[buf][(4 * lg) * SB + wn * REP_N * MFMA + li];
#endif
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int j = 0; j < REP_N; ++j)
#if defined(BSWZ)
                b[s][j] = bs[(kb + s) * SB + (bcolx[j] ^ (MFMA == 16 ? 0 : (((kb >> 2) & 1) << 5)))];
#elif defined(BSWZ1)
                b[s][j] = bs[kb * SB + browx[s] + bcolx[j]];
#else
                b[s][j] = bs[(kb + s) * SB + j * MFMA];
#endif
#endif
    };
    auto mfma_block = [&](const f32x4 (&a)[REP_M], const float (&b)[4][REP_N]) {
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int i = 0; i < REP_M; ++i)
#pragma unroll
                for (int j = 0; j < REP_N; ++j)
                    acc[i][j] = MFMA_OP(a[i][s], b[s][j], acc[i][j]);
    };
    auto compute = [&](int buf) {
#pragma unroll
        for (int kb = 0; kb < BK; kb += KBLK) {
            f32x4 a[REP_M];
            float b[4][REP_N];
            read_block(buf, kb, a, b);
            mfma_block(a, b);
        }
    };


    /* ---- main loop ------------------------------------------------------ */
    /* Tile t travels global -> register set t % PD -> LDS buffer -> MFMA.
     * While tile kt is multiplied, tiles kt+1 .. kt+PD are in registers or in
     * flight; tile kt+1 is written to LDS right after the MFMAs of tile kt. */
#if DTL
    /* tile 0 was requested above, as early as its addresses were known */
    __builtin_amdgcn_s_waitcnt(0x0F70);      /* vmcnt(0): this wavefront's part of tile 0 is in LDS */
#else
#pragma unroll
    for (int p = 0; p < PD; ++p)
        if (p < nk) load_global(p, p);
    store_lds(0, 0);
#endif
#if SK_PER > 0
    /* The arrival for the slot written at the end of the previous segment is
     * counted here, behind this tile's first loads: vector memory operations
     * retire in issue order, so the slot stores have long completed when the
     * explicit wait returns and the exchange costs this segment next to
     * nothing. */
    if (arrive_tile >= 0) SK_DRAIN_STORES();
#endif
    __syncthreads();
#if SK_PER > 0
    if (arrive_tile >= 0) {
        if (tid == 0)
            check_before = __hip_atomic_fetch_add(&sk_cnt[arrive_tile], 1u, SK_ARRIVE_ORDER, __HIP_MEMORY_SCOPE_AGENT);
        check_tile = arrive_tile;
        arrive_tile = -1;
    }
#endif
#if DTL && STAGES > 2
    /* STAGES buffers: tiles 1 .. STAGES-2 are requested right behind tile 0,
     * and tile kt+STAGES-1 while tile kt is multiplied, so STAGES-1 tiles are
     * in flight or landed ahead of the MFMAs. Loads complete in order: a wait
     * that leaves the loads of the tiles behind kt+1 outstanding has seen
     * tile kt+1 land. */
#pragma unroll
    for (int p = 1; p < STAGES - 1; ++p)
        if (p < nk) dma_tile(p, p);
    {
        int cur = 0, nxt = STAGES - 1;       /* buffers of tile kt and of tile kt+STAGES-1 */
        for (int kt = 0; kt < nk; ++kt) {
            if (kt + STAGES - 1 < nk) dma_tile(kt + STAGES - 1, nxt);
            compute(cur);
            const int behind = nk - kt - 2;  /* requested tiles behind tile kt+1 (more than STAGES-2 never are) */
            if (behind >= STAGES - 2) VMCNT((STAGES - 2) * DMA_PER_TILE);
#if STAGES > 3
            else if (behind == 1) VMCNT(DMA_PER_TILE);
#endif
            else VMCNT(0);
            __syncthreads();
            cur = (cur + 1 == STAGES) ? 0 : cur + 1;
            nxt = (nxt + 1 == STAGES) ? 0 : nxt + 1;
        }
    }
#elif DTL && FPF
    /* Two buffers, and the operands of a tile's first k block are read right behind the
     * barrier that ends the tile before it, ahead of that tile's last MFMAs: the LDS
     * latency of the first reads, which every wavefront of the workgroup would otherwise
     * sit out together after each barrier, hides behind matrix work. The barrier stands
     * before the last k block's MFMAs; all reads of the current buffer have returned by
     * then (lgkmcnt(0)), so the next iteration may overwrite it. */
    {
        f32x4 pa[REP_M];
        float pb[4][REP_N];
        read_block(0, 0, pa, pb);
        for (int kt = 0; kt < nk; ++kt) {
            const int cur = kt & 1;
            f32x4 a[2][REP_M], na[REP_M];
            float b[2][4][REP_N], nb[4][REP_N];
#pragma unroll
            for (int blk = 0; blk < BK / KBLK; ++blk) {
                /* the next tile's loads, in LSPREAD parts in front of the first LSPREAD k blocks: with
                 * few wavefronts per SIMD a wavefront that issues all of them at once keeps the
                 * matrix core waiting; spread out, they go between its MFMAs */
                if (blk < LSPREAD && kt + 1 < nk) dma_tile(kt + 1, cur ^ 1, blk, LSPREAD);
                if (blk + 1 < BK / KBLK) read_block(cur, (blk + 1) * KBLK, a[(blk + 1) & 1], b[(blk + 1) & 1]);
                if (blk == BK / KBLK - 1) {
                    __builtin_amdgcn_s_waitcnt(0x0070);      /* vmcnt(0), lgkmcnt(0) */
                    __syncthreads();
                    /* after the last tile this reads stale data that nothing uses */
                    read_block(cur ^ 1, 0, na, nb);
                }
                /* the reads above are issued before the MFMAs below, which then hide their latency
                 * (left alone, the scheduler puts each read right in front of its first use) */
                __builtin_amdgcn_sched_barrier(0);
                if (blk == 0) mfma_block(pa, pb);
                else mfma_block(a[blk & 1], b[blk & 1]);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i = 0; i < REP_M; ++i) pa[i] = na[i];
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int j = 0; j < REP_N; ++j) pb[s][j] = nb[s][j];
        }
    }
#elif DTL
    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) dma_tile(kt + 1, cur ^ 1);      /* lands while tile kt is multiplied */
        compute(cur);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
    }
#else
    for (int kt0 = 0; kt0 < nk; kt0 += PD) {
#pragma unroll
        for (int u = 0; u < PD; ++u) {
            const int kt = kt0 + u;
            if (kt < nk) {
                const int cur = (STAGES == 2) ? (kt & 1) : 0;
                if (kt + PD < nk) load_global(kt + PD, u);
                /* keep the prefetch at the top of the iteration: without this
                 * fence the scheduler sinks the loads down to their use */
                __builtin_amdgcn_sched_barrier(0);
                compute(cur);
                if (STAGES == 1) __syncthreads();
                if (kt + 1 < nk) store_lds((STAGES == 2) ? (cur ^ 1) : 0, (u + 1) % PD);
                __syncthreads();
            }
        }
    }
#endif
    /* A 16-pass MFMA's last result registers may not be read for 19 issue
     * slots, and nothing in the hardware enforces that. The compiler pads
     * the code it can follow, but in the segment loop's control flow of
     * balanced K streaming its hazard pass lost the short path from the last
     * MFMA to the first accumulator read (a full tile's store then took the
     * value from before the last MFMA), so the distance is made explicit. */
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 15\n\ts_nop 3" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

#if WAVES_K > 1
    /* ---- sum the k-groups' partial tiles through LDS --------------------- */
    /* the last barrier of the main loop has passed: tile memory is free */
    if (kg > 0) {
        float* red = smem + (kg - 1) * (NT * REP_M * REP_N * NACC);
#pragma unroll
        for (int i = 0; i < REP_M; ++i)
#pragma unroll
            for (int j = 0; j < REP_N; ++j)
#pragma unroll
                for (int v = 0; v < NACC; ++v)
                    red[((i * REP_N + j) * NACC + v) * NT + tid] = acc[i][j][v];
    }
    __syncthreads();
    if (kg > 0) return;
#pragma unroll
    for (int g = 1; g < WAVES_K; ++g) {
        const float* red = smem + (g - 1) * (NT * REP_M * REP_N * NACC);
#pragma unroll
        for (int i = 0; i < REP_M; ++i)
#pragma unroll
            for (int j = 0; j < REP_N; ++j)
#pragma unroll
                for (int v = 0; v < NACC; ++v)
                    acc[i][j][v] += red[((i * REP_N + j) * NACC + v) * NT + tid];
    }
#endif

#if SK_PER > 0
    if (nk != KT) {
        int wg_first, wg_last;
        sharers(tile, wg_first, wg_last);
        const unsigned others = (unsigned)(wg_last - wg_first);
        if (kt_lo == 0) {
            /* this workgroup holds the lowest K range and ends its run here,
             * long after the other sharers began theirs: when all of them
             * have arrived, add their slots to the registers and store */
            if (tid == 0)
                sk_arrived = __hip_atomic_load(&sk_cnt[tile], SK_LOOK_ORDER, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            const bool all_in = (sk_arrived == others);
            __syncthreads();
            if (all_in) {
                add_slots(tile, wg_first + 1, wg_last);
                if (tid == 0) atomicExch(&sk_cnt[tile], 0u);   /* ready for the next launch */
                store_c(m0, n0, gi, true);
                continue;
            }
        }
        float* mine = slot_of(wg, tile);
#pragma unroll
        for (int i = 0; i < REP_M; ++i)
#pragma unroll
            for (int j = 0; j < REP_N; ++j)
#pragma unroll
                for (int v = 0; v < NACC; ++v)
                    __hip_atomic_store(&mine[((i * REP_N + j) * NACC + v) * NT + tid], acc[i][j][v],
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (unit < unit_end) {
            arrive_tile = tile;      /* counted in the next segment's prologue */
            continue;
        }
        SK_DRAIN_STORES();
        __syncthreads();
        if (tid == 0)
            sk_arrived = __hip_atomic_fetch_add(&sk_cnt[tile], 1u, SK_ARRIVE_ORDER, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        const unsigned before_me = sk_arrived;
        __syncthreads();
        if (before_me != others) continue;
        if (tid == 0) atomicExch(&sk_cnt[tile], 0u);
        clear_acc();
        add_slots(tile, wg_first, wg_last);
    }
#endif
    store_c(m0, n0, gi, kz == 0);
    }   /* tile / segment */
#if SK_PER > 0
    if (check_tile >= 0) {
        /* the first segment's arrival: if every other sharer had arrived
         * before, the sum falls to this workgroup */
        if (tid == 0) sk_arrived = check_before;
        __syncthreads();
        int wg_first, wg_last;
        sharers(check_tile, wg_first, wg_last);
        if (sk_arrived == (unsigned)(wg_last - wg_first)) {
            if (tid == 0) atomicExch(&sk_cnt[check_tile], 0u);
            clear_acc();
            add_slots(check_tile, wg_first, wg_last);
            int m0, n0;
            tile_origin(check_tile % (TILES_M * TILES_N), m0, n0);
            store_c(m0, n0, check_tile / (TILES_M * TILES_N), true);
        }
    }
#endif
    CLK_END;
}
