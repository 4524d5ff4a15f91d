// int8 x int8 -> int32 GEMM kernel template for gfx950 (CDNA4), hiprtc-compiled.
//
//   C[M][N] = sum_k int32(A[m][k]) * int32(B[n][k])
//
// A is [M][K] and B is [N][K], both K-contiguous ("B in K-major layout"), C is
// row-major int32 — the compute of
// flextensor/test/test_tvm/legacy/gemm_int8.py:15-21.
//
// Knobs (-D constants set by the scheduler from a Config):
//   MFMA        32 -> v_mfma_i32_32x32x32_i8, 16 -> v_mfma_i32_16x16x64_i8
//   WAVES_M/N   wavefronts per workgroup along M / N
//   REP_M/N     MFMA tiles per wavefront along M / N
//   BK          bytes of K per LDS tile (multiple of the MFMA K)
//   STAGES      1 or 2 LDS buffers
//   PD          prefetch distance: global loads of tile t+PD are in flight
//               (in PD register sets) while tile t is multiplied
//   FRAGPF      1: fragment-prefetch pipeline. Tile t+1 is written to LDS at
//               the *start* of iteration t (its global loads were issued one
//               iteration earlier), the operand fragments of the next k-step
//               are read from LDS while the MFMAs of the current one run, and
//               the first fragments of tile t+1 are read right after the one
//               barrier of the iteration, so that the matrix cores have work
//               immediately after every barrier (needs STAGES 2, PD 1)
//   GROUP_M     tile-traversal group height (L2 locality)
//   XCD_REMAP   1: consecutive logical tiles stay on one XCD
//   PAD         LDS row padding in bytes (multiple of 16); -1 selects
//               unpadded rows whose 16-byte chunks are XOR-swizzled by row
//   DTL         1: tiles travel global -> LDS directly (buffer loads with the
//               lds modifier, 16 bytes per lane): no staging registers, no
//               LDS store instructions; the row swizzle is applied on the
//               global side, since a wavefront's 64 chunks land contiguously
//               DTL 3: the same data path with the instruction order of the
//               main loop written out and pinned: the LDS fragment reads of
//               the next k-step and the direct-to-LDS loads of the tile after
//               next are issued one at a time between the MFMAs of the current
//               k-step, and the one barrier of a tile sits a quarter into its
//               last k-step, so that the matrix cores always have queued work
//               (left to itself the compiler issues the fragment reads right
//               before their first use and waits for them)
//   NT_STORE    1: non-temporal stores for C
//   EARLYST     1 (with DTL 2 and two k-steps per tile): the last tile is multiplied
//               block by block instead of k-step by k-step, and every accumulator
//               block is stored as soon as its last MFMA has been issued and the
//               next group's MFMAs cover the distance to the read: the stores of C
//               start a tile's time before the workgroup's last MFMA instead of
//               behind it
//   SPLITK      grid-level split of K: SPLITK workgroups per tile, each over a
//               contiguous range of K; the partial sums meet in C (zero-filled by a
//               kernel in front) through integer atomic adds, which are exact and
//               order-independent, so the result stays bit-exact and repeatable
//   WAVES_K     split of K inside the workgroup: WAVES_K groups of WAVES_M x WAVES_N
//               wavefronts, each with its own LDS tiles and its own range of K; the
//               groups' accumulators are summed through LDS and group 0 stores
//   CVEC        1: the MFMA operands are swapped (the core computes the
//               transposed tile), so a lane holds four consecutive columns of
//               one row of C and writes them with one 128-bit store
//
// Both operands live in LDS as [rows][BK+PAD] bytes and are read as one
// 128-bit load per lane per MFMA: lane (i, g) takes the 16 bytes at
// k = kstep + 16*g of row i, identically for A and B, so whatever order the
// matrix core assigns to those 16 values inside its K dimension, A and B
// agree and the integer sum is exact.

/* Constants arrive as -DFT_<NAME>=value: single-letter macros on the command line
 * would be visible to (and break) the runtime-compilation built-in headers. */
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
#define FRAGPF FT_FRAGPF
#define GROUP_M FT_GROUP_M
#define XCD_REMAP FT_XCD_REMAP
#define PAD FT_PAD
#define NT_STORE FT_NT_STORE
#ifdef FT_DTL
#define DTL FT_DTL
#else
#define DTL 0
#endif
#ifdef FT_CVEC
#define CVEC FT_CVEC
#else
#define CVEC 0
#endif
#ifdef FT_EARLYST
#define EARLYST FT_EARLYST
#else
#define EARLYST 0
#endif
#ifdef FT_SPLITK
#define SPLITK FT_SPLITK
#else
#define SPLITK 1
#endif
#ifdef FT_WAVES_K
#define WAVES_K FT_WAVES_K
#else
#define WAVES_K 1
#endif

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));

#if MFMA == 32
typedef i32x16 acc_t;
#define NACC 16
#define MFMA_K 32
#define MFMA_RAW(a, b, c) __builtin_amdgcn_mfma_i32_32x32x32_i8((a), (b), (c), 0, 0, 0)
#elif MFMA == 16
typedef i32x4 acc_t;
#define NACC 4
#define MFMA_K 64
#define MFMA_RAW(a, b, c) __builtin_amdgcn_mfma_i32_16x16x64_i8((a), (b), (c), 0, 0, 0)
#else
#error "MFMA must be 16 or 32"
#endif
#if CVEC
#define MFMA_OP(a, b, c) MFMA_RAW((b), (a), (c))   /* rows of the result follow B's rows (n) */
#else
#define MFMA_OP(a, b, c) MFMA_RAW((a), (b), (c))
#endif

#define BM (WAVES_M * REP_M * MFMA)
#define BN (WAVES_N * REP_N * MFMA)
#define NT (WAVES_M * WAVES_N * 64)      /* threads of one k-group */
#define NTW (NT * WAVES_K)               /* threads of the workgroup */
#define CRW (BK / 16)             /* 16-byte chunks per LDS row */
#if PAD < 0
#define SROW (BK)                 /* LDS row stride in bytes */
#if CRW >= 16
#define SWZ(row) ((row) & 15)
#else
#define SWZ(row) (((row) / (16 / CRW)) & (CRW - 1))
#endif
#else
#define SROW (BK + PAD)
#define SWZ(row) 0
#endif
/* byte column c (multiple of 16) of `row` -> physical byte column */
#define PCOL(row, c) (((((c) >> 4) ^ SWZ(row)) << 4))
#define OOB 0x80000000u
#define TILES_M ((M + BM - 1) / BM)
#define TILES_N ((N + BN - 1) / BN)
/* KP = K rounded up to a multiple of 64 (host checks KP % BK == 0); chunks
 * beyond K are zero-filled by the load predicate. When K is no multiple of 16
 * the rows of A and B are not 16-byte aligned and the last chunk of a row is
 * partly beyond it (those bytes are the next row's, not zeros): the chunk is
 * then put together from dword loads (K % 4 == 0) or byte loads, each with its
 * own predicate. Register-staged pipelines only. */
#define KT (KP / BK / (SPLITK * WAVES_K))      /* tiles of one k-group (host checks divisibility) */
#if EARLYST && (SPLITK > 1 || WAVES_K > 1)
#error "early stores write finished sums: no K division"
#endif

#if BK % MFMA_K != 0
#error "BK must be a multiple of the MFMA K extent"
#endif
#if PAD >= 0 && PAD % 16 != 0
#error "PAD must be a multiple of 16 bytes"
#endif

#define CHUNKS_ROW (BK / 16)
#define A_CHUNKS (BM * CHUNKS_ROW)
#define B_CHUNKS (BN * CHUNKS_ROW)
#define EA ((A_CHUNKS + NT - 1) / NT)
#define EB ((B_CHUNKS + NT - 1) / NT)
#if DTL
#if PAD > 0 || STAGES != 2 || A_CHUNKS % NT != 0 || B_CHUNKS % NT != 0 || K % 16 != 0
#error "direct-to-LDS tiles need unpadded rows, two buffers, whole rounds of chunks and K % 16 == 0"
#endif
#if DTL == 3 && ((BK / MFMA_K) % 2 != 0 || REP_M * REP_N / 4 + REP_M + REP_N > REP_M * REP_N || REP_M * REP_N / 4 + EA + EB > REP_M * REP_N)
#error "the pinned schedule needs an even number of k-steps per tile and enough MFMAs per k-step to interleave with"
#endif
typedef __attribute__((address_space(3))) void lds_void;
#endif

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

#define A_TILE_BYTES (BM * SROW)
#define B_TILE_BYTES (BN * SROW)
#define TILE_BYTES (WAVES_K * STAGES * (A_TILE_BYTES + B_TILE_BYTES))
#define RED_BYTES ((WAVES_K - 1) * NT * REP_M * REP_N * NACC * 4)
#define SMEM_BYTES (TILE_BYTES > RED_BYTES ? TILE_BYTES : RED_BYTES)

extern "C" __global__ __launch_bounds__(NTW)
void gemm_i8(const signed char* __restrict__ A, const signed char* __restrict__ B,
             int* __restrict__ C CLK_PARAM)
{
    CLK_BEGIN
#if WAVES_K > 1
    /* every k-group has its own tiles; the memory is reused for the sum of the groups */
    __shared__ __attribute__((aligned(16))) signed char smem[SMEM_BYTES];
    const int kg = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / NT));
    const int tid = threadIdx.x - kg * NT;          /* thread index inside the k-group */
    signed char (*As)[A_TILE_BYTES] = reinterpret_cast<signed char (*)[A_TILE_BYTES]>(smem + kg * STAGES * A_TILE_BYTES);
    signed char (*Bs)[B_TILE_BYTES] = reinterpret_cast<signed char (*)[B_TILE_BYTES]>(
        smem + WAVES_K * STAGES * A_TILE_BYTES + kg * STAGES * B_TILE_BYTES);
#else
    __shared__ __attribute__((aligned(16))) signed char As[STAGES][BM * SROW];
    __shared__ __attribute__((aligned(16))) signed char Bs[STAGES][BN * SROW];
    const int kg = 0;
    const int tid = threadIdx.x;
#endif
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N;
    const int wn = wave % WAVES_N;
    const int li = lane % MFMA;
    const int lg = lane / MFMA;

    const int nblk = TILES_M * TILES_N * SPLITK;
    int bid = blockIdx.x;
#if XCD_REMAP
    if (nblk % 8 == 0) bid = (bid % 8) * (nblk / 8) + bid / 8;
#endif
#if SPLITK > 1
    const int kz = bid / (TILES_M * TILES_N);       /* which part of K */
    bid = bid % (TILES_M * TILES_N);
#else
    const int kz = 0;
#endif
    const int kbase = (kz * WAVES_K + kg) * (KT * BK);     /* first k of this group's range */
    const int grp = bid / (GROUP_M * TILES_N);
    const int first_m = grp * GROUP_M;
    const int gsz = (TILES_M - first_m) < GROUP_M ? (TILES_M - first_m) : GROUP_M;
    const int rr = bid % (GROUP_M * TILES_N);
    const int tile_m = first_m + rr % gsz;
    const int tile_n = rr / gsz;
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;

    int a_row[EA], a_col[EA], b_row[EB], b_col[EB];
#pragma unroll
    for (int e = 0; e < EA; ++e) {
        const int q = tid + e * NT;
        a_row[e] = q / CHUNKS_ROW;
#if DTL
        /* chunk q lands at byte 16*q of the tile = physical chunk q % CHUNKS_ROW
         * of its row: fetch the logical chunk that belongs there */
        a_col[e] = ((q % CHUNKS_ROW) ^ SWZ(a_row[e])) * 16;
#else
        a_col[e] = (q % CHUNKS_ROW) * 16;
#endif
    }
#pragma unroll
    for (int e = 0; e < EB; ++e) {
        const int q = tid + e * NT;
        b_row[e] = q / CHUNKS_ROW;
#if DTL
        b_col[e] = ((q % CHUNKS_ROW) ^ SWZ(b_row[e])) * 16;
#else
        b_col[e] = (q % CHUNKS_ROW) * 16;
#endif
    }

    /* raw buffer loads: an element that must read as zero (edge tile, idle
     * lane, K tail) gets an offset beyond the buffer and loads 0 */
    const __amdgpu_buffer_rsrc_t rsrc_a =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<signed char*>(A), 0, M * K, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<signed char*>(B), 0, N * K, 0x00020000);
    unsigned a_voff[EA], b_voff[EB];
#pragma unroll
    for (int e = 0; e < EA; ++e) {
        const int m = m0 + a_row[e];
        bool ok = (A_CHUNKS % NT == 0) || (tid + e * NT < A_CHUNKS);
        if (M % BM != 0) ok = ok && (m < M);
        a_voff[e] = ok ? (unsigned)(m * K + a_col[e]) : OOB;
    }
#pragma unroll
    for (int e = 0; e < EB; ++e) {
        const int n = n0 + b_row[e];
        bool ok = (B_CHUNKS % NT == 0) || (tid + e * NT < B_CHUNKS);
        if (N % BN != 0) ok = ok && (n < N);
        b_voff[e] = ok ? (unsigned)(n * K + b_col[e]) : OOB;
    }

    i32x4 areg[PD][EA], breg[PD][EB];

    /* the 16 bytes k0 + col .. k0 + col + 15 of the row whose chunk offset is vo */
    auto load_chunk = [&](__amdgpu_buffer_rsrc_t rsrc, unsigned vo, int k0, int col) -> i32x4 {
#if K % 16 == 0
        return __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)vo, k0, 0));
#elif K % 4 == 0
        i32x4 v;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const unsigned o = (vo != OOB && k0 + col + 4 * d < K) ? vo + 4 * d : OOB;
            v[d] = (int)__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)o, k0, 0);
        }
        return v;
#else
        i32x4 v = (i32x4)(0);
#pragma unroll
        for (int b = 0; b < 16; ++b) {
            const unsigned o = (vo != OOB && k0 + col + b < K) ? vo + b : OOB;
            const unsigned byte = (unsigned)__builtin_amdgcn_raw_buffer_load_b8(rsrc, (int)o, k0, 0) & 0xffu;
            v[b / 4] |= (int)(byte << (8 * (b % 4)));
        }
        return v;
#endif
    };

    auto load_global = [&](int kt, int set) {
        const int k0 = kbase + kt * BK;
#pragma unroll
        for (int e = 0; e < EA; ++e) {
            unsigned vo = a_voff[e];
            if (KP != K) vo = (k0 + a_col[e] < K) ? vo : OOB;
            areg[set][e] = load_chunk(rsrc_a, vo, k0, a_col[e]);
        }
#pragma unroll
        for (int e = 0; e < EB; ++e) {
            unsigned vo = b_voff[e];
            if (KP != K) vo = (k0 + b_col[e] < K) ? vo : OOB;
            breg[set][e] = load_chunk(rsrc_b, vo, k0, b_col[e]);
        }
    };

    auto store_lds = [&](int buf, int set) {
#pragma unroll
        for (int e = 0; e < EA; ++e)
            if ((A_CHUNKS % NT == 0) || (tid + e * NT < A_CHUNKS))
                *reinterpret_cast<i32x4*>(&As[buf][a_row[e] * SROW + PCOL(a_row[e], a_col[e])]) = areg[set][e];
#pragma unroll
        for (int e = 0; e < EB; ++e)
            if ((B_CHUNKS % NT == 0) || (tid + e * NT < B_CHUNKS))
                *reinterpret_cast<i32x4*>(&Bs[buf][b_row[e] * SROW + PCOL(b_row[e], b_col[e])]) = breg[set][e];
    };

    acc_t acc[REP_M][REP_N];
#pragma unroll
    for (int i = 0; i < REP_M; ++i)
#pragma unroll
        for (int j = 0; j < REP_N; ++j)
            acc[i][j] = (acc_t)(0);

    /* accumulator block (i, j) -> C */
    auto store_block = [&](int i, int j) {
#if CVEC
        /* swapped operands: lane (li, lg) holds C[m = li][n = 4*lg + 0..3] (16x16),
         * or C[m = li][n = 8*q + 4*lg + 0..3] in registers 4q..4q+3 (32x32) */
        const int m = m0 + (wm * REP_M + i) * MFMA + li;
#pragma unroll
        for (int q = 0; q < NACC / 4; ++q) {
#if MFMA == 32
            const int n = n0 + (wn * REP_N + j) * MFMA + 8 * q + 4 * lg;
#else
            const int n = n0 + (wn * REP_N + j) * MFMA + 4 * lg;
#endif
            bool ok = true;
            if (M % BM != 0) ok = ok && (m < M);
            if (N % BN != 0) ok = ok && (n < N);      /* N % 4 == 0: whole vectors */
            if (ok) {
                i32x4 v4;
                v4[0] = acc[i][j][4 * q + 0]; v4[1] = acc[i][j][4 * q + 1];
                v4[2] = acc[i][j][4 * q + 2]; v4[3] = acc[i][j][4 * q + 3];
#if SPLITK > 1
#pragma unroll
                for (int x = 0; x < 4; ++x) atomicAdd(C + (size_t)m * N + n + x, v4[x]);
#else
                i32x4* dst = reinterpret_cast<i32x4*>(C + (size_t)m * N + n);
#if NT_STORE
                __builtin_nontemporal_store(v4, dst);
#else
                *dst = v4;
#endif
#endif
            }
        }
#else
        const int n = n0 + (wn * REP_N + j) * MFMA + li;
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
#if SPLITK > 1
                atomicAdd(C + (size_t)m * N + n, acc[i][j][v]);
#elif NT_STORE
                __builtin_nontemporal_store(acc[i][j][v], C + (size_t)m * N + n);
#else
                C[(size_t)m * N + n] = acc[i][j][v];
#endif
            }
        }
#endif
    };

    auto compute = [&](int buf) {
        const int arow = wm * REP_M * MFMA + li;
        const int brow = wn * REP_N * MFMA + li;
        const signed char* as = &As[buf][arow * SROW];
        const signed char* bs = &Bs[buf][brow * SROW];
#pragma unroll
        for (int kk = 0; kk < BK; kk += MFMA_K) {
            i32x4 a[REP_M], b[REP_N];
#pragma unroll
            for (int i = 0; i < REP_M; ++i)
                a[i] = *reinterpret_cast<const i32x4*>(as + i * MFMA * SROW + PCOL(arow + i * MFMA, kk + 16 * lg));
#pragma unroll
            for (int j = 0; j < REP_N; ++j)
                b[j] = *reinterpret_cast<const i32x4*>(bs + j * MFMA * SROW + PCOL(brow + j * MFMA, kk + 16 * lg));
#pragma unroll
            for (int i = 0; i < REP_M; ++i)
#pragma unroll
                for (int j = 0; j < REP_N; ++j)
                    acc[i][j] = MFMA_OP(a[i], b[j], acc[i][j]);
        }
    };

#if DTL
    {
        const int wv = __builtin_amdgcn_readfirstlane(wave);
        /* The load is written as an instruction, not through the builtin: the
         * compiler makes every later LDS read wait for a direct-to-LDS load it
         * knows of (it cannot tell the two buffers apart), which would undo the
         * overlap. Completion is tracked by hand: vmcnt(0) and a barrier at
         * the end of every iteration. */
        auto descriptor = [](const signed char* base, unsigned bytes) {
            const unsigned long long p = (unsigned long long)base;
            i32x4 d;                         /* raw buffer: base, stride 0, size in bytes, untyped dwords */
            d[0] = __builtin_amdgcn_readfirstlane((int)(unsigned)p);
            d[1] = __builtin_amdgcn_readfirstlane((int)((unsigned)(p >> 32) & 0xffffu));
            d[2] = __builtin_amdgcn_readfirstlane((int)bytes);
            d[3] = 0x00020000;
            return d;
        };
        const i32x4 ra = descriptor(A, (unsigned)(M * K));
        const i32x4 rb = descriptor(B, (unsigned)(N * K));
        auto dma16 = [&](const i32x4& rsrc, const signed char* dst, unsigned vo, int so) {
            const unsigned lds_addr = (unsigned)(__UINTPTR_TYPE__)(lds_void*)dst;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :: "s"(lds_addr), "v"(vo), "s"(rsrc), "s"(so) : "memory", "m0");
        };
        auto dma_tile = [&](int kt, int buf) {
            const int k0 = kbase + kt * BK;
#pragma unroll
            for (int e = 0; e < EA; ++e) {
                unsigned vo = a_voff[e];
                if (KP != K) vo = (k0 + a_col[e] < K) ? vo : OOB;
                dma16(ra, &As[buf][(e * NT + wv * 64) * 16], vo, k0);
            }
#pragma unroll
            for (int e = 0; e < EB; ++e) {
                unsigned vo = b_voff[e];
                if (KP != K) vo = (k0 + b_col[e] < K) ? vo : OOB;
                dma16(rb, &Bs[buf][(e * NT + wv * 64) * 16], vo, k0);
            }
        };
        dma_tile(0, 0);
#if DTL != 3
        __builtin_amdgcn_s_waitcnt(0x0F70);     /* vmcnt(0): this wavefront's chunks are in LDS */
        __syncthreads();
#endif
#if DTL == 3
        /* Pinned schedule. Two fragment sets alternate by k-step parity (an even
         * number of k-steps per tile, so a tile ends on the set it began with and
         * nothing is copied). Slot m is what is issued before MFMA m of a k-step:
         *   not the last k-step:  fragment read m of the next k-step   (m < NR)
         *   last k-step:          at m == NB the wait for tile kt+1 and the barrier
         *                         (everybody has read the last fragments of tile kt
         *                         one k-step ago), then fragment read m - NB of tile
         *                         kt+1 and direct-to-LDS load m - NB of tile kt+2,
         *                         which goes into the buffer the barrier has freed
         *                         and has a whole tile period to land. */
#define NKS (BK / MFMA_K)
#define NM (REP_M * REP_N)
#define NR (REP_M + REP_N)
#define NB (NM / 4)
        const int arow = wm * REP_M * MFMA + li;
        const int brow = wn * REP_N * MFMA + li;
        i32x4 fA[2][REP_M], fB[2][REP_N];
        auto rd = [&](int buf, int kk, int set, int g) {
            if (g < REP_M)
                fA[set][g] = *reinterpret_cast<const i32x4*>(&As[buf][(arow + g * MFMA) * SROW + PCOL(arow + g * MFMA, kk + 16 * lg)]);
            else
                fB[set][g - REP_M] = *reinterpret_cast<const i32x4*>(&Bs[buf][(brow + (g - REP_M) * MFMA) * SROW + PCOL(brow + (g - REP_M) * MFMA, kk + 16 * lg)]);
        };
        auto dma_one = [&](int kt, int buf, int e) {
            const int k0 = kbase + kt * BK;
            if (e < EA) {
                unsigned vo = a_voff[e];
                if (KP != K) vo = (k0 + a_col[e] < K) ? vo : OOB;
                dma16(ra, &As[buf][(e * NT + wv * 64) * 16], vo, k0);
            } else {
                unsigned vo = b_voff[e - EA];
                if (KP != K) vo = (k0 + b_col[e - EA] < K) ? vo : OOB;
                dma16(rb, &Bs[buf][((e - EA) * NT + wv * 64) * 16], vo, k0);
            }
        };
        /* one tile; NEXT: tile kt+1 exists (its fragments are fetched), NEXT2: tile kt+2 exists */
#define I8_TILE(NEXT, NEXT2)                                                                          \
        _Pragma("unroll")                                                                             \
        for (int ks = 0; ks < NKS; ++ks) {                                                            \
            const int set = ks & 1;                                                                   \
            _Pragma("unroll")                                                                         \
            for (int m = 0; m < NM; ++m) {                                                            \
                if (ks + 1 < NKS) {                                                                   \
                    if (m < NR) rd(cur, (ks + 1) * MFMA_K, set ^ 1, m);                               \
                } else if (NEXT) {                                                                    \
                    if (m == NB) {                                                                    \
                        __builtin_amdgcn_s_waitcnt(0x0F70);                                           \
                        __syncthreads();                                                              \
                    }                                                                                 \
                    if (m >= NB && m - NB < NR) rd(cur ^ 1, 0, set ^ 1, m - NB);                      \
                    if ((NEXT2) && m >= NB && m - NB < EA + EB) dma_one(kt + 2, cur, m - NB);         \
                }                                                                                     \
                __builtin_amdgcn_sched_barrier(0);                                                    \
                acc[m / REP_N][m % REP_N] = MFMA_OP(fA[set][m / REP_N], fB[set][m % REP_N], acc[m / REP_N][m % REP_N]); \
                __builtin_amdgcn_sched_barrier(0);                                                    \
            }                                                                                         \
        }
        if (KT > 1) dma_tile(1, 1);
        /* tile 0 has landed when at most the loads of tile 1 are outstanding */
        if (KT > 1) __builtin_amdgcn_s_waitcnt(0x0F70 | ((EA + EB) & 15) | (((EA + EB) >> 4) << 14));
        else __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
#pragma unroll
        for (int g = 0; g < NR; ++g) rd(0, 0, 0, g);
        int kt = 0;
        for (; kt + 2 < KT; ++kt) {
            const int cur = kt & 1;
            I8_TILE(1, 1)
        }
        for (; kt + 1 < KT; ++kt) {
            const int cur = kt & 1;
            I8_TILE(1, 0)
        }
        {
            const int cur = kt & 1;
            I8_TILE(0, 0)
        }
#undef I8_TILE
#elif DTL == 2
        /* with fragment prefetch: the LDS reads of step t+1 are issued before
         * the MFMAs of step t, across the tile boundary as well */
        const int arow = wm * REP_M * MFMA + li;
        const int brow = wn * REP_N * MFMA + li;
        auto load_frags = [&](int buf, int kk, i32x4 (&fa)[REP_M], i32x4 (&fb)[REP_N]) {
            const signed char* as = &As[buf][arow * SROW];
            const signed char* bs = &Bs[buf][brow * SROW];
#pragma unroll
            for (int i = 0; i < REP_M; ++i)
                fa[i] = *reinterpret_cast<const i32x4*>(as + i * MFMA * SROW + PCOL(arow + i * MFMA, kk + 16 * lg));
#pragma unroll
            for (int j = 0; j < REP_N; ++j)
                fb[j] = *reinterpret_cast<const i32x4*>(bs + j * MFMA * SROW + PCOL(brow + j * MFMA, kk + 16 * lg));
        };
        i32x4 fa[REP_M], fb[REP_N];
        load_frags(0, 0, fa, fb);
#if EARLYST
#if BK != 2 * MFMA_K
#error "early stores: two k-steps per tile"
#endif
#define KT_LOOP (KT - 1)
#else
#define KT_LOOP KT
#endif
        for (int kt = 0; kt < KT_LOOP; ++kt) {
            const int cur = kt & 1;
            if (kt + 1 < KT) dma_tile(kt + 1, cur ^ 1);
#pragma unroll
            for (int kk = 0; kk < BK; kk += MFMA_K) {
                i32x4 na[REP_M], nb[REP_N];
                if (kk + MFMA_K < BK) {
                    load_frags(cur, kk + MFMA_K, na, nb);
                } else {
                    /* tile kt has been read by everybody, tile kt+1 has landed */
                    __builtin_amdgcn_s_waitcnt(0x0F70);
                    __syncthreads();
                    if (kt + 1 < KT) load_frags(cur ^ 1, 0, na, nb);
                }
#pragma unroll
                for (int i = 0; i < REP_M; ++i)
#pragma unroll
                    for (int j = 0; j < REP_N; ++j)
                        acc[i][j] = MFMA_OP(fa[i], fb[j], acc[i][j]);
                if (kk + MFMA_K < BK || kt + 1 < KT) {
#pragma unroll
                    for (int i = 0; i < REP_M; ++i) fa[i] = na[i];
#pragma unroll
                    for (int j = 0; j < REP_N; ++j) fb[j] = nb[j];
                }
            }
        }
#if EARLYST
        {
            /* the last tile, block-major: fa/fb hold the fragments of its first k-step, na/nb get
             * those of its second; blocks go in groups of EG, and the stores of a group are issued
             * behind the MFMAs of the next group, which cover the distance from an MFMA to the
             * read of its result */
            i32x4 na[REP_M], nb[REP_N];
            load_frags((KT - 1) & 1, MFMA_K, na, nb);
#define EG 4
#define NBLK (REP_M * REP_N)
#pragma unroll
            for (int g = 0; g <= (NBLK + EG - 1) / EG; ++g) {
                if (g * EG < NBLK) {
#pragma unroll
                    for (int b = g * EG; b < g * EG + EG && b < NBLK; ++b)
                        acc[b / REP_N][b % REP_N] = MFMA_OP(fa[b / REP_N], fb[b % REP_N], acc[b / REP_N][b % REP_N]);
#pragma unroll
                    for (int b = g * EG; b < g * EG + EG && b < NBLK; ++b)
                        acc[b / REP_N][b % REP_N] = MFMA_OP(na[b / REP_N], nb[b % REP_N], acc[b / REP_N][b % REP_N]);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (g > 0) {
#pragma unroll
                    for (int b = (g - 1) * EG; b < g * EG && b < NBLK; ++b)
                        store_block(b / REP_N, b % REP_N);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#endif
#else
        for (int kt = 0; kt < KT; ++kt) {
            const int cur = kt & 1;
            if (kt + 1 < KT) dma_tile(kt + 1, cur ^ 1);   /* lands while tile kt is multiplied */
            compute(cur);
            __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
        }
#endif
    }
#elif FRAGPF
    {
        const int arow = wm * REP_M * MFMA + li;
        const int brow = wn * REP_N * MFMA + li;
        auto load_frags = [&](int buf, int kk, i32x4 (&fa)[REP_M], i32x4 (&fb)[REP_N]) {
            const signed char* as = &As[buf][arow * SROW];
            const signed char* bs = &Bs[buf][brow * SROW];
#pragma unroll
            for (int i = 0; i < REP_M; ++i)
                fa[i] = *reinterpret_cast<const i32x4*>(as + i * MFMA * SROW + PCOL(arow + i * MFMA, kk + 16 * lg));
#pragma unroll
            for (int j = 0; j < REP_N; ++j)
                fb[j] = *reinterpret_cast<const i32x4*>(bs + j * MFMA * SROW + PCOL(brow + j * MFMA, kk + 16 * lg));
        };
        i32x4 fa[REP_M], fb[REP_N];
        load_global(0, 0);
        store_lds(0, 0);
        if (KT > 1) load_global(1, 0);
        __syncthreads();
        load_frags(0, 0, fa, fb);
        for (int kt = 0; kt < KT; ++kt) {
            const int cur = kt & 1;
            if (kt + 1 < KT) {
                store_lds(cur ^ 1, 0);                 /* tile kt+1, loaded during iteration kt-1 */
                __builtin_amdgcn_sched_barrier(0);
                if (kt + 2 < KT) load_global(kt + 2, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int kk = 0; kk < BK; kk += MFMA_K) {
                i32x4 na[REP_M], nb[REP_N];
                if (kk + MFMA_K < BK) {
                    load_frags(cur, kk + MFMA_K, na, nb);
                } else {
                    /* every wavefront has read tile kt and written tile kt+1 */
                    __syncthreads();
                    if (kt + 1 < KT) load_frags(cur ^ 1, 0, na, nb);
                }
#pragma unroll
                for (int i = 0; i < REP_M; ++i)
#pragma unroll
                    for (int j = 0; j < REP_N; ++j)
                        acc[i][j] = MFMA_OP(fa[i], fb[j], acc[i][j]);
                if (kk + MFMA_K < BK || kt + 1 < KT) {
#pragma unroll
                    for (int i = 0; i < REP_M; ++i) fa[i] = na[i];
#pragma unroll
                    for (int j = 0; j < REP_N; ++j) fb[j] = nb[j];
                }
            }
        }
    }
#else
    /* tile t: global -> register set t % PD -> LDS buffer -> MFMA */
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
                /* keep the prefetch at the top of the iteration: without this
                 * fence the scheduler sinks the loads down to their use */
                __builtin_amdgcn_sched_barrier(0);
                compute(cur);
                if (STAGES == 1) __syncthreads();
                if (kt + 1 < KT) store_lds((STAGES == 2) ? (cur ^ 1) : 0, (u + 1) % PD);
                __syncthreads();
            }
        }
    }

#endif
    /* The last MFMA's result registers may not be read for 19 issue slots
     * (16 passes) and the hardware does not enforce it; the compiler's hazard
     * pass can lose a short path through branchy code, so the distance from
     * the main loop to the first accumulator read is explicit. */
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 15\n\ts_nop 3" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

#if WAVES_K > 1
    /* ---- sum the k-groups' partial tiles through LDS ---- */
    __syncthreads();             /* every group has read its last fragments: tile memory is free */
    if (kg > 0) {
        int* red = reinterpret_cast<int*>(smem) + (kg - 1) * (NT * REP_M * REP_N * NACC);
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
        const int* red = reinterpret_cast<const int*>(smem) + (g - 1) * (NT * REP_M * REP_N * NACC);
#pragma unroll
        for (int i = 0; i < REP_M; ++i)
#pragma unroll
            for (int j = 0; j < REP_N; ++j)
#pragma unroll
                for (int v = 0; v < NACC; ++v)
                    acc[i][j][v] += red[((i * REP_N + j) * NACC + v) * NT + tid];
    }
#endif
#if !EARLYST
#pragma unroll
    for (int i = 0; i < REP_M; ++i)
#pragma unroll
        for (int j = 0; j < REP_N; ++j)
            store_block(i, j);
#endif
    CLK_END;
}
