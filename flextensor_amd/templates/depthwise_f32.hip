// Direct depthwise conv2d NCHW fp32 kernel template for gfx950, hiprtc-compiled.
//
//   O[b][c][h][w] = sum_{r,s} P[b][c / FACT][h*STRH + r*DILH][w*STRW + s*DILW]
//                             * Wt[c / FACT][c % FACT][r][s]
// with P the zero-padded input (padding folded into load predicates), as in
// flextensor/nn/ops.py:622-678 (weight layout [C][FACT][R][S], ops.py:630).
//
// The operator moves ~2 bytes per flop: it is bound by HBM bandwidth, not by
// arithmetic, so there is no matrix-core path. Each lane owns a TH x TW patch
// of one output plane; consecutive lanes own consecutive patches along W, then
// H, then planes, so global reads and writes of a wavefront are contiguous.
//
// Knobs (-D constants): NT threads per workgroup, TH x TW outputs per lane,
// NT_STORE (1: non-temporal stores for the output), SHFL (1: the one-column
// halo left and right of a lane's four columns comes from the neighbouring
// lanes through DPP wavefront shifts instead of two more global loads; each
// wavefront then uses a multiple of TILES_W lanes so that neighbours along W
// are always in the same wavefront), MFUSE (1: with FACT > 1 kernels per input
// channel a lane loads its input patch once and computes the patch of all
// FACT output planes from it, instead of one lane per output plane).
// LDSP > 0 selects the plane-staged variant instead: a workgroup streams LDSP
// whole planes into LDS with 128-bit loads in pure copy order (every input
// element is fetched once, no halo re-reads), computes from LDS, where a zero
// border stands for the padding, and writes the outputs in the same order.
// It needs a same-size 3x3 / stride 1 / dilation 1 / padding 1 layer with
// FACT == 1 and rows that are multiples of four floats.
// WX > 0 selects the row-exchange variant for the same kind of layer: a
// wavefront owns WXR * WX consecutive rows of one plane (WXR whole rows per
// load instruction, WX 16-byte chunks per lane), loads each chunk once, in
// copy order, all loads issued before anything else, and passes the rows
// above and below between lanes through a wavefront-private LDS window: no
// barrier, no halo re-reads from memory except the one row either side of
// the span; the padding rows arrive as the zeros of out-of-range loads.
// HAS_BIAS = 1 adds a per-output-channel bias (ops.py:673-677) to every
// result in the store, from a fourth argument; all three variants take it.
// Shape constants: CB batch, CC channels, CH x CW input, CR x CS kernel,
// STRH/STRW, PADH/PADW, DILH/DILW (rows / columns), FACT, CP x CQ output.

/* Constants arrive as -DFT_<NAME>=value: single-letter macros on the command line
 * would be visible to (and break) the runtime-compilation built-in headers. */
#define NT FT_NT
#define TH FT_TH
#define TW FT_TW
#define NT_STORE FT_NT_STORE
#define SHFL FT_SHFL
#ifdef FT_NT_LOAD
#define NT_LOAD FT_NT_LOAD
#else
#define NT_LOAD 0
#endif
#ifdef FT_IPL
#define IPL FT_IPL        /* patches per lane */
#else
#define IPL 1
#endif
#ifdef FT_LDSP
#define LDSP FT_LDSP
#else
#define LDSP 0
#endif
#ifdef FT_WX
#define WX FT_WX          /* chunks per lane of the row-exchange variant */
#else
#define WX 0
#endif
#ifdef FT_MFUSE
#define MFUSE FT_MFUSE    /* a lane computes all FACT output planes of its input patch */
#else
#define MFUSE 0
#endif
#ifdef FT_HAS_BIAS
#define HAS_BIAS FT_HAS_BIAS
#else
#define HAS_BIAS 0
#endif
#if HAS_BIAS
#define BIAS_PARAM , const float* __restrict__ Bs
#else
#define BIAS_PARAM
#endif
#define CB FT_CB
#define CC FT_CC
#define CH FT_CH
#define CW FT_CW
#define CR FT_CR
#define CS FT_CS
#define STRH FT_STRH
#define STRW FT_STRW
#define PADH FT_PADH
#define PADW FT_PADW
#define DILH FT_DILH
#define DILW FT_DILW
#define FACT FT_FACT
#define CP FT_CP
#define CQ FT_CQ

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

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

#define PLANES (CB * CC * FACT)
#define FM (MFUSE ? FACT : 1)            /* output planes per lane patch */
#define TILES_H ((CP + TH - 1) / TH)
#define TILES_W ((CQ + TW - 1) / TW)
#define ITEMS (PLANES / FM * TILES_H * TILES_W)
#define IH_T ((TH - 1) * STRH + (CR - 1) * DILH + 1)
#define IW_T ((TW - 1) * STRW + (CS - 1) * DILW + 1)

/* 128-bit path: a convolution with stride 1 or 2 along W whose output rows
 * are 1/STRW of the input rows and whose rows keep 16-byte alignment; the
 * 4 * STRW input columns from the patch's first output column on come in as
 * STRW vectors. Of a ragged last patch (CQ % 4 != 0) they run into the next
 * row. The last stored output column, CQ - 1, reads up to input column
 * CW - STRW + (CS - 1) * DILW - PADW: when that stays below CW the elements
 * from the next row only feed outputs that are not stored; otherwise columns
 * CW and beyond are padding that a stored output does read, and every vector
 * element whose column is not below CW is replaced by zero (VEC_CLIP). */
#if (TW == 4) && (STRW <= 2) && (CW % 4 == 0) && (CQ * STRW == CW) && (PADW + 4 * STRW <= IW_T)
#define VEC_IN 1
#else
#define VEC_IN 0
#endif
#define VEC_CLIP (VEC_IN && (CQ % 4 != 0) && ((CS - 1) * DILW - PADW >= STRW))
#define NVEC STRW
#if (TW == 4) && (CQ % 4 == 0)
#define VEC_OUT 1
#else
#define VEC_OUT 0
#endif
#if SHFL
#if !(VEC_IN && STRW == 1 && CS == 3 && DILW == 1 && PADW == 1 && TILES_W <= 64)
#error "SHFL needs the 128-bit input path with a 3-wide kernel, dilation 1, padding 1"
#endif
#define LPW ((64 / TILES_W) * TILES_W)   /* lanes of a wavefront that carry work */
#else
#define LPW 64
#endif

#if LDSP > 0
#if !(STRH == 1 && STRW == 1 && DILH == 1 && DILW == 1 && CR == 3 && CS == 3 && PADH == 1 && PADW == 1 && CP == CH && CQ == CW && CW % 4 == 0 && FACT == 1)
#error "the plane-staged variant needs a same-size 3x3 stride-1 pad-1 layer, FACT 1, CW % 4 == 0"
#endif
#define RS (CW + 8)                  /* LDS row: 4 zero floats, CW data, 4 zero floats */
#define PS ((CH + 2) * RS)           /* plane: zero row, CH rows, zero row */
#define Q4 (CW / 4)                  /* 128-bit chunks per row */
#define PLANE4 (CH * Q4)             /* ... per plane */
#define BORDER4 (2 * (RS / 4) + 2 * CH)   /* border chunks per plane: two rows + two per data row */

extern "C" __global__ __launch_bounds__(NT)
void depthwise_f32(const float* __restrict__ X, const float* __restrict__ Wt,
                   float* __restrict__ O BIAS_PARAM CLK_PARAM)
{
    CLK_BEGIN
    __shared__ __attribute__((aligned(16))) float sx[LDSP * PS];
    __shared__ __attribute__((aligned(16))) float sw[LDSP * 12];     /* 3 taps + 1 pad per kernel row */
    const int tid = threadIdx.x;
    const int p0 = blockIdx.x * LDSP;
    const f32x4 zero = (f32x4)(0.0f);
    /* ---- borders (the padding) ---------------------------------------- */
    for (int i = tid; i < LDSP * BORDER4; i += NT) {
        const int pl = i / BORDER4;
        const int q = i % BORDER4;
        int off;
        if (q < RS / 4) off = q * 4;                                   /* top row */
        else if (q < 2 * (RS / 4)) off = (CH + 1) * RS + (q - RS / 4) * 4;   /* bottom row */
        else {
            const int k = q - 2 * (RS / 4);                            /* left / right of a data row */
            off = (k / 2 + 1) * RS + ((k & 1) ? (CW + 4) : 0);
        }
        *reinterpret_cast<f32x4*>(&sx[pl * PS + off]) = zero;
    }
    /* ---- weights: [plane][r][s] -> [plane][r][4] ------------------------ */
    for (int i = tid; i < LDSP * 9; i += NT) {
        const int pl = i / 9, k = i % 9;
        const int plane = p0 + pl;
        sw[pl * 12 + (k / 3) * 4 + (k % 3)] = (plane < PLANES) ? Wt[(size_t)(plane % (CC * FACT)) * 9 + k] : 0.0f;   /* kernels repeat per batch entry */
    }
    /* ---- planes, in copy order ------------------------------------------ */
    const f32x4* X4 = reinterpret_cast<const f32x4*>(X);
    for (int i = tid; i < LDSP * PLANE4; i += NT) {
        const int pl = i / PLANE4;
        const int rem = i % PLANE4;
        const int plane = p0 + pl;
        f32x4 v = zero;
        if (plane < PLANES) v = NT_LOAD ? __builtin_nontemporal_load(&X4[(size_t)plane * PLANE4 + rem])
                                        : X4[(size_t)plane * PLANE4 + rem];
        *reinterpret_cast<f32x4*>(&sx[pl * PS + (rem / Q4 + 1) * RS + 4 + (rem % Q4) * 4]) = v;
    }
    __syncthreads();
    /* ---- four outputs per item, same order ------------------------------ */
    f32x4* O4 = reinterpret_cast<f32x4*>(O);
    for (int i = tid; i < LDSP * PLANE4; i += NT) {
        const int pl = i / PLANE4;
        const int rem = i % PLANE4;
        const int plane = p0 + pl;
        if (plane >= PLANES) break;
        const float* base = &sx[pl * PS + (rem / Q4) * RS + 4 + (rem % Q4) * 4];   /* input row of tap r = 0 */
        f32x4 acc = zero;
#pragma unroll
        for (int r = 0; r < 3; ++r) {
            const f32x4 w = *reinterpret_cast<const f32x4*>(&sw[pl * 12 + r * 4]);
            const f32x4 m = *reinterpret_cast<const f32x4*>(base + r * RS);
            const float l = base[r * RS - 1];
            const float g = base[r * RS + 4];
            const float in[6] = {l, m[0], m[1], m[2], m[3], g};
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int t = 0; t < 3; ++t)
                    acc[j] += in[j + t] * w[t];
        }
#if HAS_BIAS
        acc += Bs[plane % (CC * FACT)];
#endif
#if NT_STORE
        __builtin_nontemporal_store(acc, &O4[(size_t)plane * PLANE4 + rem]);
#else
        O4[(size_t)plane * PLANE4 + rem] = acc;
#endif
    }
    CLK_END;
}
#elif WX > 0
#if !(STRH == 1 && STRW == 1 && DILH == 1 && DILW == 1 && CR == 3 && CS == 3 && PADH == 1 && PADW == 1 && CP == CH && CQ == CW && CW % 4 == 0 && FACT == 1)
#error "the row-exchange variant needs a same-size 3x3 stride-1 pad-1 layer, FACT 1, CW % 4 == 0"
#endif
#define Q4 (CW / 4)                  /* 128-bit chunks per row */
#define PLANE4 (CH * Q4)             /* ... per plane */
#define NCH (PLANES * PLANE4)        /* ... of the tensor */
#define RPI FT_WXR                   /* whole rows one load instruction of a wavefront covers */
#define LPW (RPI * Q4)               /* lanes that carry work */
#define ROWS (RPI * WX)              /* rows one wavefront owns */
#define SPP ((CH + ROWS - 1) / ROWS) /* wavefronts per plane */
#define WIN ((ROWS + 2) * Q4)        /* chunks of a wavefront's LDS window: row above, rows, row below */
#if LPW > 64 || LPW < 1 || 2 * Q4 > 64
#error "row exchange: whole rows per instruction, rows of at most 128 floats"
#endif
#define OOB 0x80000000u
#define X_BYTES (NCH * 16)
#define LD_AUX (NT_LOAD ? 2 : 0)     /* bit 1 of the cache policy operand: non-temporal */
#define ST_AUX (NT_STORE ? 2 : 0)

extern "C" __global__ __launch_bounds__(NT)
void depthwise_f32(const float* __restrict__ X, const float* __restrict__ Wt,
                   float* __restrict__ O BIAS_PARAM CLK_PARAM)
{
    CLK_BEGIN
    /* window chunk ro * Q4 + col of a wavefront holds (row r0 - 1 + ro, chunk col) of its plane.
     * Idle lanes (LPW .. 63) read the chunk their own lane number points at, like the busy ones:
     * 64 consecutive chunks per read, which the LDS serves without a bank conflict (an idle lane
     * parked on one fixed chunk shares its banks with a busy lane of the same pass). What they
     * read, from the next wavefront's window or the slack behind the last one, is never used. */
    __shared__ __attribute__((aligned(16))) float sx[((NT / 64) * WIN + 64) * 4];
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(X), 0, X_BYTES, 0x00020000);
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(O, 0, X_BYTES, 0x00020000);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int wid = blockIdx.x * (NT / 64) + wave;              /* wavefront-uniform from here on */
    const int plane = wid / SPP;
    const int r0 = (wid - plane * SPP) * ROWS;                  /* first row of the span */
    const int lr = lane / Q4, col = lane - lr * Q4;
    float* win = &sx[wave * WIN * 4];
    const bool plane_ok = plane < PLANES;

    /* ---- every load first: the rows in copy order, then the rows above and below ---- */
    f32x4 v[WX];
    unsigned vo[WX];
#pragma unroll
    for (int i = 0; i < WX; ++i) {
        const int row = r0 + i * RPI + lr;
        const bool ok = plane_ok && lane < LPW && row < CH;
        vo[i] = ok ? (unsigned)(plane * PLANE4 + row * Q4 + col) * 16u : OOB;
        v[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, (int)vo[i], 0, LD_AUX));
    }
    /* lanes 0 .. Q4-1 fetch the row above the span, the next Q4 lanes the row below; rows
     * outside the plane are the padding and read as zero, like everything an idle lane asks for */
    const int hrow = lane < Q4 ? r0 - 1 : r0 + ROWS;
    const int hcol = lane < Q4 ? lane : lane - Q4;
    const bool hok = plane_ok && lane < 2 * Q4 && hrow >= 0 && hrow < CH;
    const f32x4 hv = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
        rx, (int)(hok ? (unsigned)(plane * PLANE4 + hrow * Q4 + hcol) * 16u : OOB), 0, LD_AUX));
    /* the plane's kernel: wavefront-uniform, so scalar loads */
    const int ch = __builtin_amdgcn_readfirstlane(plane_ok ? plane % CC : 0);     /* kernels repeat per batch entry */
    float w[9];
#pragma unroll
    for (int t = 0; t < 9; ++t)
        w[t] = Wt[ch * 9 + t];
#if HAS_BIAS
    const float bias = Bs[ch];
#endif

    /* ---- rows change lanes through the window -------------------------------- */
    if (lane < LPW) {
#pragma unroll
        for (int i = 0; i < WX; ++i)
            *reinterpret_cast<f32x4*>(&win[((1 + i * RPI) * Q4 + lane) * 4]) = v[i];
    }
    if (lane < 2 * Q4)
        *reinterpret_cast<f32x4*>(&win[(lane < Q4 ? lane : (ROWS + 1) * Q4 + lane - Q4) * 4]) = hv;
    /* LDS operations of one wavefront complete in order; the fences keep the compiler from
     * moving the reads below above the writes of the other lanes */
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    const bool left = col == 0, right = col == Q4 - 1;
#pragma unroll
    for (int i = 0; i < WX; ++i) {
        const float* mid = &win[((1 + i * RPI) * Q4 + lane) * 4];
        f32x4 acc = (f32x4)(0.0f);
#pragma unroll
        for (int r = 0; r < 3; ++r) {
            const float* base = mid + (r - 1) * Q4 * 4;
            const f32x4 m = r == 1 ? v[i] : *reinterpret_cast<const f32x4*>(base);
            /* the columns left and right of the four come from the neighbouring lanes' vectors
             * (DPP wavefront shifts by one lane); at the ends of a row they are the padding */
            /* (both shifts run in every lane, outside the selects: a lane switched off by a
             * branch could not be read by its neighbour) */
            const int from_below = __builtin_amdgcn_update_dpp(0, __float_as_int(m[3]), 0x138, 0xf, 0xf, false);
            const int from_above = __builtin_amdgcn_update_dpp(0, __float_as_int(m[0]), 0x130, 0xf, 0xf, false);
            const float lf = left ? 0.0f : __int_as_float(from_below);
            const float rt = right ? 0.0f : __int_as_float(from_above);
            const float in[6] = {lf, m[0], m[1], m[2], m[3], rt};
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int t = 0; t < 3; ++t)
                    acc[c] += in[c + t] * w[r * 3 + t];
        }
#if HAS_BIAS
        acc += bias;                     /* FACT == 1: the plane's channel is its output channel */
#endif
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc), ro, (int)vo[i], 0, ST_AUX);
    }
    CLK_END;
}
#else
/* Every global access of the direct kernel is a raw buffer access: an
 * element that must read as zero (padding row or column, idle lane) or must
 * not be written gets an offset beyond the buffer, for which a load returns 0
 * and a store is dropped by the hardware. Nothing branches, so the row loads
 * of a patch are all issued back to back and their round trips overlap. */
#define OOB 0x80000000u
#define X_BYTES (CB * CC * CH * CW * 4)
#define W_BYTES (CC * FACT * CR * CS * 4)
#define O_BYTES (CB * CC * FACT * CP * CQ * 4)
#define LD_AUX (NT_LOAD ? 2 : 0)     /* bit 1 of the cache policy operand: non-temporal */
#define ST_AUX (NT_STORE ? 2 : 0)

extern "C" __global__ __launch_bounds__(NT)
void depthwise_f32(const float* __restrict__ X, const float* __restrict__ Wt,
                   float* __restrict__ O BIAS_PARAM CLK_PARAM)
{
    CLK_BEGIN
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(X), 0, X_BYTES, 0x00020000);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(Wt), 0, W_BYTES, 0x00020000);
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(O, 0, O_BYTES, 0x00020000);
#if HAS_BIAS
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(Bs), 0, CC * FACT * 4, 0x00020000);
    float bias[IPL][FM];
#endif

    /* A lane works on IPL patches, NT lanes (LPW per wavefront) apart, so that a
     * workgroup covers one contiguous run of IPL * (lanes that carry work)
     * patches. Everything a patch needs is requested first, for all IPL
     * patches (phase 1); the arithmetic and the stores follow (phase 2): a
     * lane keeps IPL * (IH_T + taps) loads in flight, and fewer, longer-lived
     * wavefronts move the same bytes. */
    bool live[IPL];
    int tw[IPL], ovo[IPL], oh0[IPL];
    float wreg[IPL][FM][CR][CS];
#if (SHFL || VEC_IN)
    f32x4 rows[IPL][IH_T][NVEC];
#if !SHFL
    float halo[IPL][IH_T][IW_T];
#endif
#else
    float in_all[IPL][IH_T][IW_T];
#endif

#pragma unroll
    for (int k = 0; k < IPL; ++k) {
#if SHFL
        const int lane = threadIdx.x & 63;
        const int gid = (((blockIdx.x * IPL + k) * NT + threadIdx.x) >> 6) * LPW + lane;
        /* idle lanes stay alive (DPP reads their registers) but load and store nothing */
        live[k] = (lane < LPW) && (gid < ITEMS);
#else
        const int gid = (blockIdx.x * IPL + k) * NT + threadIdx.x;
        live[k] = gid < ITEMS;
#endif
        tw[k] = gid % TILES_W;
        const int th = (gid / TILES_W) % TILES_H;
        const int plane = gid / (TILES_W * TILES_H);
#if MFUSE
        /* plane counts input planes; its output planes are plane * FACT .. plane * FACT + FACT - 1 */
        const int co = (plane % CC) * FACT;
        const int xplane = plane * (CH * CW);
#else
        const int b = plane / (CC * FACT);
        const int co = plane % (CC * FACT);
        const int ci = co / FACT;
        const int xplane = (b * CC + ci) * (CH * CW);      /* first element of the input plane */
#endif
        oh0[k] = th * TH;
        const int ow0 = tw[k] * TW;
        const int ih0 = oh0[k] * STRH - PADH;
        const int iw0 = ow0 * STRW - PADW;
        ovo[k] = plane * FM * (CP * CQ) + oh0[k] * CQ + ow0;     /* first output element of the patch */
#pragma unroll
        for (int m = 0; m < FM; ++m) {
            /* the kernel's CR*CS taps: 128-bit loads (dword-aligned is enough for buffer loads) and a tail */
            const unsigned wo = live[k] ? (unsigned)((co + m) * (CR * CS)) * 4u : OOB;
#if HAS_BIAS
            bias[k][m] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                rb, (int)(live[k] ? (unsigned)(co + m) * 4u : OOB), 0, 0));
#endif
            float wflat[(CR * CS + 3) / 4 * 4];
#pragma unroll
            for (int t = 0; t + 4 <= CR * CS; t += 4) {
                const f32x4 v = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, (int)wo, t * 4, 0));
                wflat[t] = v[0]; wflat[t + 1] = v[1]; wflat[t + 2] = v[2]; wflat[t + 3] = v[3];
            }
#pragma unroll
            for (int t = (CR * CS) / 4 * 4; t < CR * CS; ++t)
                wflat[t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rw, (int)wo, t * 4, 0));
#pragma unroll
            for (int r = 0; r < CR; ++r)
#pragma unroll
                for (int s = 0; s < CS; ++s)
                    wreg[k][m][r][s] = wflat[r * CS + s];
        }
        /* one element of input row ih (any int), column iw (any int); zero outside the image */
        auto load1 = [&](int ih, int iw) -> float {
            const bool ok = live[k] && (unsigned)ih < (unsigned)CH && (unsigned)iw < (unsigned)CW;
            const unsigned vo = ok ? (unsigned)(xplane + ih * CW + iw) * 4u : OOB;
            return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rx, (int)vo, 0, LD_AUX));
        };
#if (SHFL || VEC_IN)
#pragma unroll
        for (int y = 0; y < IH_T; ++y) {
            /* the 4 * STRW centre columns of input row ih0 + y */
            const int ih = ih0 + y;
            const bool row_ok = live[k] && (unsigned)ih < (unsigned)CH;
            const unsigned vo = row_ok ? (unsigned)(xplane + ih * CW + ow0 * STRW) * 4u : OOB;
#pragma unroll
            for (int v = 0; v < NVEC; ++v)
                rows[k][y][v] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, (int)vo, v * 16, LD_AUX));
        }
#if !SHFL
        /* the halo columns left and right of the centre vectors */
#pragma unroll
        for (int y = 0; y < IH_T; ++y)
#pragma unroll
            for (int j = 0; j < IW_T; ++j)
                if (j < PADW || j >= PADW + 4 * NVEC) halo[k][y][j] = load1(ih0 + y, iw0 + j);
#endif
#else
#pragma unroll
        for (int y = 0; y < IH_T; ++y)
#pragma unroll
            for (int j = 0; j < IW_T; ++j) in_all[k][y][j] = load1(ih0 + y, iw0 + j);
#endif
    }

#pragma unroll
    for (int k = 0; k < IPL; ++k)
#pragma unroll
    for (int m = 0; m < FM; ++m) {
        float acc[TH][TW];
#pragma unroll
        for (int i = 0; i < TH; ++i)
#pragma unroll
            for (int j = 0; j < TW; ++j)
                acc[i][j] = 0.0f;
#pragma unroll
        for (int y = 0; y < IH_T; ++y) {
            float in[IW_T];
#if SHFL
            {
                const f32x4 v = rows[k][y][0];
                /* column ow0-1 is the last column of the lane below, column ow0+4
                 * the first column of the lane above; image borders read zero */
                const float v0 = v[0], v3 = v[3];
                const int lft = __builtin_amdgcn_update_dpp(0, __float_as_int(v3), 0x138, 0xf, 0xf, false);
                const int rgt = __builtin_amdgcn_update_dpp(0, __float_as_int(v0), 0x130, 0xf, 0xf, false);
                in[0] = (tw[k] > 0) ? __int_as_float(lft) : 0.0f;
                in[1] = v[0]; in[2] = v[1]; in[3] = v[2]; in[4] = v[3];
                in[5] = (tw[k] < TILES_W - 1) ? __int_as_float(rgt) : 0.0f;
            }
#elif VEC_IN
            {
#pragma unroll
                for (int j = 0; j < IW_T; ++j) {
                    in[j] = (j >= PADW && j < PADW + 4 * NVEC) ? rows[k][y][((j - PADW) >> 2) % NVEC][(j - PADW) & 3]
                                                               : halo[k][y][j];
#if VEC_CLIP
                    /* a ragged last patch: vector elements beyond the row's end are the right padding */
                    if (j >= PADW && j < PADW + 4 * NVEC && tw[k] * (TW * STRW) + (j - PADW) >= CW) in[j] = 0.0f;
#endif
                }
            }
#else
#pragma unroll
            for (int j = 0; j < IW_T; ++j) in[j] = in_all[k][y][j];
#endif
            /* input row y feeds output row i through tap r when y == i*STRH + r*DILH */
#pragma unroll
            for (int i = 0; i < TH; ++i) {
#pragma unroll
                for (int r = 0; r < CR; ++r) {
                    if (y == i * STRH + r * DILH) {
#pragma unroll
                        for (int j = 0; j < TW; ++j)
#pragma unroll
                            for (int s = 0; s < CS; ++s)
                                acc[i][j] += in[j * STRW + s * DILW] * wreg[k][m][r][s];
                    }
                }
            }
        }
        /* stores behind every load of the kernel: vector memory operations retire in issue
         * order, so a load issued behind a store would have to wait for the store's round trip */
#pragma unroll
        for (int i = 0; i < TH; ++i) {
            const bool row_ok = live[k] && (CP % TH == 0 || oh0[k] + i < CP);
#if HAS_BIAS
#pragma unroll
            for (int j = 0; j < TW; ++j) acc[i][j] += bias[k][m];
#endif
#if VEC_OUT
            f32x4 v;
            v[0] = acc[i][0]; v[1] = acc[i][1]; v[2] = acc[i][2]; v[3] = acc[i][3];
            const unsigned vo = row_ok ? (unsigned)(ovo[k] + m * (CP * CQ) + i * CQ) * 4u : OOB;
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), ro, (int)vo, 0, ST_AUX);
#else
#pragma unroll
            for (int j = 0; j < TW; ++j) {
                const bool ok = row_ok && (CQ % TW == 0 || tw[k] * TW + j < CQ);
                const unsigned vo = ok ? (unsigned)(ovo[k] + m * (CP * CQ) + i * CQ + j) * 4u : OOB;
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, acc[i][j]), ro, (int)vo, 0, ST_AUX);
            }
#endif
        }
    }
    CLK_END;
}
#endif
