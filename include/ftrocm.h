/*
 * ftrocm.h — C-ABI of libftrocm.so, the device runtime underneath the
 * FlexTensor-compatible scheduler for AMD Instinct MI355X (gfx950).
 *
 * The reference has no native runtime of its own: TVM's runtime plays this
 * role (tvm.build / export_library / load_module / time_evaluator / nd.array).
 * Every entry point below cites the reference call site it stands in for.
 *
 * Conventions
 *   - every function returning int returns 0 on success, non-zero on failure;
 *     ftr_last_error() then yields a thread-local, NUL-terminated message.
 *   - the library owns modules, events and compiled code blobs; the caller
 *     owns every device buffer (plain device pointers) and must keep them
 *     alive until the call (or the stream work it enqueued) has finished.
 *   - no torch types, no C++ types: plain pointers and sizes only.
 *   - a module is not safe to use from two threads at once; distinct modules
 *     are independent.
 */
#ifndef FTROCM_H
#define FTROCM_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FTR_ABI_VERSION 2

/* Return code of the calls that take a deadline when it passes. */
#define FTR_TIMEOUT 2

typedef struct ftr_module *ftr_module_t;

typedef struct ftr_props {
    char name[256];          /* marketing name */
    char arch[64];           /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
    int compute_units;       /* 256 on MI355X */
    int wave_size;           /* 64 */
    int lds_bytes_per_block; /* 163840 on gfx950 */
    int max_threads_per_block;
    int regs_per_block;
    int clock_khz;           /* peak engine clock */
    int mem_clock_khz;
    int mem_bus_bits;
    int l2_bytes;
    size_t hbm_bytes;
} ftr_props_t;

/* One kernel launch: module, geometry, dynamic LDS bytes and the kernel
 * parameters as an array of pointers to each argument value (the layout
 * hipModuleLaunchKernel's kernelParams takes). */
typedef struct ftr_launch_desc {
    ftr_module_t mod;
    unsigned grid[3];   /* workgroups per dimension */
    unsigned block[3];  /* threads per workgroup per dimension */
    unsigned lds_bytes; /* dynamic LDS */
    void **args;
} ftr_launch_desc_t;

/* ABI version of the loaded library (FTR_ABI_VERSION it was built with). */
int ftr_abi_version(void);

/* Thread-local message of the last failing call on this thread. */
const char *ftr_last_error(void);

/* Compile HIP source for `arch` (e.g. "gfx950") with hiprtc into a code
 * object held in host memory. Touches no device, so it can run in worker
 * processes or on a machine without a GPU. `opts` are extra compiler options
 * ("-DNAME=VALUE", ...). On failure the compiler log is in ftr_last_error().
 * Replaces tvm.build (flextensor/measure.py:87, flextensor/scheduler.py:91). */
int ftr_compile_to_code(const char *src, const char *arch,
                        const char *const *opts, int nopts,
                        void **code_out, size_t *size_out);

/* Release a blob returned by ftr_compile_to_code. */
void ftr_code_free(void *code);

/* Load a code object on the current device and resolve `kernel_name`
 * (an extern "C" __global__ symbol). Replaces
 * tvm.runtime.module.load_module (flextensor/measure.py:107). */
int ftr_module_load(const void *code, size_t size, const char *kernel_name,
                    ftr_module_t *out);

/* Compile for the current device's architecture and load in one call.
 * Replaces tvm.build + export_library + load_module
 * (flextensor/measure.py:87-107). */
int ftr_compile(const char *src, const char *kernel_name,
                const char *const *opts, int nopts, ftr_module_t *out);

/* Unload a module. NULL is ignored. */
void ftr_module_free(ftr_module_t mod);

/* Resource usage of the loaded kernel: registers per lane, static LDS bytes,
 * private (spill) bytes per lane, max threads per workgroup. Any out pointer
 * may be NULL. Stands in for the resource check in
 * flextensor/measure.py:8-26 (verify_code). */
int ftr_module_attrs(ftr_module_t mod, int *num_regs, int *static_lds_bytes,
                     int *private_bytes, int *max_threads);

/* Enqueue one launch on `stream` (NULL = the default stream). Asynchronous.
 * Replaces calling the built function, func(*tvm_arys)
 * (flextensor/optimize/common.py:39, README.md:151-158). */
int ftr_launch(ftr_module_t mod, const unsigned grid[3],
               const unsigned block[3], unsigned lds_bytes, void **args,
               void *stream);

/* Enqueue `n` launches in order on `stream`. Asynchronous. */
int ftr_launch_seq(const ftr_launch_desc_t *seq, int n, void *stream);

/* Mean milliseconds per launch: `warmup` untimed launches, then a hipEvent
 * pair around `iters` back-to-back launches on `stream`; synchronises the
 * stream before returning. Replaces
 * func.time_evaluator(entry, ctx, number)(*arys).mean * 1e3
 * (flextensor/measure.py:109-110). */
int ftr_time(ftr_module_t mod, const unsigned grid[3], const unsigned block[3],
             unsigned lds_bytes, void **args, int warmup, int iters,
             void *stream, float *ms_mean);

/* Mean milliseconds per iteration where one iteration is `n_per_iter`
 * launches in order (a multi-kernel plan). `seqs` holds
 * nsets * n_per_iter descriptors; iteration i runs set (i % nsets), so that
 * a caller can rotate through distinct buffers and keep a memory-bound
 * kernel's traffic in HBM rather than in the last-level cache. */
int ftr_time_seq(const ftr_launch_desc_t *seqs, int n_per_iter, int nsets,
                 int warmup, int iters, void *stream, float *ms_mean);

/* ftr_time_seq with a deadline of `timeout_s` seconds (0 = none) over the
 * whole call: the closing event is polled instead of waited for, and when the
 * deadline passes the call returns FTR_TIMEOUT with the work still enqueued
 * (device work cannot be taken back; no process is killed). Stands in for the
 * time limit the reference puts on a candidate by running it in a child
 * process that the parent gives `timeout` seconds
 * (flextensor/measure.py:63-74, flextensor/scheduler.py:742-748). */
int ftr_time_seq_deadline(const ftr_launch_desc_t *seqs, int n_per_iter,
                          int nsets, int warmup, int iters, void *stream,
                          double timeout_s, float *ms_mean);

/* Wait up to `timeout_s` seconds for `stream` to run empty: 0 when it is
 * idle, FTR_TIMEOUT when work is still pending. What a caller does after a
 * timed-out candidate before it measures the next one. */
int ftr_stream_idle(void *stream, double timeout_s);

/* Bytes of the static device workspace ftr_launch_seq_static_ws binds. */
#define FTR_STATIC_WS_BYTES (64u << 20)

/* One workspace argument of a launch sequence: the pointer-sized slot that
 * seq[launch].args[arg] points at receives the device address of bytes
 * [offset, offset + bytes) of the static workspace. offset must be a multiple
 * of 256 and bytes a multiple of 16; with zero != 0 the range is cleared on
 * the stream (by a fill kernel) before the first launch. */
typedef struct ftr_ws_bind {
    int launch;
    int arg;
    size_t offset;
    size_t bytes;
    int zero;
} ftr_ws_bind_t;

/* ftr_launch_seq for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * No counterpart in the reference, whose runtime allocates freely. The
 * workspace arguments named by `binds` (the per-tile slots and arrival
 * counters of a K-streaming plan, which ftr_launch_seq takes as caller-owned
 * buffers) are bound to a fixed FTR_STATIC_WS_BYTES array inside the
 * library's device image; the caller still passes every input and output.
 * Calls hipMalloc/hipFree never; fails with a message when a range does not
 * fit. The array is one per GPU and keeps the previous call's contents: ask
 * for zero where a kernel relies on zeros. Calls that overlap in time on one
 * GPU (two streams, two threads) race on it. The array's address is resolved
 * once per device: at the first ftr_module_load on that device, or, for a
 * device on which no module was loaded through this library yet, at the
 * first call of this entry point. */
int ftr_launch_seq_static_ws(const ftr_launch_desc_t *seq, int n,
                             const ftr_ws_bind_t *binds, int nbinds,
                             void *stream);

/* Properties of device `dev`. Stands in for the tvm device queries in
 * flextensor/measure.py:10-20. */
int ftr_device_props(int dev, ftr_props_t *out);

/* Number of visible devices (0 when there is none or no driver). */
int ftr_device_count(void);

#ifdef __cplusplus
}
#endif
#endif /* FTROCM_H */
