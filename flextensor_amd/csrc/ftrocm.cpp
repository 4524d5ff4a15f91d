// libftrocm.so — device runtime behind the C-ABI declared in include/ftrocm.h.
//
// Host-only C++: hiprtc turns kernel-template source into gfx950 code
// objects, the HIP module API loads and launches them, hipEvents time them.
// It stands where TVM's runtime stands in the reference
// (flextensor/measure.py:77-115: build, export_library, load_module,
// time_evaluator). Nothing here computes on the CPU.

#include "ftrocm.h"
#include "ftrocm_internal.h"

#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

struct ftr_module {
    hipModule_t module;
    hipFunction_t func;
};

namespace {

thread_local std::string g_err;

#define fail ftr_internal_fail

#define FTR_HIP(call)                                                         \
    do {                                                                      \
        hipError_t e_ = (call);                                               \
        if (e_ != hipSuccess) {                                               \
            (void)hipGetLastError(); /* do not leave a sticky error behind */ \
            return fail("%s failed: %s (%d)", #call, hipGetErrorString(e_),   \
                        (int)e_);                                             \
        }                                                                     \
    } while (0)

int launch_one(const ftr_launch_desc_t &d, hipStream_t s) {
    if (ftr_internal_check_desc(&d)) return 1;
    FTR_HIP(hipModuleLaunchKernel(d.mod->func, d.grid[0], d.grid[1], d.grid[2],
                                  d.block[0], d.block[1], d.block[2],
                                  d.lds_bytes, s, d.args, nullptr));
    return 0;
}

}  // namespace

int ftr_internal_check_desc(const ftr_launch_desc_t *d) {
    if (!d->mod) return fail("ftr_launch: null module");
    if (!d->args) return fail("ftr_launch: null argument array");
    for (int i = 0; i < 3; ++i)
        if (d->grid[i] == 0 || d->block[i] == 0)
            return fail("ftr_launch: zero grid/block extent in dim %d", i);
    if ((unsigned long long)d->block[0] * d->block[1] * d->block[2] > 1024ull)
        return fail("ftr_launch: more than 1024 threads per workgroup");
    return 0;
}

int ftr_internal_fail(const char *fmt, ...) {
    char buf[4096];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
    return 1;
}

extern "C" {

int ftr_abi_version(void) { return FTR_ABI_VERSION; }

const char *ftr_last_error(void) { return g_err.c_str(); }

int ftr_compile_to_code(const char *src, const char *arch,
                        const char *const *opts, int nopts, void **code_out,
                        size_t *size_out) {
    if (!src || !arch || !code_out || !size_out)
        return fail("ftr_compile_to_code: null argument");
    if (nopts < 0 || (nopts > 0 && !opts))
        return fail("ftr_compile_to_code: %d options but no option array", nopts);
    for (int i = 0; i < nopts; ++i)
        if (!opts[i]) return fail("ftr_compile_to_code: option %d is null", i);
    *code_out = nullptr;
    *size_out = 0;
    hiprtcProgram prog;
    hiprtcResult r = hiprtcCreateProgram(&prog, src, "ftr_kernel.hip", 0,
                                         nullptr, nullptr);
    if (r != HIPRTC_SUCCESS)
        return fail("hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
    std::string archopt = std::string("--offload-arch=") + arch;
    std::vector<const char *> all;
    all.push_back(archopt.c_str());
    all.push_back("-O3");
    // Packed-fp32 instruction selection is switched off for every kernel.
    all.push_back("-Xclang");
    all.push_back("-target-feature");
    all.push_back("-Xclang");
    all.push_back("-packed-fp32-ops");
    for (int i = 0; i < nopts; ++i) all.push_back(opts[i]);
    r = hiprtcCompileProgram(prog, (int)all.size(), all.data());
    if (r != HIPRTC_SUCCESS) {
        size_t n = 0;
        (void)hiprtcGetProgramLogSize(prog, &n);
        std::string log(n ? n : 1, '\0');
        if (n) (void)hiprtcGetProgramLog(prog, &log[0]);
        (void)hiprtcDestroyProgram(&prog);
        return fail("hiprtc compile failed (%s):\n%.3500s",
                    hiprtcGetErrorString(r), log.c_str());
    }
    size_t n = 0;
    r = hiprtcGetCodeSize(prog, &n);
    if (r != HIPRTC_SUCCESS || n == 0) {
        (void)hiprtcDestroyProgram(&prog);
        return fail("hiprtcGetCodeSize: %s", hiprtcGetErrorString(r));
    }
    void *buf = malloc(n);
    if (!buf) {
        (void)hiprtcDestroyProgram(&prog);
        return fail("out of host memory for %zu-byte code object", n);
    }
    r = hiprtcGetCode(prog, (char *)buf);
    (void)hiprtcDestroyProgram(&prog);
    if (r != HIPRTC_SUCCESS) {
        free(buf);
        return fail("hiprtcGetCode: %s", hiprtcGetErrorString(r));
    }
    *code_out = buf;
    *size_out = n;
    return 0;
}

void ftr_code_free(void *code) { free(code); }

int ftr_module_load(const void *code, size_t size, const char *kernel_name,
                    ftr_module_t *out) {
    if (!code || !size || !kernel_name || !out)
        return fail("ftr_module_load: null argument");
    *out = nullptr;
    hipModule_t m;
    FTR_HIP(hipModuleLoadData(&m, code));
    hipFunction_t f;
    hipError_t e = hipModuleGetFunction(&f, m, kernel_name);
    if (e != hipSuccess) {
        (void)hipModuleUnload(m);
        (void)hipGetLastError();
        return fail("kernel '%s' not found in code object: %s", kernel_name,
                    hipGetErrorString(e));
    }
    // set-up time is also when the static workspace of this device is looked
    // up, so that ftr_launch_seq_static_ws normally has nothing left to resolve.
    // Only that entry point needs the array: a device on which the look-up fails
    // still loads modules, and ftr_launch_seq_static_ws reports the failure.
    (void)ftr_internal_static_ws(nullptr);
    ftr_module *mod = new ftr_module{m, f};
    *out = mod;
    return 0;
}

int ftr_compile(const char *src, const char *kernel_name,
                const char *const *opts, int nopts, ftr_module_t *out) {
    if (!out) return fail("ftr_compile: null out");
    *out = nullptr;
    int dev = 0;
    FTR_HIP(hipGetDevice(&dev));
    hipDeviceProp_t p;
    FTR_HIP(hipGetDeviceProperties(&p, dev));
    std::string arch(p.gcnArchName);
    size_t colon = arch.find(':');
    if (colon != std::string::npos) arch.resize(colon);
    void *code = nullptr;
    size_t size = 0;
    if (ftr_compile_to_code(src, arch.c_str(), opts, nopts, &code, &size))
        return 1;
    int rc = ftr_module_load(code, size, kernel_name, out);
    free(code);
    return rc;
}

void ftr_module_free(ftr_module_t mod) {
    if (!mod) return;
    (void)hipModuleUnload(mod->module);
    delete mod;
}

int ftr_module_attrs(ftr_module_t mod, int *num_regs, int *static_lds_bytes,
                     int *private_bytes, int *max_threads) {
    if (!mod) return fail("ftr_module_attrs: null module");
    int v = 0;
    if (num_regs) {
        FTR_HIP(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_NUM_REGS, mod->func));
        *num_regs = v;
    }
    if (static_lds_bytes) {
        FTR_HIP(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES,
                                    mod->func));
        *static_lds_bytes = v;
    }
    if (private_bytes) {
        FTR_HIP(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES,
                                    mod->func));
        *private_bytes = v;
    }
    if (max_threads) {
        FTR_HIP(hipFuncGetAttribute(
            &v, HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK, mod->func));
        *max_threads = v;
    }
    return 0;
}

int ftr_launch(ftr_module_t mod, const unsigned grid[3],
               const unsigned block[3], unsigned lds_bytes, void **args,
               void *stream) {
    if (!grid || !block) return fail("ftr_launch: null geometry");
    ftr_launch_desc_t d;
    d.mod = mod;
    memcpy(d.grid, grid, sizeof d.grid);
    memcpy(d.block, block, sizeof d.block);
    d.lds_bytes = lds_bytes;
    d.args = args;
    return launch_one(d, (hipStream_t)stream);
}

int ftr_launch_seq(const ftr_launch_desc_t *seq, int n, void *stream) {
    if (!seq || n < 0) return fail("ftr_launch_seq: bad argument");
    for (int i = 0; i < n; ++i)
        if (launch_one(seq[i], (hipStream_t)stream)) return 1;
    return 0;
}

int ftr_time_seq_deadline(const ftr_launch_desc_t *seqs, int n_per_iter,
                          int nsets, int warmup, int iters, void *stream,
                          double timeout_s, float *ms_mean) {
    if (!seqs || !ms_mean || n_per_iter < 1 || nsets < 1 || iters < 1 ||
        warmup < 0 || !(timeout_s >= 0.0))
        return fail("ftr_time_seq: bad argument");
    hipStream_t s = (hipStream_t)stream;
    const auto t_begin = std::chrono::steady_clock::now();
    auto expired = [&]() {
        if (timeout_s <= 0.0) return false;
        std::chrono::duration<double> d = std::chrono::steady_clock::now() - t_begin;
        return d.count() > timeout_s;
    };
    for (int i = 0; i < warmup; ++i) {
        if (ftr_launch_seq(seqs + (size_t)(i % nsets) * n_per_iter, n_per_iter,
                           stream))
            return 1;
        // a candidate far slower than expected shows while the warm-up is
        // still being enqueued (the queue fills and launches block)
        if ((i & 63) == 63 && expired()) {
            fail("timed out after %.3f s (warm-up launch %d of %d)", timeout_s, i + 1, warmup);
            return FTR_TIMEOUT;
        }
    }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    FTR_HIP(hipEventCreate(&e0));
    hipError_t e = hipEventCreate(&e1);
    if (e != hipSuccess) {
        (void)hipEventDestroy(e0);
        return fail("hipEventCreate: %s", hipGetErrorString(e));
    }
    int rc = 0;
    bool late = false;
    float ms = 0.f;
    do {
        if ((e = hipEventRecord(e0, s)) != hipSuccess) break;
        for (int i = 0; i < iters && !rc && !late; ++i) {
            rc = ftr_launch_seq(seqs + (size_t)(i % nsets) * n_per_iter,
                                n_per_iter, stream);
            if ((i & 63) == 63 && expired()) late = true;   // stop enqueueing, too
        }
        if (rc || late) break;
        if ((e = hipEventRecord(e1, s)) != hipSuccess) break;
        if (timeout_s > 0.0) {
            // wait with a deadline: poll the closing event instead of blocking on it. The work
            // stays enqueued when the deadline passes (nothing can take it back); the caller
            // treats the candidate as failed and drains the stream before the next one.
            while ((e = hipEventQuery(e1)) == hipErrorNotReady) {
                if (expired()) {
                    late = true;
                    break;
                }
                std::this_thread::sleep_for(std::chrono::microseconds(50));
            }
            if (late) {
                (void)hipGetLastError();
                e = hipSuccess;
                break;
            }
            if (e != hipSuccess) break;
        } else if ((e = hipEventSynchronize(e1)) != hipSuccess) {
            break;
        }
        e = hipEventElapsedTime(&ms, e0, e1);
    } while (0);
    if (rc) (void)hipStreamSynchronize(s);  // drain what was enqueued before failing
    (void)hipEventDestroy(e0);              // a pending event is released when it completes
    (void)hipEventDestroy(e1);
    if (rc) return 1;
    if (late) {
        fail("timed out after %.3f s (up to %d timed launches enqueued)", timeout_s, iters * n_per_iter);
        return FTR_TIMEOUT;
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail("timing failed: %s (%d)", hipGetErrorString(e), (int)e);
    }
    *ms_mean = ms / (float)iters;
    return 0;
}

int ftr_time_seq(const ftr_launch_desc_t *seqs, int n_per_iter, int nsets,
                 int warmup, int iters, void *stream, float *ms_mean) {
    return ftr_time_seq_deadline(seqs, n_per_iter, nsets, warmup, iters, stream, 0.0, ms_mean);
}

int ftr_stream_idle(void *stream, double timeout_s) {
    const auto t_begin = std::chrono::steady_clock::now();
    for (;;) {
        hipError_t e = hipStreamQuery((hipStream_t)stream);
        if (e == hipSuccess) return 0;
        if (e != hipErrorNotReady) {
            (void)hipGetLastError();
            return fail("hipStreamQuery failed: %s (%d)", hipGetErrorString(e), (int)e);
        }
        std::chrono::duration<double> d = std::chrono::steady_clock::now() - t_begin;
        if (d.count() > timeout_s) {
            (void)hipGetLastError();
            fail("stream still busy after %.3f s", timeout_s);
            return FTR_TIMEOUT;
        }
        std::this_thread::sleep_for(std::chrono::microseconds(100));
    }
}

int ftr_time(ftr_module_t mod, const unsigned grid[3], const unsigned block[3],
             unsigned lds_bytes, void **args, int warmup, int iters,
             void *stream, float *ms_mean) {
    if (!grid || !block) return fail("ftr_time: null geometry");
    ftr_launch_desc_t d;
    d.mod = mod;
    memcpy(d.grid, grid, sizeof d.grid);
    memcpy(d.block, block, sizeof d.block);
    d.lds_bytes = lds_bytes;
    d.args = args;
    return ftr_time_seq(&d, 1, 1, warmup, iters, stream, ms_mean);
}

int ftr_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int ftr_device_props(int dev, ftr_props_t *out) {
    if (!out) return fail("ftr_device_props: null out");
    memset(out, 0, sizeof *out);
    hipDeviceProp_t p;
    FTR_HIP(hipGetDeviceProperties(&p, dev));
    snprintf(out->name, sizeof out->name, "%s", p.name);
    snprintf(out->arch, sizeof out->arch, "%.63s", p.gcnArchName);
    out->compute_units = p.multiProcessorCount;
    out->wave_size = p.warpSize;
    out->lds_bytes_per_block = (int)p.sharedMemPerBlock;
    out->max_threads_per_block = p.maxThreadsPerBlock;
    out->regs_per_block = p.regsPerBlock;
    out->clock_khz = p.clockRate;
    out->mem_clock_khz = p.memoryClockRate;
    out->mem_bus_bits = p.memoryBusWidth;
    out->l2_bytes = p.l2CacheSize;
    out->hbm_bytes = p.totalGlobalMem;
    return 0;
}

}  // extern "C"
