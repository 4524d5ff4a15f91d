// ftr_launch_seq_static_ws — the one entry point of libftrocm.so that
// allocates nothing. It is ftr_launch_seq for plans whose kernels need a
// device workspace (the per-tile slots and arrival counters of balanced K
// streaming): instead of a buffer the caller allocated, the workspace
// arguments are bound to a fixed array that lives in this library's device
// image. For callers that cannot call hipMalloc: code under HIP graph
// capture, tight serving loops, harnesses that forbid allocation.

#include "ftrocm.h"
#include "ftrocm_internal.h"

#include <hip/hip_runtime.h>

#include <cstdint>
#include <mutex>

// Device memory of the workspace. Every GPU the library runs on holds its own
// copy at its own address until the process ends. In host code the name is
// only a handle for hipGetSymbolAddress, never an address to hand to a kernel.
static __device__ __align__(256) unsigned char scratch[FTR_STATIC_WS_BYTES];

namespace {

constexpr int kMaxDevices = 64;
void *g_ws_ptr[kMaxDevices];     // per device: device address of `scratch`
bool g_ws_known[kMaxDevices];
std::mutex g_ws_mutex;

// 16 bytes per lane per step; `n16` 16-byte words starting at the 16-byte aligned `p`
__global__ void ftr_fill_zero16(uint4 *p, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
        p[i] = make_uint4(0u, 0u, 0u, 0u);
}

}  // namespace

int ftr_internal_static_ws(void **ptr_out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return ftr_internal_fail("hipGetDevice failed: %s (%d)", hipGetErrorString(e), (int)e);
    }
    if (dev < 0 || dev >= kMaxDevices)
        return ftr_internal_fail("static workspace: device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    if (!g_ws_known[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            return ftr_internal_fail("hipGetSymbolAddress(scratch) failed on device %d: %s (%d)", dev,
                                     hipGetErrorString(e), (int)e);
        }
        g_ws_ptr[dev] = p;
        g_ws_known[dev] = true;
    }
    if (ptr_out) *ptr_out = g_ws_ptr[dev];
    return 0;
}

extern "C" int ftr_launch_seq_static_ws(const ftr_launch_desc_t *seq, int n, const ftr_ws_bind_t *binds,
                                        int nbinds, void *stream) {
    if (!seq || n < 1 || nbinds < 0 || (nbinds > 0 && !binds))
        return ftr_internal_fail("ftr_launch_seq_static_ws: bad argument");
    // validate everything, launch descriptors included, before anything is enqueued or written
    for (int i = 0; i < n; ++i)
        if (ftr_internal_check_desc(&seq[i])) return 1;
    for (int b = 0; b < nbinds; ++b) {
        const ftr_ws_bind_t &w = binds[b];
        if (w.launch < 0 || w.launch >= n || w.arg < 0)
            return ftr_internal_fail("ftr_launch_seq_static_ws: bind %d names launch %d, argument %d", b,
                                     w.launch, w.arg);
        if (!seq[w.launch].args || !seq[w.launch].args[w.arg])
            return ftr_internal_fail("ftr_launch_seq_static_ws: bind %d: null argument slot", b);
        if (w.offset % 256 != 0 || w.bytes % 16 != 0)
            return ftr_internal_fail("ftr_launch_seq_static_ws: bind %d: offset must be a multiple of 256 "
                                     "and size a multiple of 16 bytes", b);
        if (w.bytes > (size_t)FTR_STATIC_WS_BYTES || w.offset > (size_t)FTR_STATIC_WS_BYTES - w.bytes)
            return ftr_internal_fail("ftr_launch_seq_static_ws: bind %d needs bytes [%zu, %zu) of the static "
                                     "workspace, which holds %zu; use ftr_launch_seq with a caller-owned buffer",
                                     b, w.offset, w.offset + w.bytes, (size_t)FTR_STATIC_WS_BYTES);
        for (int c = 0; c < b; ++c) {
            const ftr_ws_bind_t &o = binds[c];
            const bool same_slot = o.launch == w.launch && o.arg == w.arg;
            const bool overlap = w.offset < o.offset + o.bytes && o.offset < w.offset + w.bytes;
            if (same_slot || (overlap && !(o.offset == w.offset && o.bytes == w.bytes)))
                return ftr_internal_fail("ftr_launch_seq_static_ws: binds %d and %d collide", c, b);
        }
    }
    void *base = nullptr;
    if (ftr_internal_static_ws(&base)) return 1;
    hipStream_t s = (hipStream_t)stream;
    for (int b = 0; b < nbinds; ++b) {
        const ftr_ws_bind_t &w = binds[b];
        unsigned char *p = (unsigned char *)base + w.offset;
        *(void **)seq[w.launch].args[w.arg] = p;
        if (w.zero && w.bytes) {
            // a kernel, not hipMemsetAsync: the caller may be capturing a graph
            const size_t n16 = w.bytes / 16;
            const unsigned blocks = (unsigned)((n16 + 255) / 256 < 1024 ? (n16 + 255) / 256 : 1024);
            hipLaunchKernelGGL(ftr_fill_zero16, dim3(blocks), dim3(256), 0, s, (uint4 *)p, n16);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess)
                return ftr_internal_fail("static workspace clear failed: %s (%d)", hipGetErrorString(e), (int)e);
        }
    }
    return ftr_launch_seq(seq, n, stream);
}
