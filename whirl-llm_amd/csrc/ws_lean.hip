// The lean single-sweep sampler (ws_lean.h), a translation unit of its own: 1024 threads per workgroup, 128 registers a
// thread, and the three-pass code of ws_sample.h as a function for the rows it hands back.
#define WS_BLOCK 1024
#include <atomic>

#include "ws_lean.h"

namespace ws {

int prepare_lean(unsigned lds_limit) {
    // raising the dynamic LDS limit is per function and device, once per process (setting it twice does no harm)
    static std::atomic<uint64_t> attr_set{0};
    int dev = 0;
    if (const hipError_t e = hipGetDevice(&dev); e != hipSuccess) return static_cast<int>(e);
    const uint64_t bit = 1ull << (dev & 63);
    if (!(attr_set.load(std::memory_order_acquire) & bit)) {
        for (const void* f : {reinterpret_cast<const void*>(&lean_batch_kernel<false>), reinterpret_cast<const void*>(&lean_batch_kernel<true>)}) {
            const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_limit));
            if (e != hipSuccess) return static_cast<int>(e);
        }
        attr_set.fetch_or(bit, std::memory_order_release);
    }
    return 0;
}

int launch_lean(hipStream_t stream, const BatchArgs& a, unsigned rows, unsigned lds_bytes, unsigned lds_limit) {
    if (const int e = prepare_lean(lds_limit); e != 0) return e;
#ifndef WS_LEAN_UNMASKED_ONLY
    if (a.allow) hipLaunchKernelGGL(lean_batch_kernel<true>, dim3(rows), dim3(WS_BLOCK), lds_bytes, stream, a);
    else
#endif
        hipLaunchKernelGGL(lean_batch_kernel<false>, dim3(rows), dim3(WS_BLOCK), lds_bytes, stream, a);
    return static_cast<int>(hipGetLastError());
}

}  // namespace ws
