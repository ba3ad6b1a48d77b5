// The fused-sweep instantiation of the batched sampler, compiled with 512 threads per workgroup: one wave64 pair per
// SIMD leaves every thread 256 registers, enough to keep the bin index of its 320 tokens in registers (no scratch).
#define WS_BLOCK 512
#ifndef WS_KEPT_BUILD  // (the build with the kept-set dump includes this file with both set)
#define WS_KEPT_BUILD false
#define WS_LAUNCH launch_fused
#endif
#include <atomic>

#include "ws_sample.h"

namespace ws {

int WS_LAUNCH(hipStream_t stream, const BatchArgs& a, unsigned rows, unsigned lds_bytes, unsigned lds_limit) {
    // raising the dynamic LDS limit is per function and device, once per process (setting it twice does no harm, so two
    // threads that both find the bit clear may both go on)
    static std::atomic<uint64_t> attr_set{0};
    int dev = 0;
    if (const hipError_t e = hipGetDevice(&dev); e != hipSuccess) return static_cast<int>(e);
    const uint64_t bit = 1ull << (dev & 63);
    if (!(attr_set.load(std::memory_order_acquire) & bit)) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sample_batch_kernel<true, false, WS_KEPT_BUILD>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_limit));
        if (e != hipSuccess) return static_cast<int>(e);
        attr_set.fetch_or(bit, std::memory_order_release);
    }
    hipLaunchKernelGGL((sample_batch_kernel<true, false, WS_KEPT_BUILD>), dim3(rows), dim3(WS_BLOCK), lds_bytes, stream, a);
    return static_cast<int>(hipGetLastError());
}

}  // namespace ws
