// The single-sweep sampler for small batches: the same kernel as ws_fused.hip with rows split over several workgroups
// (each sweeps a slice of the row; histograms and candidates meet in global memory), a build of its own so that the
// unsplit kernel carries none of it.
#define WS_BLOCK 512
#ifndef WS_KEPT_BUILD  // (the build with the kept-set dump includes this file with both set)
#define WS_KEPT_BUILD false
#define WS_LAUNCH launch_split
#endif
#include <atomic>

#include "ws_sample.h"

namespace ws {

int WS_LAUNCH(hipStream_t stream, const BatchArgs& a, unsigned blocks, unsigned lds_bytes, unsigned lds_limit) {
    // raising the dynamic LDS limit is per function and device, once per process (setting it twice does no harm)
    static std::atomic<uint64_t> attr_set{0};
    int dev = 0;
    if (const hipError_t e = hipGetDevice(&dev); e != hipSuccess) return static_cast<int>(e);
    const uint64_t bit = 1ull << (dev & 63);
    if (!(attr_set.load(std::memory_order_acquire) & bit)) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sample_batch_kernel<true, true, WS_KEPT_BUILD>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_limit));
        if (e != hipSuccess) return static_cast<int>(e);
        attr_set.fetch_or(bit, std::memory_order_release);
    }
    hipLaunchKernelGGL((sample_batch_kernel<true, true, WS_KEPT_BUILD>), dim3(blocks), dim3(WS_BLOCK), lds_bytes, stream, a);
    return static_cast<int>(hipGetLastError());
}

}  // namespace ws
