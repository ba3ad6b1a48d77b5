// The fused-sweep instantiation of the batched sampler, compiled with 512 threads per workgroup: one wave64 pair per
// SIMD leaves every thread 256 registers, enough to keep the bin index of its 320 tokens in registers (no scratch).
#define WS_BLOCK 512
#include "ws_sample.h"

namespace ws {

int launch_fused(hipStream_t stream, const BatchArgs& a, unsigned rows, unsigned lds_bytes, unsigned lds_limit) {
    static bool attr_set = false;  // raising the dynamic LDS limit is per function, once per process
    if (!attr_set) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sample_batch_kernel<true>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_limit));
        if (e != hipSuccess) return static_cast<int>(e);
        attr_set = true;
    }
    hipLaunchKernelGGL(sample_batch_kernel<true>, dim3(rows), dim3(WS_BLOCK), lds_bytes, stream, a);
    return static_cast<int>(hipGetLastError());
}

}  // namespace ws
