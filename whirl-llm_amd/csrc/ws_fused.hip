// The fused-sweep instantiation of the batched sampler, compiled with 512 threads per workgroup: one wave64 pair per
// SIMD leaves every thread 256 registers, enough to keep the bin index of its 320 tokens in registers (no scratch).
#define WS_BLOCK 512
#ifndef WS_KEPT_BUILD  // (the build with the kept-set dump includes this file with both set)
#define WS_KEPT_BUILD false
#define WS_LAUNCH launch_fused
#define WS_PREPARE prepare_fused
#endif
#include "ws_lds_limit.h"
#include "ws_sample.h"

namespace ws {

int WS_PREPARE(unsigned lds_limit) {
    static std::atomic<uint64_t> done{0};
    return raise_lds_limit(done, {reinterpret_cast<const void*>(&sample_batch_kernel<true, false, WS_KEPT_BUILD>)}, lds_limit);
}

int WS_LAUNCH(hipStream_t stream, const BatchArgs& a, unsigned rows, unsigned lds_bytes, unsigned lds_limit) {
    if (const int e = WS_PREPARE(lds_limit); e != 0) return e;
    hipLaunchKernelGGL((sample_batch_kernel<true, false, WS_KEPT_BUILD>), dim3(rows), dim3(WS_BLOCK), lds_bytes, stream, a);
    return static_cast<int>(hipGetLastError());
}

}  // namespace ws
