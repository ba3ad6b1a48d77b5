// The single-sweep sampler for small batches: the same kernel as ws_fused.hip with rows split over several workgroups
// (each sweeps a slice of the row; histograms and candidates meet in global memory), a build of its own so that the
// unsplit kernel carries none of it.
#define WS_BLOCK 512
#ifndef WS_KEPT_BUILD  // (the build with the kept-set dump includes this file with both set)
#define WS_KEPT_BUILD false
#define WS_LAUNCH launch_split
#define WS_PREPARE prepare_split
#endif
#include "ws_lds_limit.h"
#include "ws_sample.h"

namespace ws {

int WS_PREPARE(unsigned lds_limit) {
    static std::atomic<uint64_t> done{0};
    return raise_lds_limit(done, {reinterpret_cast<const void*>(&sample_batch_kernel<true, true, WS_KEPT_BUILD>)}, lds_limit);
}

int WS_LAUNCH(hipStream_t stream, const BatchArgs& a, unsigned blocks, unsigned lds_bytes, unsigned lds_limit) {
    if (const int e = WS_PREPARE(lds_limit); e != 0) return e;
    hipLaunchKernelGGL((sample_batch_kernel<true, true, WS_KEPT_BUILD>), dim3(blocks), dim3(WS_BLOCK), lds_bytes, stream, a);
    return static_cast<int>(hipGetLastError());
}

}  // namespace ws
