// The lean single-sweep sampler (ws_lean.h), a translation unit of its own (fp32 and bf16 rows, with and without an allow
// mask: four kernels): 1024 threads per workgroup, 128 registers a thread, and the three-pass code of ws_sample.h as a function for the rows it hands back.
#define WS_BLOCK 1024
#include "ws_lds_limit.h"
#include "ws_lean.h"

namespace ws {

int prepare_lean(unsigned lds_limit) {
    static std::atomic<uint64_t> done{0};
    return raise_lds_limit(done,
                           {reinterpret_cast<const void*>(&lean_batch_kernel<false, 0>), reinterpret_cast<const void*>(&lean_batch_kernel<true, 0>),
                            reinterpret_cast<const void*>(&lean_batch_kernel<false, 1>), reinterpret_cast<const void*>(&lean_batch_kernel<true, 1>)},
                           lds_limit);
}

int launch_lean(hipStream_t stream, const BatchArgs& a, unsigned rows, unsigned lds_bytes, unsigned lds_limit) {
    if (const int e = prepare_lean(lds_limit); e != 0) return e;
    const dim3 grid(rows), block(WS_BLOCK);
    if (a.dtype == 0) {
        if (a.allow) hipLaunchKernelGGL((lean_batch_kernel<true, 0>), grid, block, lds_bytes, stream, a);
        else hipLaunchKernelGGL((lean_batch_kernel<false, 0>), grid, block, lds_bytes, stream, a);
    } else {
        if (a.allow) hipLaunchKernelGGL((lean_batch_kernel<true, 1>), grid, block, lds_bytes, stream, a);
        else hipLaunchKernelGGL((lean_batch_kernel<false, 1>), grid, block, lds_bytes, stream, a);
    }
    return static_cast<int>(hipGetLastError());
}

}  // namespace ws
