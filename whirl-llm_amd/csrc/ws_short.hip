// The short-list sampler (ws_short.h), a translation unit of its own: 1024 threads per workgroup; fp32 and bf16 rows,
// with and without an allow mask; the three-pass code of ws_sample.h as a function for the rows it hands back.
#define WS_BLOCK 1024
#include "ws_lds_limit.h"
#include "ws_short.h"

namespace ws {

int prepare_short(unsigned lds_limit) {
    static std::atomic<uint64_t> done{0};
    return raise_lds_limit(done,
                           {reinterpret_cast<const void*>(&short_batch_kernel<0, false>), reinterpret_cast<const void*>(&short_batch_kernel<0, true>),
                            reinterpret_cast<const void*>(&short_batch_kernel<1, false>), reinterpret_cast<const void*>(&short_batch_kernel<1, true>)},
                           lds_limit);
}

int launch_short(hipStream_t stream, const BatchArgs& a, unsigned blocks, unsigned lds_bytes, unsigned lds_limit) {
    if (const int e = prepare_short(lds_limit); e != 0) return e;
    const dim3 g(blocks), b(WS_BLOCK);
    if (a.dtype == 0) {
        if (a.allow) hipLaunchKernelGGL((short_batch_kernel<0, true>), g, b, lds_bytes, stream, a);
        else hipLaunchKernelGGL((short_batch_kernel<0, false>), g, b, lds_bytes, stream, a);
    } else {
        if (a.allow) hipLaunchKernelGGL((short_batch_kernel<1, true>), g, b, lds_bytes, stream, a);
        else hipLaunchKernelGGL((short_batch_kernel<1, false>), g, b, lds_bytes, stream, a);
    }
    return static_cast<int>(hipGetLastError());
}

}  // namespace ws
