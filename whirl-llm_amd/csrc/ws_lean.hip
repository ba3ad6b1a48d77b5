// The lean single-sweep sampler (ws_lean.h), a translation unit of its own: 1024 threads per workgroup, 128 registers a
// thread, and the three-pass code of ws_sample.h as a function for the rows it hands back.
#define WS_BLOCK 1024
#include "ws_lds_limit.h"
#include "ws_lean.h"

namespace ws {

int prepare_lean(unsigned lds_limit) {
    static std::atomic<uint64_t> done{0};
    return raise_lds_limit(done, {reinterpret_cast<const void*>(&lean_batch_kernel<false>), reinterpret_cast<const void*>(&lean_batch_kernel<true>)}, lds_limit);
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
