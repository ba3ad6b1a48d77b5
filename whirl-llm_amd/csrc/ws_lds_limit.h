// Raising a kernel's dynamic LDS limit above the default 64 KiB: per function and device, once per process. Shared by
// the translation units that launch such kernels; ws_probe() calls every one of the prepare_* functions built on this,
// so that a launch under stream capture finds nothing left to set.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <initializer_list>

namespace ws {

// `done`: one bit per device (setting the attribute twice does no harm, so two threads that both find the bit clear may
// both go on). Returns 0 or the hipError_t.
inline int raise_lds_limit(std::atomic<uint64_t>& done, std::initializer_list<const void*> kernels, unsigned lds_limit) {
    int dev = 0;
    if (const hipError_t e = hipGetDevice(&dev); e != hipSuccess) return static_cast<int>(e);
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return 0;
    for (const void* f : kernels) {
        const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_limit));
        if (e != hipSuccess) return static_cast<int>(e);
    }
    done.fetch_or(bit, std::memory_order_release);
    return 0;
}

}  // namespace ws
