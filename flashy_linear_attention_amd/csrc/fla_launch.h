// Host-side launch helpers shared by every kernel of the library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <tuple>
#include <utility>

namespace fla {

// Launches `kern` and returns the status of this launch alone.  (hipGetLastError after a
// triple-chevron launch would also hand back -- and clear -- an error that some earlier,
// unrelated call of the host program left behind.)
template <typename... KArgs, typename... Args>
inline hipError_t launch_kernel(void (*kern)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream,
                                Args &&...args) {
    static_assert(sizeof...(KArgs) == sizeof...(Args), "one argument per kernel parameter");
    std::tuple<std::decay_t<KArgs>...> vals{static_cast<std::decay_t<KArgs>>(std::forward<Args>(args))...};
    void *ptrs[sizeof...(KArgs) > 0 ? sizeof...(KArgs) : 1];
    std::apply([&](auto &...v) { int i = 0; ((ptrs[i++] = static_cast<void *>(&v)), ...); }, vals);
    return hipLaunchKernel(reinterpret_cast<const void *>(kern), grid, block, ptrs, lds_bytes, stream);
}

// Raises the dynamic LDS limit of kernel `Kern` to `bytes`, once per device and process: the
// attribute call costs a few microseconds of host time, which matters for launches of 30 us.
template <auto Kern>
inline hipError_t ensure_dynamic_lds(int bytes) {
    static std::atomic<uint64_t> done{0};  // one bit per device ordinal below 64
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = dev >= 0 && dev < 64 ? (uint64_t)1 << dev : 0;
    if (bit && (done.load(std::memory_order_acquire) & bit)) return hipSuccess;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(Kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && bit) done.fetch_or(bit, std::memory_order_release);
    return e;
}

}  // namespace fla
