// Host-side launch helpers shared by every kernel of the library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <tuple>
#include <utility>

#if defined(FLA_TRACE_LAUNCHES)
// Host-only build that makes no launch: every launch_kernel call is written down instead -- kernel
// (with its template arguments), grid, block, dynamic LDS and every argument field by field -- so
// that the launch plan of an operator call can be enumerated and checked on a machine without a GPU.
#include "fla_trace.h"
#endif

namespace fla {

// Launches `Kern` and returns the status of this launch alone.  (hipGetLastError after a
// triple-chevron launch would also hand back -- and clear -- an error that some earlier,
// unrelated call of the host program left behind.)
template <typename... KArgs, typename... Args>
inline hipError_t launch_kernel_ptr(void (*kern)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream,
                                    Args &&...args) {
    static_assert(sizeof...(KArgs) == sizeof...(Args), "one argument per kernel parameter");
    std::tuple<std::decay_t<KArgs>...> vals{static_cast<std::decay_t<KArgs>>(std::forward<Args>(args))...};
    void *ptrs[sizeof...(KArgs) > 0 ? sizeof...(KArgs) : 1];
    std::apply([&](auto &...v) { int i = 0; ((ptrs[i++] = static_cast<void *>(&v)), ...); }, vals);
    return hipLaunchKernel(reinterpret_cast<const void *>(kern), grid, block, ptrs, lds_bytes, stream);
}

#if defined(FLA_TRACE_LAUNCHES)
template <typename... KArgs, typename... Args>
inline hipError_t trace_kernel_ptr(const char *name, void (*)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes,
                                   Args &&...args) {
    static_assert(sizeof...(KArgs) == sizeof...(Args), "one argument per kernel parameter");
    std::tuple<std::decay_t<KArgs>...> vals{static_cast<std::decay_t<KArgs>>(std::forward<Args>(args))...};
    trace::Record rec(name, grid.x, grid.y, grid.z, block.x, lds_bytes);
    std::apply([&](auto &...v) { int i = 0; ((trace_describe(rec, i++, v)), ...); }, vals);
    rec.commit();
    return hipSuccess;
}
#endif

template <auto Kern, typename... Args>
inline hipError_t launch_kernel(dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream, Args &&...args) {
#if defined(FLA_TRACE_LAUNCHES)
    (void)stream;
    return trace_kernel_ptr(trace::kernel_name<Kern>(), Kern, grid, block, lds_bytes, std::forward<Args>(args)...);
#else
    return launch_kernel_ptr(Kern, grid, block, lds_bytes, stream, std::forward<Args>(args)...);
#endif
}

// Raises the dynamic LDS limit of kernel `Kern` to `bytes`, once per device and process: the
// attribute call costs a few microseconds of host time, which matters for launches of 30 us.
template <auto Kern>
inline hipError_t ensure_dynamic_lds(int bytes) {
#if defined(FLA_TRACE_LAUNCHES)
    trace::note_lds_limit(trace::kernel_name<Kern>(), bytes);
    return hipSuccess;
#else
    static std::atomic<uint64_t> done{0};  // one bit per device ordinal below 64
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = dev >= 0 && dev < 64 ? (uint64_t)1 << dev : 0;
    if (bit && (done.load(std::memory_order_acquire) & bit)) return hipSuccess;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(Kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && bit) done.fetch_or(bit, std::memory_order_release);
    return e;
#endif
}

}  // namespace fla
