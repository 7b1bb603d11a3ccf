// Element-wise feature maps applied while operands are loaded: q = phi(xq), k = phi(xk) never
// exist in memory.  phi is one of the positive maps callers of the reference put in front of
// its operators (README.md:27-30 of the reference leaves the map to the caller; its tests use
// softplus, flashlinear/test_attn.py:36-40, the linear-attention literature elu(x) + 1).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "fla_tri_kernel.h"

namespace fla {

constexpr int kMapNone = 0, kMapElu1 = 1, kMapSoftplus = 2;

// phi(x) in fp32, the map a compile-time constant
template <int MAP>
__device__ __forceinline__ float feature_value_c(float x) {
    static_assert(MAP == kMapElu1 || MAP == kMapSoftplus, "unknown feature map");
    if constexpr (MAP == kMapElu1) return x > 0.f ? x + 1.f : __expf(x);
    // softplus: log(1 + e^x); e^x itself where 1 + e^x would round to 1, x where e^x overflows the sum
    const float e = __expf(x);
    return x > 20.f ? x : (x < -10.f ? e : __logf(1.f + e));
}

// phi'(x) in fp32, from y = phi(x) (the value the forward pass left in memory; x itself is not
// needed again): elu(x) + 1 has slope 1 where y >= 1 and e^x = y below; softplus has slope
// sigmoid(x) = e^x / (1 + e^x) = 1 - e^{-y}.
template <int MAP>
__device__ __forceinline__ float feature_slope_c(float y) {
    static_assert(MAP == kMapElu1 || MAP == kMapSoftplus, "unknown feature map");
    if constexpr (MAP == kMapElu1) return y >= 1.f ? 1.f : y;
    return 1.f - __expf(-y);
}

// f(std::integral_constant<int, MAP>) for the map that `map` names (not kMapNone): one uniform branch
// around a whole loop instead of one per element
template <typename F>
__device__ __forceinline__ void feature_dispatch(int map, F &&f) {
    if (map == kMapElu1)
        f(std::integral_constant<int, kMapElu1>{});
    else
        f(std::integral_constant<int, kMapSoftplus>{});
}

__device__ __forceinline__ float feature_value(int map, float x) {
    return map == kMapElu1 ? feature_value_c<kMapElu1>(x) : feature_value_c<kMapSoftplus>(x);
}
__device__ __forceinline__ float feature_slope_from_value(int map, float y) {
    return map == kMapElu1 ? feature_slope_c<kMapElu1>(y) : feature_slope_c<kMapSoftplus>(y);
}

// phi on eight packed 16-bit values (one rounding to the storage type)
template <typename T, int MAP>
__device__ __forceinline__ u32x4 feature_map8_c(u32x4 raw) {
    typedef T v8 __attribute__((ext_vector_type(8)));
    v8 v = __builtin_bit_cast(v8, raw);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = static_cast<T>(feature_value_c<MAP>(static_cast<float>(v[e])));
    return __builtin_bit_cast(u32x4, v);
}
template <typename T>
__device__ __forceinline__ u32x4 feature_map8(int map, u32x4 raw) {
    return map == kMapElu1 ? feature_map8_c<T, kMapElu1>(raw) : feature_map8_c<T, kMapSoftplus>(raw);
}

}  // namespace fla
