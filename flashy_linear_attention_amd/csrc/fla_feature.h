// Element-wise feature maps applied while operands are loaded: q = phi(xq), k = phi(xk) never
// exist in memory.  phi is one of the positive maps callers of the reference put in front of
// its operators (README.md:27-30 of the reference leaves the map to the caller; its tests use
// softplus, flashlinear/test_attn.py:36-40, the linear-attention literature elu(x) + 1).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fla_tri_kernel.h"

namespace fla {

constexpr int kMapNone = 0, kMapElu1 = 1, kMapSoftplus = 2;

// phi(x) in fp32
__device__ __forceinline__ float feature_value(int map, float x) {
    if (map == kMapElu1) return x > 0.f ? x + 1.f : __expf(x);
    // softplus: log(1 + e^x); e^x itself where 1 + e^x would round to 1, x where e^x overflows the sum
    const float e = __expf(x);
    return x > 20.f ? x : (x < -10.f ? e : __logf(1.f + e));
}

// phi'(x) in fp32, from y = phi(x) (the value the forward pass left in memory; x itself is not
// needed again): elu(x) + 1 has slope 1 where y >= 1 and e^x = y below; softplus has slope
// sigmoid(x) = e^x / (1 + e^x) = 1 - e^{-y}.
__device__ __forceinline__ float feature_slope_from_value(int map, float y) {
    if (map == kMapElu1) return y >= 1.f ? 1.f : y;
    return 1.f - __expf(-y);
}

// phi on eight packed 16-bit values (one rounding to the storage type)
template <typename T>
__device__ __forceinline__ u32x4 feature_map8(int map, u32x4 raw) {
    typedef T v8 __attribute__((ext_vector_type(8)));
    v8 v = __builtin_bit_cast(v8, raw);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = static_cast<T>(feature_value(map, static_cast<float>(v[e])));
    return __builtin_bit_cast(u32x4, v);
}

}  // namespace fla
