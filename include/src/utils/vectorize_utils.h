// Vec<T>: the packed type the reference's kernels use per element type (src/utils/vectorize_utils.h:
// 43-57): half -> half2 (2 elements), float -> float4 (4 elements).  The gfx950 kernels do not use
// it (they move 16 bytes per lane whatever the type); it is kept so code written against the
// reference's headers compiles unchanged.
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

template <typename T>
struct Vec {
    using Type = T;
    static constexpr int size = 0;
};
template <>
struct Vec<half> {
    using Type = half2;
    static constexpr int size = 2;
};
template <>
struct Vec<float> {
    using Type = float4;
    static constexpr int size = 4;
};

struct TwoFloat2 {
    float2 x;
    float2 y;
};

// broadcast a scalar into every slot of a packed type
template <typename T_OUT, typename T_IN>
inline __host__ __device__ T_OUT scalar_cast_vec(T_IN val) {
    return val;
}
template <>
inline __host__ __device__ half2 scalar_cast_vec<half2, float>(float val) {
    return __float2half2_rn(val);
}
template <>
inline __host__ __device__ float4 scalar_cast_vec<float4, float>(float val) {
    return make_float4(val, val, val, val);
}
template <>
inline __host__ __device__ float2 scalar_cast_vec<float2, float>(float val) {
    return make_float2(val, val);
}
template <>
inline __host__ __device__ half2 scalar_cast_vec<half2, half>(half val) {
    return __half2half2(val);
}
