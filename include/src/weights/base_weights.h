// Weight descriptors with the reference's names (src/weights/base_weights.h:29-35).  The pointers
// are zero-initialised here (the reference leaves them indeterminate), so an unset `bias` reads as
// "no bias" instead of garbage.
#pragma once
#include <hip/hip_fp16.h>

#include <cstdint>
#include <type_traits>
#include <vector>

enum class WeightType { FP32_W, FP16_W, INT8_W, UNSUPPORTED_W };

template <typename T>
inline WeightType getWeightType() {
    using U = typename std::remove_cv<T>::type;
    if (std::is_same<U, float>::value) return WeightType::FP32_W;
    if (std::is_same<U, half>::value) return WeightType::FP16_W;
    if (std::is_same<U, int8_t>::value) return WeightType::INT8_W;
    return WeightType::UNSUPPORTED_W;
}

template <typename T>
struct BaseWeight {
    std::vector<int> shape;
    T* data = nullptr;
    WeightType type = getWeightType<T>();
    T* bias = nullptr;
};
