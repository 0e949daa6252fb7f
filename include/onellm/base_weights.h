// src/weights/base_weights.h:5-49 restated: weight carrier handed to the decode attention launcher.
#pragma once
#include <vector>
#include <cstdint>
#include <type_traits>
#include <hip/hip_fp16.h>

enum class WeightType
{
    FP32_W,
    FP16_W,
    INT8_W,
    UNSUPPORTED_W
};

inline int getBitNum(WeightType type)
{
    switch (type) {
        case WeightType::FP32_W: return 32;
        case WeightType::FP16_W: return 16;
        case WeightType::INT8_W: return 8;
        default: return 0;
    }
}

template<typename T>
inline WeightType getWeightType()
{
    using U = typename std::remove_const<T>::type;
    if (std::is_same<U, float>::value)  return WeightType::FP32_W;
    if (std::is_same<U, half>::value)   return WeightType::FP16_W;
    if (std::is_same<U, int8_t>::value) return WeightType::INT8_W;
    return WeightType::UNSUPPORTED_W;
}

struct BaseWeight {
    std::vector<int> shape;
    void*            data;
    WeightType       type;
    void*            bias;
};
