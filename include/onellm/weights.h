// Weight carriers of the decode path, with the member names, order and types the oneLLM layers fill
// in, so that code written against them compiles unchanged:
//   WeightType, getBitNum, getWeightType<T>, BaseWeight   <- src/weights/base_weights.h:5-49
//   LayerNormWeight                                         <- src/weights/llama/norm_weights.h:2-4
// A BaseWeight never owns `data` or `bias`; both are device pointers (bias may be null).
#pragma once
#include <cstdint>
#include <type_traits>
#include <vector>
#include <hip/hip_fp16.h>

enum class WeightType { FP32_W, FP16_W, INT8_W, UNSUPPORTED_W };

// storage bits of one weight element; 0 for an unsupported type
inline int getBitNum(WeightType type)
{
    return type == WeightType::FP32_W ? 32 : type == WeightType::FP16_W ? 16 : type == WeightType::INT8_W ? 8 : 0;
}

template<typename T>
inline WeightType getWeightType()
{
    using U = typename std::remove_const<T>::type;
    return std::is_same<U, float>::value    ? WeightType::FP32_W
           : std::is_same<U, half>::value   ? WeightType::FP16_W
           : std::is_same<U, int8_t>::value ? WeightType::INT8_W
                                            : WeightType::UNSUPPORTED_W;
}

// one projection: `data` is the matrix (used by the GEMMs, never by this backend), `bias` the fused
// bias vector the attention kernels read
struct BaseWeight {
    std::vector<int> shape;
    void*            data;
    WeightType       type;
    void*            bias;
};

// RMSNorm scale.  The field is `float*` in oneLLM; for FP16 activations the launcher reads fp16
// values behind the same pointer.
struct LayerNormWeight {
    float* gamma;
};
