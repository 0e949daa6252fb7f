// Boundary carrier types of the decode path, restated from the oneLLM tree so that code
// written against src/utils/tensor.h:12-144 compiles against this backend unchanged:
// same enumerator order, same field order and types.  A Tensor never owns `data`
// (src/utils/tensor.h:79-85).
#pragma once
#include <algorithm>
#include <functional>
#include <numeric>
#include <string>
#include <type_traits>
#include <vector>
#include <cstdint>
#include <hip/hip_fp16.h>
#include "onellm/macro.h"

enum Device
{
    CPU_PINNED,
    CPU,
    GPU
};

enum DataType
{
    FP32,
    FP16,
    INT8,
    INT32,
    BOOL,
    BYTES,
    UNSUPPORTED
};

// src/utils/tensor.h:30-54
template<typename T>
DataType getTensorType()
{
    using U = typename std::remove_const<T>::type;
    if (std::is_same<U, float>::value)  return FP32;
    if (std::is_same<U, half>::value)   return FP16;
    if (std::is_same<U, int>::value)    return INT32;
    if (std::is_same<U, int8_t>::value) return INT8;
    if (std::is_same<U, bool>::value)   return BOOL;
    if (std::is_same<U, char>::value)   return BYTES;
    return UNSUPPORTED;
}

// src/utils/tensor.h:56-144
struct Tensor {
    Device           location;
    DataType         dtype;
    std::vector<int> shape;
    void*            data;

    Tensor() = default;

    Tensor(const Device location_, const DataType dtype_, const std::vector<int> shape_):
        location(location_), dtype(dtype_), shape(shape_), data(nullptr) {}

    Tensor(const Device location_, const DataType dtype_, const std::vector<int> shape_, void* data_):
        location(location_), dtype(dtype_), shape(shape_), data(data_) {}

    int size() const
    {
        if (data == nullptr || shape.empty()) {
            return 0;
        }
        return std::accumulate(shape.begin(), shape.end(), 1, std::multiplies<int>());
    }

    template<typename T>
    inline T getVal(int id) const { return ((T*)data)[id]; }

    // host-resident scalars only (src/utils/tensor.h:100-107)
    template<typename T>
    inline T getVal() const
    {
        ONELLM_CHECK(location == CPU);
        return getVal<T>(0);
    }

    template<typename T>
    inline T* getPtr() const { return (T*)data; }

    template<typename T>
    inline T* getPtrByOffset(int offset) const { return (T*)data + offset; }

    std::string DeviceString() const
    {
        return location == CPU ? "CPU" : (location == CPU_PINNED ? "CPU_PINNED" : "GPU");
    }

    std::string toString() const
    {
        std::string s = "Tensor[where=" + DeviceString() + ", type=";
        s += dtype == FP32 ? "FP32" : dtype == FP16 ? "FP16" : dtype == INT8 ? "INT8" : dtype == INT32 ? "INT32" : "OTHER";
        s += ", shape=(";
        for (size_t i = 0; i < shape.size(); ++i) {
            s += std::to_string(shape[i]);
            if (i + 1 < shape.size()) s += ", ";
        }
        s += ")]";
        return s;
    }

    friend bool operator==(Tensor& t1, Tensor& t2);
};

// src/utils/tensor.h:86,146-160: element-wise comparison of two host-readable FP32 tensors of equal size (the
// reference dereferences `data` as float on the host whatever the element type or location are; so does this).
// Sizes that differ, or an empty tensor on either side with a non-empty one on the other, compare unequal.
inline bool operator==(Tensor& t1, Tensor& t2)
{
    if (t1.size() != t2.size()) return false;
    const float* a = static_cast<const float*>(t1.data);
    const float* b = static_cast<const float*>(t2.data);
    for (int i = 0; i < t1.size(); ++i) {
        if (a[i] != b[i]) return false;
    }
    return true;
}
