// Address of a file-scope __device__ array on the current GPU.  In host code the array's name is only a handle for
// hipGetSymbolAddress; every GPU holds its own copy at its own address, so the address is resolved once per device,
// under a lock, and kept.  Nothing is allocated, launched or synchronised.
#pragma once
#include <mutex>
#include <hip/hip_runtime.h>
#include "onellm_hip.h"

namespace onellm {

class DeviceSymbol {
public:
    // `handle` is HIP_SYMBOL(the array).  Returns 0, a hipError_t, or ONELLM_EUNSUPPORTED for a device ordinal
    // beyond kMaxDevices.
    int address(const void* handle, void** out)
    {
        int dev = -1;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return static_cast<int>(e);
        if (dev < 0 || dev >= kMaxDevices) return ONELLM_EUNSUPPORTED;
        std::lock_guard<std::mutex> lock(mu_);
        if (!known_[dev]) {
            void* p = nullptr;
            e = hipGetSymbolAddress(&p, handle);
            if (e != hipSuccess) return static_cast<int>(e);
            if (!p) return static_cast<int>(hipErrorInvalidSymbol);
            known_[dev] = p;
        }
        *out = known_[dev];
        return 0;
    }

private:
    static constexpr int kMaxDevices = 64;
    std::mutex mu_;
    void* known_[kMaxDevices] = {};
};

}  // namespace onellm
