// Buffer source of the layers, with the interface the oneLLM layers call
// (src/memory/allocator/base_allocator.h:5-17): Malloc<T>(ptr, bytes, is_host), deviceMalloc, deviceFree.
// HipAllocator is a small size-bucketed recycler over hipMalloc / hipHostMalloc: a decode step asks for the same
// handful of sizes every time, so after the first step no call reaches the driver.  It is not the block-pool
// allocator of src/memory/allocator/cuda_allocator.h (that subsystem is outside the decode path).
#pragma once
#include <cstddef>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>
#include <hip/hip_runtime_api.h>
#include "onellm/macro.h"

class BaseAllocator {
public:
    virtual ~BaseAllocator() {}
    template<typename T>
    void* Malloc(T* ptr, size_t size, bool is_host) { return deviceMalloc((void*)ptr, size, is_host); }
    virtual void* deviceMalloc(void* ptr, size_t size, bool is_host = false) = 0;
    virtual void  deviceFree(void* ptr, bool is_host = false) = 0;
};

class HipAllocator: public BaseAllocator {
public:
    ~HipAllocator() override
    {
        for (auto& b : live_) release(b.first, b.second.second);
        for (auto& bucket : idle_)
            for (void* p : bucket.second) release(p, bucket.first.second);
    }
    // `ptr` is ignored (the reference passes the previous value of the field it assigns to)
    void* deviceMalloc(void* /*ptr*/, size_t size, bool is_host = false) override
    {
        const size_t bytes = (size + 255) & ~size_t(255);
        std::lock_guard<std::mutex> g(mu_);
        auto& bucket = idle_[{bytes, is_host}];
        void* p = nullptr;
        if (!bucket.empty()) {
            p = bucket.back();
            bucket.pop_back();
        } else {
            const hipError_t e = is_host ? hipHostMalloc(&p, bytes, hipHostMallocDefault) : hipMalloc(&p, bytes);
            ONELLM_CHECK_WITH_INFO(e == hipSuccess, std::string("allocation failed: ") + hipGetErrorString(e));
        }
        live_[p] = {bytes, is_host};
        return p;
    }
    // returns the buffer to its bucket; work already queued on a stream may still be using it, which is safe as
    // long as the next user queues on the same stream (the layers use one)
    void deviceFree(void* ptr, bool /*is_host*/ = false) override
    {
        if (!ptr) return;
        std::lock_guard<std::mutex> g(mu_);
        auto it = live_.find(ptr);
        if (it == live_.end()) return;
        idle_[{it->second.first, it->second.second}].push_back(ptr);
        live_.erase(it);
    }

private:
    static void release(void* p, bool is_host)
    {
        if (is_host) (void)hipHostFree(p);
        else (void)hipFree(p);
    }
    std::mutex mu_;
    std::unordered_map<void*, std::pair<size_t, bool>> live_;
    std::map<std::pair<size_t, bool>, std::vector<void*>> idle_;
};
