// Error convention of the decode path, restated from src/utils/macro.h:6-106 for HIP:
// launchers return void; precondition failures and HIP errors become std::runtime_error.
#pragma once
#include <stdexcept>
#include <string>
#include <cstdio>
#include <cstdlib>
#include <hip/hip_runtime_api.h>

// src/utils/macro.h:6-20 (unit-test style: print and exit)
#define CHECK(call)                                                     \
do {                                                                    \
    const hipError_t error_code = call;                                 \
    if (error_code != hipSuccess) {                                     \
        printf("HIP Error:\n");                                         \
        printf("    File:       %s\n", __FILE__);                       \
        printf("    Line:       %d\n", __LINE__);                       \
        printf("    Error code: %d\n", error_code);                     \
        printf("    Error text: %s\n", hipGetErrorString(error_code));  \
        exit(1);                                                        \
    }                                                                   \
} while (0)

// src/utils/macro.h:59-70: status check of a BLAS-library call.  The layers here call the GEMM through
// onellm_linear (which reports through its return code), so nothing in this backend uses it; it is kept so that layer
// sources written against the reference (`CHECK_CUBLAS(cublasXxx(...))`) compile unchanged when the call they wrap
// returns a hipblasStatus_t / hipError_t-like integer: non-zero throws, as in the reference.
template<typename T>
void check(T result, char const* const func, const char* const file, int const line)
{
    if (result) {
        throw std::runtime_error(std::string("[TM][ERROR] HIP runtime error: status ") + std::to_string((long long)result)
                                 + " from " + func + " " + file + ":" + std::to_string(line) + " \n");
    }
}
#define CHECK_CUBLAS(val) check((val), #val, __FILE__, __LINE__)

// src/utils/macro.h:74-84
inline void syncAndCheck(const char* const file, int const line)
{
    hipError_t result = hipDeviceSynchronize();
    if (result == hipSuccess) result = hipGetLastError();
    if (result) {
        throw std::runtime_error(std::string("[TM][ERROR] HIP runtime error: ") + hipGetErrorString(result) + " "
                                 + file + ":" + std::to_string(line) + " \n");
    }
}
#define DeviceSyncAndCheckCudaError() syncAndCheck(__FILE__, __LINE__)

// src/utils/macro.h:86-106
[[noreturn]] inline void throwRuntimeError(const char* const file, int const line, std::string const& info = "")
{
    throw std::runtime_error(std::string("[oneLLM][ERROR] ") + info + " Assertion fail: " + file + ":"
                             + std::to_string(line) + " \n");
}

inline void onellmAssert(bool result, const char* const file, int const line, std::string const& info = "")
{
    if (!result) {
        throwRuntimeError(file, line, info);
    }
}

#define ONELLM_CHECK(val) onellmAssert(val, __FILE__, __LINE__)
#define ONELLM_CHECK_WITH_INFO(val, info)                           \
    do {                                                            \
        bool is_valid_val = (val);                                  \
        if (!is_valid_val) {                                        \
            onellmAssert(is_valid_val, __FILE__, __LINE__, (info)); \
        }                                                           \
    } while (0)
