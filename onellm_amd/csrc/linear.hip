// y = x . W for the projections around the decode path: hipBLASLt with a per-device handle and cached
// plans, plus a plain kernel for shapes the library declines.
#include <map>
#include <mutex>
#include <tuple>
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hipblaslt/hipblaslt.h>
#include "onellm_gemm.h"

namespace onellm {
namespace {

constexpr size_t kWorkspaceBytes = 32u << 20;

template <typename T> __device__ __forceinline__ float ld(const T* p, size_t i);
template <> __device__ __forceinline__ float ld<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ __forceinline__ float ld<__half>(const __half* p, size_t i) { return __half2float(p[i]); }
template <typename T> __device__ __forceinline__ void st(T* p, size_t i, float v);
template <> __device__ __forceinline__ void st<float>(float* p, size_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void st<__half>(__half* p, size_t i, float v) { p[i] = __float2half(v); }

// One thread per output element, serial over K: a correctness path for shapes without a library kernel
// (tiny or oddly sized matrices), not a tuned one.
template <typename T>
__global__ __launch_bounds__(256)
void linear_plain_kernel(const T* __restrict__ x, const T* __restrict__ w, T* __restrict__ y, int M, int K, int N, int ldy,
                         int w_is_nk)
{
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)M * N) return;
    const int m = (int)(idx / N), n = (int)(idx % N);
    float acc = 0.f;
    if (w_is_nk) {
        for (int k = 0; k < K; ++k) acc = fmaf(ld(x, (size_t)m * K + k), ld(w, (size_t)n * K + k), acc);
    } else {
        for (int k = 0; k < K; ++k) acc = fmaf(ld(x, (size_t)m * K + k), ld(w, (size_t)k * N + n), acc);
    }
    st(y, (size_t)m * ldy + n, acc);
}

struct Plan {
    bool usable = false;
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
    hipblasLtMatmulHeuristicResult_t heur{};
};

struct DeviceState {
    hipblasLtHandle_t handle = nullptr;
    bool handle_failed = false;
    // key: dtype, M, K, N, ldy, w_is_nk, workspace available
    std::map<std::tuple<int, int, int, int, int, int, int>, Plan> plans;
};

std::mutex g_mu;
std::map<int, DeviceState> g_devices;
thread_local int t_last_path = 0;

// Row-major y[M,N] = x[M,K].W[K,N] is, read column-major, y^T[N,M] = W^T[N,K] . x^T[K,M]: the buffers are passed
// as they are with A = W (leading dimension N, or K with a transpose when W is [N,K]) and B = x.
Plan make_plan(hipblasLtHandle_t h, int dtype, int M, int K, int N, int ldy, int w_is_nk, size_t ws_bytes)
{
    Plan p;
    const hipDataType dt = dtype == ONELLM_FP16 ? HIP_R_16F : HIP_R_32F;
    if (hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return p;
    const hipblasOperation_t opa = w_is_nk ? HIPBLAS_OP_T : HIPBLAS_OP_N, opb = HIPBLAS_OP_N;
    hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &opa, sizeof(opa));
    hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &opb, sizeof(opb));
    bool ok = true;
    if (w_is_nk) ok &= hipblasLtMatrixLayoutCreate(&p.la, dt, K, N, K) == HIPBLAS_STATUS_SUCCESS;
    else ok &= hipblasLtMatrixLayoutCreate(&p.la, dt, N, K, N) == HIPBLAS_STATUS_SUCCESS;
    ok &= hipblasLtMatrixLayoutCreate(&p.lb, dt, K, M, K) == HIPBLAS_STATUS_SUCCESS;
    ok &= hipblasLtMatrixLayoutCreate(&p.lc, dt, N, M, ldy) == HIPBLAS_STATUS_SUCCESS;
    if (!ok) return p;
    hipblasLtMatmulPreference_t pref = nullptr;
    if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return p;
    const uint64_t max_ws = ws_bytes;
    hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws));
    int found = 0;
    const hipblasStatus_t s = hipblasLtMatmulAlgoGetHeuristic(h, p.desc, p.la, p.lb, p.lc, p.lc, pref, 1, &p.heur, &found);
    hipblasLtMatmulPreferenceDestroy(pref);
    p.usable = s == HIPBLAS_STATUS_SUCCESS && found > 0 && p.heur.workspaceSize <= ws_bytes;
    return p;
}

template <typename T>
int run_plain(const void* x, const void* w, void* y, int M, int K, int N, int ldy, int w_is_nk, hipStream_t st)
{
    const size_t total = (size_t)M * N;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    hipLaunchKernelGGL((linear_plain_kernel<T>), dim3(blocks), dim3(256), 0, st, static_cast<const T*>(x),
                       static_cast<const T*>(w), static_cast<T*>(y), M, K, N, ldy, w_is_nk);
    return (int)hipGetLastError();
}

}  // namespace
}  // namespace onellm

extern "C" size_t onellm_linear_workspace_bytes(void) { return onellm::kWorkspaceBytes; }

extern "C" int onellm_linear_last_path(void) { return onellm::t_last_path; }

extern "C" int onellm_linear(int dtype, const void* x, const void* w, void* y, int M, int K, int N, int ldy, int w_is_nk,
                             void* workspace, size_t workspace_bytes, onellm_stream_t stream)
{
    using namespace onellm;
    if (dtype != ONELLM_FP32 && dtype != ONELLM_FP16) return ONELLM_EINVAL;
    if (M < 0 || K <= 0 || N <= 0) return ONELLM_EINVAL;
    if (ldy == 0) ldy = N;
    if (ldy < N) return ONELLM_EINVAL;
    if (M == 0) return 0;
    if (!x || !w || !y) return ONELLM_EINVAL;
    if ((size_t)M * N > 0x7fffffffu * (size_t)256) return ONELLM_EUNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (!workspace) workspace_bytes = 0;
    if (workspace_bytes > kWorkspaceBytes) workspace_bytes = kWorkspaceBytes;
    w_is_nk = w_is_nk ? 1 : 0;

    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;

    Plan plan;
    hipblasLtHandle_t handle = nullptr;
    {
        std::lock_guard<std::mutex> g(g_mu);
        DeviceState& ds = g_devices[dev];
        if (!ds.handle && !ds.handle_failed) {
            if (hipblasLtCreate(&ds.handle) != HIPBLAS_STATUS_SUCCESS) {
                ds.handle = nullptr;
                ds.handle_failed = true;
            }
        }
        handle = ds.handle;
        if (handle) {
            const auto key = std::make_tuple(dtype, M, K, N, ldy, w_is_nk, workspace_bytes ? 1 : 0);
            auto it = ds.plans.find(key);
            if (it == ds.plans.end()) it = ds.plans.emplace(key, make_plan(handle, dtype, M, K, N, ldy, w_is_nk, workspace_bytes)).first;
            plan = it->second;
            if (plan.usable && plan.heur.workspaceSize > workspace_bytes) plan.usable = false;
        }
    }
    if (plan.usable) {
        const float alpha = 1.f, beta = 0.f;
        const hipblasStatus_t s = hipblasLtMatmul(handle, plan.desc, &alpha, w, plan.la, x, plan.lb, &beta, y, plan.lc, y,
                                                  plan.lc, &plan.heur.algo, workspace, workspace_bytes, st);
        if (s == HIPBLAS_STATUS_SUCCESS) {
            t_last_path = 1;
            return 0;
        }
    }
    t_last_path = 0;
    return dtype == ONELLM_FP16 ? run_plain<__half>(x, w, y, M, K, N, ldy, w_is_nk, st)
                                : run_plain<float>(x, w, y, M, K, N, ldy, w_is_nk, st);
}
