// y = x . W for the projections around the decode path: hipBLASLt with a per-device handle and cached
// plans, this library's own kernel for a decode step's few rows where timing finds it faster (skinny_gemm.hip),
// plus a plain kernel for shapes the library declines.
#include <algorithm>
#include <atomic>
#include <map>
#include <mutex>
#include <tuple>
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hipblaslt/hipblaslt.h>
#include "onellm_gemm.h"
#include "skinny_gemm.hpp"

namespace onellm {
int tune_get(const char* key);     // libonellm_hip.so's tuning table
namespace {

constexpr size_t kWorkspaceBytes = 32u << 20;
// The plain kernel runs one thread per output element: fine for the tiny matrices of unit tests and example
// drivers, about a hundred times slower than the library on a projection of a real model.  Up to this many
// multiply-adds it is used without asking; a larger problem the library declines is an error unless the caller
// has allowed the plain kernel (onellm_linear_allow_plain).
constexpr unsigned long long kPlainQuietMacs = 1ull << 24;
std::atomic<int> g_allow_plain{0};

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
    bool usable = false;                     // the library's objects below are there
    SkinnyConfig skinny;                     // set by the tuning run when this library's few-row kernel won
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
    hipblasLtMatmulHeuristicResult_t heur{};
};

// gives the library's objects of a plan back (a plan that is replaced, or one whose set-up failed half way)
void destroy_plan(Plan& p)
{
    if (p.desc) (void)hipblasLtMatmulDescDestroy(p.desc);
    if (p.la) (void)hipblasLtMatrixLayoutDestroy(p.la);
    if (p.lb) (void)hipblasLtMatrixLayoutDestroy(p.lb);
    if (p.lc) (void)hipblasLtMatrixLayoutDestroy(p.lc);
    p = Plan{};
}

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
// Descriptor and layouts of one problem; `heur` is filled by the callers below.
Plan make_problem(int dtype, int M, int K, int N, int ldy, int w_is_nk)
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
    if (!ok) destroy_plan(p);
    else p.usable = true;
    return p;
}

// the library's ranked candidates for a problem (at most `want`), those that fit the workspace
int candidates(hipblasLtHandle_t h, const Plan& p, size_t ws_bytes, hipblasLtMatmulHeuristicResult_t* out, int want)
{
    hipblasLtMatmulPreference_t pref = nullptr;
    if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return 0;
    const uint64_t max_ws = ws_bytes;
    hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws));
    int found = 0;
    const hipblasStatus_t s = hipblasLtMatmulAlgoGetHeuristic(h, p.desc, p.la, p.lb, p.lc, p.lc, pref, want, out, &found);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (s != HIPBLAS_STATUS_SUCCESS) return 0;
    int kept = 0;
    for (int i = 0; i < found; ++i)
        if (out[i].workspaceSize <= ws_bytes) out[kept++] = out[i];
    return kept;
}

// the library's first suggestion for a problem
Plan make_plan(hipblasLtHandle_t h, int dtype, int M, int K, int N, int ldy, int w_is_nk, size_t ws_bytes)
{
    Plan p = make_problem(dtype, M, K, N, ldy, w_is_nk);
    if (!p.usable) return p;
    if (candidates(h, p, ws_bytes, &p.heur, 1) != 1) destroy_plan(p);       // (an unusable plan holds nothing)
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

namespace onellm {
namespace {
// caller holds g_mu
hipblasLtHandle_t device_handle(DeviceState& ds)
{
    if (!ds.handle && !ds.handle_failed) {
        if (hipblasLtCreate(&ds.handle) != HIPBLAS_STATUS_SUCCESS) {
            ds.handle = nullptr;
            ds.handle_failed = true;
        }
    }
    return ds.handle;
}
}  // namespace
}  // namespace onellm

extern "C" int onellm_linear_tune(int dtype, int M, int K, int N, int ldy, int w_is_nk, void* workspace, size_t workspace_bytes,
                                  onellm_stream_t stream, float* best_us, float* first_us)
{
    using namespace onellm;
    if (dtype != ONELLM_FP32 && dtype != ONELLM_FP16) return ONELLM_EINVAL;
    if (M <= 0 || K <= 0 || N <= 0) return ONELLM_EINVAL;
    if (ldy == 0) ldy = N;
    if (ldy < N) return ONELLM_EINVAL;
    if (!workspace) workspace_bytes = 0;
    if (workspace_bytes > kWorkspaceBytes) workspace_bytes = kWorkspaceBytes;
    w_is_nk = w_is_nk ? 1 : 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;

    hipblasLtHandle_t handle = nullptr;
    {
        std::lock_guard<std::mutex> g(g_mu);
        handle = device_handle(g_devices[dev]);
    }
    if (!handle) return ONELLM_EUNSUPPORTED;
    Plan p = make_problem(dtype, M, K, N, ldy, w_is_nk);
    if (!p.usable) return ONELLM_EUNSUPPORTED;
    constexpr int kWant = 32;
    hipblasLtMatmulHeuristicResult_t cand[kWant];
    const int n = candidates(handle, p, workspace_bytes, cand, kWant);
    constexpr int kWantOwn = 64;
    SkinnyConfig own[kWantOwn];
    const int n_own = (tune_get("gemm_skinny") != 0 && skinny_shape_ok(dtype, M, K, N, ldy, w_is_nk))
                          ? skinny_candidates(M, K, N, workspace_bytes, own, kWantOwn) : 0;
    if (n == 0 && n_own == 0) {
        destroy_plan(p);
        return ONELLM_EUNSUPPORTED;
    }
    // the timing runs allocate, synchronise and launch: none of that may happen on a stream that is being captured
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &capturing) != hipSuccess) (void)hipGetLastError();
    if (capturing != hipStreamCaptureStatusNone) {
        destroy_plan(p);
        return ONELLM_ECAPTURING;
    }

    // stand-in operands of the right size (values do not matter for the timing; 0x3c3c.. is ~1.06 in fp16 and a
    // small normal number in fp32)
    // The weights of a model are far larger than the chip's caches, so a projection always meets its matrix cold.  A
    // timing loop over one matrix would not: it stays in the 256 MB memory-side cache and every candidate looks up to
    // twice as fast as it will be (a 7B down projection, 90 MB: 29 us warm, 50 us cold with the same algorithm).  The
    // runs therefore rotate over enough copies of W to exceed that cache.
    const size_t esz = dtype == ONELLM_FP16 ? 2 : 4;
    const size_t w_bytes = (size_t)K * N * esz;
    constexpr size_t kColdBytes = 640u << 20;
    constexpr int kMaxCopies = 16;
    const int copies = (int)std::min<size_t>(kMaxCopies, std::max<size_t>(2, (kColdBytes + w_bytes - 1) / w_bytes));
    void *x = nullptr, *y = nullptr, *w[kMaxCopies] = {};
    hipEvent_t t0 = nullptr, t1 = nullptr;
    int rc = 0;
    auto cleanup = [&] {
        if (x) (void)hipFree(x);
        for (void* c : w)
            if (c) (void)hipFree(c);
        if (y) (void)hipFree(y);
        if (t0) (void)hipEventDestroy(t0);
        if (t1) (void)hipEventDestroy(t1);
    };
    e = hipMalloc(&x, (size_t)M * K * esz);
    for (int c = 0; c < copies && e == hipSuccess; ++c) e = hipMalloc(&w[c], w_bytes);
    if (e != hipSuccess || (e = hipMalloc(&y, (size_t)M * ldy * esz)) != hipSuccess || (e = hipEventCreate(&t0)) != hipSuccess ||
        (e = hipEventCreate(&t1)) != hipSuccess) {
        cleanup();
        destroy_plan(p);
        return (int)e;
    }
    (void)hipMemsetAsync(x, 0x3c, (size_t)M * K * esz, st);
    for (int c = 0; c < copies; ++c) (void)hipMemsetAsync(w[c], 0x3c, w_bytes, st);
    const float alpha = 1.f, beta = 0.f;
    int best = -1, best_own = -1;
    float best_ms = 0.f, first_ms = 0.f, best_own_ms = 0.f;
    constexpr int kWarm = 2;
    const int runs = std::max(8, copies);
    // candidate i of the library (i < n) or of this library's kernel (i >= n), timed over `runs` launches
    for (int i = 0; i < n + n_own; ++i) {
        bool ok = true;
        for (int r = 0; r < kWarm + runs && ok; ++r) {
            if (r == kWarm) (void)hipEventRecord(t0, st);
            const void* wc = w[r % copies];
            if (i < n)
                ok = hipblasLtMatmul(handle, p.desc, &alpha, wc, p.la, x, p.lb, &beta, y, p.lc, y, p.lc, &cand[i].algo, workspace,
                                     workspace_bytes, st) == HIPBLAS_STATUS_SUCCESS;
            else
                ok = skinny_launch(own[i - n], x, wc, y, M, K, N, ldy, workspace, workspace_bytes, st) == 0;
        }
        (void)hipEventRecord(t1, st);
        if ((e = hipEventSynchronize(t1)) != hipSuccess) {
            rc = (int)e;
            break;
        }
        if (!ok) continue;
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, t0, t1);
        ms /= runs;
        if (i == 0) first_ms = ms;
        if (i < n) {
            if (best < 0 || ms < best_ms) {
                best = i;
                best_ms = ms;
            }
        } else if (best_own < 0 || ms < best_own_ms) {
            best_own = i - n;
            best_own_ms = ms;
        }
    }
    cleanup();
    if (rc != 0 || (best < 0 && best_own < 0)) {
        destroy_plan(p);
        return rc != 0 ? rc : ONELLM_EUNSUPPORTED;
    }
    if (best >= 0) p.heur = cand[best];
    else destroy_plan(p);                    // (the library has nothing for this problem: the plan is this library's kernel alone)
    // this library's kernel is taken when it is clearly ahead (3 %: two near-equal timings should not flip a plan)
    if (best_own >= 0 && (best < 0 || best_own_ms < 0.97f * best_ms)) {
        p.skinny = own[best_own];
        best_ms = best_own_ms;
    }
    {
        // (a plan in the table is only ever used under this lock or as a copy taken under it by a call that was
        // queued before this one returns: the stream was synchronised above, so the old objects are idle)
        std::lock_guard<std::mutex> g(g_mu);
        Plan& slot = g_devices[dev].plans[std::make_tuple(dtype, M, K, N, ldy, w_is_nk, workspace_bytes ? 1 : 0)];
        destroy_plan(slot);
        slot = p;
    }
    if (best_us) *best_us = best_ms * 1e3f;
    if (first_us) *first_us = first_ms * 1e3f;
    return 0;
}

extern "C" size_t onellm_linear_workspace_bytes(void) { return onellm::kWorkspaceBytes; }

extern "C" int onellm_linear_last_path(void) { return onellm::t_last_path; }

extern "C" int onellm_linear_allow_plain(int allow) { return onellm::g_allow_plain.exchange(allow ? 1 : 0); }

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
        device_handle(ds);
        handle = ds.handle;
        if (handle) {
            const auto key = std::make_tuple(dtype, M, K, N, ldy, w_is_nk, workspace_bytes ? 1 : 0);
            auto it = ds.plans.find(key);
            if (it == ds.plans.end()) it = ds.plans.emplace(key, make_plan(handle, dtype, M, K, N, ldy, w_is_nk, workspace_bytes)).first;
            plan = it->second;
            if (plan.usable && plan.heur.workspaceSize > workspace_bytes) plan.usable = false;
        }
    }
    if (tune_get("gemm_no_library") == 1) plan.usable = false;
    // this library's few-row kernel: where the tuning run chose it (tuning key gemm_skinny = 0: never; 1: wherever it
    // takes the problem, with a default configuration if none was timed)
    {
        const int want = tune_get("gemm_skinny");
        SkinnyConfig c = plan.skinny;
        if (want == 0) c = SkinnyConfig{};
        else if (want == 1 && skinny_shape_ok(dtype, M, K, N, ldy, w_is_nk)) {
            const int pick = tune_get("gemm_skinny_config");             // 100 * variant + slices along K (tests)
            if (pick >= 0) c = SkinnyConfig{pick / 100, pick % 100};
            else if (c.variant < 0) c = skinny_default(M, K, N, workspace_bytes);
        }
        if (c.variant >= 0) {
            const int rc = skinny_launch(c, x, w, y, M, K, N, ldy, workspace, workspace_bytes, st);
            if (rc == 0) {
                t_last_path = 2;
                return 0;
            }
            if (rc != ONELLM_EUNSUPPORTED) return rc;        // (declined as given - alignment, workspace: on to the library)
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
    // no library kernel (or the library refused at run time): the plain kernel, unless that would be a silent
    // hundredfold slowdown
    if ((unsigned long long)M * (unsigned long long)K * (unsigned long long)N > kPlainQuietMacs && !g_allow_plain.load())
        return ONELLM_ENOGEMMKERNEL;
    t_last_path = 0;
    return dtype == ONELLM_FP16 ? run_plain<__half>(x, w, y, M, K, N, ldy, w_is_nk, st)
                                : run_plain<float>(x, w, y, M, K, N, ldy, w_is_nk, st);
}
