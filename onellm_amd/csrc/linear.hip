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

namespace onellm {
namespace {

// Stand-in operands for a timing run (values do not matter; 0x3c3c.. is ~1.06 in fp16 and a small normal number in
// fp32), two events, and the loop that times one candidate.
//
// The weights of a model are far larger than the chip's caches, so a projection always meets its matrix cold.  A
// timing loop over one matrix would not: it stays in the 256 MB memory-side cache and every candidate looks up to
// twice as fast as it will be (a 7B down projection, 90 MB: 29 us warm, 50 us cold with the same algorithm).  The
// runs therefore rotate over enough copies of W to exceed that cache.
struct TimingRig {
    static constexpr int kMaxCopies = 16;
    static constexpr size_t kColdBytes = 640u << 20;
    void *x = nullptr, *y = nullptr, *w[kMaxCopies] = {};
    int copies = 0;
    hipEvent_t t0 = nullptr, t1 = nullptr;

    hipError_t make(size_t x_bytes, size_t y_bytes, size_t w_bytes, hipStream_t st)
    {
        copies = (int)std::min<size_t>(kMaxCopies, std::max<size_t>(2, (kColdBytes + w_bytes - 1) / w_bytes));
        copies &= ~1;                                            // (pairs of matrices for the two-problem launch)
        hipError_t e = hipMalloc(&x, x_bytes);
        for (int c = 0; c < copies && e == hipSuccess; ++c) e = hipMalloc(&w[c], w_bytes);
        if (e == hipSuccess) e = hipMalloc(&y, y_bytes);
        if (e == hipSuccess) e = hipEventCreate(&t0);
        if (e == hipSuccess) e = hipEventCreate(&t1);
        if (e != hipSuccess) return e;
        (void)hipMemsetAsync(x, 0x3c, x_bytes, st);
        for (int c = 0; c < copies; ++c) (void)hipMemsetAsync(w[c], 0x3c, w_bytes, st);
        return hipSuccess;
    }
    ~TimingRig()
    {
        if (x) (void)hipFree(x);
        for (void* c : w)
            if (c) (void)hipFree(c);
        if (y) (void)hipFree(y);
        if (t0) (void)hipEventDestroy(t0);
        if (t1) (void)hipEventDestroy(t1);
    }
    // milliseconds per call of run(r) (true: queued), over `runs` calls after two that do not count; negative when a
    // call was refused; rc receives a hipError_t if the stream failed
    template <typename F>
    float time(F&& run, int runs, hipStream_t st, int& rc)
    {
        constexpr int kWarm = 2;
        bool ok = true;
        for (int r = 0; r < kWarm + runs && ok; ++r) {
            if (r == kWarm) (void)hipEventRecord(t0, st);
            ok = run(r);
        }
        (void)hipEventRecord(t1, st);
        const hipError_t e = hipEventSynchronize(t1);
        if (e != hipSuccess) {
            rc = (int)e;
            return -1.f;
        }
        if (!ok) return -1.f;
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, t0, t1);
        return ms / runs;
    }
};

// what runs the two projections of a feed-forward block that share their input: key (M, K, N, ldy, workspace or not);
// variant -1: two ordinary calls
std::map<std::tuple<int, int, int, int, int, int, int>, SkinnyConfig> g_pair_plans;      // (device, element type, M, K, N, ldy, workspace or not)

bool stream_capturing(hipStream_t st)
{
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &capturing) != hipSuccess) (void)hipGetLastError();
    return capturing != hipStreamCaptureStatusNone;
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
                          ? skinny_candidates(dtype, M, K, N, workspace_bytes, 1, own, kWantOwn) : 0;
    if (n == 0 && n_own == 0) {
        destroy_plan(p);
        return ONELLM_EUNSUPPORTED;
    }
    // the timing runs allocate, synchronise and launch: none of that may happen on a stream that is being captured
    if (stream_capturing(st)) {
        destroy_plan(p);
        return ONELLM_ECAPTURING;
    }
    const size_t esz = dtype == ONELLM_FP16 ? 2 : 4;
    int rc = 0;
    int best = -1, best_own = -1;
    float best_ms = 0.f, first_ms = 0.f, best_own_ms = 0.f;
    {
        TimingRig rig;
        if ((e = rig.make((size_t)M * K * esz, (size_t)M * ldy * esz, (size_t)K * N * esz, st)) != hipSuccess) {
            destroy_plan(p);
            return (int)e;
        }
        const float alpha = 1.f, beta = 0.f;
        const int runs = std::max(8, rig.copies);
        // candidate i of the library (i < n) or of this library's kernel (i >= n)
        for (int i = 0; i < n + n_own && rc == 0; ++i) {
            const float ms = rig.time([&](int r) {
                const void* wc = rig.w[r % rig.copies];
                if (i < n)
                    return hipblasLtMatmul(handle, p.desc, &alpha, wc, p.la, rig.x, p.lb, &beta, rig.y, p.lc, rig.y, p.lc, &cand[i].algo,
                                           workspace, workspace_bytes, st) == HIPBLAS_STATUS_SUCCESS;
                return skinny_launch(own[i - n], dtype, rig.x, wc, rig.y, nullptr, nullptr, M, K, N, ldy, workspace, workspace_bytes, st) == 0;
            }, runs, st, rc);
            if (ms < 0.f) continue;
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
    }
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

extern "C" int onellm_linear_pair_tune(int dtype, int M, int K, int N, int ldy, int w_is_nk, void* workspace, size_t workspace_bytes,
                                       onellm_stream_t stream, float* best_us, float* two_calls_us)
{
    using namespace onellm;
    // the single projection first: the two-call sequence below is what the pair has to beat
    int rc = onellm_linear_tune(dtype, M, K, N, ldy, w_is_nk, workspace, workspace_bytes, stream, nullptr, nullptr);
    if (rc != 0) return rc;
    if (ldy == 0) ldy = N;
    if (!workspace) workspace_bytes = 0;
    if (workspace_bytes > kWorkspaceBytes) workspace_bytes = kWorkspaceBytes;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    constexpr int kWantOwn = 64;
    SkinnyConfig own[kWantOwn];
    const int n_own = (tune_get("gemm_skinny") != 0 && skinny_shape_ok(dtype, M, K, N, ldy, w_is_nk))
                          ? skinny_candidates(dtype, M, K, N, workspace_bytes, 2, own, kWantOwn) : 0;
    const size_t esz = dtype == ONELLM_FP16 ? 2 : 4;
    float two_ms = -1.f, best_ms = -1.f;
    SkinnyConfig chosen;
    {
        TimingRig rig;
        // (two outputs of M rows each, one after the other)
        if ((e = rig.make((size_t)M * K * esz, 2 * (size_t)M * ldy * esz, (size_t)K * N * esz, st)) != hipSuccess) return (int)e;
        void* y_second = static_cast<char*>(rig.y) + (size_t)M * ldy * esz;
        const int runs = std::max(8, rig.copies);
        two_ms = rig.time([&](int r) {
            const void *w0 = rig.w[(2 * r) % rig.copies], *w1 = rig.w[(2 * r + 1) % rig.copies];
            return onellm_linear(dtype, rig.x, w0, rig.y, M, K, N, ldy, w_is_nk, workspace, workspace_bytes, stream) == 0 &&
                   onellm_linear(dtype, rig.x, w1, y_second, M, K, N, ldy, w_is_nk, workspace, workspace_bytes, stream) == 0;
        }, runs, st, rc);
        if (rc != 0) return rc;
        if (two_ms < 0.f) return ONELLM_EUNSUPPORTED;
        best_ms = two_ms;
        for (int i = 0; i < n_own && rc == 0; ++i) {
            const float ms = rig.time([&](int r) {
                const void *w0 = rig.w[(2 * r) % rig.copies], *w1 = rig.w[(2 * r + 1) % rig.copies];
                return skinny_launch(own[i], dtype, rig.x, w0, rig.y, w1, y_second, M, K, N, ldy, workspace, workspace_bytes, st) == 0;
            }, runs, st, rc);
            if (ms >= 0.f && ms < 0.97f * two_ms && ms < best_ms) {
                best_ms = ms;
                chosen = own[i];
            }
        }
        if (rc != 0) return rc;
    }
    {
        std::lock_guard<std::mutex> g(g_mu);
        g_pair_plans[std::make_tuple(dev, dtype, M, K, N, ldy, workspace_bytes ? 1 : 0)] = chosen;
    }
    if (best_us) *best_us = best_ms * 1e3f;
    if (two_calls_us) *two_calls_us = two_ms * 1e3f;
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
    bool no_counter_set = false;
    // this library's few-row kernel: where the tuning run chose it (tuning key gemm_skinny = 0: never; 1: wherever it
    // takes the problem, with a default configuration if none was timed)
    {
        const int want = tune_get("gemm_skinny");
        SkinnyConfig c = plan.skinny;
        if (want == 0) c = SkinnyConfig{};
        else if (want == 1 && skinny_shape_ok(dtype, M, K, N, ldy, w_is_nk)) {
            const int pick = tune_get("gemm_skinny_config");             // 100 * variant + slices along K (tests)
            if (pick >= 0) c = SkinnyConfig{pick / 100, pick % 100};
            else if (c.variant < 0) c = skinny_default(dtype, M, K, N, workspace_bytes, 1);
        }
        if (c.variant >= 0) {
            int rc = skinny_launch(c, dtype, x, w, y, nullptr, nullptr, M, K, N, ldy, workspace, workspace_bytes, st);
            if (rc == 0) {
                t_last_path = 2;
                return 0;
            }
            if (rc == kSkinnyNoCounterSet) {
                // the cut run found no arrival-counter set free: the same variant uncut, else the library; either way
                // the caller can see it (paths 4 and 5)
                no_counter_set = true;
                rc = skinny_launch(SkinnyConfig{c.variant, 1}, dtype, x, w, y, nullptr, nullptr, M, K, N, ldy, workspace, workspace_bytes, st);
                if (rc == 0) {
                    t_last_path = 4;
                    return 0;
                }
            }
            if (rc != ONELLM_EUNSUPPORTED) return rc;        // (declined as given - alignment, workspace: on to the library)
        }
    }
    if (plan.usable) {
        const float alpha = 1.f, beta = 0.f;
        const hipblasStatus_t s = hipblasLtMatmul(handle, plan.desc, &alpha, w, plan.la, x, plan.lb, &beta, y, plan.lc, y,
                                                  plan.lc, &plan.heur.algo, workspace, workspace_bytes, st);
        if (s == HIPBLAS_STATUS_SUCCESS) {
            t_last_path = no_counter_set ? 5 : 1;
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

extern "C" int onellm_linear_pair(int dtype, const void* x, const void* w_first, const void* w_second, void* y_first, void* y_second,
                                  int M, int K, int N, int ldy, int w_is_nk, void* workspace, size_t workspace_bytes,
                                  onellm_stream_t stream)
{
    using namespace onellm;
    if (dtype != ONELLM_FP32 && dtype != ONELLM_FP16) return ONELLM_EINVAL;
    if (M < 0 || K <= 0 || N <= 0) return ONELLM_EINVAL;
    if (ldy == 0) ldy = N;
    if (ldy < N) return ONELLM_EINVAL;
    if (M == 0) return 0;
    if (!x || !w_first || !w_second || !y_first || !y_second) return ONELLM_EINVAL;
    if (!workspace) workspace_bytes = 0;
    if (workspace_bytes > kWorkspaceBytes) workspace_bytes = kWorkspaceBytes;
    const int want = tune_get("gemm_skinny");
    if (want != 0 && skinny_shape_ok(dtype, M, K, N, ldy, w_is_nk)) {
        SkinnyConfig c;
        int dev = 0;
        const hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return (int)e;
        {
            std::lock_guard<std::mutex> g(g_mu);
            auto it = g_pair_plans.find(std::make_tuple(dev, dtype, M, K, N, ldy, workspace_bytes ? 1 : 0));
            if (it != g_pair_plans.end()) c = it->second;
        }
        if (want == 1) {
            const int pick = tune_get("gemm_skinny_config");
            if (pick >= 0) c = SkinnyConfig{pick / 100, pick % 100};
            else if (c.variant < 0) c = skinny_default(dtype, M, K, N, workspace_bytes, 2);
        }
        if (c.variant >= 0) {
            int rc = skinny_launch(c, dtype, x, w_first, y_first, w_second, y_second, M, K, N, ldy, workspace, workspace_bytes,
                                   static_cast<hipStream_t>(stream));
            if (rc == 0) {
                t_last_path = 3;
                return 0;
            }
            if (rc == kSkinnyNoCounterSet) {
                rc = skinny_launch(SkinnyConfig{c.variant, 1}, dtype, x, w_first, y_first, w_second, y_second, M, K, N, ldy, workspace,
                                   workspace_bytes, static_cast<hipStream_t>(stream));
                if (rc == 0) {
                    t_last_path = 4;
                    return 0;
                }
            }
            if (rc != ONELLM_EUNSUPPORTED) return rc;
        }
    }
    const int rc = onellm_linear(dtype, x, w_first, y_first, M, K, N, ldy, w_is_nk, workspace, workspace_bytes, stream);
    if (rc != 0) return rc;
    return onellm_linear(dtype, x, w_second, y_second, M, K, N, ldy, w_is_nk, workspace, workspace_bytes, stream);
}
