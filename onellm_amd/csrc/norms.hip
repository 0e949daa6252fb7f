// RMSNorm and fused add-bias-residual-RMSNorm for gfx950.
//
// Both are one-pass row kernels: a row is read from HBM once with 16-byte loads, kept in
// registers, reduced with DPP (plus one LDS hop when more than one wave shares a row), scaled
// and written back.  Algorithmic traffic: RMSNorm 2*N*H*e + H*e bytes, fused 4*N*H*e + 2*H*e.
// A row is owned by TPR threads (64 = one wave per row, no barrier at all; 256 or 1024 = one
// workgroup per row) holding NV 16-byte vectors each.
#include "common.hpp"

namespace onellm {
namespace {

// Sums over the TPR threads that share a row, for RPT rows at once; smem holds RPT floats per
// wave of the block.  Teams of a block reach the barrier together (callers keep whole blocks alive).
template <int TPR, int RPT>
__device__ __forceinline__ void row_sums(float (&v)[RPT], float* smem, int tid)
{
#pragma unroll
    for (int k = 0; k < RPT; ++k) v[k] = wave_sum(v[k]);
    if constexpr (TPR > kWave) {
        constexpr int NWAVE = TPR / kWave;
        const int wave = tid / kWave;
        if ((tid & (kWave - 1)) == 0) {
#pragma unroll
            for (int k = 0; k < RPT; ++k) smem[wave * RPT + k] = v[k];
        }
        __syncthreads();
        const int first = wave / NWAVE * NWAVE;
#pragma unroll
        for (int k = 0; k < RPT; ++k) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < NWAVE; ++w) s += smem[(first + w) * RPT + k];
            v[k] = s;
        }
    }
}

// A team of TPR threads owns RPT rows at a time and each thread holds NV 16-byte vectors of each:
// all RPT*NV loads (twice that when FUSED) are issued before anything is consumed, so a thread
// keeps up to 8 KiB-per-wave-sized bursts in flight; then one reduction serves the RPT rows.
// FUSED selects the add-bias-residual form at compile time.
template <typename T, int NV, int TPR, int RPT, bool FUSED>
__global__ __launch_bounds__(TPR > 256 ? TPR : 256)
void norm_rows_kernel(T* __restrict__ out, T* __restrict__ residual, const T* __restrict__ bias,
                      const T* __restrict__ gamma, float eps, int N, int H)
{
    constexpr int VEC = Elt<T>::kVec;
    constexpr int BLOCK = TPR > 256 ? TPR : 256;
    constexpr int TPB = BLOCK / TPR;             // teams per block
    __shared__ float smem[BLOCK / kWave * RPT];
    const int tid = threadIdx.x;
    const int lane = tid % TPR;
    const int row0 = (blockIdx.x * TPB + tid / TPR) * RPT;
    // one wave per team: a wave past the end simply leaves (no barrier is ever used);
    // several waves per team: every team stays for the barrier, rows past the end are empty
    if (TPR <= kWave && row0 >= N) return;
    const int nvec = H / VEC;

    // mean = sum * (1/H) instead of a division (ten instructions per thread); a zero the compiler cannot see through
    // keeps gamma * x a mixed-precision fma on the fp16 values themselves (v_fma_mix_f32: no widening instructions)
    const float inv_h = 1.0f / (float)H;
    const float zero = eps * 0.0f;
    const float one = 1.0f + zero;
    Vec16<T> x[RPT][NV];
    float ss[RPT];
    // gamma is requested with the row, not after the reduction: by then it has arrived, instead of
    // costing every workgroup a second memory round trip between its barrier and its stores
    Vec16<T> g[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int idx = lane + j * TPR;
        if (idx < nvec) g[j] = load16(gamma + idx * VEC);
    }
#pragma unroll
    for (int k = 0; k < RPT; ++k) {
        ss[k] = 0.f;
        const bool live = row0 + k < N;
        const T* orow = out + (size_t)(live ? row0 + k : 0) * H;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int idx = lane + j * TPR;
            if (live && idx < nvec) x[k][j] = load16_stream(orow + idx * VEC);
        }
    }
    if constexpr (FUSED) {
        // r = (out + residual) + bias is kept in fp32 in place of the raw inputs
        float r[RPT][NV][VEC];
        {
            Vec16<T> y[RPT][NV];
#pragma unroll
            for (int k = 0; k < RPT; ++k) {
                const bool live = row0 + k < N;
                const T* rrow = residual + (size_t)(live ? row0 + k : 0) * H;
#pragma unroll
                for (int j = 0; j < NV; ++j) {
                    const int idx = lane + j * TPR;
                    if (live && idx < nvec) y[k][j] = load16_stream(rrow + idx * VEC);
                }
            }
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const int idx = lane + j * TPR;
                Vec16<T> b;
                if (bias && idx < nvec) b = load16(bias + idx * VEC);
#pragma unroll
                for (int k = 0; k < RPT; ++k) {
                    if (row0 + k < N && idx < nvec) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) {
                            // (out + residual) + bias, in this order; the multiplications by a one the compiler
                            // cannot see through keep the additions mixed-precision fmas on the stored values
                            float v = __builtin_fmaf(x[k][j].get(e), one, y[k][j].get(e));
                            if (bias) v = __builtin_fmaf(b.get(e), one, v);
                            r[k][j][e] = v;
                            y[k][j].set(e, v);
                            ss[k] = fmaf(v, v, ss[k]);
                        }
                        store16_stream(residual + (size_t)(row0 + k) * H + idx * VEC, y[k][j]);
                    }
                }
            }
        }
        row_sums<TPR, RPT>(ss, smem, tid);
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int idx = lane + j * TPR;
            if (idx < nvec) {
#pragma unroll
                for (int k = 0; k < RPT; ++k) {
                    if (row0 + k < N) {
                        const float inv = rsqrtf(__builtin_fmaf(ss[k], inv_h, eps));
#pragma unroll
                        for (int e = 0; e < VEC; ++e) x[k][j].set(e, g[j].get(e) * r[k][j][e] * inv);
                        store16_stream(out + (size_t)(row0 + k) * H + idx * VEC, x[k][j]);
                    }
                }
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < RPT; ++k)
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const int idx = lane + j * TPR;
                if (row0 + k < N && idx < nvec) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const float v = x[k][j].get(e);
                        ss[k] = fmaf(v, v, ss[k]);
                    }
                }
            }
        row_sums<TPR, RPT>(ss, smem, tid);
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int idx = lane + j * TPR;
            if (idx < nvec) {
#pragma unroll
                for (int k = 0; k < RPT; ++k) {
                    if (row0 + k < N) {
                        const float inv = rsqrtf(__builtin_fmaf(ss[k], inv_h, eps));
#pragma unroll
                        for (int e = 0; e < VEC; ++e) x[k][j].set(e, __builtin_fmaf(g[j].get(e), x[k][j].get(e), zero) * inv);
                        store16_stream(out + (size_t)(row0 + k) * H + idx * VEC, x[k][j]);
                    }
                }
            }
        }
    }
}

// Any H, any alignment: scalar accesses, the row is read twice.  Not a performance path.
template <typename T, bool FUSED>
__global__ __launch_bounds__(256)
void norm_rows_generic_kernel(T* __restrict__ out, T* __restrict__ residual, const T* __restrict__ bias,
                              const T* __restrict__ gamma, float eps, int N, int H)
{
    __shared__ float smem[4];
    const int row = blockIdx.x, tid = threadIdx.x;
    T* orow = out + (size_t)row * H;
    T* rrow = FUSED ? residual + (size_t)row * H : nullptr;
    float ss = 0.f;
    for (int i = tid; i < H; i += 256) {
        float v = to_f32(orow[i]);
        if constexpr (FUSED) {
            v += to_f32(rrow[i]);
            if (bias) v += to_f32(bias[i]);
        }
        ss = fmaf(v, v, ss);
    }
    float sv[1] = {ss};
    row_sums<256, 1>(sv, smem, tid);
    const float inv = rsqrtf(sv[0] / (float)H + eps);
    for (int i = tid; i < H; i += 256) {
        float v = to_f32(orow[i]);
        if constexpr (FUSED) {
            v += to_f32(rrow[i]);
            if (bias) v += to_f32(bias[i]);
            rrow[i] = from_f32<T>(v);
        }
        orow[i] = from_f32<T>(to_f32(gamma[i]) * v * inv);
    }
}

template <typename T, int TPR, int RPT, bool FUSED>
int launch_team(T* out, T* residual, const T* bias, const T* gamma, float eps, int N, int H, hipStream_t st)
{
    constexpr int VEC = Elt<T>::kVec;
    constexpr int BLOCK = TPR > 256 ? TPR : 256;
    constexpr int RPB = BLOCK / TPR * RPT;       // rows per block
    const int nvec = H / VEC;
    const int need = (nvec + TPR - 1) / TPR;
    const dim3 grid((N + RPB - 1) / RPB), block(BLOCK);
#define ONELLM_NORM_CASE(nv)                                                                                          \
    hipLaunchKernelGGL((norm_rows_kernel<T, nv, TPR, RPT, FUSED>), grid, block, 0, st, out, residual, bias, gamma, eps, N, H)
    if (need <= 1) ONELLM_NORM_CASE(1);
    else if (need <= 2) ONELLM_NORM_CASE(2);
    else if (need <= 4) ONELLM_NORM_CASE(4);
    else if (need <= 8) ONELLM_NORM_CASE(8);
    else if (need <= 16) ONELLM_NORM_CASE(16);
    else return ONELLM_EUNSUPPORTED;
#undef ONELLM_NORM_CASE
    return launch_status();
}

template <typename T, int RPT, bool FUSED>
int launch_tpr(int tpr, T* out, T* residual, const T* bias, const T* gamma, float eps, int N, int H, hipStream_t st)
{
    if (tpr == 64) return launch_team<T, 64, RPT, FUSED>(out, residual, bias, gamma, eps, N, H, st);
    if (tpr == 128) return launch_team<T, 128, RPT, FUSED>(out, residual, bias, gamma, eps, N, H, st);
    if (tpr == 256) return launch_team<T, 256, RPT, FUSED>(out, residual, bias, gamma, eps, N, H, st);
    if (tpr == 512) return launch_team<T, 512, RPT, FUSED>(out, residual, bias, gamma, eps, N, H, st);
    return launch_team<T, 1024, RPT, FUSED>(out, residual, bias, gamma, eps, N, H, st);
}

template <typename T, bool FUSED>
int launch_norm(T* out, T* residual, const T* bias, const T* gamma, float eps, int N, int H, hipStream_t st)
{
    constexpr int VEC = Elt<T>::kVec;
    if (N == 0) return 0;
    const bool vec_ok = (H % VEC == 0) && aligned16(out) && aligned16(gamma) && (!FUSED || aligned16(residual))
                        && (!bias || aligned16(bias)) && (H / VEC) <= 1024 * 16;
    if (!vec_ok) {
        hipLaunchKernelGGL((norm_rows_generic_kernel<T, FUSED>), dim3(N), dim3(256), 0, st, out, residual, bias, gamma, eps, N, H);
        return launch_status();
    }
    const int nvec = H / VEC;
    // team size: one 16-byte vector per thread and row up to 512 threads, then more vectors per thread
    // (8 KiB fp16 rows -> 512 threads x 1: 23.3 / 44.4 us plain / fused at 8192 rows against 23.5 / 45.6 with
    // 256 x 2; 16 KiB rows -> 512 x 2: 44.7 / 90.8 against 47.2 / 90.4 with 1024 x 1)
    int tpr = tune_get("norm_tpr");
    if (tpr != 64 && tpr != 128 && tpr != 256 && tpr != 512 && tpr != 1024) {
        tpr = 64;
        while (tpr < 512 && nvec > tpr) tpr *= 2;
    }
    while (tpr < 1024 && nvec > tpr * 16) tpr *= 2;
    // several rows per team (2 or 4, all loads issued up front) were measured too and gave nothing
    // over one row per team on MI355X: the plateau is the read/write mix at the memory, not latency
    return launch_tpr<T, 1, FUSED>(tpr, out, residual, bias, gamma, eps, N, H, st);
}

}  // namespace
}  // namespace onellm

extern "C" int onellm_rmsnorm(int dtype, void* x, const void* gamma, float eps, int N, int H, onellm_stream_t stream)
{
    using namespace onellm;
    if (N == 0 && H > 0) return 0;   // nothing to do; an empty tensor may come with a null pointer
    if (!x || !gamma || N < 0 || H <= 0) return ONELLM_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == ONELLM_FP32)
        return launch_norm<float, false>((float*)x, nullptr, nullptr, (const float*)gamma, eps, N, H, st);
    if (dtype == ONELLM_FP16)
        return launch_norm<__half, false>((__half*)x, nullptr, nullptr, (const __half*)gamma, eps, N, H, st);
    return ONELLM_EINVAL;
}

extern "C" int onellm_fused_add_bias_residual_rmsnorm(int dtype, void* residual, void* out, const void* bias,
                                                      const void* gamma, float eps, int N, int H,
                                                      onellm_stream_t stream)
{
    using namespace onellm;
    if (N == 0 && H > 0) return 0;
    if (!residual || !out || !gamma || N < 0 || H <= 0) return ONELLM_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == ONELLM_FP32)
        return launch_norm<float, true>((float*)out, (float*)residual, (const float*)bias, (const float*)gamma, eps, N, H, st);
    if (dtype == ONELLM_FP16)
        return launch_norm<__half, true>((__half*)out, (__half*)residual, (const __half*)bias, (const __half*)gamma, eps, N, H, st);
    return ONELLM_EINVAL;
}
