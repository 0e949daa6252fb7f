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

template <int TPR>
__device__ __forceinline__ float row_sum(float v, float* smem, int tid)
{
    v = wave_sum(v);
    if constexpr (TPR > kWave) {
        constexpr int NWAVE = TPR / kWave;
        if ((tid & (kWave - 1)) == 0) smem[tid / kWave] = v;
        __syncthreads();
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < NWAVE; ++w) s += smem[w];
        v = s;
    }
    return v;
}

// residual == nullptr-free: FUSED selects the add-bias-residual form at compile time.
template <typename T, int NV, int TPR, bool FUSED>
__global__ __launch_bounds__(TPR > 256 ? TPR : 256)
void norm_rows_kernel(T* __restrict__ out, T* __restrict__ residual, const T* __restrict__ bias,
                      const T* __restrict__ gamma, float eps, int N, int H)
{
    constexpr int VEC = Elt<T>::kVec;
    constexpr int BLOCK = TPR > 256 ? TPR : 256;
    constexpr int RPB = BLOCK / TPR;
    __shared__ float smem[TPR > kWave ? TPR / kWave : 1];
    const int tid = threadIdx.x;
    const int row = blockIdx.x * RPB + tid / TPR;
    const int lane = tid % TPR;
    if (row >= N) return;   // whole row-teams leave together; TPR > 64 means one team per block
    const int nvec = H / VEC;
    T* orow = out + (size_t)row * H;
    T* rrow = FUSED ? residual + (size_t)row * H : nullptr;

    Vec16<T> x[NV];
    float r[NV][VEC];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int idx = lane + j * TPR;
        if (idx < nvec) x[j] = load16_stream(orow + idx * VEC);
    }
    if constexpr (FUSED) {
        Vec16<T> y[NV];
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int idx = lane + j * TPR;
            if (idx < nvec) y[j] = load16_stream(rrow + idx * VEC);
        }
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int idx = lane + j * TPR;
            if (idx < nvec) {
                Vec16<T> b;
                if (bias) b = load16(bias + idx * VEC);
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    float v = x[j].get(e) + y[j].get(e);        // (out + residual) + bias, in this order
                    if (bias) v += b.get(e);
                    r[j][e] = v;
                    y[j].set(e, v);
                    ss = fmaf(v, v, ss);
                }
                store16_stream(rrow + idx * VEC, y[j]);
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int idx = lane + j * TPR;
            if (idx < nvec) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    r[j][e] = x[j].get(e);
                    ss = fmaf(r[j][e], r[j][e], ss);
                }
            }
        }
    }
    ss = row_sum<TPR>(ss, smem, tid);
    const float inv = rsqrtf(ss / (float)H + eps);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int idx = lane + j * TPR;
        if (idx < nvec) {
            const Vec16<T> g = load16(gamma + idx * VEC);
#pragma unroll
            for (int e = 0; e < VEC; ++e) x[j].set(e, g.get(e) * r[j][e] * inv);
            store16_stream(orow + idx * VEC, x[j]);
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
    ss = row_sum<256>(ss, smem, tid);
    const float inv = rsqrtf(ss / (float)H + eps);
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

template <typename T, int TPR, bool FUSED>
int launch_tpr(T* out, T* residual, const T* bias, const T* gamma, float eps, int N, int H, hipStream_t st)
{
    constexpr int VEC = Elt<T>::kVec;
    constexpr int BLOCK = TPR > 256 ? TPR : 256;
    constexpr int RPB = BLOCK / TPR;
    const int nvec = H / VEC;
    const int need = (nvec + TPR - 1) / TPR;
    const dim3 grid((N + RPB - 1) / RPB), block(BLOCK);
#define ONELLM_NORM_CASE(nv)                                                                                     \
    hipLaunchKernelGGL((norm_rows_kernel<T, nv, TPR, FUSED>), grid, block, 0, st, out, residual, bias, gamma, eps, N, H)
    if (need <= 1) ONELLM_NORM_CASE(1);
    else if (need <= 2) ONELLM_NORM_CASE(2);
    else if (need <= 4) ONELLM_NORM_CASE(4);
    else if (need <= 8) ONELLM_NORM_CASE(8);
    else if (need <= 16) ONELLM_NORM_CASE(16);
    else return ONELLM_EUNSUPPORTED;
#undef ONELLM_NORM_CASE
    return launch_status();
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
    int tpr = tune_get("norm_tpr");
    if (tpr != 64 && tpr != 256 && tpr != 1024) {
        // one wave per row once there are enough rows to fill the chip with independent waves and
        // the row fits a wave's registers; otherwise a workgroup per row
        const int wave_nv_cap = FUSED ? 8 : 16;
        if (N >= 2048 && nvec <= kWave * wave_nv_cap) tpr = 64;
        else if (nvec <= 256 * 16) tpr = 256;
        else tpr = 1024;
    }
    if (tpr == 64 && nvec > 64 * 16) tpr = 256;
    if (tpr == 256 && nvec > 256 * 16) tpr = 1024;
    if (tpr == 64) return launch_tpr<T, 64, FUSED>(out, residual, bias, gamma, eps, N, H, st);
    if (tpr == 256) return launch_tpr<T, 256, FUSED>(out, residual, bias, gamma, eps, N, H, st);
    return launch_tpr<T, 1024, FUSED>(out, residual, bias, gamma, eps, N, H, st);
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
