// RMSNorm and fused add-bias-residual-RMSNorm for gfx950.
//
// Both are one-pass row kernels: a row is read from HBM once with 16-byte loads, kept in registers, reduced with
// DPP (plus one LDS hop when more than one wave shares a row), scaled and written back.  Algorithmic traffic:
// RMSNorm 2*N*H*e + H*e bytes, fused 4*N*H*e + 2*H*e.  A row is owned by a team of TPR threads holding NV 16-byte
// vectors each: one wave (no barrier at all) or two waves for short rows, several teams to a 256-thread workgroup;
// a whole workgroup of 256, 512 or 1024 threads for rows of more than 128 vectors.
#include "common.hpp"

namespace onellm {
namespace {

// ---------------------------------------------------------------- buffer accesses
//
// A team of TPR threads per row, NV vectors per thread.  Loads and stores are raw buffer accesses whose
// descriptor covers exactly the row, so a lane past the row's end reads zeros and stores nothing - there is no
// branch anywhere - and the cache policy is chosen per access: the row is read non-temporally and written
// non-temporally + write-through (measured on MI355X with a read-reduce-write kernel of this shape over 64 MiB:
// 24.6 us with plain accesses, 21.5 us non-temporal both ways, 21.1 us with the write-through bit on the store).
// The arithmetic is kept to what the memory pipeline leaves room for: the sum of squares of fp16 pairs is one
// dot instruction per pair (exact products, fp32 accumulation), gamma is folded into the row's scale once
// (gamma * inv as a mixed-precision fma on the stored fp16 value), and the result is one mixed-precision fma and
// half a packed conversion per element.

constexpr int kAuxPlain = 0;
constexpr int kAuxStreamLoad = 2;        // nt
constexpr int kAuxStreamStore = 2 | 16;  // nt + sc1

__device__ __forceinline__ __amdgpu_buffer_rsrc_t row_descriptor(const void* base, unsigned bytes)
{
    // raw buffer (stride 0): an access is dropped when offset + size exceeds `bytes`
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

typedef int i32x4 __attribute__((ext_vector_type(4)));

template <typename T, int AUX>
__device__ __forceinline__ Vec16<T> buffer_load16(__amdgpu_buffer_rsrc_t r, unsigned byte_offset)
{
    Vec16<T> v;
    v.raw = __builtin_bit_cast(decltype(v.raw), __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_offset, 0, AUX));
    return v;
}
template <typename T, int AUX>
__device__ __forceinline__ void buffer_store16(__amdgpu_buffer_rsrc_t r, unsigned byte_offset, const Vec16<T>& v)
{
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, v.raw), r, (int)byte_offset, 0, AUX);
}

// sum of the squares of the 16 bytes' elements, added to acc
__device__ __forceinline__ float sum_squares(const Vec16<float>& v, float acc)
{
#pragma unroll
    for (int e = 0; e < 4; ++e) acc = fmaf(v.raw[e], v.raw[e], acc);
    return acc;
}
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float sum_squares(const Vec16<__half>& v, float acc)
{
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
        const f16x2 pr = {v.raw[e], v.raw[e + 1]};
        acc = __builtin_amdgcn_fdot2(pr, pr, acc, false);
    }
    return acc;
}

// Total over the wave, valid in lane 63 only: row sums by DPP, then the two row broadcasts.
__device__ __forceinline__ float wave_sum_in_last_lane(float v)
{
    v += dpp_f32<kDppQuadXor1>(v);
    v += dpp_f32<kDppQuadXor2>(v);
    v += dpp_f32<kDppRowHalfMirror>(v);
    v += dpp_f32<kDppRowMirror>(v);
    // row_bcast:15 into rows 1 and 3, row_bcast:31 into rows 2 and 3 (lanes of the other rows keep their value)
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xA, 0xF, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xC, 0xF, false));
    return v;
}

template <typename T, int NV, int TPR, bool FUSED>
__global__ __launch_bounds__(TPR > 256 ? TPR : 256)
void norm_row_kernel(T* __restrict__ out, T* __restrict__ residual, const T* __restrict__ bias,
                     const T* __restrict__ gamma, float eps, int N, int H)
{
    constexpr int VEC = Elt<T>::kVec;
    constexpr int BLOCK = TPR > 256 ? TPR : 256;
    constexpr int TPB = BLOCK / TPR;              // teams (rows) per workgroup
    constexpr int NWAVE = TPR / kWave;            // waves per team
    __shared__ float smem[BLOCK / kWave];
    const int tid = threadIdx.x;
    const int lane = tid % TPR;
    // the row a wave works on is the same for all its lanes: say so, the descriptors live in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int row_id = blockIdx.x * TPB + wave / NWAVE;
    // a team past the last row keeps running with empty descriptors (every load gives zeros, every store is
    // dropped), so that all waves of the workgroup reach the barrier
    const unsigned row_bytes = row_id < N ? (unsigned)H * (unsigned)sizeof(T) : 0u;
    const size_t row = (size_t)(row_id < N ? row_id : 0) * H;
    const __amdgpu_buffer_rsrc_t d_out = row_descriptor(out + row, row_bytes);
    const __amdgpu_buffer_rsrc_t d_gamma = row_descriptor(gamma, row_bytes);
    const float inv_h = 1.0f / (float)H;
    const float zero = eps * 0.0f;          // a zero and a one the compiler cannot see through keep the fp16
    const float one = 1.0f + zero;          // operands inside mixed-precision fmas (no widening instructions)

    // gamma is requested right behind the row, so that it has arrived when the reduction is done - except in the
    // one form whose registers that would overflow (fused, fp16, eight vectors per thread: rows beyond 32 Ki elements)
    constexpr bool kLateGamma = FUSED && NV >= 8 && sizeof(T) == 2;
    Vec16<T> g[NV], x[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) x[j] = buffer_load16<T, kAuxStreamLoad>(d_out, (unsigned)(lane + j * TPR) * 16u);
    if constexpr (!kLateGamma) {
#pragma unroll
        for (int j = 0; j < NV; ++j) g[j] = buffer_load16<T, kAuxPlain>(d_gamma, (unsigned)(lane + j * TPR) * 16u);
    }
    float ss = 0.f;
    float r[FUSED ? NV : 1][VEC];
    if constexpr (FUSED) {
        const __amdgpu_buffer_rsrc_t d_res = row_descriptor(residual + row, row_bytes);
        const __amdgpu_buffer_rsrc_t d_bias = row_descriptor(bias, bias ? row_bytes : 0u);   // no bias: zeros
        Vec16<T> y[NV], b[NV];
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const unsigned off = (unsigned)(lane + j * TPR) * 16u;
            y[j] = buffer_load16<T, kAuxStreamLoad>(d_res, off);
            if constexpr (!kLateGamma) b[j] = buffer_load16<T, kAuxPlain>(d_bias, off);
        }
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            // (the register-bound form fetches its bias vector by vector, a cache hit each)
            if constexpr (kLateGamma) b[j] = buffer_load16<T, kAuxPlain>(d_bias, (unsigned)(lane + j * TPR) * 16u);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                // (out + residual) + bias in fp32, in this order
                float v = __builtin_fmaf(x[j].get(e), one, y[j].get(e));
                v = __builtin_fmaf(b[j].get(e), one, v);
                r[j][e] = v;
                y[j].set(e, v);
                ss = fmaf(v, v, ss);
            }
            buffer_store16<T, kAuxStreamStore>(d_res, (unsigned)(lane + j * TPR) * 16u, y[j]);
        }
    } else {
#pragma unroll
        for (int j = 0; j < NV; ++j) ss = sum_squares(x[j], ss);
    }
    float total;
    if constexpr (NWAVE == 1) {
        total = wave_sum(ss);
    } else {
        ss = wave_sum_in_last_lane(ss);
        if ((tid & (kWave - 1)) == kWave - 1) smem[wave] = ss;
        __syncthreads();
        total = 0.f;
        const int first = wave / NWAVE * NWAVE;
#pragma unroll
        for (int w = 0; w < NWAVE; ++w) total += smem[first + w];
    }
    const float inv = rsqrtf(__builtin_fmaf(total, inv_h, eps));
    if constexpr (kLateGamma) {
#pragma unroll
        for (int j = 0; j < NV; ++j) g[j] = buffer_load16<T, kAuxPlain>(d_gamma, (unsigned)(lane + j * TPR) * 16u);
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float gs = __builtin_fmaf(g[j].get(e), inv, zero);
            if constexpr (FUSED) x[j].set(e, r[j][e] * gs);
            else x[j].set(e, __builtin_fmaf(x[j].get(e), gs, zero));
        }
        buffer_store16<T, kAuxStreamStore>(d_out, (unsigned)(lane + j * TPR) * 16u, x[j]);
    }
}

template <typename T, int NV, int TPR, bool FUSED>
int launch_row(T* out, T* residual, const T* bias, const T* gamma, float eps, int N, int H, hipStream_t st)
{
    constexpr int BLOCK = TPR > 256 ? TPR : 256;
    constexpr int TPB = BLOCK / TPR;
    hipLaunchKernelGGL((norm_row_kernel<T, NV, TPR, FUSED>), dim3((N + TPB - 1) / TPB), dim3(BLOCK), 0, st,
                       out, residual, bias, gamma, eps, N, H);
    return launch_status();
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
    ss = wave_sum(ss);
    if ((tid & (kWave - 1)) == 0) smem[tid / kWave] = ss;
    __syncthreads();
    const float inv = rsqrtf((smem[0] + smem[1] + smem[2] + smem[3]) / (float)H + eps);
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

// Team size and vectors per thread: a wave or two for short rows; 256 threads up to 256 vectors, 512 threads up
// to 2048 (one, two or four vectors each: measured best on MI355X at 8 KiB and 16 KiB rows - 256 threads x 2 and
// 1024 x 1 are 0.5-45 % slower), 1024 threads with four or eight beyond.  `forced` (a tuning knob) picks the
// team size where the row fits it.
template <typename T, bool FUSED>
int launch_norm(T* out, T* residual, const T* bias, const T* gamma, float eps, int N, int H, hipStream_t st)
{
    constexpr int VEC = Elt<T>::kVec;
    if (N == 0) return 0;
    const int nvec = H / VEC;
    const bool vec_ok = (H % VEC == 0) && aligned16(out) && aligned16(gamma) && (!FUSED || aligned16(residual))
                        && (!bias || aligned16(bias)) && nvec <= 1024 * 8;
    if (!vec_ok) {
        hipLaunchKernelGGL((norm_rows_generic_kernel<T, FUSED>), dim3(N), dim3(256), 0, st, out, residual, bias, gamma, eps, N, H);
        return launch_status();
    }
    int tpr = nvec <= 64 ? 64 : nvec <= 128 ? 128 : nvec <= 256 ? 256 : nvec <= 2048 ? 512 : 1024;
    const int forced = tune_get("norm_tpr");
    if ((forced == 64 || forced == 128 || forced == 256 || forced == 512 || forced == 1024)
        && nvec <= forced * (forced >= 1024 ? 8 : forced >= 256 ? 4 : 1))
        tpr = forced;
    const int nv = (nvec + tpr - 1) / tpr;
#define ONELLM_NORM_CASE(NV, TPR) return launch_row<T, NV, TPR, FUSED>(out, residual, bias, gamma, eps, N, H, st)
    switch (tpr) {
        case 64: ONELLM_NORM_CASE(1, 64);
        case 128: ONELLM_NORM_CASE(1, 128);
        case 256:
            if (nv <= 1) ONELLM_NORM_CASE(1, 256);
            if (nv <= 2) ONELLM_NORM_CASE(2, 256);
            ONELLM_NORM_CASE(4, 256);
        case 512:
            if (nv <= 1) ONELLM_NORM_CASE(1, 512);
            if (nv <= 2) ONELLM_NORM_CASE(2, 512);
            ONELLM_NORM_CASE(4, 512);
        default:
            if (nv <= 1) ONELLM_NORM_CASE(1, 1024);
            if (nv <= 2) ONELLM_NORM_CASE(2, 1024);
            if (nv <= 4) ONELLM_NORM_CASE(4, 1024);
            ONELLM_NORM_CASE(8, 1024);
    }
#undef ONELLM_NORM_CASE
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
