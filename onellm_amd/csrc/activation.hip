// SwiGLU gate for gfx950: out[b, i] = silu(in[b, 0, i]) * in[b, 1, i], silu(x) = x / (1 + exp(-x)) in
// fp32.  One or two 16-byte pieces of the output per thread, non-temporal streams; HBM-bound: 3*B*I*e bytes.
#include "common.hpp"

namespace onellm {
namespace {

// the reciprocal is the hardware's (v_rcp_f32, 1 ulp) rather than an IEEE division: ten instructions fewer per
// element in a kernel whose vector ALU is more than half busy
__device__ __forceinline__ float silu_mul(float x, float y) { return (x * __builtin_amdgcn_rcpf(1.0f + __expf(-x))) * y; }

template <typename T, int NV>
__global__ __launch_bounds__(256)
void silu_and_mul_kernel(T* __restrict__ out, const T* __restrict__ in, int I)
{
    constexpr int VEC = Elt<T>::kVec;
    const int b = blockIdx.y;
    const int nvec = I / VEC;
    const T* row = in + (size_t)b * 2 * I;
    Vec16<T> x[NV], y[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int v = (blockIdx.x * NV + j) * 256 + threadIdx.x;
        if (v < nvec) {
            x[j] = load16_stream(row + v * VEC);
            y[j] = load16_stream(row + I + v * VEC);
        }
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int v = (blockIdx.x * NV + j) * 256 + threadIdx.x;
        if (v < nvec) {
            Vec16<T> o;
#pragma unroll
            for (int e = 0; e < VEC; ++e) o.set(e, silu_mul(x[j].get(e), y[j].get(e)));
            store16_stream(out + (size_t)b * I + v * VEC, o);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256)
void silu_and_mul_scalar_kernel(T* __restrict__ out, const T* __restrict__ in, int I)
{
    const int b = blockIdx.y;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= I) return;
    const T* row = in + (size_t)b * 2 * I;
    out[(size_t)b * I + i] = from_f32<T>(silu_mul(to_f32(row[i]), to_f32(row[I + i])));
}

template <typename T>
int launch_act(const T* in, T* out, int B, int I, hipStream_t st)
{
    constexpr int VEC = Elt<T>::kVec;
    if (B > 65535) return ONELLM_EUNSUPPORTED;
    if (I % VEC == 0 && aligned16(in) && aligned16(out)) {
        // two pieces per thread (four loads in flight) where a row has more than 256 pieces: 86.2 us against 89-90 us
        // with one piece at 8192 x 11008 fp16 (four pieces: 105 us, the row's last workgroup is then mostly idle)
        if (I / VEC > 256) hipLaunchKernelGGL((silu_and_mul_kernel<T, 2>), dim3((I / VEC + 511) / 512, B), dim3(256), 0, st, out, in, I);
        else hipLaunchKernelGGL((silu_and_mul_kernel<T, 1>), dim3((I / VEC + 255) / 256, B), dim3(256), 0, st, out, in, I);
    } else {
        hipLaunchKernelGGL((silu_and_mul_scalar_kernel<T>), dim3((I + 255) / 256, B), dim3(256), 0, st, out, in, I);
    }
    return launch_status();
}

}  // namespace
}  // namespace onellm

extern "C" int onellm_silu_and_mul(int dtype, const void* input, void* out, int B, int I, onellm_stream_t stream)
{
    using namespace onellm;
    if (B == 0 && I > 0) return 0;
    if (!input || !out || B < 0 || I <= 0) return ONELLM_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == ONELLM_FP32) return launch_act<float>((const float*)input, (float*)out, B, I, st);
    if (dtype == ONELLM_FP16) return launch_act<__half>((const __half*)input, (__half*)out, B, I, st);
    return ONELLM_EINVAL;
}
