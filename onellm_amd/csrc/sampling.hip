// Top-K sampling for gfx950: one lane per batch row walks the K (value, id) pairs the beam top-K
// left, draws one uniform from a counter-based generator and picks a token.  A few hundred bytes of
// traffic: launch-bound.  exp and the generator are fixed fp32 / integer operation sequences
// (Philox4x32-10, key = seed, counter = batch row), so a CPU computes the same token ids.
#include "common.hpp"

namespace onellm {
namespace {

__device__ __forceinline__ unsigned philox_first_word(unsigned c0, unsigned k0, unsigned k1)
{
    unsigned c1 = 0, c2 = 0, c3 = 0;
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const unsigned long long p0 = (unsigned long long)0xD2511F53u * c0, p1 = (unsigned long long)0xCD9E8D57u * c2;
        const unsigned n0 = (unsigned)(p1 >> 32) ^ c1 ^ k0, n1 = (unsigned)p1;
        const unsigned n2 = (unsigned)(p0 >> 32) ^ c3 ^ k1, n3 = (unsigned)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return c0;
}

// e^x for x <= 0: n = rint(x*log2 e), r = x - n*ln2 (two fma), degree-6 Horner with fma, 2^n through
// the exponent field, 0 below 2^-126
__device__ __forceinline__ float exp_fixed(float x)
{
    const float n = __builtin_rintf(x * 0x1.715476p+0f);
    float r = __builtin_fmaf(-n, 0x1.62e400p-1f, x);
    r = __builtin_fmaf(-n, 0x1.7f7d1cp-20f, r);
    float p = __builtin_fmaf(0x1.6c16c2p-10f, r, 0x1.111112p-7f);
    p = __builtin_fmaf(p, r, 0x1.555556p-5f);
    p = __builtin_fmaf(p, r, 0x1.555556p-3f);
    p = __builtin_fmaf(p, r, 0.5f);
    p = __builtin_fmaf(p, r, 1.0f);
    p = __builtin_fmaf(p, r, 1.0f);
    const int e = (int)n;
    if (e < -126) return 0.0f;
    return p * __uint_as_float((unsigned)(e + 127) << 23);
}

__global__ __launch_bounds__(64)
void topk_sample_kernel(const int* __restrict__ topk_id, const float* __restrict__ topk_val, int* __restrict__ output_id,
                        int* __restrict__ seqlen, unsigned char* __restrict__ is_finished, int B, int K,
                        unsigned seed_lo, unsigned seed_hi, int end_id, int vocab_size)
{
    const int b = blockIdx.x * 64 + threadIdx.x;
    if (b >= B) return;
    const float* v = topk_val + (size_t)b * K;
    const float v0 = v[0];
    float sum = 0.0f;
    for (int i = 0; i < K; ++i) sum += exp_fixed(v[i] - v0);
    const unsigned x = philox_first_word((unsigned)b, seed_lo, seed_hi);
    float thr = __builtin_fmaf((float)x, 0x1.0p-32f, 0x1.0p-32f) * sum;       // u in (0, 1]
    int pick = K - 1;
    for (int i = 0; i < K; ++i) {
        thr -= exp_fixed(v[i] - v0);
        if (thr < 0) {
            pick = i;
            break;
        }
    }
    const int id = topk_id[(size_t)b * K + pick] % vocab_size;
    output_id[b] = id;
    if (!is_finished[b]) seqlen[b] += 1;
    is_finished[b] = id == end_id ? 1 : 0;
}

}  // namespace
}  // namespace onellm

extern "C" int onellm_topk_sample(const int* topk_id, const float* topk_val, int* output_id, int* seqlen,
                                  unsigned char* is_finished, int B, int K, unsigned long long seed, int end_id,
                                  int vocab_size, onellm_stream_t stream)
{
    using namespace onellm;
    if (B == 0 && K > 0) return 0;
    if (!topk_id || !topk_val || !output_id || !seqlen || !is_finished || B < 0 || K <= 0 || vocab_size <= 0) return ONELLM_EINVAL;
    hipLaunchKernelGGL(topk_sample_kernel, dim3((B + 63) / 64), dim3(64), 0, static_cast<hipStream_t>(stream), topk_id, topk_val,
                       output_id, seqlen, is_finished, B, K, (unsigned)seed, (unsigned)(seed >> 32), end_id, vocab_size);
    return launch_status();
}
