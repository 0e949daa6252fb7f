// RoPE pieces shared by the decode and the prefill kernels: the frequency table that travels to a
// kernel by value, and sin/cos as a fixed operation sequence.
#pragma once
#include <math.h>
#include "common.hpp"

namespace onellm {

constexpr int kMaxPairs = 256;                 // D <= 512
struct RopeFreqs { float f[kMaxPairs]; };      // f[i] = base^(2i/rotary_dim), filled on the host

// sin/cos as a fixed sequence of fp32 IEEE operations: 3-term Cody-Waite reduction by pi/2, the
// single-precision minimax polynomials on [-pi/4, pi/4], quadrant from the multiple.  Every
// multiply-add is an explicit fma so that a host implementation of the same sequence gives the
// same bits (the K row written to the cache is bit-reproducible on a CPU).
__device__ __forceinline__ void sincos_fixed(float x, float& s_out, float& c_out)
{
    const float j = __builtin_rintf(x * 0x1.45f306p-1f);
    float r = __builtin_fmaf(-j, 0x1.921fb6p+0f, x);
    r = __builtin_fmaf(-j, -0x1.777a5cp-25f, r);
    r = __builtin_fmaf(-j, -0x1.0p-49f, r);
    const float r2 = r * r;
    float ps = __builtin_fmaf(-1.9515295891e-4f, r2, 8.3321608736e-3f);
    ps = __builtin_fmaf(ps, r2, -1.6666654611e-1f);
    const float sr = __builtin_fmaf(r * r2, ps, r);
    float pc = __builtin_fmaf(2.443315711809948e-5f, r2, -1.388731625493765e-3f);
    pc = __builtin_fmaf(pc, r2, 4.166664568298827e-2f);
    const float cr = __builtin_fmaf(r2 * r2, pc, __builtin_fmaf(-0.5f, r2, 1.0f));
    const int q = (int)j & 3;
    float s = (q & 1) ? cr : sr;
    float c = (q & 1) ? sr : cr;
    if (q & 2) s = -s;
    if ((q + 1) & 2) c = -c;
    s_out = s;
    c_out = c;
}

// rotate the pair (x0, x1) of index `pair` at position pos
__device__ __forceinline__ void rope_pair(float& x0, float& x1, int pair, int pos, const RopeFreqs& fr)
{
    const float ang = (float)pos / fr.f[pair];
    float s, c;
    sincos_fixed(ang, s, c);
    const float a = __builtin_fmaf(x0, c, -(x1 * s));
    const float b = __builtin_fmaf(x1, c, x0 * s);
    x0 = a;
    x1 = b;
}


// freq[i] = base^(2i/rotary_dim) for the pairs that exist (2i < rotary_dim, 2i+1 < D), with libm powf on the host
inline void fill_rope_freqs(RopeFreqs& fr, int D, int rotary_dim, float base)
{
    for (int i = 0; 2 * i < rotary_dim && 2 * i + 1 < D && i < kMaxPairs; ++i)
        fr.f[i] = powf(base, (float)(2 * i) / (float)rotary_dim);
}

}  // namespace onellm
