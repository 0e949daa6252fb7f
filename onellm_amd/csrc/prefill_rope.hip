// Context-phase fused QKV bias + RoPE + un-pad transpose for gfx950: the producer of the K/V rows the
// decode kernel streams.  A workgroup takes a few consecutive packed tokens: the sin/cos of their
// positions are computed once into LDS (the same fixed fp32 sequence as the decode kernel, so prefill
// and decode agree bit for bit), then every (head, token, 16-byte piece) is read once, biased, rotated
// (q and k heads) and stored at its [batch, head, position] place.  HBM-bound:
// 2 * token_num * (Hq+2Hkv) * D * e bytes.
#include "common.hpp"
#include "rope.hpp"

namespace onellm {
namespace {

struct PrefillArgs {
    void* q_buf;
    void* k_buf;
    void* v_buf;
    const void* qkv;
    const void* bias;
    const int* padding_offset;
    const int* history_length;
    int B, seq_len, Hq, Hkv, D, rotary_dim;
};

constexpr int kTokensPerGroup = 4;

// A workgroup handles kTokensPerGroup consecutive packed tokens.  Pieces are dealt so that, for one
// head, the lanes of a wave cover the same columns of consecutive tokens: the tokens of a sequence sit
// next to each other in [batch, head, position, D], so the transposed stores of a wave are contiguous
// (1 KiB at D = 128 fp16) instead of one 256-byte piece per head.
// VECTOR: 16-byte accesses (needs D % (16/e) == 0 and aligned buffers); otherwise one pair per access.
template <typename T, bool VECTOR>
__global__ __launch_bounds__(256)
void qkv_bias_rope_transpose_kernel(const PrefillArgs a, const RopeFreqs fr, int token_num)
{
    constexpr int VEC = VECTOR ? Elt<T>::kVec : 2;
    constexpr int TT = kTokensPerGroup;
    __shared__ float ssin[TT][kMaxPairs], scos[TT][kMaxPairs];
    __shared__ long s_dst[TT];        // destination row of each token inside [B, *, seq_len, D], -1 = skip
    __shared__ int s_b[TT];
    const int tok0 = blockIdx.x * TT, tid = threadIdx.x;
    const int D = a.D, QKVH = a.Hq + 2 * a.Hkv;
    const int npair = min(a.rotary_dim, D) / 2;          // pairs (2p, 2p+1) with 2p < rotary_dim inside the head
    if (tid < TT) {
        const int tok = tok0 + tid;
        long srow = -1;
        int bb = 0;
        if (tok < token_num) {
            const long dst = (long)tok + a.padding_offset[tok];
            const long b = dst / a.seq_len;
            if (dst >= 0 && b < a.B) {                    // a token outside the batch touches nothing
                srow = dst % a.seq_len;
                bb = (int)b;
            }
        }
        s_dst[tid] = srow;
        s_b[tid] = bb;
    }
    __syncthreads();
    for (int i = tid; i < TT * npair; i += 256) {
        const int tl = i / npair, p = i % npair;
        if (s_dst[tl] >= 0) {
            const int pos = a.history_length[s_b[tl]] + (int)s_dst[tl];
            float sn, cs;
            sincos_fixed((float)pos / fr.f[p], sn, cs);
            ssin[tl][p] = sn;
            scos[tl][p] = cs;
        }
    }
    __syncthreads();
    const T* bias = static_cast<const T*>(a.bias);
    const int nvec = D / VEC;
    const int total = QKVH * TT * nvec;
    for (int i = tid; i < total; i += 256) {
        const int c = (i % nvec) * VEC;
        const int tl = (i / nvec) % TT;
        const int h = i / (nvec * TT);
        const long s = s_dst[tl];
        if (s < 0) continue;
        const int b = s_b[tl];
        const T* in = static_cast<const T*>(a.qkv) + ((size_t)(tok0 + tl) * QKVH + h) * D + c;
        float x[VEC];
        if constexpr (VECTOR) {
            const Vec16<T> v = load16_stream(in);
#pragma unroll
            for (int e = 0; e < VEC; ++e) x[e] = v.get(e);
            if (bias) {
                const Vec16<T> bv = load16(bias + (size_t)h * D + c);
#pragma unroll
                for (int e = 0; e < VEC; ++e) x[e] += bv.get(e);
            }
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                x[e] = to_f32(in[e]);
                if (bias) x[e] += to_f32(bias[(size_t)h * D + c + e]);
            }
        }
        T* out;
        if (h < a.Hq) {
            out = static_cast<T*>(a.q_buf) + (((size_t)b * a.Hq + h) * a.seq_len + (size_t)s) * D;
        } else if (h < a.Hq + a.Hkv) {
            out = static_cast<T*>(a.k_buf) + (((size_t)b * a.Hkv + (h - a.Hq)) * a.seq_len + (size_t)s) * D;
        } else {
            out = static_cast<T*>(a.v_buf) + (((size_t)b * a.Hkv + (h - a.Hq - a.Hkv)) * a.seq_len + (size_t)s) * D;
        }
        if (h < a.Hq + a.Hkv) {
#pragma unroll
            for (int e = 0; e < VEC; e += 2) {
                const int p = (c + e) >> 1;
                if (p < npair) {
                    const float sn = ssin[tl][p], cs = scos[tl][p];
                    const float r0 = __builtin_fmaf(x[e], cs, -(x[e + 1] * sn));
                    const float r1 = __builtin_fmaf(x[e + 1], cs, x[e] * sn);
                    x[e] = r0;
                    x[e + 1] = r1;
                }
            }
        }
        if constexpr (VECTOR) {
            Vec16<T> o;
#pragma unroll
            for (int e = 0; e < VEC; ++e) o.set(e, x[e]);
            store16_stream(out + c, o);
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) out[c + e] = from_f32<T>(x[e]);
        }
    }
}

// The same work for head sizes whose rows are a power-of-two number of 16-byte pieces (NVEC of them,
// at most 64): a thread then keeps one (token, piece) for the whole workgroup and only walks the
// heads, so its destination row and the sin/cos of its pairs are computed once into registers (no
// LDS, no barrier, no index division in the loop), and the loads of UNROLL heads are issued before
// any of them is used.  With 8 tokens per workgroup a head's rows leave as 2 KiB contiguous stores.
// 5.55 TB/s against 5.15 TB/s for the loop above at 4 x 2048 tokens x 96 heads x 128 fp16; results are
// bit-identical to it.
template <typename T, int NVEC, int TT>
__global__ __launch_bounds__(256)
void qkv_bias_rope_transpose_rows_kernel(const PrefillArgs a, const RopeFreqs fr, int token_num)
{
    constexpr int VEC = Elt<T>::kVec;
    constexpr int GROUP = NVEC * TT;              // threads that share a head
    constexpr int HPP = 256 / GROUP;              // heads per pass of the workgroup
    constexpr int UNROLL = 8;
    static_assert(GROUP >= 1 && GROUP <= 256 && 256 % GROUP == 0, "pieces per row");
    const int tid = threadIdx.x;
    const int c = (tid % NVEC) * VEC, tl = (tid / NVEC) % TT, h0 = tid / GROUP;
    const int D = NVEC * VEC, QKVH = a.Hq + 2 * a.Hkv;
    const int tok = blockIdx.x * TT + tl;
    if (tok >= token_num) return;
    // the first heads of the token are requested before its destination is known: where it goes (padding
    // offset -> sequence -> history length, two dependent loads) and the sin / cos of its pairs are worked out
    // while they travel - every workgroup of the launch starts at the same time, so nothing else covers that wait
    const T* in = static_cast<const T*>(a.qkv) + (size_t)tok * (a.Hq + 2 * a.Hkv) * (NVEC * VEC) + c;
    const T* bias = static_cast<const T*>(a.bias);
    Vec16<T> v[UNROLL], bv[UNROLL];
    auto request = [&](int hb) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int h = hb + u * HPP;
            if (h < a.Hq + 2 * a.Hkv) {
                v[u] = load16_stream(in + (size_t)h * (NVEC * VEC));
                if (bias) bv[u] = load16(bias + (size_t)h * (NVEC * VEC) + c);
            }
        }
    };
    request(h0);
    const long dst = (long)tok + a.padding_offset[tok];
    const long b = dst / a.seq_len;
    if (dst < 0 || b >= a.B) return;              // a token outside the batch touches nothing
    const long srow = dst % a.seq_len;
    const int pos = a.history_length[b] + (int)srow;
    const int npair = min(a.rotary_dim, D) / 2;
    float sn[VEC / 2], cs[VEC / 2];
#pragma unroll
    for (int e = 0; e < VEC / 2; ++e) {
        const int p = (c >> 1) + e;
        sn[e] = 0.f;
        cs[e] = 1.f;
        if (p < npair) sincos_fixed((float)pos / fr.f[p], sn[e], cs[e]);
    }
    T* qo = static_cast<T*>(a.q_buf) + ((size_t)b * a.Hq * a.seq_len + (size_t)srow) * D + c;
    T* ko = static_cast<T*>(a.k_buf) + ((size_t)b * a.Hkv * a.seq_len + (size_t)srow) * D + c;
    T* vo = static_cast<T*>(a.v_buf) + ((size_t)b * a.Hkv * a.seq_len + (size_t)srow) * D + c;
    const size_t head_step = (size_t)a.seq_len * D;
    for (int hb = h0; hb < QKVH; hb += HPP * UNROLL) {
        if (hb != h0) request(hb);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int h = hb + u * HPP;
            if (h >= QKVH) break;
            float x[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) x[e] = v[u].get(e);
            if (bias) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) x[e] += bv[u].get(e);
            }
            const bool rotate = h < a.Hq + a.Hkv;
#pragma unroll
            for (int e = 0; e < VEC; e += 2) {
                // the pairs past rotary_dim keep sin = 0, cos = 1 but must stay untouched bit for bit
                const bool on = rotate && ((c + e) >> 1) < npair;
                const float r0 = __builtin_fmaf(x[e], cs[e / 2], -(x[e + 1] * sn[e / 2]));
                const float r1 = __builtin_fmaf(x[e + 1], cs[e / 2], x[e] * sn[e / 2]);
                x[e] = on ? r0 : x[e];
                x[e + 1] = on ? r1 : x[e + 1];
            }
            T* out = h < a.Hq ? qo + (size_t)h * head_step
                              : (h < a.Hq + a.Hkv ? ko + (size_t)(h - a.Hq) * head_step : vo + (size_t)(h - a.Hq - a.Hkv) * head_step);
            Vec16<T> o;
#pragma unroll
            for (int e = 0; e < VEC; ++e) o.set(e, x[e]);
            store16_stream(out, o);
        }
    }
}

// Tokens per workgroup: 8 where a row has at most 32 pieces (4 x 2048 tokens x 96 heads x 128 fp16: 72.5 us with 8,
// 76-77 us with 4 or 16; splitting the heads of a token over several workgroups only loses), else 4.
template <typename T, int NVEC>
void launch_rows(const PrefillArgs& a, const RopeFreqs& fr, int token_num, hipStream_t st)
{
    constexpr int TT = NVEC * 8 <= 256 ? 8 : kTokensPerGroup;
    hipLaunchKernelGGL((qkv_bias_rope_transpose_rows_kernel<T, NVEC, TT>), dim3((token_num + TT - 1) / TT), dim3(256), 0, st, a, fr,
                       token_num);
}

template <typename T>
int launch_prefill(const PrefillArgs& a, const RopeFreqs& fr, int token_num, bool vec, hipStream_t st)
{
    const dim3 grid((token_num + kTokensPerGroup - 1) / kTokensPerGroup);
    if (vec && tune_get("prefill_generic") != 1) {
        const int nvec = a.D / Elt<T>::kVec;
        bool done = true;
        switch (nvec) {
            case 1: launch_rows<T, 1>(a, fr, token_num, st); break;
            case 2: launch_rows<T, 2>(a, fr, token_num, st); break;
            case 4: launch_rows<T, 4>(a, fr, token_num, st); break;
            case 8: launch_rows<T, 8>(a, fr, token_num, st); break;
            case 16: launch_rows<T, 16>(a, fr, token_num, st); break;
            case 32: launch_rows<T, 32>(a, fr, token_num, st); break;
            case 64: launch_rows<T, 64>(a, fr, token_num, st); break;
            default: done = false; break;
        }
        if (done) return launch_status();
    }
    if (vec) hipLaunchKernelGGL((qkv_bias_rope_transpose_kernel<T, true>), grid, dim3(256), 0, st, a, fr, token_num);
    else hipLaunchKernelGGL((qkv_bias_rope_transpose_kernel<T, false>), grid, dim3(256), 0, st, a, fr, token_num);
    return launch_status();
}

}  // namespace
}  // namespace onellm

extern "C" int onellm_qkv_bias_rope_transpose(int dtype, void* q_buf, void* k_buf, void* v_buf, const void* qkv,
                                              const void* qkv_bias, const int* padding_offset, const int* history_length,
                                              int B, int seq_len, int token_num, int Hq, int Hkv, int D,
                                              int rotary_dim, float rope_base, onellm_stream_t stream)
{
    using namespace onellm;
    if (token_num == 0 && B > 0) return 0;
    if (!q_buf || !k_buf || !v_buf || !qkv || !padding_offset || !history_length) return ONELLM_EINVAL;
    if (B <= 0 || seq_len <= 0 || token_num < 0 || Hq <= 0 || Hkv <= 0 || D <= 0) return ONELLM_EINVAL;
    if (dtype != ONELLM_FP32 && dtype != ONELLM_FP16) return ONELLM_EINVAL;
    if (rotary_dim < 0 || (rotary_dim > 0 && !(rope_base > 0.f))) return ONELLM_EINVAL;
    if ((D & 1) || D > 2 * kMaxPairs) return ONELLM_EUNSUPPORTED;
    const int vec_elts = dtype == ONELLM_FP16 ? 8 : 4;
    const bool vec = D % vec_elts == 0 && aligned16(q_buf) && aligned16(k_buf) && aligned16(v_buf) && aligned16(qkv)
                     && (!qkv_bias || aligned16(qkv_bias));
    PrefillArgs a{q_buf, k_buf, v_buf, qkv, qkv_bias, padding_offset, history_length, B, seq_len, Hq, Hkv, D, rotary_dim};
    RopeFreqs fr;
    fill_rope_freqs(fr, D, rotary_dim, rope_base);
    hipStream_t st = static_cast<hipStream_t>(stream);
    return dtype == ONELLM_FP16 ? launch_prefill<__half>(a, fr, token_num, vec, st)
                                : launch_prefill<float>(a, fr, token_num, vec, st);
}
