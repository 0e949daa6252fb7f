// Decode attention on the vector ALU: rows of LPR lanes x 16 bytes, DPP dot products, one softmax state per row group.
// (part of decode_attn.hip, which is the only file that includes it: everything here sits in its anonymous namespace)
#pragma once
#include <type_traits>
#include "attn_finish.hpp"

namespace onellm {
namespace {

// DP = 16-byte pieces a cache row really has (D = DP * VEC); LPR = the lanes that share a row, the
// power of two at or above DP.  With DP < LPR (head sizes 80, 96, 160, 192, ...) the surplus lanes of
// a row group re-read the row's first piece with a zero q (they add nothing to the dot product) and
// keep no result; the memory traffic is unchanged, a load instruction just carries fewer distinct bytes.
template <typename T, int LPR, int DP, int GT, int U, int NW>
__device__ __forceinline__ void split_unit(const AttnArgs& a, const RopeFreqs& fr, const Unit& u, float* lds)
{
    static_assert(DP >= 1 && DP <= LPR && 2 * DP > LPR, "pieces per row and lanes per row");
    constexpr int VEC = Elt<T>::kVec;
    constexpr int D = DP * VEC;
    constexpr int RPW = kWave / LPR;            // cache rows per wave per load instruction
    constexpr int NRG = NW * RPW;               // row groups (independent softmax states) per workgroup
    constexpr int NTHR = NW * kWave;

    float* sq = lds;                            // [GT][D]   roped q * qscale
    float* sk = sq + GT * D;                    // [D]       new k row (as stored)
    float* sv = sk + D;                         // [D]       new v row (as stored)
    float* snew = sv + D;                       // [GT]      score of the new row
    float* st_ml = snew + GT;                   // [NRG][GT][2]
    float* st_acc = st_ml + NRG * GT * 2;       // [NRG][GT][D]

    const int tid = lane_id_per_unit();
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int r0 = u.r0, r1 = u.r1;
    const size_t head_off = a.slab + ((size_t)u.b * a.Hkv + u.kvh) * (size_t)a.S * D;
    T* kc = static_cast<T*>(a.k_cache) + head_off;
    T* vc = static_cast<T*>(a.v_cache) + head_off;

    // ---- the first rows of the chunk are requested before anything else: they do not depend on q,
    // and their latency then hides the q / new-row set-up below
    const bool owner = DP == LPR || lane % LPR < DP;        // this lane owns VEC columns of the row
    const int col = owner ? (lane % LPR) * VEC : 0;         // first of this lane's VEC columns
    const int rg = wave * RPW + lane / LPR;     // row group of this lane
    constexpr int RPI = U * NRG;                // rows per workgroup iteration
    const T* kp = kc + col;
    const T* vp = vc + col;
    // loads of one iteration: U cache rows of K and of V per row group
    auto issue = [&](Vec16<T> (&kv)[U], Vec16<T> (&vv)[U], int rbase) {
#pragma unroll
        for (int u_ = 0; u_ < U; ++u_) {
            const int row = rbase + u_ * NRG + rg;
            kv[u_] = load16_stream(kp + (size_t)row * D);
            vv[u_] = load16_stream(vp + (size_t)row * D);
        }
    };
    // the same for the chunk's last, partial iteration: rows past the end are read from the last valid row (and
    // masked when they are consumed)
    auto issue_any = [&](Vec16<T> (&kv)[U], Vec16<T> (&vv)[U], int rbase) {
        if (rbase + RPI <= r1) {
            issue(kv, vv, rbase);
        } else {
#pragma unroll
            for (int u_ = 0; u_ < U; ++u_) {
                const int row = min(rbase + u_ * NRG + rg, r1 - 1);
                kv[u_] = load16_stream(kp + (size_t)row * D);
                vv[u_] = load16_stream(vp + (size_t)row * D);
            }
        }
    };
    const int nfull = r1 > r0 ? (r1 - r0) / RPI : 0;
    const int nb = r1 > r0 ? (r1 - r0 + RPI - 1) / RPI : 0;     // iterations, the partial one included
    Vec16<T> ka[U], va[U], kb[U], vb[U];
    if (nb > 0) issue_any(ka, va, r0);

    stage_q_and_new_row<T, D, GT, NTHR>(a, fr, u, kc, vc, sq, sk, sv, snew);

    float qr[GT][VEC];
#pragma unroll
    for (int g = 0; g < GT; ++g)
#pragma unroll
        for (int e = 0; e < VEC; ++e) qr[g][e] = owner ? sq[g * D + col + e] : 0.f;

    // ---- stream the history rows of this chunk
    float m[GT], l[GT], acc[GT][VEC];
#pragma unroll
    for (int g = 0; g < GT; ++g) {
        m[g] = -INFINITY;
        l[g] = 0.f;
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[g][e] = 0.f;
    }

    // scores, online softmax and weighted V sum for the rows held in (kv, vv); `valid` masks rows
    // past the end of the chunk in the tail iteration
    auto consume = [&](const Vec16<T> (&kv)[U], const Vec16<T> (&vv)[U], const bool (&valid)[U], auto masked_tag) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        float s[GT][U];
#pragma unroll
        for (int g = 0; g < GT; ++g)
#pragma unroll
            for (int u_ = 0; u_ < U; ++u_) {
                float part = 0.f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) part = fmaf(qr[g][e], kv[u_].get(e), part);
                part = group_sum<LPR>(part);
                if constexpr (MASKED) part = valid[u_] ? part : -INFINITY;
                s[g][u_] = part;
            }
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            float mx = m[g];
#pragma unroll
            for (int u_ = 0; u_ < U; ++u_) mx = fmaxf(mx, s[g][u_]);
            float mref = mx;
            if constexpr (MASKED) mref = (mx == -INFINITY) ? 0.f : mx;   // nothing seen yet: keep zeros
            const float alpha = __builtin_amdgcn_exp2f(m[g] - mref);
            float psum = 0.f;
            float p[U];
#pragma unroll
            for (int u_ = 0; u_ < U; ++u_) {
                p[u_] = __builtin_amdgcn_exp2f(s[g][u_] - mref);
                psum += p[u_];
            }
            l[g] = fmaf(l[g], alpha, psum);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float v = acc[g][e] * alpha;
#pragma unroll
                for (int u_ = 0; u_ < U; ++u_) v = fmaf(p[u_], vv[u_].get(e), v);
                acc[g][e] = v;
            }
            m[g] = mx;
        }
    };

    int look = -1;                              // (fused finish: the other pieces' arrivals, asked near the end)
    if (nfull == 0) look = first_look(a, u);
    if (nb > 0) {
        // Iterations are software-pipelined over two register buffers - iteration k in buffer k % 2, the loads of
        // the next one in flight while the current one is consumed - the chunk's last, partial iteration included
        // (asked for after the last full one was consumed, it was a memory round trip with nothing else in flight
        // at the end of every chunk: Llama-7B shape at 512 rows 24.2 -> 23.6 us).  While two more full iterations lie
        // ahead the loop holds nothing conditional, so the compiler waits for exactly the loads a product needs.
        const bool none[U] = {};
        if (nb > 1) issue_any(kb, vb, r0 + RPI);
        int k = 0;
        for (; k + 4 <= nfull; k += 2) {
            const int rbase = r0 + k * RPI;
            consume(ka, va, none, std::false_type{});
            issue(ka, va, rbase + 2 * RPI);
            consume(kb, vb, none, std::false_type{});
            issue(kb, vb, rbase + 3 * RPI);
        }
        for (; k < nfull; k += 2) {
            if (k + 2 >= nfull) look = first_look(a, u);
            const int rbase = r0 + k * RPI;
            consume(ka, va, none, std::false_type{});
            if (k + 2 < nb) issue_any(ka, va, rbase + 2 * RPI);
            if (k + 1 < nfull) {
                consume(kb, vb, none, std::false_type{});
                if (k + 3 < nb) issue_any(kb, vb, rbase + 3 * RPI);
            }
        }
        if (nb > nfull) {
            const int rbase = r0 + nfull * RPI;
            bool valid[U];
#pragma unroll
            for (int u_ = 0; u_ < U; ++u_) valid[u_] = rbase + u_ * NRG + rg < r1;
            if (nfull & 1) consume(kb, vb, valid, std::true_type{});
            else consume(ka, va, valid, std::true_type{});
        }
    }

    // ---- merge the row-group states of the workgroup
#pragma unroll
    for (int g = 0; g < GT; ++g) {
        if (lane % LPR == 0) {
            st_ml[(rg * GT + g) * 2] = m[g];
            st_ml[(rg * GT + g) * 2 + 1] = l[g];
        }
        if (owner) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) st_acc[(size_t)(rg * GT + g) * D + col + e] = acc[g][e];
        }
    }
    __syncthreads();
    finish_unit<T, D, GT, NRG, NTHR>(a, u, st_ml, st_acc, snew, sv, look);
}

// (the single-head fp16 kernel at D = 128 - the Llama-7B shape - is held to the registers of four waves per SIMD: it
// sits within two or three registers of that bound, and the fourth resident workgroup per compute unit is worth more)
template <typename T, int LPR, int GT, int U, int NW, bool BALANCED>
__global__ __launch_bounds__(NW * kWave, (GT == 1 && LPR == 16 && sizeof(T) == 2) ? 4 : 1)
void decode_attn_split_kernel(const AttnArgs a, const RopeFreqs fr)
{
    extern __shared__ float lds[];
    stamp_entry(a);
    for_each_unit<GT, BALANCED>(a, [&](const Unit& u) { split_unit<T, LPR, LPR, GT, U, NW>(a, fr, u, lds); });
    stamp_end(a);
}

// the same kernel for rows that do not fill their lanes (grid schedule only)
template <typename T, int LPR, int DP, int GT>
__global__ __launch_bounds__(4 * kWave)
void decode_attn_split_padded_kernel(const AttnArgs a, const RopeFreqs fr)
{
    extern __shared__ float lds[];
    for_each_unit<GT, false>(a, [&](const Unit& u) { split_unit<T, LPR, DP, GT, 4, 4>(a, fr, u, lds); });
}

}  // namespace
}  // namespace onellm
