// Fused masked decoder self-attention for one new token per sequence, gfx950 (wave64).
//
// One launch fuses: q/k/v bias add, RoPE of q and k, the KV-cache write of row t-1, the scaled
// scores against rows 0..t-1, the softmax and the weighted V sum.  The work is memory-bound (the
// K and V history is read exactly once: 2*Hkv*(t-1)*D*e bytes per sequence), so the design is
// about bytes in flight, not matrix cores:
//
//   * split over the sequence ("flash-decoding"): grid = (kv-head x head-tile, splits, batch); each
//     workgroup streams one contiguous chunk of cache rows of one (sequence, kv-head) and keeps an
//     online-softmax state (running max m, sum l, weighted V accumulator) per query head;
//   * grouped-query heads are fused on the read side: a workgroup applies every K/V row it loads to
//     up to GT query heads of the group, so the cache is never repeated in memory;
//   * lane mapping: a cache row of D elements is LPR = D*sizeof(T)/16 lanes x 16 bytes, so a wave
//     reads 64/LPR whole rows per global_load_dwordx4 (fully coalesced 1 KiB per instruction); the
//     q.k dot product is finished by an LPR-lane DPP reduction, no LDS;
//   * every group of LPR lanes owns an independent softmax state for the rows it sees; the states
//     of a workgroup are merged once, through LDS, at the end of the chunk;
//   * partial results (m, l, unnormalised acc) go to a workspace and a second tiny kernel merges
//     the splits; with a single split the first kernel writes the output directly.
//
// Arithmetic is fp32 throughout; T is only the storage type of qkv, bias, cache and output.
//
// The device code lives in four headers that only this file includes: attn_schedule.hpp (arguments, units, the
// grid and balanced schedules), attn_finish.hpp (set-up and finish of a unit, fused finish), attn_valu.hpp (the
// vector-ALU kernels) and attn_mfma.hpp (the matrix-core kernels for grouped-query heads).  Here: the merge
// kernels, the scalar kernel for any head size, the launch selection and the C entry points.
#include <math.h>
#include "common.hpp"
#include "device_symbol.hpp"
#include "rope.hpp"
#include "attn_schedule.hpp"
#include "attn_finish.hpp"
#include "attn_valu.hpp"
#include "attn_mfma.hpp"

namespace onellm {
namespace {

// Merge the per-split partial states of one (sequence, query head) and normalise: one wave per
// (sequence, head).  Lane s holds split s's (m, l), so the maximum, the weights and the denominator
// are two wave reductions instead of loops of dependent loads; the weighted sum over splits then
// runs with the loads of several splits in flight.
template <typename T>
__global__ __launch_bounds__(kWave)
void decode_attn_merge_kernel(const AttnArgs a, int D)
{
    constexpr int PRE = 16;                                    // splits whose partial sums are requested up front
    const int bh = blockIdx.x, lane = threadIdx.x;
    const int b = bh / a.Hq;
    const float* ml = a.part_ml + (size_t)bh * a.nsplit * 2;
    const float* po = a.part_o + (size_t)bh * a.nsplit * D;
    // everything that does not depend on the length is requested before the length is looked at: the
    // (m, l) pairs of all splits and the first block of partial sums.  Entries of splits past the
    // sequence's end hold stale bytes; they are selected away below, never multiplied.
    float m_raw = 0.f, l_raw = 0.f;
    if (lane < a.nsplit) {
        m_raw = ml[lane * 2];
        l_raw = ml[lane * 2 + 1];
    }
    const int npre = min(a.nsplit, PRE);
    float o_pre[PRE];
#pragma unroll
    for (int s = 0; s < PRE; ++s) o_pre[s] = (s < npre && lane < D) ? po[(size_t)s * D + lane] : 0.f;
    const int t = a.t_dev ? a.t_dev[b] : a.t_host;
    if (t < 1 || t > a.S) return;
    const int nvalid = min((t - 1) / a.chunk + 1, a.nsplit);   // t above max_t is out of contract: stay in bounds
    const float m = lane < nvalid ? m_raw : -INFINITY;
    const float l = lane < nvalid ? l_raw : 0.f;
    float M = m;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) M = fmaxf(M, __shfl_xor(M, off, kWave));
    const float w = __builtin_amdgcn_exp2f(m - M);          // 0 for the lanes without a split
    const float invL = 1.0f / wave_sum(l * w);
    // the loops are uniform over the wave (the weights travel by lane exchange); only the accesses are guarded
    for (int d0 = 0; d0 < D; d0 += kWave) {
        const int d = d0 + lane;
        float O = 0.f;
        int s = 0;
        if (d0 == 0) {
#pragma unroll
            for (; s < PRE; ++s) {
                const float ws = __shfl(w, s, kWave);
                if (s < nvalid) O = fmaf(o_pre[s], ws, O);
            }
        }
        for (; s < nvalid; ++s) {
            const float ws = __shfl(w, s, kWave);
            if (d < D) O = fmaf(po[(size_t)s * D + d], ws, O);
        }
        if (d < D) static_cast<T*>(a.out)[(size_t)bh * D + d] = from_f32<T>(O * invL);
    }
}

// The same merge for the balanced schedule: the workgroups that touched the unit of (sequence,
// head) are found from the lengths exactly as the attention kernel found its shares; a unit one
// workgroup saw whole was already written by it.  A unit can have more than 64 partial states
// (one long sequence among short ones), so the passes run over blocks of 64 of them.
template <typename T>
__global__ __launch_bounds__(kWave)
void decode_attn_merge_balanced_kernel(const AttnArgs a, int D)
{
    __shared__ float w_s[kWave];
    const int bh = blockIdx.x, lane = threadIdx.x;
    const int b = bh / a.Hq, h = bh % a.Hq;
    const int t = a.t_dev ? a.t_dev[b] : a.t_host;
    const int items = seq_items(a, t);
    if (items == 0) return;
    unsigned total, before;
    count_items(a, b, total, before);
    const int ngt = (a.G + a.gt - 1) / a.gt;
    const int nunits = a.Hkv * ngt;
    const int gi = h % a.G;
    const int uib = (h / a.G) * ngt + gi / a.gt;
    const int g = gi % a.gt;
    const unsigned W = total * (unsigned)nunits;
    const unsigned first = before * (unsigned)nunits + (unsigned)uib * (unsigned)items;
    const int N = balanced_workgroups(a, W);
    const int i0 = item_owner(first + (unsigned)a.unit_cost, W, N), i1 = item_owner(first + (unsigned)items - 1u, W, N);   // (the items that hold rows)
    if (i0 == i1) return;
    const int n = i1 - i0 + 1;
    // entry of workgroup i0 + s: (i0 + s + global unit) * gt + g
    const size_t e0 = ((size_t)i0 + (size_t)b * nunits + uib) * a.gt + g;
    const float* ml = a.part_ml + e0 * 2;
    const float* po = a.part_o + e0 * D;
    const size_t step = (size_t)a.gt;
    float M = -INFINITY;
    for (int s = lane; s < n; s += kWave) M = fmaxf(M, ml[(size_t)s * step * 2]);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) M = fmaxf(M, __shfl_xor(M, off, kWave));
    float L = 0.f;
    for (int s = lane; s < n; s += kWave)
        L = fmaf(ml[(size_t)s * step * 2 + 1], __builtin_amdgcn_exp2f(ml[(size_t)s * step * 2] - M), L);
    const float invL = 1.0f / wave_sum(L);
    float O[8];                                               // D <= 512: 8 columns per lane
#pragma unroll
    for (int j = 0; j < 8; ++j) O[j] = 0.f;
    for (int s0 = 0; s0 < n; s0 += kWave) {
        const int cnt = min(kWave, n - s0);
        __syncthreads();
        w_s[lane] = lane < cnt ? __builtin_amdgcn_exp2f(ml[(size_t)(s0 + lane) * step * 2] - M) : 0.f;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int d = lane + j * kWave;
            if (d < D) {
                float acc = O[j];
#pragma unroll 4
                for (int s = 0; s < cnt; ++s) acc = fmaf(po[(size_t)(s0 + s) * step * D + d], w_s[s], acc);
                O[j] = acc;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int d = lane + j * kWave;
        if (d < D) static_cast<T*>(a.out)[(size_t)bh * D + d] = from_f32<T>(O[j] * invL);
    }
}

// Any head size up to 512 and any alignment: one workgroup per (sequence, query head), scalar
// accesses, no sequence split, grouped-query heads each re-read their kv-head's rows.  Same
// arithmetic and the same cache write as the tiled kernel; a correctness path for head sizes
// whose rows are not a power-of-two number of bytes (96, 80, ...), not a performance path.
template <typename T>
__global__ __launch_bounds__(256)
void decode_attn_generic_kernel(const AttnArgs a, const RopeFreqs fr, int D)
{
    constexpr int NW = 4, MAXJ = 2 * kMaxPairs / kWave;       // elements of a row per lane
    extern __shared__ float lds[];
    float* sq = lds;                  // [D]
    float* sk = sq + D;               // [D]
    float* sv = sk + D;               // [D]
    float* st_ml = sv + D;            // [NW][2]
    float* st_acc = st_ml + NW * 2;   // [NW][D]
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int h = blockIdx.x, b = blockIdx.y;
    const int kvh = h / a.G;
    const int t = a.t_dev ? a.t_dev[b] : a.t_host;
    if (t < 1 || t > a.S) return;
    const int pos = t + a.pos_offset;
    const T* qkv = static_cast<const T*>(a.qkv) + (size_t)b * (a.Hq + 2 * a.Hkv) * D;
    const T* bias = static_cast<const T*>(a.bias);
    const size_t head_off = a.slab + ((size_t)b * a.Hkv + kvh) * (size_t)a.S * D;
    T* kc = static_cast<T*>(a.k_cache) + head_off;
    T* vc = static_cast<T*>(a.v_cache) + head_off;
    const bool store = (h % a.G) == 0 && !(a.flags & ONELLM_ATTN_NO_CACHE_WRITE);

    // q, new k, new v: bias, RoPE on the pairs that exist, staging in LDS (an odd last element is not rotated)
    for (int p = tid; 2 * p < D; p += 256) {
        const bool pair = 2 * p + 1 < D;
        const int oq = h * D + 2 * p, ok = (a.Hq + kvh) * D + 2 * p;
        float q0 = to_f32(qkv[oq]), q1 = pair ? to_f32(qkv[oq + 1]) : 0.f;
        float k0 = to_f32(qkv[ok]), k1 = pair ? to_f32(qkv[ok + 1]) : 0.f;
        if (bias) {
            q0 += to_f32(bias[oq]);
            k0 += to_f32(bias[ok]);
            if (pair) {
                q1 += to_f32(bias[oq + 1]);
                k1 += to_f32(bias[ok + 1]);
            }
        }
        if (pair && 2 * p < a.rotary_dim) {
            rope_pair(q0, q1, p, pos, fr);
            rope_pair(k0, k1, p, pos, fr);
        }
        sq[2 * p] = q0 * a.qscale;
        const T ks0 = from_f32<T>(k0);
        sk[2 * p] = to_f32(ks0);
        if (store) kc[(size_t)(t - 1) * D + 2 * p] = ks0;
        if (pair) {
            sq[2 * p + 1] = q1 * a.qscale;
            const T ks1 = from_f32<T>(k1);
            sk[2 * p + 1] = to_f32(ks1);
            if (store) kc[(size_t)(t - 1) * D + 2 * p + 1] = ks1;
        }
    }
    for (int d = tid; d < D; d += 256) {
        const int o = (a.Hq + a.Hkv + kvh) * D + d;
        float x = to_f32(qkv[o]);
        if (bias && !(a.flags & ONELLM_ATTN_NO_V_BIAS)) x += to_f32(bias[o]);
        const T v = from_f32<T>(x);
        sv[d] = to_f32(v);
        if (store) vc[(size_t)(t - 1) * D + d] = v;
    }
    __syncthreads();

    float qr[MAXJ], acc[MAXJ];
#pragma unroll
    for (int j = 0; j < MAXJ; ++j) {
        const int d = lane + j * kWave;
        qr[j] = d < D ? sq[d] : 0.f;
        acc[j] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    auto row_step = [&](auto&& kget, auto&& vget) {
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < MAXJ; ++j) {
            const int d = lane + j * kWave;
            if (d < D) part = fmaf(qr[j], kget(d), part);
        }
        const float sc = wave_sum(part);
        const float mx = fmaxf(m, sc);
        const float alpha = __builtin_amdgcn_exp2f(m - mx), pr = __builtin_amdgcn_exp2f(sc - mx);
        l = fmaf(l, alpha, pr);
#pragma unroll
        for (int j = 0; j < MAXJ; ++j) {
            const int d = lane + j * kWave;
            if (d < D) acc[j] = fmaf(pr, vget(d), acc[j] * alpha);
        }
        m = mx;
    };
    for (int r = wave; r < t - 1; r += NW) {
        const T* kr = kc + (size_t)r * D;
        const T* vr = vc + (size_t)r * D;
        row_step([&](int d) { return to_f32(kr[d]); }, [&](int d) { return to_f32(vr[d]); });
    }
    if (wave == 0) row_step([&](int d) { return sk[d]; }, [&](int d) { return sv[d]; });   // the new token's row

    if (lane == 0) {
        st_ml[wave * 2] = m;
        st_ml[wave * 2 + 1] = l;
    }
#pragma unroll
    for (int j = 0; j < MAXJ; ++j) {
        const int d = lane + j * kWave;
        if (d < D) st_acc[wave * D + d] = acc[j];
    }
    __syncthreads();
    for (int d = tid; d < D; d += 256) {
        float M = -INFINITY;
        for (int w = 0; w < NW; ++w) M = fmaxf(M, st_ml[w * 2]);      // wave 0 always holds the new row: M is finite
        float L = 0.f, O = 0.f;
        for (int w = 0; w < NW; ++w) {
            const float wt = __builtin_amdgcn_exp2f(st_ml[w * 2] - M);
            L = fmaf(st_ml[w * 2 + 1], wt, L);
            O = fmaf(st_acc[w * D + d], wt, O);
        }
        static_cast<T*>(a.out)[((size_t)b * a.Hq + h) * D + d] = from_f32<T>(O / L);
    }
}

template <typename T>
int launch_generic(const AttnArgs& a, const RopeFreqs& fr, int D, hipStream_t st)
{
    const size_t lds_bytes = sizeof(float) * (size_t)(3 * D + 8 + 4 * D);
    hipLaunchKernelGGL((decode_attn_generic_kernel<T>), dim3(a.Hq, a.B), dim3(256), lds_bytes, st, a, fr, D);
    return launch_status();
}

constexpr int kMaxSplits = 64;      // upper bound of splits the workspace is sized for
constexpr int kMinChunk = 64;       // never split finer than this many cache rows

template <typename T, int LPR, int GT, int U, int NW>
int launch_split(const AttnArgs& a, const RopeFreqs& fr, hipStream_t st)
{
    constexpr int D = LPR * Elt<T>::kVec;
    constexpr int NRG = NW * (kWave / LPR);
    const size_t lds_bytes = sizeof(float) * (size_t)(GT * D + 2 * D + GT + NRG * GT * 2 + (size_t)NRG * GT * D);
    if (lds_bytes > 64 * 1024) return ONELLM_EUNSUPPORTED;
    const int ngt = (a.G + GT - 1) / GT;
    const dim3 grid(a.Hkv * ngt, a.nsplit, a.B), block(NW * kWave);
    if (a.bal_nwg > 0)
        hipLaunchKernelGGL((decode_attn_split_kernel<T, LPR, GT, U, NW, true>), dim3(a.bal_nwg), block, lds_bytes, st, a, fr);
    else
        hipLaunchKernelGGL((decode_attn_split_kernel<T, LPR, GT, U, NW, false>), grid, block, lds_bytes, st, a, fr);
    return launch_status();
}

template <typename T, int LPR, int DP, int GT>
int launch_padded(const AttnArgs& a, const RopeFreqs& fr, hipStream_t st)
{
    constexpr int D = DP * Elt<T>::kVec;
    constexpr int NRG = 4 * (kWave / LPR);
    const size_t lds_bytes = sizeof(float) * (size_t)(GT * D + 2 * D + GT + NRG * GT * 2 + (size_t)NRG * GT * D);
    if (lds_bytes > 64 * 1024) return ONELLM_EUNSUPPORTED;
    const int ngt = (a.G + GT - 1) / GT;
    const dim3 grid(a.Hkv * ngt, a.nsplit, a.B), block(4 * kWave);
    hipLaunchKernelGGL((decode_attn_split_padded_kernel<T, LPR, DP, GT>), grid, block, lds_bytes, st, a, fr);
    return launch_status();
}

// head sizes between the powers of two that the tiled kernel is built for, in 16-byte pieces per row
constexpr bool padded_pieces(int dp) { return dp == 10 || dp == 12 || dp == 20 || dp == 24 || dp == 40 || dp == 48; }

template <typename T, int LPR, int DP>
int launch_padded_gt(const AttnArgs& a, const RopeFreqs& fr, hipStream_t st)
{
    return a.G == 1 ? launch_padded<T, LPR, DP, 1>(a, fr, st) : launch_padded<T, LPR, DP, 4>(a, fr, st);
}

template <typename T>
int launch_padded_dp(int dp, const AttnArgs& a, const RopeFreqs& fr, hipStream_t st)
{
    switch (dp) {
        case 10: return launch_padded_gt<T, 16, 10>(a, fr, st);
        case 12: return launch_padded_gt<T, 16, 12>(a, fr, st);
        case 20: return launch_padded_gt<T, 32, 20>(a, fr, st);
        case 24: return launch_padded_gt<T, 32, 24>(a, fr, st);
        case 40: return launch_padded_gt<T, 64, 40>(a, fr, st);
        case 48: return launch_padded_gt<T, 64, 48>(a, fr, st);
        default: return ONELLM_EUNSUPPORTED;
    }
}

template <typename T, int LPR, int GT>
int launch_shape(const AttnArgs& a, const RopeFreqs& fr, hipStream_t st)
{
    // 4 waves per workgroup and 4 cache rows per row group and iteration measured best on MI355X for
    // both the single-head and the grouped-query form (8 or 16 waves, 2 or 8 rows: 3-30 % slower).
    return launch_split<T, LPR, GT, 4, 4>(a, fr, st);
}

// head sizes the matrix-core kernel is built for (fp16 caches)
constexpr bool mfma_head_size(int D) { return D == 64 || D == 128 || D == 256; }

// shapes that run on the matrix cores: fp16 caches with three or more query heads per kv head at those head
// sizes, fp32 caches at D = 64 or 128 with more than four.  With two heads per kv head the vector ALU keeps up with
// the stream, and which kernel is faster depends on how long a unit streams between its set-up and its finish:
// at D = 128 the matrix-core kernel wins from about 2048 rows (16 q / 8 kv heads, batch 32: 8192 rows 158.2 -> 152.3
// us, lengths 1024..8192 94.9 -> 92.2, 2048 rows 44.2 -> 43.8; 64 q / 32 kv heads, batch 16, 4096 rows 159.0 ->
// 157.8) and loses below (512 rows 15.1 -> 15.6, lengths 256..2048 at batch 96 76.4 -> 78.8), so it takes steps whose
// longest sequence has 4096 rows or more; at D = 64 (82.4 against 86.7) and D = 256 (lengths 512..4096: 96.5 against
// 98.9) the vector-ALU kernel stays.  One head per kv head: equal from 4096 rows (157.7 both at the Llama-2-7B shape),
// the vector ALU ahead below (512 rows 23.7 against 24.6), so it keeps all of them.
// Tuning key attn_gqa_valu: 1 = never the matrix cores, 0 = always where a matrix-core kernel exists.
bool on_matrix_cores(bool fp16, int D, int G, int max_t)
{
    if (tune_get("attn_gqa_valu") == 1) return false;
    if (tune_get("attn_gqa_valu") == 0 && fp16 && mfma_head_size(D)) return true;
    if (!fp16) return G > 4 && (D == 128 || D == 64);
    return mfma_head_size(D) && (G > 2 || (G == 2 && D == 128 && max_t >= 4096));
}

// query heads one workgroup serves (they share every K/V row it reads)
int heads_per_tile(bool fp16, int D, int G, int max_t)
{
    if (G == 1 && !on_matrix_cores(fp16, D, G, max_t)) return 1;       // one head: memory-bound on either kernel (measured equal), keep the lighter one
    // three or more query heads per kv head, fp16: both products on the matrix cores, where up to 16
    // heads cost the same as 4 (8 at D = 256: the per-wave states of 16 heads would not fit 64 KiB of LDS)
    if (on_matrix_cores(fp16, D, G, max_t)) {
        const int cap = D == 256 ? 8 : 16;
        const int gt = G <= 4 ? 4 : (G <= 8 ? 8 : 16);
        return gt < cap ? gt : cap;
    }
    // fp32 caches: a lane holds 4 columns, so 8 heads per tile still fit the registers and more than 4 heads
    // per kv head need no second pass over the rows
    if (!fp16 && G > 4) return 8;
    return G == 2 ? 2 : 4;
}

template <typename T, int LPR>
int launch_gt(const AttnArgs& a, const RopeFreqs& fr, hipStream_t st)
{
    constexpr bool kHalf = std::is_same<T, __half>::value;
    constexpr int D = LPR * Elt<T>::kVec;
    const int gt = a.gt;
    if constexpr (!kHalf && (D == 128 || D == 64)) {
        if (a.on_mfma) return gt == 8 ? launch_gqa_mfma_f32<D, 8>(a, fr, st) : launch_gqa_mfma_f32<D, 16>(a, fr, st);
    }
    if constexpr (kHalf && mfma_head_size(D)) {
        if (a.on_mfma) {
            switch (gt) {
                case 4: return launch_gqa_mfma<D, 4>(a, fr, st);
                case 8: return launch_gqa_mfma<D, 8>(a, fr, st);
                case 16:
                    if constexpr (D <= 128) return launch_gqa_mfma<D, 16>(a, fr, st);
                    break;
                default: break;
            }
            return ONELLM_EUNSUPPORTED;
        }
    }
    switch (gt) {
        case 1: return launch_shape<T, LPR, 1>(a, fr, st);
        case 2: return launch_shape<T, LPR, 2>(a, fr, st);
        case 8:
            if constexpr (!kHalf) return launch_shape<T, LPR, 8>(a, fr, st);
            return ONELLM_EUNSUPPORTED;
        default: return launch_shape<T, LPR, 4>(a, fr, st);
    }
}

template <typename T>
int launch_lpr(int lpr, const AttnArgs& a, const RopeFreqs& fr, hipStream_t st)
{
    switch (lpr) {
        case 1: return launch_gt<T, 1>(a, fr, st);
        case 2: return launch_gt<T, 2>(a, fr, st);
        case 4: return launch_gt<T, 4>(a, fr, st);
        case 8: return launch_gt<T, 8>(a, fr, st);
        case 16: return launch_gt<T, 16>(a, fr, st);
        case 32: return launch_gt<T, 32>(a, fr, st);
        case 64: return launch_gt<T, 64>(a, fr, st);
        default: return ONELLM_EUNSUPPORTED;
    }
}


// rows per work item of the balanced schedule: one workgroup iteration of the kernel that runs
int item_rows_for(bool fp16, int D, int G, int max_t)
{
    if (on_matrix_cores(fp16, D, G, max_t)) return 64;
    const int lpr = D * (fp16 ? 2 : 4) / 16;
    const int rpi = 1024 / lpr;               // 4 waves x (64 / lpr) rows x 4 per row group
    return rpi < 64 ? 64 : rpi;
}

// When the balanced schedule is the default (tuning knob attn_balanced = 1 / 0 forces it on / off): per-sequence
// lengths on the matrix-core kernels.  Measured on MI355X against the grid schedule (us per step, lengths uniform
// in [S/8, S]): 32 q / 8 kv heads, batch 32, S 8192: 117 -> 98; 64 q / 8 kv, batch 16: 81 -> 57; batch 8, S 16384:
// 97 -> 61; D = 256, batch 16, S 4096: 90 -> 64; and, since the shares are equal in cost, with more units than
// workgroups too: batch 72, S 4096: 131 -> 118; batch 96, S 2048: 101 -> 87; batch 256, S 1024: 155 -> 118.  With
// equal lengths a grid that fills the chip evenly needs no merge and is as fast or faster; on the vector-ALU kernel
// (which keeps four workgroups per compute unit resident) the hardware dispatcher balances the grid schedule's
// chunks about as well as the fixed shares do (batch 24 x 32 heads: 157.5 / 153.8; batch 16: 94.4 / 97.4).  Nor for
// a small step (fewer than kBalancedMinItems items
// if every length were the longest): the walk's set-up and its serial unit changes are then most of the time and
// the grid schedule with the fused finish is faster (8 sequences of 256..2048 rows: 24.9 against 17.6 us; 4 of
// 512..4096: 25.2 / 19.6; even at 3500..4100 items; the balanced schedule is ahead from ~7000: 16 sequences of
// 1024..8192 rows 56.7 / 67.6).
bool balanced_by_default(bool ragged, bool mfma, int G, long long max_items, long units, int max_t)
{
    // (two heads per kv head on the vector-ALU kernel: 32 sequences of 1024..8192 rows 105.4 -> 98.1 us.  One head,
    // where the dispatcher keeps four workgroups per compute unit busy with the grid schedule's chunks: a tie up to
    // ~16000 items, then 3-6 % - 16 sequences x 32 heads of 512..4096 rows 105 -> 100 us, 64 of 128..2048: 184 -> 174)
    if (!ragged) return false;
    // (matrix-core kernels: fewer than 128 units of fewer than 4000 rows are cut into few chunks by the grid schedule
    // and finish faster there - 12 sequences x 8 kv heads of 256..2048 / 375..3000 rows 18.9 / 21.9 us on equal shares,
    // 16.7 / 19.3 on the grid - while 16 sequences of 256..2048 rows, 21.5 / 24.9, and 12 of 500..4000, 24.9 / 30.8, go
    // the other way)
    if (mfma) return max_items >= kBalancedMinItems && (units >= 128 || max_t >= 4000);
    // (two heads per tile on the vector-ALU kernel: 16 sequences x 8 kv heads of 256..2048 / 375..3000 rows, 4096 / 6016
    // items, 21.3 / 25.4 us on equal shares against 17.9 / 22.1 on the grid; from 8192 items the shares are ahead)
    if (G == 2) return max_items >= 8192;
    return max_items >= 16384;
}

int max_splits(int max_t)
{
    int n = (max_t + kMinChunk - 1) / kMinChunk;
    return n < 1 ? 1 : (n > kMaxSplits ? kMaxSplits : n);
}

}  // namespace
}  // namespace onellm

// Built-in scratch of onellm_decode_attn_static: arrival counters + split partials, one copy per GPU, held from
// the moment the library is loaded on that GPU until the process ends.  Zero at load; every call leaves the
// counter region at zero again.  In host code this name is only a handle for hipGetSymbolAddress: the device
// address it resolves to (one per GPU) is what kernels and fills are given.
static __device__ __align__(256) unsigned char scratch[ONELLM_DECODE_ATTN_STATIC_SCRATCH_BYTES];

namespace onellm {
namespace {

// Address of the current device's copy of `scratch`, resolved once per device.  Nothing is launched or allocated:
// the array is zero when the module is loaded and every call leaves its counter region at zero again.
DeviceSymbol g_scratch_address;
int static_scratch(void** out) { return g_scratch_address.address(HIP_SYMBOL(scratch), out); }

}  // namespace
}  // namespace onellm

#ifdef ONELLM_ATTN_STAMPS
namespace onellm { namespace { long long* g_stamp_buffer = nullptr; } }
// timeline build only: device buffer of 4 * (workgroups of the launch) int64 words, or NULL to stop recording
extern "C" void onellm_attn_set_stamp_buffer(void* buffer) { onellm::g_stamp_buffer = static_cast<long long*>(buffer); }
#endif

extern "C" size_t onellm_decode_attn_workspace_bytes(int B, int Hq, int Hkv, int D, int max_t)
{
    (void)Hkv;
    if (B <= 0 || Hq <= 0 || D <= 0 || max_t <= 0) return 256;
    // grid schedule: one partial state per (sequence, head, split); balanced schedule: one per
    // (workgroup + unit) and tile head - at most 16 heads per tile, and the padded tiles of all
    // units hold less than twice the query heads
    const size_t grid_entries = (size_t)B * Hq * onellm::max_splits(max_t);
    const size_t bal_entries = (size_t)onellm::kBalancedWorkgroups * 2 * 16 + (size_t)B * Hq * 2;
    const size_t n = onellm::kCounterBytes + (grid_entries > bal_entries ? grid_entries : bal_entries) * (size_t)(D + 2) * sizeof(float);
    return (n + 255) & ~(size_t)255;
}

extern "C" int onellm_decode_attn(int dtype, const void* qkv, const void* qkv_bias, void* k_cache, void* v_cache,
                                  void* out, int B, int Hq, int Hkv, int D, int S, int layer, int num_layers,
                                  int t_host, const int* t_dev, int max_t, int rotary_dim, float rope_base,
                                  int rope_pos_offset, unsigned flags, void* workspace, size_t workspace_bytes,
                                  onellm_stream_t stream)
{
    using namespace onellm;
    if (!qkv || !k_cache || !v_cache || !out) return ONELLM_EINVAL;
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || S <= 0 || num_layers <= 0) return ONELLM_EINVAL;
    if (layer < 0 || layer >= num_layers || Hq % Hkv) return ONELLM_EINVAL;
    if (dtype != ONELLM_FP32 && dtype != ONELLM_FP16) return ONELLM_EINVAL;
    if (!t_dev) max_t = t_host;
    if (max_t < 1 || max_t > S || (!t_dev && (t_host < 1 || t_host > S))) return ONELLM_EINVAL;
    if (rotary_dim < 0 || (rotary_dim > 0 && !(rope_base > 0.f))) return ONELLM_EINVAL;
    const int esz = dtype == ONELLM_FP16 ? 2 : 4;
    const int row_bytes = D * esz;
    if (D > 2 * kMaxPairs || B > 65535) return ONELLM_EUNSUPPORTED;
    // rows of a power-of-two number of bytes - or of 10, 12, 20, 24, 40 or 48 16-byte pieces (head sizes 80, 96,
    // 160, 192, ... in fp16) - in 16-byte aligned caches take the tiled kernels; any other head size or alignment
    // takes the scalar kernel
    const bool padded = row_bytes % 16 == 0 && padded_pieces(row_bytes / 16);
    // (... and qkv / bias aligned to a pair of elements: the set-up reads them a pair at a time)
    const uintptr_t pair_mask = (uintptr_t)(2 * esz - 1);
    const bool pairs_aligned = !(reinterpret_cast<uintptr_t>(qkv) & pair_mask) && !(reinterpret_cast<uintptr_t>(qkv_bias) & pair_mask);
    const bool tiled = row_bytes >= 16 && row_bytes <= 1024 && (!(row_bytes & (row_bytes - 1)) || padded)
                       && aligned16(k_cache) && aligned16(v_cache) && pairs_aligned;
    const int lpr = row_bytes / 16;

    AttnArgs a{};
    a.qkv = qkv; a.bias = qkv_bias; a.k_cache = k_cache; a.v_cache = v_cache; a.out = out;
    a.t_dev = t_dev; a.t_host = t_host;
    a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.G = Hq / Hkv; a.S = S;
    a.rotary_dim = rotary_dim; a.pos_offset = rope_pos_offset; a.flags = flags;
#ifdef ONELLM_ATTN_STAMPS
    a.stamps = g_stamp_buffer;
#endif
    a.turns = tune_get("attn_turns") != 0;
    a.ordered = tune_get("attn_ordered_finish") == 1;
    a.early_look = 0;
    a.qscale = (1.0f / sqrtf((float)D)) * 1.4426950408889634f;
    a.slab = (size_t)layer * B * Hkv * (size_t)S * D;

    if (!tiled) {
        RopeFreqs frg;
        fill_rope_freqs(frg, D, rotary_dim, rope_base);
        hipStream_t stg = static_cast<hipStream_t>(stream);
        return dtype == ONELLM_FP16 ? launch_generic<__half>(a, frg, D, stg) : launch_generic<float>(a, frg, D, stg);
    }

    // Sequence split, from sweeps on MI355X.  Equal lengths (t_dev == NULL): about one workgroup per
    // compute unit with chunks of at least 512 rows (more, smaller workgroups only add per-workgroup
    // set-up and merge work); a shape that already has that many workgroups is not split at all and
    // needs no merge pass.  Per-sequence lengths: finer chunks (about 16 workgroups per compute unit,
    // at least 256 rows each) so that the dispatcher can balance ragged work.
    const int G = a.G;
    const int gt = padded ? (G == 1 ? 1 : 4) : heads_per_tile(dtype == ONELLM_FP16, D, G, max_t);
    const int ngt = (G + gt - 1) / gt;
    const long base_wgs = (long)B * Hkv * ngt;
    const int user_target = tune_get("attn_target_wgs");
    // (the matrix-core kernel at D = 64 has half the bytes in flight per workgroup: two per compute unit)
    const bool mfma_kernel = !padded && on_matrix_cores(dtype == ONELLM_FP16, D, G, max_t);
    const bool mfma64 = D == 64 && mfma_kernel && dtype == ONELLM_FP16;
    const int target = user_target > 0 ? user_target : (t_dev ? 4096 : (mfma64 ? 512 : 256));
    int nsplit = (int)((target + base_wgs - 1) / base_wgs);
    int cap = max_splits(max_t);
    if (user_target <= 0) {
        // (a handful of units - one or two sequences - is latency-bound: chunks down to 128 rows, so that the
        // chip has work at all: batch 1, 8 kv heads, 2048 rows 16.6 -> 11.8 us)
        const bool cheap_finish = (flags & ONELLM_ATTN_ZEROED_WORKSPACE) && tune_get("attn_fused_finish") != 0;
        const int min_rows = t_dev ? 256 : (base_wgs < 128 ? (cheap_finish ? 128 : 256) : 512);
        const int by_rows = max_t / min_rows;
        cap = by_rows < cap ? by_rows : cap;
    }
    if (nsplit > cap) nsplit = cap;
    if (nsplit < 1) nsplit = 1;
    // Equal lengths, a little fewer units than compute units: whole units on that many compute units, no split.  The
    // active units already draw what the memory system gives (vector-ALU kernel: 43 GB/s each, 7 TB/s from 160 units),
    // and a split would put every unit in two pieces.  Measured against two pieces per unit on equal shares: 192 / 224
    // single-head units of 4096 rows 65.8 -> 60.3 / 75.5 -> 70.4 us, of 1024 rows 21.6 -> 19.9 / 23.1 -> 22.0; 160 units:
    // 20.6 -> 18.5 (1024 rows), 54.9 -> 55.9 (4096).  A matrix-core workgroup draws ~30 GB/s alone, so there it takes
    // more units or shorter rows: 224 units 149.2 -> 142.9 (8192 rows), 46.6 -> 42.3 (2048); 192 units 42.1 -> 39.5
    // (2048) but 127.8 -> 136.8 (8192); 160 units 106 -> 132.  The vector-ALU kernel with several heads per tile is
    // as heavy per row (fp32 caches, 32 q / 8 kv heads, 192 units of 4096 rows: 127.8 -> 142.4; 224 units 148.0 -> 146.0)
    // and takes the matrix-core kernel's bounds.
    const bool light_rows = !mfma_kernel && gt == 1;
    if (user_target <= 0 && !t_dev && !mfma64 && nsplit == 2 && base_wgs < 256
        && (light_rows ? (base_wgs >= 176 || (base_wgs >= 160 && max_t <= 2048)) : (base_wgs >= 208 || (base_wgs >= 176 && max_t <= 2048))))
        nsplit = 1;
    const int forced = tune_get("attn_nsplit");
    if (forced > 0) nsplit = forced > max_splits(max_t) ? max_splits(max_t) : forced;
    int chunk = (max_t + nsplit - 1) / nsplit;
    chunk = (chunk + kMinChunk - 1) / kMinChunk * kMinChunk;
    nsplit = (max_t + chunk - 1) / chunk;
    a.chunk = chunk;
    a.nsplit = nsplit;
    a.gt = gt;
    a.on_mfma = mfma_kernel;

    // Balanced schedule: a fixed number of workgroups (what the chip holds at once) share the rows
    // of the step equally, whatever the lengths and however the units divide among compute units.
    const long nunits = (long)Hkv * ngt;
    bool merge_needed = nsplit > 1;
    // arrival counters of the fused finish sit at the front of a workspace the caller keeps zeroed
    // (the region has one size for every shape and is set aside whether or not this call uses it, so
    // that calls of any shapes, with and without the flag, can share one workspace)
    const size_t counter_bytes = kCounterBytes;
    const bool fused_finish = (flags & ONELLM_ATTN_ZEROED_WORKSPACE) && tune_get("attn_fused_finish") != 0
                              && (size_t)B * nunits * sizeof(int) <= kCounterBytes;
    float* const partials = reinterpret_cast<float*>(static_cast<char*>(workspace) + counter_bytes);
    const int bal = tune_get("attn_balanced");
    // (the step's size in work items if every sequence had the longest length: all the host knows)
    const int item_rows = item_rows_for(dtype == ONELLM_FP16, D, G, max_t);
    const long long items = (max_t - 1 + item_rows - 1) / item_rows;
    const long long wmax = (long long)B * nunits * (items < 1 ? 1 : items);
    // Equal lengths whose grid does not fill the chip evenly - between one and two workgroups per compute unit (one
    // and one and a half on the vector-ALU kernel, which loses less when a unit holds one workgroup): some units would
    // run two workgroups and the rest one.  One equal share per compute unit instead (measured: 40 heads x batch 8 =
    // 320 units 116 -> 101 us; 8 kv heads x batch 10, cut in four = 320 workgroups 75 -> 59 us; 8 kv heads x batch 48
    // = 384 units 144 -> 130 us; 384 single-head units 121.5 -> 124.6, hence the lower bound there).
    const long grid_wgs = base_wgs * nsplit;
    // (the matrix-core kernels hold two workgroups per unit at most, so any grid that is not a whole number of such
    // rounds ends with part of the chip idle: 576 units 227 -> 190 us, 640 units 265 -> 212, 768 units 284 -> 249)
    // (the vector-ALU kernel keeps four workgroups per unit resident, so a grid a little above a whole number of
    // workgroups per compute unit runs them all at once and ends with the few units that hold one more, alone, at a
    // fraction of the bandwidth: 544 / 576 / 800 / 832 single-head units of 4096 rows 192.9 / 195.2 / 269.6 / 271.4 us
    // against 178.4 / 182.8 / 250.0 / 260.0 on 512 equal shares; of 1024 rows 51.9 / 52.7 / 71.1 / 71.8 against 49.6 /
    // 52.3 / 70.4 / 70.1; with 96 units or more over the multiple the grid is as fast - 608, 640 units - or faster)
    const bool zeroed_ws = (flags & ONELLM_ATTN_ZEROED_WORKSPACE) && tune_get("attn_fused_finish") != 0;
    const bool valu_tail = grid_wgs > 512 && grid_wgs < 2048 && grid_wgs % 256 != 0 && grid_wgs % 256 <= 80
                           && (max_t >= 2048 || (zeroed_ws && max_t >= 1024));
    const bool uneven_grid = !t_dev && wmax >= 2048 && grid_wgs > 256
                             && (mfma_kernel ? (grid_wgs % 512 != 0 && grid_wgs < 4096) : (grid_wgs < 384 || valu_tail));
    // (the walk counts items in 32 bits: a step of more items than that allows - hundreds of millions of rows -
    // stays on the grid schedule)
    const int cost_bound = tune_get("attn_balanced_cost") > 6 ? tune_get("attn_balanced_cost") : 6;
    const bool walk_fits = (wmax + (long long)B * nunits * cost_bound) * (kBalancedWorkgroups * 2) < (long long)kBalancedMaxItemsTimesWorkgroups;
    // Per-sequence lengths on the vector-ALU kernel, a step of middling size (2048 rows or more at the longest, 128..800
    // MiB of K rows): one equal share per compute unit.  Measured against the default it replaces (the grid
    // schedule below 16384 items, 512 shares above), single-head units, lengths uniform in [S/8, S]: 8 sequences x 32
    // heads, S 2048 / 4096: 31.3 -> 28.7 / 53.2 -> 51.3 us; 12 sequences: 37.5 -> 35.7 / 64.7 -> 63.1 / (S 8192) 122.6 ->
    // 119.9; 16 sequences: 46.6 -> 44.3 / 84.6 -> 81.1; 24 sequences, S 4096: 124.0 -> 121.6.  Not for shorter rows (8 x 32
    // units of 128..1024 rows: 17.1 -> 19.4) nor beyond (16 sequences of 1024..8192 rows: 159.4 -> 161.2).
    // The bounds are in bytes of K rows if every sequence had the longest length (8192..50000 items of 64 rows of 256 bytes),
    // which carries over to the other row sizes: fp32 caches, head size 128 (512-byte rows), 4 / 8 / 16 sequences x 32 heads
    // of 512..4096 / 256..2048 rows 41.4 -> 38.5 / 51.6 -> 49.8 / 84.4 -> 81.4 us, 32 q / 8 kv heads x 16 / 32 sequences of
    // 512..4096 rows 53.2 -> 48.7 / 100.4 -> 94.3; fp16, head size 64, 8 sequences x 32 heads of 512..4096 rows 33.7 -> 28.7;
    // head size 256, 16 sequences x 16 heads of 256..2048 rows 48.1 -> 43.3.
    const long long wbytes = wmax * item_rows * row_bytes;
    const bool valu_mid_ragged = t_dev && !mfma_kernel && max_t >= 2048 && wbytes >= (128ll << 20) && wbytes <= (800ll << 20);
    if (forced <= 0 && !padded && walk_fits
        && (bal == 1 || (bal != 0 && (uneven_grid || valu_mid_ragged || balanced_by_default(t_dev != nullptr, mfma_kernel, G, wmax, (long)B * nunits, max_t))))) {
        a.item_rows = item_rows;
        // (what a change of unit costs a workgroup, in items: measured on the matrix-core kernel, where workgroups whose
        // equal-row shares held one / two / three units finished at 82 / 90 / 94 us of a 101 us step)
        const int user_cost = tune_get("attn_balanced_cost");
        const int user_wgs = tune_get("attn_balanced_wgs");
        // Few long units with per-sequence lengths on the fp16 D = 128 matrix-core kernel (no more units than compute
        // units, 4096 rows or more at the longest): one workgroup per compute unit, and a unit change charged six items.
        // Two co-resident workgroups stream ~3 % more per unit of time, but do not finish together - measured finish
        // times of 512 equal shares: mean 86, first 60-70, last 96 us of a 97 us step, against mean 88, last 94 with one
        // workgroup per compute unit (config 3: 96.9 -> 94.3 us; 64 q / 8 kv heads, batch 16: 66.5 -> 64.3; lengths
        // 7000..8192: 159 -> 155).  Many short units go the other way (96 sequences of 256..2048 rows: 79 against 86 us;
        // D = 64, with half the bytes in flight per workgroup: 66 against 85), so they keep two per compute unit.
        // (with half as many units as compute units or fewer it holds for shorter rows too: 16 sequences x 8 kv heads of
        // 256..2048 / 500..4000 rows 23.9 -> 21.5 / 32.0 -> 29.6 us, 12 sequences of 500..4000 rows 27.2 -> 24.9)
        const bool few_long_units = t_dev && mfma_kernel && dtype == ONELLM_FP16 && D == 128
                                    && ((long)B * nunits <= kBalancedWorkgroups / 4
                                        || ((long)B * nunits <= kBalancedWorkgroups / 2 && items >= 64));
        a.unit_cost = user_cost >= 0 ? user_cost : (few_long_units ? 6 : (valu_mid_ragged && bal != 1 ? 5 : 3));
        const long long wmax_cost = wmax + (long long)B * nunits * a.unit_cost;
        // (an uneven grid of SHORT units keeps two shares per compute unit: with a share of a few hundred rows the second
        // workgroup covers the first one's set-up and finish - 288 single-head units of 600 rows 23.1 -> 21.2 us, 36
        // sequences x 8 kv heads of 600 rows 28.4 -> 26.2; from about 1200 rows on one share per unit is as fast or faster)
        // (fp32 caches on the matrix-core kernel, head size 128: its one register buffer is a pipeline of its own since K
        // and V rows are requested separately, and one share per compute unit is ahead - 64 q / 8 kv heads, 8 / 16 / 32
        // sequences of 1024..8192 / 512..4096 rows: 57.7 -> 56.3 / 92.0 -> 88.6 / 104.2 -> 98.9 us; not for rows shorter than
        // 2048: 96 sequences of 128..1024 rows 93.1 -> 96.6)
        const bool fp32_mfma_shares = t_dev && mfma_kernel && dtype == ONELLM_FP32 && D == 128 && max_t >= 2048 && bal != 1;
        const bool one_share_per_unit = (uneven_grid && bal != 1 && grid_wgs < 512 && max_t >= 1024) || few_long_units
                                        || (valu_mid_ragged && bal != 1) || fp32_mfma_shares;
        long long nwg = user_wgs > 0 ? user_wgs : (one_share_per_unit ? kBalancedWorkgroups / 2 : kBalancedWorkgroups);
        // (the matrix-core kernel for D = 256 keeps one workgroup per compute unit resident: a second 256 would only
        // queue behind the first - 16 sequences of 512..4096 rows x 4 kv heads: 65.7 -> 47.1 us)
        if (user_wgs <= 0 && mfma_kernel && dtype == ONELLM_FP16 && D == 256 && nwg > kBalancedWorkgroups / 2) nwg = kBalancedWorkgroups / 2;
        if (nwg > kBalancedWorkgroups * 2) nwg = kBalancedWorkgroups * 2;
        // no workgroup for fewer than four items; between one and two workgroups per compute unit some units would
        // get two shares and the rest one, so one larger share each (6 sequences of 1024..4096 rows: 28.9 -> 25.3 us)
        if (nwg > (wmax_cost + 3) / 4) nwg = (wmax_cost + 3) / 4;
        if (user_wgs <= 0 && nwg > kBalancedWorkgroups / 2 && nwg < kBalancedWorkgroups) nwg = kBalancedWorkgroups / 2;
        // equal lengths and as many units as workgroups or more: whole units per workgroup when they divide evenly
        a.bal_nwg = (int)nwg;
        a.nsplit = 1;
        merge_needed = !(!t_dev && (B * nunits) % nwg == 0);
        const size_t entries = ((size_t)a.bal_nwg + (size_t)B * nunits) * gt;
        if (merge_needed) {
            const size_t need = counter_bytes + entries * (size_t)(D + 2) * sizeof(float);
            if (!workspace || workspace_bytes < need) return ONELLM_EWORKSPACE;
            a.part_o = partials;
            a.part_ml = a.part_o + entries * D;
        }
    } else if (nsplit > 1) {
        const size_t need = counter_bytes + (size_t)B * Hq * nsplit * (size_t)(D + 2) * sizeof(float);
        if (!workspace || workspace_bytes < need) return ONELLM_EWORKSPACE;
        a.part_o = partials;
        a.part_ml = a.part_o + (size_t)B * Hq * nsplit * D;
    }
    // Not with the grid schedule's fine chunks for per-sequence lengths when the step is large: thousands of
    // pieces each pay the counter round trip and the merge launch is cheaper (batch 32 x 32 heads, lengths
    // 512..4096: 181 -> 191 us; 32 q / 8 kv heads, 32 sequences of 512..4096 rows: 79.3 -> 81.8).  With a few
    // hundred workgroups it saves 2-5 us per step (batch 4, 32 q / 8 kv heads, 8192 rows: 30.8 -> 27.5; 8
    // sequences of 256..2048 rows: 20.8 -> 17.6).
    if (merge_needed && fused_finish && (a.bal_nwg > 0 || !t_dev || wmax <= kFusedGridMaxItems || tune_get("attn_fused_finish") == 1)) {
        a.counters = static_cast<int*>(workspace);
        merge_needed = false;                          // the last piece of every unit finishes it
    }

    // The first look pays where the pieces of a unit end at very different times - the balanced schedule, whose
    // shared units are begun by one workgroup at the start of its share and ended by its neighbour at the end of
    // its own (config 3 ragged 97.9 -> 96.8 us, 36 sequences x 8 kv heads of 600 rows 31.5 -> 29.9).  The pieces of
    // the grid schedule end together: the look finds nothing, and costs (8 sequences of 256..2048 rows 19.2 -> 20.3).
    const int look = tune_get("attn_early_look");
    a.early_look = look >= 0 ? look : (a.bal_nwg > 0 ? 1 : 0);

    RopeFreqs fr;
    fill_rope_freqs(fr, D, rotary_dim, rope_base);

    hipStream_t st = static_cast<hipStream_t>(stream);
    int rc;
    if (padded) rc = dtype == ONELLM_FP16 ? launch_padded_dp<__half>(lpr, a, fr, st) : launch_padded_dp<float>(lpr, a, fr, st);
    else rc = dtype == ONELLM_FP16 ? launch_lpr<__half>(lpr, a, fr, st) : launch_lpr<float>(lpr, a, fr, st);
    if (rc != 0) return rc;
    if (merge_needed) {
        if (a.bal_nwg > 0) {
            if (dtype == ONELLM_FP16)
                hipLaunchKernelGGL((decode_attn_merge_balanced_kernel<__half>), dim3(B * Hq), dim3(kWave), 0, st, a, D);
            else
                hipLaunchKernelGGL((decode_attn_merge_balanced_kernel<float>), dim3(B * Hq), dim3(kWave), 0, st, a, D);
        } else if (dtype == ONELLM_FP16) {
            hipLaunchKernelGGL((decode_attn_merge_kernel<__half>), dim3(B * Hq), dim3(kWave), 0, st, a, D);
        } else {
            hipLaunchKernelGGL((decode_attn_merge_kernel<float>), dim3(B * Hq), dim3(kWave), 0, st, a, D);
        }
        rc = launch_status();
    }
    return rc;
}

extern "C" int onellm_decode_attn_static(int dtype, const void* qkv, const void* qkv_bias, void* k_cache, void* v_cache,
                                         void* out, int B, int Hq, int Hkv, int D, int S, int layer, int num_layers,
                                         int t_host, const int* t_dev, int max_t, int rotary_dim, float rope_base,
                                         int rope_pos_offset, unsigned flags, onellm_stream_t stream)
{
    void* ws = nullptr;
    int rc = onellm::static_scratch(&ws);
    if (rc != 0) return rc;
    // the library owns this buffer and nothing else writes it: its counters are zero between calls
    rc = onellm_decode_attn(dtype, qkv, qkv_bias, k_cache, v_cache, out, B, Hq, Hkv, D, S, layer, num_layers, t_host, t_dev,
                            max_t, rotary_dim, rope_base, rope_pos_offset, flags | ONELLM_ATTN_ZEROED_WORKSPACE, ws,
                            (size_t)ONELLM_DECODE_ATTN_STATIC_SCRATCH_BYTES, stream);
    return rc == ONELLM_EWORKSPACE ? ONELLM_ESCRATCH : rc;
}
