// Decode attention: set-up of a unit (q, the new k/v row) and its finish (merge of the workgroup's states, partial states, fused finish).
// (part of decode_attn.hip, which is the only file that includes it: everything here sits in its anonymous namespace)
#pragma once
#include "attn_schedule.hpp"
#include "rope.hpp"

namespace onellm {
namespace {

// Two consecutive elements of a row fetched with one access, and one element fetched into a register of its own.
// (Two fp16 loads that fill the two halves of one register depend on each other - the second has to wait for the first
// to land - so element-by-element loads of a pair cost a memory round trip each; a 32-bit load of the pair, and a
// zero-extending 16-bit load of a single element, keep every load of the set-up independent of the others.)
template <typename T> struct RawPair;
template <> struct RawPair<__half> {
    unsigned w = 0;
    __device__ __forceinline__ float first() const { return __half2float(__ushort_as_half((unsigned short)(w & 0xFFFFu))); }
    __device__ __forceinline__ float second() const { return __half2float(__ushort_as_half((unsigned short)(w >> 16))); }
};
template <> struct RawPair<float> {
    float a = 0.f, b = 0.f;
    __device__ __forceinline__ float first() const { return a; }
    __device__ __forceinline__ float second() const { return b; }
};
__device__ __forceinline__ RawPair<__half> load_pair(const __half* p)
{
    RawPair<__half> r;
    r.w = *reinterpret_cast<const unsigned*>(p);
    return r;
}
__device__ __forceinline__ RawPair<float> load_pair(const float* p)
{
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const f32x2 v = *reinterpret_cast<const f32x2*>(p);
    RawPair<float> r;
    r.a = v[0];
    r.b = v[1];
    return r;
}
template <typename T> struct RawOne;
template <> struct RawOne<__half> {
    unsigned w = 0;
    __device__ __forceinline__ float value() const { return __half2float(__ushort_as_half((unsigned short)w)); }
};
template <> struct RawOne<float> {
    float v = 0.f;
    __device__ __forceinline__ float value() const { return v; }
};
__device__ __forceinline__ RawOne<__half> load_one(const __half* p)
{
    RawOne<__half> r;
    r.w = *reinterpret_cast<const unsigned short*>(p);
    return r;
}
__device__ __forceinline__ RawOne<float> load_one(const float* p)
{
    RawOne<float> r;
    r.v = *p;
    return r;
}

// What a unit's set-up reads from memory - q of the tile's heads and, in the unit's last piece, the new k and v row,
// each with its bias - as it sits in registers between the request and the use.  Everything is requested before
// any of it is used or anything is stored: one memory round trip instead of three in a row (q; then k behind the
// stores of q's results; then v), which every workgroup pays before its first score (5.0 -> 2.4 us after entry
// with cold caches at 32 heads x 128).  The matrix-core kernels request the next unit's rows while the current
// unit is still being finished, so that round trip disappears from a change of unit altogether.
// (qkv and bias must be aligned to a pair of elements: the tiled kernels are only taken for such pointers)
template <typename T, int D, int GT, int NTHR>
struct SetupRows {
    static constexpr int QI = (GT * (D / 2) + NTHR - 1) / NTHR;      // q pairs per thread
    static constexpr int KI = (D / 2 + NTHR - 1) / NTHR;             // k pairs per thread
    static constexpr int VI = (D + NTHR - 1) / NTHR;                 // v elements per thread
    RawPair<T> q[QI], qb[QI], k[KI], kb[KI];
    RawOne<T> v[VI], vb[VI];
};

template <typename T, int D, int GT, int NTHR>
__device__ __forceinline__ void request_setup_rows(const AttnArgs& a, const Unit& u, SetupRows<T, D, GT, NTHR>& r)
{
    using R = SetupRows<T, D, GT, NTHR>;
    const int tid = lane_id_per_unit();
    const T* qkv = static_cast<const T*>(a.qkv) + (size_t)u.b * (a.Hq + 2 * a.Hkv) * D;
    const T* bias = static_cast<const T*>(a.bias);
    const bool v_bias = bias && !(a.flags & ONELLM_ATTN_NO_V_BIAS);
#pragma unroll
    for (int k = 0; k < R::QI; ++k) {
        const int i = tid + k * NTHR;
        const int g = i / (D / 2), p = i % (D / 2);
        r.q[k] = RawPair<T>();
        r.qb[k] = RawPair<T>();
        if (i < GT * (D / 2) && u.g0 + g < a.G) {
            const int o = (u.kvh * a.G + u.g0 + g) * D + 2 * p;
            r.q[k] = load_pair(qkv + o);
            if (bias) r.qb[k] = load_pair(bias + o);
        }
    }
    if (u.is_last) {
#pragma unroll
        for (int k = 0; k < R::KI; ++k) {
            const int p = tid + k * NTHR;
            r.k[k] = RawPair<T>();
            r.kb[k] = RawPair<T>();
            if (p < D / 2) {
                const int o = (a.Hq + u.kvh) * D + 2 * p;
                r.k[k] = load_pair(qkv + o);
                if (bias) r.kb[k] = load_pair(bias + o);
            }
        }
#pragma unroll
        for (int k = 0; k < R::VI; ++k) {
            const int d = tid + k * NTHR;
            r.v[k] = RawOne<T>();
            r.vb[k] = RawOne<T>();
            if (d < D) {
                const int o = (a.Hq + a.Hkv + u.kvh) * D + d;
                r.v[k] = load_one(qkv + o);
                if (v_bias) r.vb[k] = load_one(bias + o);
            }
        }
    }
    // (the requests stay here: the compiler may not move a load past this point towards its use)
    asm volatile("" ::: "memory");
}

// The set-up proper, from the requested rows: bias, RoPE, staging in LDS; the last piece also stores the new row
// to the cache and leaves its scores in snew.  Ends with the whole workgroup synchronised on sq / sk / sv (snew is
// ready after the caller's next barrier).
template <typename T, int D, int GT, int NTHR>
__device__ __forceinline__ void stage_setup_rows(const AttnArgs& a, const RopeFreqs& fr, const Unit& u, const SetupRows<T, D, GT, NTHR>& r,
                                                 T* kc, T* vc, float* sq, float* sk, float* sv, float* snew)
{
    using R = SetupRows<T, D, GT, NTHR>;
    const int tid = lane_id_per_unit();
    const T* bias = static_cast<const T*>(a.bias);
    const bool v_bias = bias && !(a.flags & ONELLM_ATTN_NO_V_BIAS);
#pragma unroll
    for (int k = 0; k < R::QI; ++k) {
        const int i = tid + k * NTHR;
        if (i < GT * (D / 2)) {
            const int g = i / (D / 2), p = i % (D / 2);
            float x0 = r.q[k].first(), x1 = r.q[k].second();     // (zeros for a head past the group's end)
            if (bias) {
                x0 += r.qb[k].first();
                x1 += r.qb[k].second();
            }
            if (u.g0 + g < a.G && 2 * p < a.rotary_dim) rope_pair(x0, x1, p, u.pos, fr);
            sq[g * D + 2 * p] = x0 * a.qscale;
            sq[g * D + 2 * p + 1] = x1 * a.qscale;
        }
    }
    if (u.is_last) {
        const bool store = u.g0 == 0 && !(a.flags & ONELLM_ATTN_NO_CACHE_WRITE);
#pragma unroll
        for (int k = 0; k < R::KI; ++k) {
            const int p = tid + k * NTHR;
            if (p < D / 2) {
                float x0 = r.k[k].first(), x1 = r.k[k].second();
                if (bias) {
                    x0 += r.kb[k].first();
                    x1 += r.kb[k].second();
                }
                if (2 * p < a.rotary_dim) rope_pair(x0, x1, p, u.pos, fr);
                const T r0 = from_f32<T>(x0), r1 = from_f32<T>(x1);
                sk[2 * p] = to_f32(r0);
                sk[2 * p + 1] = to_f32(r1);
                if (store) {
                    kc[(size_t)(u.t - 1) * D + 2 * p] = r0;
                    kc[(size_t)(u.t - 1) * D + 2 * p + 1] = r1;
                }
            }
        }
#pragma unroll
        for (int k = 0; k < R::VI; ++k) {
            const int d = tid + k * NTHR;
            if (d < D) {
                float x = r.v[k].value();
                if (v_bias) x += r.vb[k].value();
                const T v = from_f32<T>(x);
                sv[d] = to_f32(v);
                if (store) vc[(size_t)(u.t - 1) * D + d] = v;
            }
        }
    }
    __syncthreads();
    if (u.is_last) {
        // the new row's score with each head of the tile: the heads are dealt to the waves (one wave doing them all
        // in turn started its rows a microsecond after the others, and the unit's finish waits for the last wave)
        const int lane = tid & (kWave - 1);
        for (int g = tid / kWave; g < GT; g += NTHR / kWave) {
            float part = 0.f;
            for (int d = lane; d < D; d += kWave) part = fmaf(sq[g * D + d], sk[d], part);
            part = wave_sum(part);
            if (lane == 0) snew[g] = part;
        }
    }
}

// request + set-up in one go (the kernels that do not look ahead to their next unit)
template <typename T, int D, int GT, int NTHR>
__device__ __forceinline__ void stage_q_and_new_row(const AttnArgs& a, const RopeFreqs& fr, const Unit& u, T* kc, T* vc,
                                                    float* sq, float* sk, float* sv, float* snew)
{
    SetupRows<T, D, GT, NTHR> rows;
    request_setup_rows<T, D, GT, NTHR>(a, u, rows);
    stage_setup_rows<T, D, GT, NTHR>(a, fr, u, rows, kc, vc, sq, sk, sv, snew);
}

// device-scope accesses for data that workgroups on different chip quarters hand to each other
__device__ __forceinline__ void publish(float* p, float v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float fetch(const float* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The fused finish's last step: the piece that arrived last reads the states of all pieces of its unit
// (device-scope loads, BATCH pieces in flight at a time) and writes the unit's output.
template <typename T, int D, int GT, int NTHR, int BATCH>
__device__ __forceinline__ void merge_pieces(const AttnArgs& a, const Unit& u, int tid)
{
    for (int i = tid; i < GT * D; i += NTHR) {
        const int g = i / D, d = i % D;
        if (u.g0 + g >= a.G) continue;
        const size_t e0 = u.p0 + (size_t)g * u.pstride;
        float M = -INFINITY, L = 0.f, O = 0.f;
        for (int s0 = 0; s0 < u.npieces; s0 += BATCH) {
            float mm[BATCH], ll[BATCH], oo[BATCH];
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                const size_t e = e0 + (size_t)min(s0 + j, u.npieces - 1) * u.sstride;
                mm[j] = fetch(a.part_ml + e * 2);
                ll[j] = fetch(a.part_ml + e * 2 + 1);
                oo[j] = fetch(a.part_o + e * D + d);
            }
            float bm = M;
#pragma unroll
            for (int j = 0; j < BATCH; ++j) bm = s0 + j < u.npieces ? fmaxf(bm, mm[j]) : bm;
            const float keep = __builtin_amdgcn_exp2f(M - bm);   // every piece has a finite maximum
            L *= keep;
            O *= keep;
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                const float wgt = s0 + j < u.npieces ? __builtin_amdgcn_exp2f(mm[j] - bm) : 0.f;
                L = fmaf(ll[j], wgt, L);
                O = fmaf(oo[j], wgt, O);
            }
            M = bm;
        }
        const int h = u.kvh * a.G + u.g0 + g;
        static_cast<T*>(a.out)[((size_t)u.b * a.Hq + h) * D + d] = from_f32<T>(O / L);
    }
}

// The same for a unit with many pieces (a long sequence of a small batch is cut into up to 64).  Read one float at a
// time, 32 pieces x 2 KiB take a workgroup 4.5-5 us however the loads are batched: 384 load instructions of 256
// bytes from one compute unit, two thirds of them for (m, l) pairs every thread of a head reads again.  Here the
// pairs go through LDS first - one round trip, one 8-byte load per (piece, head) - where each head's maximum, its
// pieces' weights and its sum are worked out once, a head per wave at a time; and the partial sums are read 16
// bytes at a time by the threads that own four consecutive output elements (the first batch is requested together
// with the pairs).  The order of every sum is fixed, so the result does not depend on which piece arrived last.
// `lds` holds (2 * npieces + 1) * GT floats.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t device_scope_window(const void* base)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7FFFFFFF, 0x00020000);
}
constexpr int kDeviceScopeLoad = 16;          // sc1
__device__ __forceinline__ f32x4 fetch16(__amdgpu_buffer_rsrc_t w, unsigned byte_offset)
{
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(w, byte_offset, 0, kDeviceScopeLoad));
}

template <typename T, int D, int GT, int NTHR>
__device__ __forceinline__ void merge_pieces_vec(const AttnArgs& a, const Unit& u, int tid, float* lds)
{
    static_assert(D % 4 == 0, "four consecutive elements of a head per thread");
    constexpr int NQ = GT * D / 4;                            // groups of four output elements
    constexpr int E = (NQ + NTHR - 1) / NTHR;                 // groups per thread
    constexpr int BATCH = E >= 4 ? 4 : (E == 2 ? 8 : 16);     // pieces in flight: 16 loads of 16 bytes per thread
    constexpr int NWAVE = NTHR / kWave;
    const int P = u.npieces;
    float* lw = lds;                                          // [P][GT]: m, then the weight 2^(m - max)
    float* ll = lds + P * GT;                                 // [P][GT]: l
    float* lL = ll + P * GT;                                  // [GT]: the head's sum
    const __amdgpu_buffer_rsrc_t wo = device_scope_window(a.part_o + u.p0 * D);
    const __amdgpu_buffer_rsrc_t wml = device_scope_window(a.part_ml + u.p0 * 2);
    bool valid[E];
    int hg[E];
    unsigned off[E];                                          // byte offset of the group in piece 0's entry
    f32x4 O[E];
#pragma unroll
    for (int k = 0; k < E; ++k) {
        const int q = tid + k * NTHR;
        hg[k] = (4 * q) / D;
        valid[k] = q < NQ && u.g0 + hg[k] < a.G;
        if (!valid[k]) hg[k] = 0;                             // (reads the tile's first head and stores nothing: no branches around the loads)
        off[k] = (unsigned)(((size_t)hg[k] * u.pstride * D + (valid[k] ? (4 * q) % D : 0)) * sizeof(float));
        O[k] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const unsigned piece_step = (unsigned)((size_t)u.sstride * D * sizeof(float));
    f32x4 oo[E][BATCH];
    auto request = [&](int s0) {
#pragma unroll
        for (int k = 0; k < E; ++k)
#pragma unroll
            for (int j = 0; j < BATCH; ++j) oo[k][j] = fetch16(wo, off[k] + (unsigned)min(s0 + j, P - 1) * piece_step);
    };
    request(0);
    for (int p = tid; p < P * GT; p += NTHR) {
        const int sp = p / GT, g = p % GT;
        if (u.g0 + g < a.G) {
            const unsigned e = (unsigned)(((size_t)g * u.pstride + (size_t)sp * u.sstride) * 2 * sizeof(float));
            const auto ml = __builtin_amdgcn_raw_buffer_load_b64(wml, e, 0, kDeviceScopeLoad);
            lw[p] = __uint_as_float(ml[0]);
            ll[p] = __uint_as_float(ml[1]);
        }
    }
    __syncthreads();
    {
        const int lane = tid & (kWave - 1);
        for (int g = tid / kWave; g < GT; g += NWAVE) {       // (uniform over the wave)
            if (u.g0 + g >= a.G) continue;
            float M = -INFINITY;
            for (int sp = lane; sp < P; sp += kWave) M = fmaxf(M, lw[sp * GT + g]);
#pragma unroll
            for (int o = 32; o >= 1; o >>= 1) M = fmaxf(M, __shfl_xor(M, o, kWave));
            float L = 0.f;
            for (int sp = lane; sp < P; sp += kWave) {
                const float wgt = __builtin_amdgcn_exp2f(lw[sp * GT + g] - M);   // every piece has a finite maximum
                lw[sp * GT + g] = wgt;
                L = fmaf(ll[sp * GT + g], wgt, L);
            }
            L = wave_sum(L);
            if (lane == 0) lL[g] = L;
        }
    }
    __syncthreads();
    for (int s0 = 0; s0 < P; s0 += BATCH) {
        if (s0 > 0) request(s0);
#pragma unroll
        for (int k = 0; k < E; ++k)
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                const float wgt = s0 + j < P ? lw[min(s0 + j, P - 1) * GT + hg[k]] : 0.f;
#pragma unroll
                for (int c = 0; c < 4; ++c) O[k][c] = fmaf(oo[k][j][c], wgt, O[k][c]);
            }
    }
#pragma unroll
    for (int k = 0; k < E; ++k)
        if (valid[k]) {
            const int q = tid + k * NTHR;
            const int h = u.kvh * a.G + u.g0 + hg[k];
            const float L = lL[hg[k]];
            T* out = static_cast<T*>(a.out) + ((size_t)u.b * a.Hq + h) * D + (4 * q) % D;
#pragma unroll
            for (int c = 0; c < 4; ++c) out[c] = from_f32<T>(O[k][c] / L);
        }
}

// Fused finish, first look: how many of the unit's other pieces have arrived.  Asked a streaming iteration or two
// before the piece ends and looked at in finish_unit, so the answer's round trip costs nothing.  Thread 0 only
// (-1 elsewhere, and for units that are not shared or have more pieces than the register-held merge takes).
__device__ __forceinline__ int first_look(const AttnArgs& a, const Unit& u)
{
    if (u.direct || !a.counters || !a.early_look || u.npieces > 8 || lane_id_per_unit() != 0) return -1;
    return __hip_atomic_load(a.counters + u.counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The merge of a unit's pieces by a piece that still holds its own state in registers: piece `mine` is taken from
// (Ms, Ls, Os), the others are read with device-scope loads, and the arithmetic is that of merge_pieces with all
// pieces read from memory - same batches, same order - so the unit's output does not depend on which piece merged it.
template <typename T, int D, int GT, int NTHR, int BATCH, int E>
__device__ __forceinline__ void merge_pieces_local(const AttnArgs& a, const Unit& u, int tid, int mine,
                                                   const float (&Ms)[E], const float (&Ls)[E], const float (&Os)[E])
{
#pragma unroll
    for (int k = 0; k < E; ++k) {
        const int i = tid + k * NTHR;
        const int g = i / D, d = i % D;
        if (i >= GT * D || u.g0 + g >= a.G) continue;
        const size_t e0 = u.p0 + (size_t)g * u.pstride;
        float M = -INFINITY, L = 0.f, O = 0.f;
        for (int s0 = 0; s0 < u.npieces; s0 += BATCH) {
            float mm[BATCH], ll[BATCH], oo[BATCH];
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                const int sp = min(s0 + j, u.npieces - 1);
                const size_t e = e0 + (size_t)sp * u.sstride;
                // (the loads of the own piece are issued like the others and their result dropped: no branch around a load)
                const float pm = fetch(a.part_ml + e * 2), pl = fetch(a.part_ml + e * 2 + 1), po = fetch(a.part_o + e * D + d);
                mm[j] = sp == mine ? Ms[k] : pm;
                ll[j] = sp == mine ? Ls[k] : pl;
                oo[j] = sp == mine ? Os[k] : po;
            }
            float bm = M;
#pragma unroll
            for (int j = 0; j < BATCH; ++j) bm = s0 + j < u.npieces ? fmaxf(bm, mm[j]) : bm;
            const float keep = __builtin_amdgcn_exp2f(M - bm);
            L *= keep;
            O *= keep;
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                const float wgt = s0 + j < u.npieces ? __builtin_amdgcn_exp2f(mm[j] - bm) : 0.f;
                L = fmaf(ll[j], wgt, L);
                O = fmaf(oo[j], wgt, O);
            }
            M = bm;
        }
        const int h = u.kvh * a.G + u.g0 + g;
        static_cast<T*>(a.out)[((size_t)u.b * a.Hq + h) * D + d] = from_f32<T>(O / L);
    }
}

// Merge the NST softmax states the workgroup left in LDS (plus the new token's row in the last
// split) and write either the output (single split) or this split's partial state.  The caller has
// synchronised the workgroup on st_ml / st_acc / snew.
template <typename T, int D, int GT, int NST, int NTHR>
__device__ __forceinline__ void finish_unit(const AttnArgs& a, const Unit& u, float* st_ml, float* st_acc,
                                            const float* snew, const float* sv, int arrived_before)
{
    constexpr int E = (GT * D + NTHR - 1) / NTHR;             // elements per thread
    const int tid = lane_id_per_unit();
    float Ms[E], Ls[E], Os[E];
#pragma unroll
    for (int k = 0; k < E; ++k) {
        const int i = tid + k * NTHR;
        const int g = i / D, d = i % D;
        Ms[k] = -INFINITY;
        Ls[k] = Os[k] = 0.f;
        if (i >= GT * D || u.g0 + g >= a.G) continue;
        float M = u.is_last ? snew[g] : -INFINITY;
        for (int r = 0; r < NST; ++r) M = fmaxf(M, st_ml[(r * GT + g) * 2]);
        float L = 0.f, O = 0.f;
        for (int r = 0; r < NST; ++r) {
            const float w = __builtin_amdgcn_exp2f(st_ml[(r * GT + g) * 2] - M);
            L = fmaf(st_ml[(r * GT + g) * 2 + 1], w, L);
            O = fmaf(st_acc[(size_t)(r * GT + g) * D + d], w, O);
        }
        if (u.is_last) {
            const float w = __builtin_amdgcn_exp2f(snew[g] - M);
            L += w;
            O = fmaf(sv[d], w, O);
        }
        Ms[k] = M;
        Ls[k] = L;
        Os[k] = O;
        const int h = u.kvh * a.G + u.g0 + g;
        if (u.direct) {
            static_cast<T*>(a.out)[((size_t)u.b * a.Hq + h) * D + d] = from_f32<T>(O / L);
        } else if (!a.counters) {
            const size_t pi = u.pbase + (size_t)g * u.pstride;
            a.part_o[pi * D + d] = O;
            if (d == 0) {
                a.part_ml[pi * 2] = M;
                a.part_ml[pi * 2 + 1] = L;
            }
        }
    }
    if (u.direct || !a.counters) return;

    // ---- fused finish.  Every piece of the unit has written its state with agent-scope stores and then, once all
    // of its threads' stores have completed, adds one to the unit's counter.  The piece whose add finds all the
    // others there reads their states back with agent-scope loads and merges them.  Nobody waits on anybody.
    //
    // What orders the hand-over.  By default nothing in the source language does: the stores, the add and the loads
    // are relaxed, so the ordering between a piece's state and its counter add rests on what these instructions do
    // on gfx950, which is this.  (1) An agent-scope store is `global_store ... sc1`: it is written through this chip
    // quarter's L2 to memory, and the wave's vmcnt drops only when that write has been acknowledged; the explicit
    // `s_waitcnt vmcnt(0)` + barrier below therefore mean every thread's state is in memory before thread 0 issues
    // the add.  That wait is exactly the instruction sequence the compiler emits for an agent-scope release, minus
    // `buffer_wbl2 sc1` - the write-back of lines that ordinary stores left dirty in L2, of which the state has
    // none.  (2) The add is an L2-bypassing device atomic executed at memory, so the piece that reads
    // `npieces - 1` issues its loads after all the other pieces' adds, hence after their acknowledged writes.
    // (3) An agent-scope load is `global_load ... sc1`: it is served from memory, not from a line another chip
    // quarter's write could have left stale in this quarter's L2 or this unit's L1 - which is all that the
    // `buffer_inv sc1` of an acquire would add, for ordinary loads.  The formally ordered form (release on the add,
    // an acquire fence in the merging piece: `a.ordered`, tuning key attn_ordered_finish) is kept and tested; its two
    // cache-maintenance instructions cost 8 % on a one-sequence step and 34 % on a 32-sequence ragged step on
    // MI355X (17.2 -> 18.5 us, 96 -> 129 us), which is why it is not the default.
    //
    // The piece that finds all the others already there at its first look does not publish anything: it holds
    // its own state in registers, reads the others (which were acknowledged before their adds, which came before
    // the look) and writes the unit's output - two memory round trips fewer on the path of the piece that ends
    // last, which with equal shares is the end of the kernel.
    int* arrived = reinterpret_cast<int*>(st_ml);                  // the merged states are no longer needed: reuse a word
    __syncthreads();                                            // st_ml / st_acc no longer read by anyone
    if (tid == 0) *arrived = arrived_before;
    __syncthreads();
    if (*arrived == u.npieces - 1) {
        if (tid == 0) __hip_atomic_store(a.counters + u.counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // zero for the next call
        if (a.ordered) {
            if (tid == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            __syncthreads();
        }
        const int mine = (int)((u.pbase - u.p0) / (size_t)u.sstride);
        if (u.npieces <= 2) merge_pieces_local<T, D, GT, NTHR, 2, E>(a, u, tid, mine, Ms, Ls, Os);
        else if (u.npieces <= 4) merge_pieces_local<T, D, GT, NTHR, 4, E>(a, u, tid, mine, Ms, Ls, Os);
        else merge_pieces_local<T, D, GT, NTHR, 8, E>(a, u, tid, mine, Ms, Ls, Os);
        return;
    }
#pragma unroll
    for (int k = 0; k < E; ++k) {
        const int i = tid + k * NTHR;
        const int g = i / D, d = i % D;
        if (i >= GT * D || u.g0 + g >= a.G) continue;
        const size_t pi = u.pbase + (size_t)g * u.pstride;
        publish(a.part_o + pi * D + d, Os[k]);
        if (d == 0) {
            publish(a.part_ml + pi * 2, Ms[k]);
            publish(a.part_ml + pi * 2 + 1, Ls[k]);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();                                            // all stores done
    if (tid == 0) {
        if (a.ordered) *arrived = __hip_atomic_fetch_add(a.counters + u.counter, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        else *arrived = __hip_atomic_fetch_add(a.counters + u.counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (*arrived != u.npieces - 1) return;
    if (tid == 0) __hip_atomic_store(a.counters + u.counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // zero for the next call
    if (a.ordered) {
        if (tid == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        __syncthreads();
    }
    // (pieces whose loads are in flight together: 16 at most, no more than the unit has - most have two or three -
    // rounded up to a power of two; the surplus slots of a batch repeat the last piece's loads)
    if (u.npieces <= 2) merge_pieces<T, D, GT, NTHR, 2>(a, u, tid);
    else if (u.npieces <= 4) merge_pieces<T, D, GT, NTHR, 4>(a, u, tid);
    else if (u.npieces <= 8) merge_pieces<T, D, GT, NTHR, 8>(a, u, tid);
    // (more than eight: 16-byte loads and the pairs through LDS - st_acc: NST * GT * D floats, free by now)
    else if (2 * u.npieces + 1 <= NST * D) merge_pieces_vec<T, D, GT, NTHR>(a, u, tid, st_acc);
    else merge_pieces<T, D, GT, NTHR, 16>(a, u, tid);
}

}  // namespace
}  // namespace onellm
