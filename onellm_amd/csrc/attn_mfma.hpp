// Decode attention for grouped-query heads on the matrix cores (fp16 and fp32 caches).
// (part of decode_attn.hip, which is the only file that includes it: everything here sits in its anonymous namespace)
#pragma once
#include <type_traits>
#include "attn_finish.hpp"

namespace onellm {
namespace {

// ---------------------------------------------------------------------------------------------
// Grouped-query form on the matrix cores (fp16 storage, D = 128; GT = 4, 8 or 16 query heads per
// kv head and workgroup).
//
// With one query head the scores are a matrix-vector product and the vector ALU keeps up with the
// memory stream (it is ~17 % busy).  With four query heads sharing every K/V row the same loop is
// ~65 % VALU-busy and becomes the limiter, and more than four heads need a second pass over the
// rows.  Here both products of a batch of 16 cache rows run on v_mfma_f32_16x16x16_f16 and the
// vector ALU only does the softmax bookkeeping:
//   scores  S[16 rows x 16] = K[16 x 128] . Qt[128 x 16]: A = K as loaded, B = q with the GT heads
//           repeated across the 16 columns; lane L ends up with rows 4*(L/16) + {0..3} of head L % GT;
//   output  O[16 x 128] += P[16 x 16 rows] . V[16 x 128]: A = P, exactly the registers the score tile
//           left in each lane, B = V, again straight from the load registers (a lane loads 8 columns
//           of rows 4*(L/16) + {0..3}; product c takes column c of each).
// No lane exchange is needed between the two products, the accumulators are 8 result tiles (32
// registers: 8 columns of up to 16 heads, spread over the four lane rows) instead of 128, and nothing
// has to be summed across lanes at the end.  q and P are fp32 values: each is split into an fp16 high
// part and an fp16 remainder and every product is issued for both, so they enter at ~2^-22 instead
// of being rounded to fp16; K and V are fp16 in memory, the accumulation is fp32.  The running
// maximum is per head and wave-wide; it moves rarely, so its update (two cross-row exchanges and
// the rescale) sits behind a wave-uniform branch.
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

template <int D, int GT, int NW>
__device__ __forceinline__ void gqa_mfma_unit(const AttnArgs& a, const RopeFreqs& fr, const Unit& u, float* lds, int& ev)
{
    stamp_event(a, ev);
    using T = __half;
    static_assert(GT == 4 || GT == 8 || GT == 16, "heads per tile");
    static_assert(D == 64 || D == 128 || D == 256, "head size");
    constexpr int VEC = 8;
    constexpr int NKB = D / 16;                 // k-blocks of the score product
    constexpr int NKJ = D / 32;                 // 16-byte pieces of a K row per lane
    constexpr int CG = D > 128 ? D / 128 : 1;   // groups of 128 output columns (16 lanes x 8)
    constexpr int VSLOTS = D / VEC < 16 ? D / VEC : 16;   // lanes of a row of 16 that own distinct V columns
    constexpr int NTHR = NW * kWave;
    constexpr int RPI = NW * 16;                // rows per workgroup iteration

    float* sq = lds;                            // [GT][D]
    float* sk = sq + GT * D;                    // [D]
    float* sv = sk + D;                         // [D]
    float* snew = sv + D;                       // [GT]
    float* st_ml = snew + GT;                   // [NW][GT][2]
    float* st_acc = st_ml + NW * GT * 2;        // [NW][GT][D]

    const int tid = lane_id_per_unit();
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int slot = lane & 15;
    const int grp = lane >> 4;
    const int vslot = slot % VSLOTS;            // D = 64: lanes 8..15 of a row repeat lanes 0..7 (their results are unused)
    const int r0 = u.r0, r1 = u.r1;
    const size_t head_off = a.slab + ((size_t)u.b * a.Hkv + u.kvh) * (size_t)a.S * D;
    T* kc = static_cast<T*>(a.k_cache) + head_off;
    T* vc = static_cast<T*>(a.v_cache) + head_off;
    // K: lane (slot, grp) holds row `slot` of the batch, 16-byte pieces grp + 4*jp (columns grp*8 + jp*32 ..)
    // V: lane (slot, grp) holds rows 4*grp + e of the batch, columns (cg*16 + slot)*8 .. +7
    const T* kp = kc + (size_t)(wave * 16 + slot) * D + grp * VEC;
    const T* vp = vc + (size_t)(wave * 16 + 4 * grp) * D + vslot * VEC;

    // One register buffer, K and V requested separately: the K registers are free once the batch's scores are computed
    // and the V registers once its output products are, so the next batch's K rows are on their way during this batch's
    // softmax and output products and its V rows during the next batch's scores.  The partial last batch takes the
    // same road, its row indices held at the piece's last row and its scores masked.  Measured at D = 256 against
    // requesting both after the whole batch was consumed: 32 q / 8 kv heads, batch 16 / 32, 4096 rows 90.5 -> 86.2 /
    // 159.5 -> 155.8 us; lengths 512..4096, batch 32: 102.5 -> 98.0; 12 q / 4 kv heads, batch 16: 52.1 -> 47.7; batch 4,
    // 8192 rows 54.1 -> 49.2; batch 64, 1024 rows 97.7 -> 90.1.
    auto issue_k = [&](Vec16<T> (&kv)[NKJ], int rbase) {
#pragma unroll
        for (int j = 0; j < NKJ; ++j) kv[j] = load16_stream(kp + (size_t)rbase * D + j * 32);
    };
    auto issue_v = [&](Vec16<T> (&vv)[CG * 4], int rbase) {
#pragma unroll
        for (int cg = 0; cg < CG; ++cg)
#pragma unroll
            for (int e = 0; e < 4; ++e) vv[cg * 4 + e] = load16_stream(vp + (size_t)(rbase + e) * D + cg * 128);
    };
    auto issue_k_clamped = [&](Vec16<T> (&kv)[NKJ], int rbase) {
        const int krow = min(rbase + wave * 16 + slot, r1 - 1);
#pragma unroll
        for (int j = 0; j < NKJ; ++j) kv[j] = load16_stream(kc + (size_t)krow * D + grp * VEC + j * 32);
    };
    auto issue_v_clamped = [&](Vec16<T> (&vv)[CG * 4], int rbase) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int vrow = min(rbase + wave * 16 + 4 * grp + e, r1 - 1);
#pragma unroll
            for (int cg = 0; cg < CG; ++cg) vv[cg * 4 + e] = load16_stream(vc + (size_t)vrow * D + vslot * VEC + cg * 128);
        }
    };
    const int nfull = r1 > r0 ? (r1 - r0) / RPI : 0;
    const bool partial = r1 > r0 && r0 + nfull * RPI < r1;
    Vec16<T> ka[NKJ], va[CG * 4];
    if (nfull > 0) {
        issue_k(ka, r0);
        issue_v(va, r0);
    } else if (partial) {
        issue_k_clamped(ka, r0);
        issue_v_clamped(va, r0);
    }

    stage_q_and_new_row<T, D, GT, NTHR>(a, fr, u, kc, vc, sq, sk, sv, snew);

    // B operand of the score product: column (lane % 16) is head (lane % GT); k slots 4*grp + e of
    // k-block (jp, h) are the columns grp*8 + jp*32 + 4*h + e — the ones the K registers hold there
    f16x4 qhi[NKB], qlo[NKB];
    {
        const float* qh = sq + (lane % GT) * D + grp * VEC;
#pragma unroll
        for (int jp = 0; jp < NKJ; ++jp)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float v = qh[jp * 32 + 4 * h + e];
                    const _Float16 hi = (_Float16)v;
                    qhi[jp * 2 + h][e] = hi;
                    qlo[jp * 2 + h][e] = (_Float16)(v - (float)hi);
                }
    }

    stamp_event(a, ev);
    // per lane: head (lane % GT); m is the same in every lane of a head, l is this lane's share
    float m = -INFINITY, l = 0.f;
    f32x4 o[CG * VEC];                          // o[cg*8 + c][r]: head (4*grp + r) % GT, column (cg*16 + slot)*8 + c
#pragma unroll
    for (int c = 0; c < CG * VEC; ++c) o[c] = f32x4{0.f, 0.f, 0.f, 0.f};

    // scores of the batch at rbase (row 4*grp + r of the batch, head lane % GT); after it the K registers are free
    auto scores = [&](const Vec16<T> (&kv)[NKJ], int rbase, float (&s)[4], auto masked_tag) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int jp = 0; jp < NKJ; ++jp) {
            const f16x4 k0 = __builtin_shufflevector(kv[jp].raw, kv[jp].raw, 0, 1, 2, 3);
            const f16x4 k1 = __builtin_shufflevector(kv[jp].raw, kv[jp].raw, 4, 5, 6, 7);
            s0 = __builtin_amdgcn_mfma_f32_16x16x16f16(k0, qhi[jp * 2], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x16f16(k0, qlo[jp * 2], s1, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x16f16(k1, qhi[jp * 2 + 1], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x16f16(k1, qlo[jp * 2 + 1], s1, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            s[r] = s0[r] + s1[r];
            if constexpr (MASKED) s[r] = (rbase + wave * 16 + 4 * grp + r < r1) ? s[r] : -INFINITY;
        }
    };
    // softmax update and output products of the batch; after it the V registers are free
    auto accumulate = [&](const float (&s)[4], const Vec16<T> (&vv)[CG * 4]) {
        float bm = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
        if (__builtin_amdgcn_ballot_w64(bm > m) != 0) {
            bm = fmaxf(bm, __shfl_xor(bm, 16, kWave));
            bm = fmaxf(bm, __shfl_xor(bm, 32, kWave));
            const float mnew = fmaxf(m, bm);    // finite: some row of the batch is valid
            const float alpha = __builtin_amdgcn_exp2f(m - mnew);
            l *= alpha;
            // accumulator register r belongs to head (4*grp + r) % GT: fetch that head's factor from a
            // lane that tracks it (lane % GT == head)
            float al[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) al[r] = __shfl(alpha, (lane & 48) | ((4 * grp + r) % GT), kWave);
#pragma unroll
            for (int c = 0; c < CG * VEC; ++c)
#pragma unroll
                for (int r = 0; r < 4; ++r) o[c][r] *= al[r];
            m = mnew;
        }
        f16x4 phi, plo;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float p = __builtin_amdgcn_exp2f(s[r] - m);
            l += p;
            const _Float16 hi = (_Float16)p;
            phi[r] = hi;
            plo[r] = (_Float16)(p - (float)hi);
        }
#pragma unroll
        for (int cg = 0; cg < CG; ++cg) {
            u32x4 vw[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) vw[e] = __builtin_bit_cast(u32x4, vv[cg * 4 + e].raw);
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                // column c of the four rows: one byte-permute per pair of rows
                constexpr unsigned kLow = 0x05040100u, kHigh = 0x07060302u;
                const unsigned sel = (c & 1) ? kHigh : kLow;
                const u32x2 packed = {__builtin_amdgcn_perm(vw[1][c / 2], vw[0][c / 2], sel),
                                      __builtin_amdgcn_perm(vw[3][c / 2], vw[2][c / 2], sel)};
                const f16x4 vcol = __builtin_bit_cast(f16x4, packed);
                o[cg * VEC + c] = __builtin_amdgcn_mfma_f32_16x16x16f16(phi, vcol, o[cg * VEC + c], 0, 0, 0);
                o[cg * VEC + c] = __builtin_amdgcn_mfma_f32_16x16x16f16(plo, vcol, o[cg * VEC + c], 0, 0, 0);
            }
        }
    };

    int look = -1;                              // (fused finish: the other pieces' arrivals, asked near the end)
    if (nfull == 0) look = first_look(a, u);
    if (r1 > r0) {
        int rbase = r0;
        float s[4];
        int it = 0;
        // while two more full batches lie ahead the loop holds nothing conditional (a load requested under a condition -
        // the look below is one - makes the compiler wait for every load in flight, each time round)
        for (; it + 2 < nfull; ++it) {
            take_turns(a);
            scores(ka, rbase, s, std::false_type{});
            issue_k(ka, rbase + RPI);
            accumulate(s, va);
            issue_v(va, rbase + RPI);
            rbase += RPI;
        }
        for (; it < nfull; ++it) {              // the last two full batches; the partial one is requested behind them
            take_turns(a);
            if (it + 2 == nfull || nfull == 1) look = first_look(a, u);
            scores(ka, rbase, s, std::false_type{});
            if (it + 1 < nfull) issue_k(ka, rbase + RPI);
            else if (partial) issue_k_clamped(ka, rbase + RPI);
            accumulate(s, va);
            if (it + 1 < nfull) issue_v(va, rbase + RPI);
            else if (partial) issue_v_clamped(va, rbase + RPI);
            rbase += RPI;
        }
        // a wave whose rows of the partial batch are all past the end must not touch its state (its scores are all -inf)
        if (partial && rbase + wave * 16 < r1) {
            scores(ka, rbase, s, std::true_type{});
            accumulate(s, va);
        }
    }

    stamp_event(a, ev);
    // ---- one state per wave: l is summed over the four row quarters, o is already complete
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    if (grp == 0 && slot < GT) {
        st_ml[(wave * GT + slot) * 2] = m;
        st_ml[(wave * GT + slot) * 2 + 1] = l;
    }
    if (4 * grp < GT && slot < VSLOTS) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int cg = 0; cg < CG; ++cg)
#pragma unroll
                for (int c = 0; c < VEC; ++c)
                    st_acc[(size_t)(wave * GT + 4 * grp + r) * D + (cg * 16 + slot) * VEC + c] = o[cg * VEC + c][r];
    }
    __syncthreads();
    finish_unit<T, D, GT, NW, NTHR>(a, u, st_ml, st_acc, snew, sv, look);
    stamp_event(a, ev);
}

// ---- the unit with two register buffers (D = 64, 128), both schedules.
//
// Differences from gqa_mfma_unit above (one buffer: D = 256), each measured on MI355X:
//   * a unit's last, partial batch of rows (read from the last valid row where it reaches past the end, and masked)
//     goes through the same two buffers as the full ones instead of being asked for after the last full batch was
//     consumed - a memory round trip with nothing else in flight at the end of every unit;
//   * the second batch sets out right behind the set-up instead of inside the loop;
//   * while two more full batches lie ahead, the loop holds nothing conditional, so the compiler waits for exactly
//     the loads a product needs (with a conditional request in the loop it waits for all loads: both buffers).
// 4 sequences x 8 kv heads of 8192 rows in eight pieces each 28.1 -> 26.8 us; 8 sequences of 256..2048 rows 16.4 ->
// 15.4; 64 q / 8 kv heads x 16 sequences x 8192 rows 85.4 -> 83.7; 32 sequences x 8 kv heads x 8192 rows 153.6 -> 152.0.
// Also built and measured, and not kept: a look-ahead at the next unit inside the balanced walk (the schedule state
// of two units no longer fits the scalar registers: config 3 ragged 93.3 -> 93.9, 96 sequences of 256..2048 rows
// 80.9 -> 83.3), and asking for the next piece's rows before the current piece is finished, at the end of its
// streaming loop or right behind the counter add of a piece that is handed over.  A piece's finish waits for its
// stores to be acknowledged with `s_waitcnt vmcnt(0)`, which also waits for every load in flight (64 KiB per
// workgroup: the finish went from 2.5 to 4.7-5.8 us and ate what the set-up saved), and the registers that stay live
// across the finish cost the second wave per SIMD (96 sequences of 256..2048 rows: 80 -> 105 us).
template <int D>
struct KvBatch {
    static constexpr int NKJ = D / 32;
    static constexpr int CG = D > 128 ? D / 128 : 1;
    Vec16<__half> k[NKJ], v[CG * 4];
};

// A lane's place in a unit's K and V rows: K, lane (slot, grp): row `slot` of the wave's 16, 16-byte pieces
// grp + 4 * j; V, lane (slot, grp): rows 4 * grp + e, columns (cg * 16 + slot) * 8 .. + 7.  Worked out once per unit.
template <int D>
struct KvLane {
    const __half* kp;       // row `wave * 16 + slot` of the unit's K rows, piece grp
    const __half* vp;       // row `wave * 16 + 4 * grp` of its V rows, this lane's columns
    int row0;               // wave * 16
    int slot, grp;
};

template <int D>
__device__ __forceinline__ KvLane<D> kv_lane(const __half* kc, const __half* vc)
{
    constexpr int VEC = 8, VSLOTS = D / VEC < 16 ? D / VEC : 16;
    const int tid = lane_id_per_unit();
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    KvLane<D> p;
    p.slot = lane & 15;
    p.grp = lane >> 4;
    p.row0 = wave * 16;
    p.kp = kc + (size_t)(p.row0 + p.slot) * D + p.grp * VEC;
    p.vp = vc + (size_t)(p.row0 + 4 * p.grp) * D + (p.slot % VSLOTS) * VEC;
    return p;
}

// rows [rbase, rbase + NW * 16) of a unit whose rows end at r1, into `r`; a batch that reaches past r1 reads the last
// valid row instead (the caller masks those scores)
template <int D>
__device__ __forceinline__ void issue_full_batch(KvBatch<D>& r, const KvLane<D>& p, int rbase)
{
    constexpr int NKJ = D / 32, CG = D > 128 ? D / 128 : 1;
    const __half* kp = p.kp + (size_t)rbase * D;
    const __half* vp = p.vp + (size_t)rbase * D;
#pragma unroll
    for (int j = 0; j < NKJ; ++j) r.k[j] = load16_stream(kp + j * 32);
#pragma unroll
    for (int cg = 0; cg < CG; ++cg)
#pragma unroll
        for (int e = 0; e < 4; ++e) r.v[cg * 4 + e] = load16_stream(vp + (size_t)e * D + cg * 128);
}

template <int D, int NW>
__device__ __forceinline__ void issue_batch(KvBatch<D>& r, const KvLane<D>& p, int rbase, int r1)
{
    constexpr int NKJ = D / 32, CG = D > 128 ? D / 128 : 1;
    if (rbase + NW * 16 <= r1) {
        issue_full_batch<D>(r, p, rbase);
    } else {
        // (p.kp / p.vp point at rows row0 + slot / row0 + 4 * grp of the unit: step back or forth to the clamped row)
        const int krow = min(rbase + p.row0 + p.slot, r1 - 1) - (p.row0 + p.slot);
#pragma unroll
        for (int j = 0; j < NKJ; ++j) r.k[j] = load16_stream(p.kp + (ptrdiff_t)krow * D + j * 32);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int vrow = min(rbase + p.row0 + 4 * p.grp + e, r1 - 1) - (p.row0 + 4 * p.grp);
#pragma unroll
            for (int cg = 0; cg < CG; ++cg) r.v[cg * 4 + e] = load16_stream(p.vp + (ptrdiff_t)vrow * D + cg * 128);
        }
    }
}

template <int D, int GT, int NW>
__device__ __forceinline__ void gqa_mfma_grid_unit(const AttnArgs& a, const RopeFreqs& fr, const Unit& u, float* lds, int& ev)
{
    using T = __half;
    static_assert(GT == 4 || GT == 8 || GT == 16, "heads per tile");
    static_assert(D == 64 || D == 128, "head size (two register buffers)");
    constexpr int VEC = 8;
    constexpr int NKB = D / 16;                 // k-blocks of the score product
    constexpr int NKJ = D / 32;                 // 16-byte pieces of a K row per lane
    constexpr int CG = 1;
    constexpr int VSLOTS = D / VEC < 16 ? D / VEC : 16;
    constexpr int NTHR = NW * kWave;
    constexpr int RPI = NW * 16;                // rows per batch

    float* sq = lds;                            // [GT][D]
    float* sk = sq + GT * D;                    // [D]
    float* sv = sk + D;                         // [D]
    float* snew = sv + D;                       // [GT]
    float* st_ml = snew + GT;                   // [NW][GT][2]
    float* st_acc = st_ml + NW * GT * 2;        // [NW][GT][D]

    auto cache_of = [&](const Unit& x, T*& kc, T*& vc) {
        const size_t head_off = a.slab + ((size_t)x.b * a.Hkv + x.kvh) * (size_t)a.S * D;
        kc = static_cast<T*>(a.k_cache) + head_off;
        vc = static_cast<T*>(a.v_cache) + head_off;
    };
    auto batches_of = [](const Unit& x) { return x.r1 > x.r0 ? (x.r1 - x.r0 + RPI - 1) / RPI : 0; };

    KvBatch<D> ba, bb;
    {
        stamp_event(a, ev);
        const int tid = lane_id_per_unit();
        const int lane = tid & (kWave - 1);
        const int wave = tid / kWave;
        const int slot = lane & 15;
        const int grp = lane >> 4;
        const int r0 = u.r0, r1 = u.r1;
        T *kc, *vc;
        cache_of(u, kc, vc);
        const KvLane<D> at = kv_lane<D>(kc, vc);
        const int nb = batches_of(u);
        const int nfull = r1 > r0 ? (r1 - r0) / RPI : 0;

        // the first batch of rows sets out before the set-up's own loads, the second behind them (the set-up then
        // waits for one batch, not two)
        if (nb > 0) issue_batch<D, NW>(ba, at, r0, r1);
        {
            SetupRows<T, D, GT, NTHR> rows;
            request_setup_rows<T, D, GT, NTHR>(a, u, rows);
            stage_setup_rows<T, D, GT, NTHR>(a, fr, u, rows, kc, vc, sq, sk, sv, snew);
        }
        if (nb > 1) issue_batch<D, NW>(bb, at, r0 + RPI, r1);

        // B operand of the score product: column (lane % 16) is head (lane % GT); k slots 4*grp + e of
        // k-block (jp, h) are the columns grp*8 + jp*32 + 4*h + e - the ones the K registers hold there
        f16x4 qhi[NKB], qlo[NKB];
        {
            const float* qh = sq + (lane % GT) * D + grp * VEC;
#pragma unroll
            for (int jp = 0; jp < NKJ; ++jp)
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float v = qh[jp * 32 + 4 * h + e];
                        const _Float16 hi = (_Float16)v;
                        qhi[jp * 2 + h][e] = hi;
                        qlo[jp * 2 + h][e] = (_Float16)(v - (float)hi);
                    }
        }

        stamp_event(a, ev);
        float m = -INFINITY, l = 0.f;           // per lane: head (lane % GT); m is the same in every lane of a head, l this lane's share
        f32x4 o[CG * VEC];                      // o[c][r]: head (4*grp + r) % GT, column slot*8 + c
#pragma unroll
        for (int c = 0; c < CG * VEC; ++c) o[c] = f32x4{0.f, 0.f, 0.f, 0.f};

        auto consume = [&](const KvBatch<D>& kv, int rbase, auto masked_tag) {
            constexpr bool MASKED = decltype(masked_tag)::value;
            f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int jp = 0; jp < NKJ; ++jp) {
                const f16x4 k0 = __builtin_shufflevector(kv.k[jp].raw, kv.k[jp].raw, 0, 1, 2, 3);
                const f16x4 k1 = __builtin_shufflevector(kv.k[jp].raw, kv.k[jp].raw, 4, 5, 6, 7);
                s0 = __builtin_amdgcn_mfma_f32_16x16x16f16(k0, qhi[jp * 2], s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_16x16x16f16(k0, qlo[jp * 2], s1, 0, 0, 0);
                s0 = __builtin_amdgcn_mfma_f32_16x16x16f16(k1, qhi[jp * 2 + 1], s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_16x16x16f16(k1, qlo[jp * 2 + 1], s1, 0, 0, 0);
            }
            // (rows past the unit's end - only in its last, partial batch - were read from the last valid row: masked here)
            float s[4];
            float bm = -INFINITY;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                s[r] = s0[r] + s1[r];           // score of row 4*grp + r of the batch, head lane % GT
                if constexpr (MASKED) s[r] = (rbase + wave * 16 + 4 * grp + r < r1) ? s[r] : -INFINITY;
                bm = fmaxf(bm, s[r]);
            }
            if (__builtin_amdgcn_ballot_w64(bm > m) != 0) {
                bm = fmaxf(bm, __shfl_xor(bm, 16, kWave));
                bm = fmaxf(bm, __shfl_xor(bm, 32, kWave));
                const float mnew = fmaxf(m, bm);    // finite: some row of the wave's batch is valid
                const float alpha = __builtin_amdgcn_exp2f(m - mnew);
                l *= alpha;
                // accumulator register r belongs to head (4*grp + r) % GT: fetch that head's factor from a
                // lane that tracks it (lane % GT == head)
                float al[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) al[r] = __shfl(alpha, (lane & 48) | ((4 * grp + r) % GT), kWave);
#pragma unroll
                for (int c = 0; c < CG * VEC; ++c)
#pragma unroll
                    for (int r = 0; r < 4; ++r) o[c][r] *= al[r];
                m = mnew;
            }
            f16x4 phi, plo;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float p = __builtin_amdgcn_exp2f(s[r] - m);
                l += p;
                const _Float16 hi = (_Float16)p;
                phi[r] = hi;
                plo[r] = (_Float16)(p - (float)hi);
            }
            u32x4 vw[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) vw[e] = __builtin_bit_cast(u32x4, kv.v[e].raw);
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                // column c of the four rows: one byte-permute per pair of rows
                constexpr unsigned kLow = 0x05040100u, kHigh = 0x07060302u;
                const unsigned sel = (c & 1) ? kHigh : kLow;
                const u32x2 packed = {__builtin_amdgcn_perm(vw[1][c / 2], vw[0][c / 2], sel),
                                      __builtin_amdgcn_perm(vw[3][c / 2], vw[2][c / 2], sel)};
                const f16x4 vcol = __builtin_bit_cast(f16x4, packed);
                o[c] = __builtin_amdgcn_mfma_f32_16x16x16f16(phi, vcol, o[c], 0, 0, 0);
                o[c] = __builtin_amdgcn_mfma_f32_16x16x16f16(plo, vcol, o[c], 0, 0, 0);
            }
        };
        // Batch k sits in buffer k % 2 (the first two were requested before this unit's set-up).  Full batches go in
        // pairs; the last batch of a piece may be partial: a wave whose rows of it are all past the end must not touch
        // its state (its scores would all be -inf).
        int look = -1;                          // (fused finish: the other pieces' arrivals, asked near the end)
        if (nfull == 0) look = first_look(a, u);
        int k = 0;
        // (while the two batches after the pair in flight are full ones, nothing in the loop is conditional: the
        // compiler then waits for exactly the loads a product needs and leaves the other buffer's on their way)
        for (; k + 4 <= nfull; k += 2) {
            take_turns(a);
            const int rbase = r0 + k * RPI;
            consume(ba, rbase, std::false_type{});
            issue_full_batch<D>(ba, at, rbase + 2 * RPI);
            consume(bb, rbase + RPI, std::false_type{});
            issue_full_batch<D>(bb, at, rbase + 3 * RPI);
        }
        for (; k < nfull; k += 2) {
            take_turns(a);
            if (k + 2 >= nfull) look = first_look(a, u);
            const int rbase = r0 + k * RPI;
            consume(ba, rbase, std::false_type{});
            if (k + 2 < nb) issue_batch<D, NW>(ba, at, rbase + 2 * RPI, r1);
            if (k + 1 < nfull) {
                consume(bb, rbase + RPI, std::false_type{});
                if (k + 3 < nb) issue_batch<D, NW>(bb, at, rbase + 3 * RPI, r1);
            }
        }
        if (nb > nfull) {
            const int rbase = r0 + nfull * RPI;
            if (rbase + wave * 16 < r1) {
                if (nfull & 1) consume(bb, rbase, std::true_type{});
                else consume(ba, rbase, std::true_type{});
            }
        }

        stamp_event(a, ev);
        // ---- one state per wave: l is summed over the four row quarters, o is already complete
        l += __shfl_xor(l, 16, kWave);
        l += __shfl_xor(l, 32, kWave);
        if (grp == 0 && slot < GT) {
            st_ml[(wave * GT + slot) * 2] = m;
            st_ml[(wave * GT + slot) * 2 + 1] = l;
        }
        if (4 * grp < GT && slot < VSLOTS) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c = 0; c < VEC; ++c) st_acc[(size_t)(wave * GT + 4 * grp + r) * D + slot * VEC + c] = o[c][r];
        }
        __syncthreads();
        finish_unit<T, D, GT, NW, NTHR>(a, u, st_ml, st_acc, snew, sv, look);
        stamp_event(a, ev);
    }
}

template <int D, int GT, int NW, bool DOUBLE_BUFFER, bool BALANCED>
__global__ __launch_bounds__(NW * kWave)
void decode_attn_gqa_mfma_kernel(const AttnArgs a, const RopeFreqs fr)
{
    extern __shared__ float lds[];
    stamp_entry(a);
    int ev = 0;
    if constexpr (DOUBLE_BUFFER) {
        for_each_unit<GT, BALANCED>(a, [&](const Unit& u) { gqa_mfma_grid_unit<D, GT, NW>(a, fr, u, lds, ev); });
    } else {
        for_each_unit<GT, BALANCED>(a, [&](const Unit& u) { gqa_mfma_unit<D, GT, NW>(a, fr, u, lds, ev); });
    }
    stamp_end(a);
}

template <int D, int GT>
int launch_gqa_mfma(const AttnArgs& a, const RopeFreqs& fr, hipStream_t st)
{
    constexpr int NW = 4;
    // rows of 512 bytes: one register buffer (two would not leave room for two waves per SIMD)
    constexpr bool kDouble = D <= 128;
    const size_t lds_bytes = sizeof(float) * (size_t)(GT * D + 2 * D + GT + NW * GT * 2 + NW * GT * D);
    if (lds_bytes > 64 * 1024) return ONELLM_EUNSUPPORTED;
    const int ngt = (a.G + GT - 1) / GT;
    const dim3 grid(a.Hkv * ngt, a.nsplit, a.B), block(NW * kWave);
    if (a.bal_nwg > 0)
        hipLaunchKernelGGL((decode_attn_gqa_mfma_kernel<D, GT, NW, kDouble, true>), dim3(a.bal_nwg), block, lds_bytes, st, a, fr);
    else
        hipLaunchKernelGGL((decode_attn_gqa_mfma_kernel<D, GT, NW, kDouble, false>), grid, block, lds_bytes, st, a, fr);
    return launch_status();
}

// ---------------------------------------------------------------------------------------------
// The same for fp32 caches (D = 64 or 128, more than four query heads per kv head): both products on
// v_mfma_f32_16x16x4_f32, every operand an fp32 register exactly as loaded - no splitting, no
// packing.  A K load register of lane (slot, grp) holds four columns of row `slot`; each of them is
// the A operand of one product (k = grp); q sits in 32 B-operand registers (column by column, the GT
// heads repeated over the 16 tile columns).  The score tile leaves lane (slot, grp) with rows
// 4*grp + {0..3} of head slot % GT, and score register r is the A operand of output product r
// (k = grp <-> row 4*grp + r), against V loaded as rows 4*grp + {0..3}, four columns per lane.
// 64 products of 32 cycles per 16 rows (16 KiB of K and V): about a third of what the memory stream
// leaves per SIMD.  One register buffer (two would leave one wave per SIMD), K and V requested separately as in
// gqa_mfma_unit.  Measured against requesting both after the whole batch was consumed: 64 q / 8 kv heads, batch 8,
// 8192 rows 87.3 -> 85.0 us; D = 64, batch 16: 97.5 -> 81.9; batch 4: 51.1 -> 48.7; 32 sequences of 256..2048 rows
// 64.3 -> 62.6; 128 q / 8 kv heads, batch 8, 4096 rows 56.1 -> 56.8.  (A first version with the look inside the
// steady-state loop was 8-12 % slower than before: the conditional load made every wait a wait for all loads.)
template <int D, int GT, int NW>
__device__ __forceinline__ void gqa_mfma_f32_unit(const AttnArgs& a, const RopeFreqs& fr, const Unit& u, float* lds)
{
    using T = float;
    static_assert(GT == 8 || GT == 16, "heads per tile");
    static_assert(D == 64 || D == 128, "head size");
    constexpr int VEC = 4;
    constexpr int NKJ = D / VEC / 4;            // 16-byte pieces of a K row per lane: 8
    constexpr int CG = D / (16 * VEC);          // groups of 64 output columns (16 lanes x 4): 2
    constexpr int NTHR = NW * kWave;
    constexpr int RPI = NW * 16;                // rows per workgroup iteration

    float* sq = lds;                            // [GT][D]
    float* sk = sq + GT * D;                    // [D]
    float* sv = sk + D;                         // [D]
    float* snew = sv + D;                       // [GT]
    float* st_ml = snew + GT;                   // [NW][GT][2]
    float* st_acc = st_ml + NW * GT * 2;        // [NW][GT][D]

    const int tid = lane_id_per_unit();
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int slot = lane & 15;
    const int grp = lane >> 4;
    const int r0 = u.r0, r1 = u.r1;
    const size_t head_off = a.slab + ((size_t)u.b * a.Hkv + u.kvh) * (size_t)a.S * D;
    T* kc = static_cast<T*>(a.k_cache) + head_off;
    T* vc = static_cast<T*>(a.v_cache) + head_off;
    // K: lane (slot, grp) holds row `slot` of the batch, pieces grp + 4*j (columns (grp + 4*j)*4 ..)
    // V: lane (slot, grp) holds rows 4*grp + e of the batch, columns (cg*16 + slot)*4 .. +3
    const T* kp = kc + (size_t)(wave * 16 + slot) * D + grp * VEC;
    const T* vp = vc + (size_t)(wave * 16 + 4 * grp) * D + slot * VEC;

    // K and V of a batch are requested separately: the K registers are free once the batch's scores are computed and
    // the V registers once its output products are, so the next batch's K rows are on their way during this batch's
    // softmax and output products and its V rows during the next batch's scores - a pipeline in the one register
    // buffer (two would leave one wave per SIMD).  The partial last batch takes the same road, with its row indices
    // held at the piece's last row and its scores masked.
    auto issue_k = [&](Vec16<T> (&kv)[NKJ], int rbase) {
#pragma unroll
        for (int j = 0; j < NKJ; ++j) kv[j] = load16_stream(kp + (size_t)rbase * D + j * 16);
    };
    auto issue_v = [&](Vec16<T> (&vv)[CG * 4], int rbase) {
#pragma unroll
        for (int cg = 0; cg < CG; ++cg)
#pragma unroll
            for (int e = 0; e < 4; ++e) vv[cg * 4 + e] = load16_stream(vp + (size_t)(rbase + e) * D + cg * 64);
    };
    auto issue_k_clamped = [&](Vec16<T> (&kv)[NKJ], int rbase) {
        const int krow = min(rbase + wave * 16 + slot, r1 - 1);
#pragma unroll
        for (int j = 0; j < NKJ; ++j) kv[j] = load16_stream(kc + (size_t)krow * D + grp * VEC + j * 16);
    };
    auto issue_v_clamped = [&](Vec16<T> (&vv)[CG * 4], int rbase) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int vrow = min(rbase + wave * 16 + 4 * grp + e, r1 - 1);
#pragma unroll
            for (int cg = 0; cg < CG; ++cg) vv[cg * 4 + e] = load16_stream(vc + (size_t)vrow * D + slot * VEC + cg * 64);
        }
    };
    const int nfull = r1 > r0 ? (r1 - r0) / RPI : 0;
    const bool partial = r1 > r0 && r0 + nfull * RPI < r1;
    Vec16<T> ka[NKJ], va[CG * 4];
    if (nfull > 0) {
        issue_k(ka, r0);
        issue_v(va, r0);
    } else if (partial) {
        issue_k_clamped(ka, r0);
        issue_v_clamped(va, r0);
    }

    stage_q_and_new_row<T, D, GT, NTHR>(a, fr, u, kc, vc, sq, sk, sv, snew);

    // B operand of the score products: column (lane % 16) is head (lane % GT); product (j, e) reduces
    // over the columns (grp + 4*j)*4 + e, grp = 0..3 - the ones the K registers hold there
    float qb[NKJ][VEC];
    {
        const float* qh = sq + (lane % GT) * D + grp * VEC;
#pragma unroll
        for (int j = 0; j < NKJ; ++j)
#pragma unroll
            for (int e = 0; e < VEC; ++e) qb[j][e] = qh[j * 16 + e];
    }

    float m = -INFINITY, l = 0.f;               // per lane: head lane % GT; l is this lane's share
    f32x4 o[CG * VEC];                          // o[cg*4 + c][r]: head (4*grp + r) % GT, column (cg*16 + slot)*4 + c
#pragma unroll
    for (int c = 0; c < CG * VEC; ++c) o[c] = f32x4{0.f, 0.f, 0.f, 0.f};

    // scores of the batch at rbase (row 4*grp + r of the batch, head lane % GT); after it the K registers are free
    auto scores = [&](const Vec16<T> (&kv)[NKJ], int rbase, float (&s)[4], auto masked_tag) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        f32x4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < NKJ; ++j)
#pragma unroll
            for (int e = 0; e < VEC; ++e) sc = __builtin_amdgcn_mfma_f32_16x16x4f32(kv[j].raw[e], qb[j][e], sc, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            s[r] = sc[r];
            if constexpr (MASKED) s[r] = (rbase + wave * 16 + 4 * grp + r < r1) ? s[r] : -INFINITY;
        }
    };
    // softmax update and output products of the batch; after it the V registers are free
    auto accumulate = [&](const float (&s)[4], const Vec16<T> (&vv)[CG * 4]) {
        float bm = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
        if (__builtin_amdgcn_ballot_w64(bm > m) != 0) {
            bm = fmaxf(bm, __shfl_xor(bm, 16, kWave));
            bm = fmaxf(bm, __shfl_xor(bm, 32, kWave));
            const float mnew = fmaxf(m, bm);    // finite: some row of the batch is valid
            const float alpha = __builtin_amdgcn_exp2f(m - mnew);
            l *= alpha;
            float al[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) al[r] = __shfl(alpha, (lane & 48) | ((4 * grp + r) % GT), kWave);
#pragma unroll
            for (int c = 0; c < CG * VEC; ++c)
#pragma unroll
                for (int r = 0; r < 4; ++r) o[c][r] *= al[r];
            m = mnew;
        }
        float p[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            p[r] = __builtin_amdgcn_exp2f(s[r] - m);
            l += p[r];
        }
#pragma unroll
        for (int cg = 0; cg < CG; ++cg)
#pragma unroll
            for (int c = 0; c < VEC; ++c)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    o[cg * VEC + c] = __builtin_amdgcn_mfma_f32_16x16x4f32(p[r], vv[cg * 4 + r].raw[c], o[cg * VEC + c], 0, 0, 0);
    };

    int look = -1;                              // (fused finish: the other pieces' arrivals, asked near the end)
    if (nfull == 0) look = first_look(a, u);
    if (r1 > r0) {
        int rbase = r0;
        float s[4];
        int it = 0;
        // while two more full batches lie ahead the loop holds nothing conditional (a load requested under a condition -
        // the look below is one - makes the compiler wait for every load in flight, each time round)
        for (; it + 2 < nfull; ++it) {
            take_turns(a);
            scores(ka, rbase, s, std::false_type{});
            issue_k(ka, rbase + RPI);
            accumulate(s, va);
            issue_v(va, rbase + RPI);
            rbase += RPI;
        }
        for (; it < nfull; ++it) {              // the last two full batches; the partial one is requested behind them
            take_turns(a);
            if (it + 2 == nfull || nfull == 1) look = first_look(a, u);
            scores(ka, rbase, s, std::false_type{});
            if (it + 1 < nfull) issue_k(ka, rbase + RPI);
            else if (partial) issue_k_clamped(ka, rbase + RPI);
            accumulate(s, va);
            if (it + 1 < nfull) issue_v(va, rbase + RPI);
            else if (partial) issue_v_clamped(va, rbase + RPI);
            rbase += RPI;
        }
        if (partial && rbase + wave * 16 < r1) {
            scores(ka, rbase, s, std::true_type{});
            accumulate(s, va);
        }
    }

    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    if (grp == 0 && slot < GT) {
        st_ml[(wave * GT + slot) * 2] = m;
        st_ml[(wave * GT + slot) * 2 + 1] = l;
    }
    if (4 * grp < GT) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int cg = 0; cg < CG; ++cg)
#pragma unroll
                for (int c = 0; c < VEC; ++c)
                    st_acc[(size_t)(wave * GT + 4 * grp + r) * D + (cg * 16 + slot) * VEC + c] = o[cg * VEC + c][r];
    }
    __syncthreads();
    finish_unit<T, D, GT, NW, NTHR>(a, u, st_ml, st_acc, snew, sv, look);
}

template <int D, int GT, int NW, bool BALANCED>
__global__ __launch_bounds__(NW * kWave)
void decode_attn_gqa_mfma_f32_kernel(const AttnArgs a, const RopeFreqs fr)
{
    extern __shared__ float lds[];
    for_each_unit<GT, BALANCED>(a, [&](const Unit& u) { gqa_mfma_f32_unit<D, GT, NW>(a, fr, u, lds); });
}

template <int D, int GT>
int launch_gqa_mfma_f32(const AttnArgs& a, const RopeFreqs& fr, hipStream_t st)
{
    constexpr int NW = 4;
    const size_t lds_bytes = sizeof(float) * (size_t)(GT * D + 2 * D + GT + NW * GT * 2 + NW * GT * D);
    const int ngt = (a.G + GT - 1) / GT;
    const dim3 grid(a.Hkv * ngt, a.nsplit, a.B), block(NW * kWave);
    if (a.bal_nwg > 0)
        hipLaunchKernelGGL((decode_attn_gqa_mfma_f32_kernel<D, GT, NW, true>), dim3(a.bal_nwg), block, lds_bytes, st, a, fr);
    else
        hipLaunchKernelGGL((decode_attn_gqa_mfma_f32_kernel<D, GT, NW, false>), grid, block, lds_bytes, st, a, fr);
    return launch_status();
}

}  // namespace
}  // namespace onellm
