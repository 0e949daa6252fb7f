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
#include <math.h>
#include "common.hpp"
#include "rope.hpp"

namespace onellm {
namespace {

constexpr size_t kCounterBytes = 64 * 1024; // arrival counters of the fused finish: the first bytes of every workspace
constexpr int kBalancedWorkgroups = 512;   // two 4-wave workgroups per compute unit: what the register budgets keep resident
constexpr long long kBalancedMinItems = 3072;   // the balanced schedule is not the default for a smaller step
constexpr long long kFusedGridMaxItems = 8192;  // per-sequence lengths on the grid schedule: fused finish up to this size

struct AttnArgs {
    const void* qkv;
    const void* bias;
    void* k_cache;
    void* v_cache;
    void* out;
    float* part_o;        // [B, Hq, nsplit, D]
    float* part_ml;       // [B, Hq, nsplit, 2]
    const int* t_dev;
    int t_host;
    int B, Hq, Hkv, G, S;
    int chunk;            // cache rows per split
    int nsplit;           // grid.x
    int rotary_dim;
    int pos_offset;
    unsigned flags;
    float qscale;         // log2(e) / sqrt(D), folded into q
    size_t slab;          // element offset of the layer slab inside the cache
    // balanced schedule (bal_nwg > 0): the grid is bal_nwg workgroups and each takes an equal,
    // contiguous share of all work items (an item = item_rows history rows of one unit)
    int bal_nwg;
    int item_rows;
    int gt;               // query heads per tile, for the merge kernel
    // fused finish (counters != NULL): one arrival counter per unit, zero between calls; the piece
    // that arrives last merges the unit's partial states itself and no merge kernel is launched
    int* counters;
};

// What one workgroup works on: a chunk of the history of one (sequence, kv-head) for up to GT query heads.
struct Unit {
    int b, kvh, g0;        // sequence, kv head, first query head of the tile inside the group
    int t, pos;            // attended positions of the sequence; RoPE position of the new token
    int split, last;       // this workgroup's split and the sequence's last split
    int r0, r1;            // history rows [r0, r1) of this split
    bool is_last;          // the last split also owns the new token's row
    bool direct;           // the workgroup sees the whole unit: it writes the output, not a partial state
    size_t pbase;          // partial-state entry of tile head g: pbase + g * pstride
    int pstride;
    // for the fused finish: the unit's pieces are entries p0 + g * pstride + s * sstride, s < npieces
    size_t p0;
    int sstride, npieces, counter;
};

// Workgroups are dealt to the 8 XCDs round-robin in linear block order.  The kv-head index is the
// fastest grid dimension so that every XCD sees the same mix of sequences and splits, and the split
// index is rotated by the sequence index so that, with ragged lengths, the splits every sequence has
// (the low ones) do not all land on the same XCDs.  Returns false when there is nothing to do.
template <int GT>
__device__ __forceinline__ bool locate_unit(const AttnArgs& a, Unit& u)
{
    const int ngt = (a.G + GT - 1) / GT;
    u.kvh = blockIdx.x / ngt;
    u.g0 = (blockIdx.x % ngt) * GT;
    u.b = blockIdx.z;
    u.split = (blockIdx.y + u.b) % a.nsplit;
    u.t = a.t_dev ? a.t_dev[u.b] : a.t_host;
    if (u.t < 1 || u.t > a.S) return false;      // out-of-contract length: touch nothing
    u.last = (u.t - 1) / a.chunk;
    if (u.split > u.last) return false;
    u.is_last = u.split == u.last;
    u.r0 = u.split * a.chunk;
    u.r1 = min(u.r0 + a.chunk, u.t - 1);
    u.pos = u.t + a.pos_offset;
    u.direct = a.nsplit == 1 || (a.counters && u.last == 0);    // (with the fused finish a one-piece sequence needs no partial)
    u.p0 = ((size_t)u.b * a.Hq + u.kvh * a.G + u.g0) * a.nsplit;
    u.pbase = u.p0 + u.split;
    u.pstride = a.nsplit;
    u.sstride = 1;
    u.npieces = min(u.last + 1, a.nsplit);       // (a length above max_t is out of contract: stay consistent)
    u.counter = u.b * (a.Hkv * ngt) + blockIdx.x;
    return true;
}

// ---- balanced schedule -----------------------------------------------------------------------
// All work of a step is cut into items of item_rows history rows; a unit (sequence, kv head, head
// tile) of a sequence with t attended positions has max(1, ceil((t-1)/item_rows)) of them (the
// last one also carries the new token's row).  Items are numbered sequence-major, then unit, then
// row order, and workgroup i of N takes items [i*W/N, (i+1)*W/N): every workgroup streams the same
// number of rows whatever the lengths are, crossing from one unit into the next where its share
// does.  A unit seen whole by one workgroup is finished by it; otherwise each workgroup that
// touches it leaves a partial state in entry (workgroup + global unit index) - unique, because
// along the walk either the workgroup or the unit advances - and whoever merges them (the merge
// kernel, or the piece that arrives last when the finish is fused) derives the same boundaries from
// the same lengths.
__device__ __forceinline__ int seq_items(const AttnArgs& a, int t)
{
    if (t < 1 || t > a.S) return 0;               // out-of-contract length: no work, nothing touched
    const int n = (t - 1 + a.item_rows - 1) / a.item_rows;
    return n < 1 ? 1 : n;
}

// The schedule is the same in every lane; saying so keeps it in scalar registers (the kernels that
// walk it are short of vector registers).
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ long long uniform(long long v)
{
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(unsigned long long)v);
    const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)((unsigned long long)v >> 32));
    return (long long)(((unsigned long long)hi << 32) | lo);
}

// Thread index as a value the compiler takes as new each time it is asked for: everything a unit
// derives from it (addresses, masks, lane roles) is then recomputed per unit instead of being
// hoisted out of the loop over units and held in registers across the streaming loop.
__device__ __forceinline__ int lane_id_per_unit()
{
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    return tid;
}

__device__ __forceinline__ long long wave_sum_i64(long long v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// items of all sequences, and of the sequences before `before` (every lane gets both)
__device__ __forceinline__ void count_items(const AttnArgs& a, int before, long long& total, long long& prefix)
{
    if (!a.t_dev) {
        const int it = seq_items(a, a.t_host);
        total = (long long)a.B * it;
        prefix = (long long)before * it;
        return;
    }
    const int lane = threadIdx.x & (kWave - 1);
    long long tot = 0, pre = 0;
    for (int bb = lane; bb < a.B; bb += kWave) {
        const int it = seq_items(a, a.t_dev[bb]);
        tot += it;
        if (bb < before) pre += it;
    }
    total = uniform(wave_sum_i64(tot));
    prefix = uniform(wave_sum_i64(pre));
}

// workgroup that owns item x when W items are dealt to N workgroups as [i*W/N, (i+1)*W/N)
__device__ __forceinline__ int item_owner(long long x, long long W, int N)
{
    return (int)(((x + 1) * N - 1) / W);
}

// Workgroups that take part: never more than there are items, so that no share is empty and the
// workgroups of a unit are consecutive - and, as the host sizes the grid for the longest length it
// was given while the real lengths may be much shorter: no workgroup for fewer than four items, and
// not between one and two workgroups per compute unit (some units would get two shares, the rest one:
// better one larger share each).  The launch has one workgroup per compute unit or two (or what a sweep
// asked for, taken as it is).
__device__ __forceinline__ int balanced_workgroups(const AttnArgs& a, long long W)
{
    long long n = (W + 3) / 4;
    if (n > a.bal_nwg) n = a.bal_nwg;
    if (a.bal_nwg == kBalancedWorkgroups && n > kBalancedWorkgroups / 2 && n < kBalancedWorkgroups) n = kBalancedWorkgroups / 2;
    return (int)n;
}

struct Walk {
    long long W;           // items of the whole step
    int N;                 // workgroups that share them
    long long cur, hi;     // next item of this workgroup, end of its share
    long long base;        // first item of sequence b
    int b, items;          // current sequence and its items per unit
    int nunits;            // units per sequence
};

// Positions the walk at the first item of workgroup blockIdx.x; false when its share is empty.
__device__ __forceinline__ bool walk_begin(const AttnArgs& a, int nunits, Walk& w)
{
    const int lane = threadIdx.x & (kWave - 1);
    long long total, unused;
    count_items(a, 0, total, unused);
    const long long W = total * nunits;
    const int N = balanced_workgroups(a, W);
    if ((int)blockIdx.x >= N) return false;
    w.nunits = nunits;
    w.W = W;
    w.N = N;
    w.cur = uniform((long long)blockIdx.x * W / N);
    w.hi = uniform((long long)(blockIdx.x + 1) * W / N);         // > cur, because N <= W
    const long long target = w.cur / nunits;       // the sequence that holds item `cur` holds per-unit item `target`
    if (!a.t_dev) {
        w.items = seq_items(a, a.t_host);
        w.b = uniform((int)(target / w.items));
        w.base = (long long)w.b * w.items * nunits;
        return true;
    }
    long long run = 0;
    for (int c = 0; c < a.B; c += kWave) {
        const int bb = c + lane;
        const int it = bb < a.B ? seq_items(a, a.t_dev[bb]) : 0;
        long long inc = it;
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const long long v = __shfl_up(inc, off, kWave);
            if (lane >= off) inc += v;
        }
        const long long tot = __shfl(inc, kWave - 1, kWave);
        if (run + tot > target) {
            const unsigned long long hit = __builtin_amdgcn_ballot_w64(run + inc > target);
            const int f = __builtin_ctzll(hit);
            w.b = c + f;
            w.items = uniform(__shfl(it, f, kWave));
            w.base = (run + uniform(__shfl(inc, f, kWave)) - w.items) * nunits;
            return true;
        }
        run += uniform(tot);
    }
    return false;                                   // not reached: target < total
}

// The unit piece at the walk's position (as many of the unit's remaining items as the share allows).
template <int GT>
__device__ __forceinline__ void walk_unit(const AttnArgs& a, const Walk& w, Unit& u, int& nitems)
{
    const int ngt = (a.G + GT - 1) / GT;
    const long long rel = w.cur - w.base;
    const int uib = uniform((int)(rel / w.items));
    const int item = uniform((int)(rel - (long long)uib * w.items));
    const long long left = w.hi - w.cur;
    nitems = w.items - item;
    if (left < nitems) nitems = (int)left;
    nitems = uniform(nitems);
    u.b = w.b;
    u.kvh = uib / ngt;
    u.g0 = (uib % ngt) * GT;
    u.t = uniform(a.t_dev ? a.t_dev[w.b] : a.t_host);
    u.pos = u.t + a.pos_offset;
    u.split = 0;
    u.last = 0;
    u.r0 = item * a.item_rows;
    u.r1 = min(u.r0 + nitems * a.item_rows, u.t - 1);
    u.is_last = item + nitems == w.items;
    u.direct = item == 0 && u.is_last;
    const size_t unit_index = (size_t)w.b * w.nunits + uib;
    u.pbase = ((size_t)blockIdx.x + unit_index) * GT;
    u.pstride = 1;
    u.p0 = 0;
    u.sstride = GT;
    u.npieces = 1;
    u.counter = (int)unit_index;
    if (!u.direct && a.counters) {
        const long long first = w.base + (long long)uib * w.items;
        const int i0 = uniform(item_owner(first, w.W, w.N)), i1 = uniform(item_owner(first + w.items - 1, w.W, w.N));
        u.p0 = ((size_t)i0 + unit_index) * GT;
        u.npieces = i1 - i0 + 1;
    }
}

// Moves past nitems items; steps to the next sequence that has work when the current one is done.
__device__ __forceinline__ void walk_advance(const AttnArgs& a, Walk& w, int nitems)
{
    w.cur += nitems;
    if (w.cur >= w.hi) return;
    if (w.cur == w.base + (long long)w.items * w.nunits) {
        w.base = w.cur;
        do {
            if (++w.b >= a.B) {                      // lengths changed under the kernel (out of contract): stop
                w.cur = w.hi;
                return;
            }
            w.items = uniform(seq_items(a, a.t_dev ? a.t_dev[w.b] : a.t_host));
        } while (w.items == 0);                      // cur < hi <= W: a later sequence has items
    }
}

// Runs `body(unit)` for the one unit of the grid schedule, or for every unit piece of this
// workgroup's share of the balanced schedule.
template <int GT, bool BALANCED, typename F>
__device__ __forceinline__ void for_each_unit(const AttnArgs& a, F&& body)
{
    Unit u;
    if constexpr (!BALANCED) {
        if (locate_unit<GT>(a, u)) body(u);
    } else {
        Walk w;
        if (!walk_begin(a, a.Hkv * ((a.G + GT - 1) / GT), w)) return;
        while (w.cur < w.hi) {
            int nitems;
            walk_unit<GT>(a, w, u, nitems);
            body(u);
            walk_advance(a, w, nitems);
            if (w.cur < w.hi) __syncthreads();       // the next unit reuses the LDS staging
        }
    }
}

// q of the tile's heads (and, in the last split, the new k/v row): bias, RoPE, staging in LDS; the
// last split also stores the new row to the cache and leaves its scores in snew.  Ends with the
// whole workgroup synchronised on sq / sk / sv (snew is ready after the caller's next barrier).
template <typename T, int D, int GT, int NTHR>
__device__ __forceinline__ void stage_q_and_new_row(const AttnArgs& a, const RopeFreqs& fr, const Unit& u, T* kc, T* vc,
                                                    float* sq, float* sk, float* sv, float* snew)
{
    const int tid = lane_id_per_unit();
    const T* qkv = static_cast<const T*>(a.qkv) + (size_t)u.b * (a.Hq + 2 * a.Hkv) * D;
    const T* bias = static_cast<const T*>(a.bias);
    // Everything this set-up reads from memory - q, the new k and v row, their biases - is requested before any
    // of it is used or anything is stored: one memory round trip instead of three in a row (q; then k behind the
    // stores of q's results; then v), which every workgroup pays before its first score (5.0 -> 2.4 us after
    // entry with cold caches at 32 heads x 128).
    constexpr int QI = (GT * (D / 2) + NTHR - 1) / NTHR;      // q pairs per thread
    constexpr int KI = (D / 2 + NTHR - 1) / NTHR;             // k pairs per thread
    constexpr int VI = (D + NTHR - 1) / NTHR;                 // v elements per thread
    T q0[QI], q1[QI], qb0[QI], qb1[QI], k0[KI], k1[KI], kb0[KI], kb1[KI], v0[VI], vb0[VI];
    const bool v_bias = bias && !(a.flags & ONELLM_ATTN_NO_V_BIAS);
#pragma unroll
    for (int k = 0; k < QI; ++k) {
        const int i = tid + k * NTHR;
        const int g = i / (D / 2), p = i % (D / 2);
        q0[k] = q1[k] = qb0[k] = qb1[k] = from_f32<T>(0.f);
        if (i < GT * (D / 2) && u.g0 + g < a.G) {
            const int o = (u.kvh * a.G + u.g0 + g) * D + 2 * p;
            q0[k] = qkv[o];
            q1[k] = qkv[o + 1];
            if (bias) {
                qb0[k] = bias[o];
                qb1[k] = bias[o + 1];
            }
        }
    }
    if (u.is_last) {
#pragma unroll
        for (int k = 0; k < KI; ++k) {
            const int p = tid + k * NTHR;
            k0[k] = k1[k] = kb0[k] = kb1[k] = from_f32<T>(0.f);
            if (p < D / 2) {
                const int o = (a.Hq + u.kvh) * D + 2 * p;
                k0[k] = qkv[o];
                k1[k] = qkv[o + 1];
                if (bias) {
                    kb0[k] = bias[o];
                    kb1[k] = bias[o + 1];
                }
            }
        }
#pragma unroll
        for (int k = 0; k < VI; ++k) {
            const int d = tid + k * NTHR;
            v0[k] = vb0[k] = from_f32<T>(0.f);
            if (d < D) {
                const int o = (a.Hq + a.Hkv + u.kvh) * D + d;
                v0[k] = qkv[o];
                if (v_bias) vb0[k] = bias[o];
            }
        }
    }
#pragma unroll
    for (int k = 0; k < QI; ++k) {
        const int i = tid + k * NTHR;
        if (i < GT * (D / 2)) {
            const int g = i / (D / 2), p = i % (D / 2);
            float x0 = to_f32(q0[k]), x1 = to_f32(q1[k]);     // (zeros for a head past the group's end)
            if (bias) {
                x0 += to_f32(qb0[k]);
                x1 += to_f32(qb1[k]);
            }
            if (u.g0 + g < a.G && 2 * p < a.rotary_dim) rope_pair(x0, x1, p, u.pos, fr);
            sq[g * D + 2 * p] = x0 * a.qscale;
            sq[g * D + 2 * p + 1] = x1 * a.qscale;
        }
    }
    if (u.is_last) {
        const bool store = u.g0 == 0 && !(a.flags & ONELLM_ATTN_NO_CACHE_WRITE);
#pragma unroll
        for (int k = 0; k < KI; ++k) {
            const int p = tid + k * NTHR;
            if (p < D / 2) {
                float x0 = to_f32(k0[k]), x1 = to_f32(k1[k]);
                if (bias) {
                    x0 += to_f32(kb0[k]);
                    x1 += to_f32(kb1[k]);
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
        for (int k = 0; k < VI; ++k) {
            const int d = tid + k * NTHR;
            if (d < D) {
                float x = to_f32(v0[k]);
                if (v_bias) x += to_f32(vb0[k]);
                const T v = from_f32<T>(x);
                sv[d] = to_f32(v);
                if (store) vc[(size_t)(u.t - 1) * D + d] = v;
            }
        }
    }
    __syncthreads();
    if (u.is_last && tid < kWave) {
        const int lane = tid;
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            float part = 0.f;
            for (int d = lane; d < D; d += kWave) part = fmaf(sq[g * D + d], sk[d], part);
            part = wave_sum(part);
            if (lane == 0) snew[g] = part;
        }
    }
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

// The same for a unit with many pieces (a long sequence of a small batch is cut into up to 64): the (m, l)
// pairs of all pieces go through LDS first - one round trip - where each head's maximum, its pieces' weights
// and its sum are worked out once, a head per wave at a time; then only the partial sums are read, about 64
// loads in flight per thread over all of its elements, instead of one element and sixteen pieces at a time
// (eight round trips become two at 64 pieces and two elements per thread: the first batch of sums is
// requested together with the pairs).  The order of every sum is
// fixed, so the result does not depend on which piece arrived last.  `lds` holds (2 * npieces + 1) * GT floats.
template <typename T, int D, int GT, int NTHR, int INFLIGHT>
__device__ __forceinline__ void merge_pieces_wide(const AttnArgs& a, const Unit& u, int tid, float* lds)
{
    constexpr int E = (GT * D + NTHR - 1) / NTHR;             // elements per thread
    constexpr int BATCH = INFLIGHT / E < 4 ? 4 : (INFLIGHT / E > 32 ? 32 : INFLIGHT / E);   // (more would cost the single-head kernel registers)
    constexpr int NWAVE = NTHR / kWave;
    const int P = u.npieces;
    float* lw = lds;                                          // [P][GT]: m, then the weight 2^(m - max)
    float* ll = lds + P * GT;                                 // [P][GT]: l
    float* lL = ll + P * GT;                                  // [GT]: the head's sum
    bool valid[E];
    int hg[E];
    const float* po[E];
    float O[E];
#pragma unroll
    for (int k = 0; k < E; ++k) {
        const int i = tid + k * NTHR;
        hg[k] = i / D;
        valid[k] = i < GT * D && u.g0 + hg[k] < a.G;
        if (!valid[k]) hg[k] = 0;                             // (a thread without an element reads the tile's first head and stores nothing:
        po[k] = a.part_o + (u.p0 + (size_t)hg[k] * u.pstride) * D + i % D;   //  the loads below stay free of branches)
        O[k] = 0.f;
    }
    float oo[E][BATCH];
    auto request = [&](int s0) {
#pragma unroll
        for (int k = 0; k < E; ++k)
#pragma unroll
            for (int j = 0; j < BATCH; ++j)
                oo[k][j] = fetch(po[k] + (size_t)min(s0 + j, P - 1) * u.sstride * D);
    };
    // the first batch of partial sums travels together with the (m, l) pairs
    request(0);
    for (int p = tid; p < P * GT; p += NTHR) {
        const int sp = p / GT, g = p % GT;
        if (u.g0 + g < a.G) {
            const size_t e = u.p0 + (size_t)g * u.pstride + (size_t)sp * u.sstride;
            lw[p] = fetch(a.part_ml + e * 2);
            ll[p] = fetch(a.part_ml + e * 2 + 1);
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
            for (int off = 32; off >= 1; off >>= 1) M = fmaxf(M, __shfl_xor(M, off, kWave));
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
                const float wgt = lw[min(s0 + j, P - 1) * GT + hg[k]];
                O[k] = fmaf(oo[k][j], s0 + j < P ? wgt : 0.f, O[k]);
            }
    }
#pragma unroll
    for (int k = 0; k < E; ++k)
        if (valid[k]) {
            const int i = tid + k * NTHR;
            const int h = u.kvh * a.G + u.g0 + hg[k];
            static_cast<T*>(a.out)[((size_t)u.b * a.Hq + h) * D + i % D] = from_f32<T>(O[k] / lL[hg[k]]);
        }
}

// Merge the NST softmax states the workgroup left in LDS (plus the new token's row in the last
// split) and write either the output (single split) or this split's partial state.  The caller has
// synchronised the workgroup on st_ml / st_acc / snew.
template <typename T, int D, int GT, int NST, int NTHR>
__device__ __forceinline__ void finish_unit(const AttnArgs& a, const Unit& u, float* st_ml, float* st_acc,
                                            const float* snew, const float* sv)
{
    for (int i = lane_id_per_unit(); i < GT * D; i += NTHR) {
        const int g = i / D, d = i % D;
        if (u.g0 + g >= a.G) continue;
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
        } else {
            const size_t pi = u.pbase + (size_t)g * u.pstride;
            publish(a.part_o + pi * D + d, O);
            if (d == 0) {
                publish(a.part_ml + pi * 2, M);
                publish(a.part_ml + pi * 2 + 1, L);
            }
        }
    }
    if (u.direct || !a.counters) return;

    // ---- fused finish.  Every piece of the unit has written its state with device-scope stores
    // (written through to memory, not left in this chip quarter's L2) and then, once all of its
    // threads' stores have completed, adds one to the unit's counter.  The piece whose add finds
    // all the others there reads their states back with device-scope loads and merges them.  No
    // cache write-back or invalidation is involved: the only data that crosses between workgroups
    // moves through these scoped accesses, and nobody waits on anybody.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();                                            // all stores done; st_ml no longer read
    int* arrived = reinterpret_cast<int*>(st_ml);                  // the merged states are no longer needed: reuse a word
    const int tid = lane_id_per_unit();
    if (tid == 0)
        *arrived = __hip_atomic_fetch_add(a.counters + u.counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*arrived != u.npieces - 1) return;
    if (tid == 0) __hip_atomic_store(a.counters + u.counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // zero for the next call
    // (pieces whose loads are in flight together: 16 at most, no more than the unit has - most have two or three -
    // rounded up to a power of two; the surplus slots of a batch repeat the last piece's loads)
    if (u.npieces <= 2) merge_pieces<T, D, GT, NTHR, 2>(a, u, tid);
    else if (u.npieces <= 4) merge_pieces<T, D, GT, NTHR, 4>(a, u, tid);
    else if (u.npieces <= 8) merge_pieces<T, D, GT, NTHR, 8>(a, u, tid);
    // (where a thread has 128 partial sums or more to read - measured: 32 q / 8 kv heads, batch 1, 8192 rows, 64 pieces x 2
    // elements 16.9 -> 16.5 us; 64 q heads, 32768 rows, 32 x 4: 35.4 -> 32.3; batch 2, 32 x 2: 20.0 -> 21.1, hence
    // not there.  st_acc: NST * GT * D floats, free by now)
    else if (u.npieces * ((GT * D + NTHR - 1) / NTHR) >= 128 && 2 * u.npieces + 1 <= NST * D)
        merge_pieces_wide<T, D, GT, NTHR, 64>(a, u, tid, st_acc);
    else merge_pieces<T, D, GT, NTHR, 16>(a, u, tid);
}

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
    const int nfull = r1 > r0 ? (r1 - r0) / RPI : 0;
    Vec16<T> ka[U], va[U], kb[U], vb[U];
    if (nfull > 0) issue(ka, va, r0);

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

    if (r1 > r0) {
        // Full iterations are software-pipelined over two register buffers: the loads of the next
        // iteration are in flight while the current one is consumed, so a wave never sits with an
        // empty memory queue.  The (at most one) partial iteration at the end is masked.
        const bool none[U] = {};
        int rbase = r0;
        for (int it = 0; it < nfull; it += 2) {
            if (it + 1 < nfull) issue(kb, vb, rbase + RPI);
            consume(ka, va, none, std::false_type{});
            if (it + 1 < nfull) {
                if (it + 2 < nfull) issue(ka, va, rbase + 2 * RPI);
                consume(kb, vb, none, std::false_type{});
            }
            rbase += 2 * RPI;
        }
        rbase = r0 + nfull * RPI;
        if (rbase < r1) {
            bool valid[U];
#pragma unroll
            for (int u_ = 0; u_ < U; ++u_) {
                int row = rbase + u_ * NRG + rg;
                valid[u_] = row < r1;
                row = min(row, r1 - 1);
                ka[u_] = load16_stream(kp + (size_t)row * D);
                va[u_] = load16_stream(vp + (size_t)row * D);
            }
            consume(ka, va, valid, std::true_type{});
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
    finish_unit<T, D, GT, NRG, NTHR>(a, u, st_ml, st_acc, snew, sv);
}

template <typename T, int LPR, int GT, int U, int NW, bool BALANCED>
__global__ __launch_bounds__(NW * kWave)
void decode_attn_split_kernel(const AttnArgs a, const RopeFreqs fr)
{
    extern __shared__ float lds[];
    for_each_unit<GT, BALANCED>(a, [&](const Unit& u) { split_unit<T, LPR, LPR, GT, U, NW>(a, fr, u, lds); });
}

// the same kernel for rows that do not fill their lanes (grid schedule only)
template <typename T, int LPR, int DP, int GT>
__global__ __launch_bounds__(4 * kWave)
void decode_attn_split_padded_kernel(const AttnArgs a, const RopeFreqs fr)
{
    extern __shared__ float lds[];
    for_each_unit<GT, false>(a, [&](const Unit& u) { split_unit<T, LPR, DP, GT, 4, 4>(a, fr, u, lds); });
}

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

template <int D, int GT, int NW, bool DOUBLE_BUFFER>
__device__ __forceinline__ void gqa_mfma_unit(const AttnArgs& a, const RopeFreqs& fr, const Unit& u, float* lds)
{
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

    auto issue = [&](Vec16<T> (&kv)[NKJ], Vec16<T> (&vv)[CG * 4], int rbase) {
#pragma unroll
        for (int j = 0; j < NKJ; ++j) kv[j] = load16_stream(kp + (size_t)rbase * D + j * 32);
#pragma unroll
        for (int cg = 0; cg < CG; ++cg)
#pragma unroll
            for (int e = 0; e < 4; ++e) vv[cg * 4 + e] = load16_stream(vp + (size_t)(rbase + e) * D + cg * 128);
    };
    const int nfull = r1 > r0 ? (r1 - r0) / RPI : 0;
    Vec16<T> ka[NKJ], va[CG * 4], kb[DOUBLE_BUFFER ? NKJ : 1], vb[DOUBLE_BUFFER ? CG * 4 : 1];
    if (nfull > 0) issue(ka, va, r0);

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

    // per lane: head (lane % GT); m is the same in every lane of a head, l is this lane's share
    float m = -INFINITY, l = 0.f;
    f32x4 o[CG * VEC];                          // o[cg*8 + c][r]: head (4*grp + r) % GT, column (cg*16 + slot)*8 + c
#pragma unroll
    for (int c = 0; c < CG * VEC; ++c) o[c] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto consume = [&](const Vec16<T> (&kv)[NKJ], const Vec16<T> (&vv)[CG * 4], int rbase, auto masked_tag) {
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
        float s[4];
        float bm = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            s[r] = s0[r] + s1[r];               // score of row 4*grp + r of the batch, head lane % GT
            if constexpr (MASKED) s[r] = (rbase + wave * 16 + 4 * grp + r < r1) ? s[r] : -INFINITY;
            bm = fmaxf(bm, s[r]);
        }
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

    if (r1 > r0) {
        int rbase = r0;
        if constexpr (DOUBLE_BUFFER) {
            for (int it = 0; it < nfull; it += 2) {
                if (it + 1 < nfull) issue(kb, vb, rbase + RPI);
                consume(ka, va, rbase, std::false_type{});
                if (it + 1 < nfull) {
                    if (it + 2 < nfull) issue(ka, va, rbase + 2 * RPI);
                    consume(kb, vb, rbase + RPI, std::false_type{});
                }
                rbase += 2 * RPI;
            }
        } else {
            // one register buffer: the other waves of the compute unit cover the load latency
            for (int it = 0; it < nfull; ++it) {
                consume(ka, va, rbase, std::false_type{});
                rbase += RPI;
                if (it + 1 < nfull) issue(ka, va, rbase);
            }
        }
        rbase = r0 + nfull * RPI;
        if (rbase < r1) {
            // partial batch: rows past the end are read from the last valid row and masked
            const int krow = min(rbase + wave * 16 + slot, r1 - 1);
#pragma unroll
            for (int j = 0; j < NKJ; ++j) ka[j] = load16_stream(kc + (size_t)krow * D + grp * VEC + j * 32);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int vrow = min(rbase + wave * 16 + 4 * grp + e, r1 - 1);
#pragma unroll
                for (int cg = 0; cg < CG; ++cg) va[cg * 4 + e] = load16_stream(vc + (size_t)vrow * D + vslot * VEC + cg * 128);
            }
            // a wave whose rows are all past the end must not touch its state (its scores are all -inf)
            if (rbase + wave * 16 < r1) consume(ka, va, rbase, std::true_type{});
        }
    }

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
    finish_unit<T, D, GT, NW, NTHR>(a, u, st_ml, st_acc, snew, sv);
}

template <int D, int GT, int NW, bool DOUBLE_BUFFER, bool BALANCED>
__global__ __launch_bounds__(NW * kWave)
void decode_attn_gqa_mfma_kernel(const AttnArgs a, const RopeFreqs fr)
{
    extern __shared__ float lds[];
    for_each_unit<GT, BALANCED>(a, [&](const Unit& u) { gqa_mfma_unit<D, GT, NW, DOUBLE_BUFFER>(a, fr, u, lds); });
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
// leaves per SIMD.  One register buffer (two would leave one wave per SIMD).
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

    auto issue = [&](Vec16<T> (&kv)[NKJ], Vec16<T> (&vv)[CG * 4], int rbase) {
#pragma unroll
        for (int j = 0; j < NKJ; ++j) kv[j] = load16_stream(kp + (size_t)rbase * D + j * 16);
#pragma unroll
        for (int cg = 0; cg < CG; ++cg)
#pragma unroll
            for (int e = 0; e < 4; ++e) vv[cg * 4 + e] = load16_stream(vp + (size_t)(rbase + e) * D + cg * 64);
    };
    const int nfull = r1 > r0 ? (r1 - r0) / RPI : 0;
    Vec16<T> ka[NKJ], va[CG * 4];
    if (nfull > 0) issue(ka, va, r0);

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

    auto consume = [&](const Vec16<T> (&kv)[NKJ], const Vec16<T> (&vv)[CG * 4], int rbase, auto masked_tag) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        f32x4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < NKJ; ++j)
#pragma unroll
            for (int e = 0; e < VEC; ++e) sc = __builtin_amdgcn_mfma_f32_16x16x4f32(kv[j].raw[e], qb[j][e], sc, 0, 0, 0);
        float s[4];
        float bm = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            s[r] = sc[r];                       // score of row 4*grp + r of the batch, head lane % GT
            if constexpr (MASKED) s[r] = (rbase + wave * 16 + 4 * grp + r < r1) ? s[r] : -INFINITY;
            bm = fmaxf(bm, s[r]);
        }
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

    if (r1 > r0) {
        int rbase = r0;
        // one register buffer: the other waves of the compute unit cover the load latency
        for (int it = 0; it < nfull; ++it) {
            consume(ka, va, rbase, std::false_type{});
            rbase += RPI;
            if (it + 1 < nfull) issue(ka, va, rbase);
        }
        rbase = r0 + nfull * RPI;
        if (rbase < r1) {
            // partial batch: rows past the end are read from the last valid row and masked
            const int krow = min(rbase + wave * 16 + slot, r1 - 1);
#pragma unroll
            for (int j = 0; j < NKJ; ++j) ka[j] = load16_stream(kc + (size_t)krow * D + grp * VEC + j * 16);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int vrow = min(rbase + wave * 16 + 4 * grp + e, r1 - 1);
#pragma unroll
                for (int cg = 0; cg < CG; ++cg) va[cg * 4 + e] = load16_stream(vc + (size_t)vrow * D + slot * VEC + cg * 64);
            }
            if (rbase + wave * 16 < r1) consume(ka, va, rbase, std::true_type{});
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
    finish_unit<T, D, GT, NW, NTHR>(a, u, st_ml, st_acc, snew, sv);
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
    long long total, before;
    count_items(a, b, total, before);
    const int ngt = (a.G + a.gt - 1) / a.gt;
    const int nunits = a.Hkv * ngt;
    const int gi = h % a.G;
    const int uib = (h / a.G) * ngt + gi / a.gt;
    const int g = gi % a.gt;
    const long long W = total * nunits;
    const long long first = before * nunits + (long long)uib * items;
    const int N = balanced_workgroups(a, W);
    const int i0 = item_owner(first, W, N), i1 = item_owner(first + items - 1, W, N);
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

// shapes that run on the matrix cores: fp16 caches with two or more query heads per kv head at those head
// sizes; fp32 caches at D = 64 or 128 with more than four (up to four the vector ALU keeps up with the stream)
bool on_matrix_cores(bool fp16, int D, int G)
{
    if (tune_get("attn_gqa_valu") == 1) return false;
    return fp16 ? (G > 1 && mfma_head_size(D)) : (G > 4 && (D == 128 || D == 64));
}

// query heads one workgroup serves (they share every K/V row it reads)
int heads_per_tile(bool fp16, int D, int G)
{
    if (G == 1) return 1;       // one head: memory-bound on either kernel (measured equal), keep the lighter one
    // two or more query heads per kv head, fp16: both products on the matrix cores, where up to 16
    // heads cost the same as 4 (8 at D = 256: the per-wave states of 16 heads would not fit 64 KiB of LDS)
    if (on_matrix_cores(fp16, D, G)) {
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
    const int gt = heads_per_tile(kHalf, D, a.G);
    if constexpr (!kHalf && (D == 128 || D == 64)) {
        if (on_matrix_cores(false, D, a.G)) return gt == 8 ? launch_gqa_mfma_f32<D, 8>(a, fr, st) : launch_gqa_mfma_f32<D, 16>(a, fr, st);
    }
    if constexpr (kHalf && mfma_head_size(D)) {
        if (on_matrix_cores(true, D, a.G)) {
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
int item_rows_for(bool fp16, int D, int G)
{
    if (on_matrix_cores(fp16, D, G)) return 64;
    const int lpr = D * (fp16 ? 2 : 4) / 16;
    const int rpi = 1024 / lpr;               // 4 waves x (64 / lpr) rows x 4 per row group
    return rpi < 64 ? 64 : rpi;
}

// When the balanced schedule is the default (tuning knob attn_balanced = 1 / 0 forces it on / off): per-sequence
// lengths on the matrix-core kernel with no more units than workgroups.  Measured on MI355X against the grid
// schedule (us per step, lengths uniform in [S/8, S]): 32 q / 8 kv heads, batch 32, S 8192: 117 -> 102; 64 q / 8 kv,
// batch 16: 81 -> 57; batch 8, S 16384: 97 -> 61; D = 256, batch 16, S 4096: 90 -> 74.  With equal lengths the grid
// schedule needs no merge launch and is as fast or faster; with more units than workgroups (batch 128) and on the
// vector-ALU kernel (which keeps four workgroups per compute unit resident) the hardware dispatcher balances the
// grid schedule's chunks as well as the fixed shares do.  Nor for a small step (fewer than kBalancedMinItems items
// if every length were the longest): the walk's set-up and its serial unit changes are then most of the time and
// the grid schedule with the fused finish is faster (8 sequences of 256..2048 rows: 24.9 against 17.6 us; 4 of
// 512..4096: 25.2 / 19.6; even at 3500..4100 items; the balanced schedule is ahead from ~7000: 16 sequences of
// 1024..8192 rows 56.7 / 67.6).
bool balanced_by_default(bool ragged, bool mfma, long units, long long max_items)
{
    return ragged && mfma && units <= kBalancedWorkgroups && max_items >= kBalancedMinItems;
}

int max_splits(int max_t)
{
    int n = (max_t + kMinChunk - 1) / kMinChunk;
    return n < 1 ? 1 : (n > kMaxSplits ? kMaxSplits : n);
}

}  // namespace
}  // namespace onellm

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
    const bool tiled = row_bytes >= 16 && row_bytes <= 1024 && (!(row_bytes & (row_bytes - 1)) || padded)
                       && aligned16(k_cache) && aligned16(v_cache);
    const int lpr = row_bytes / 16;

    AttnArgs a{};
    a.qkv = qkv; a.bias = qkv_bias; a.k_cache = k_cache; a.v_cache = v_cache; a.out = out;
    a.t_dev = t_dev; a.t_host = t_host;
    a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.G = Hq / Hkv; a.S = S;
    a.rotary_dim = rotary_dim; a.pos_offset = rope_pos_offset; a.flags = flags;
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
    const int gt = padded ? (G == 1 ? 1 : 4) : heads_per_tile(dtype == ONELLM_FP16, D, G);
    const int ngt = (G + gt - 1) / gt;
    const long base_wgs = (long)B * Hkv * ngt;
    const int user_target = tune_get("attn_target_wgs");
    // (the matrix-core kernel at D = 64 has half the bytes in flight per workgroup: two per compute unit)
    const bool mfma64 = dtype == ONELLM_FP16 && D == 64 && G > 1 && tune_get("attn_gqa_valu") != 1;
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
    const int forced = tune_get("attn_nsplit");
    if (forced > 0) nsplit = forced > max_splits(max_t) ? max_splits(max_t) : forced;
    int chunk = (max_t + nsplit - 1) / nsplit;
    chunk = (chunk + kMinChunk - 1) / kMinChunk * kMinChunk;
    nsplit = (max_t + chunk - 1) / chunk;
    a.chunk = chunk;
    a.nsplit = nsplit;
    a.gt = gt;

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
    const int item_rows = item_rows_for(dtype == ONELLM_FP16, D, G);
    const long long items = (max_t - 1 + item_rows - 1) / item_rows;
    const long long wmax = (long long)B * nunits * (items < 1 ? 1 : items);
    if (forced <= 0 && !padded && (bal == 1 || (bal != 0 && balanced_by_default(t_dev != nullptr, on_matrix_cores(dtype == ONELLM_FP16, D, G), (long)B * nunits, wmax)))) {
        a.item_rows = item_rows;
        const int user_wgs = tune_get("attn_balanced_wgs");
        long long nwg = user_wgs > 0 ? user_wgs : kBalancedWorkgroups;
        if (nwg > kBalancedWorkgroups * 2) nwg = kBalancedWorkgroups * 2;
        // no workgroup for fewer than four items; between one and two workgroups per compute unit some units would
        // get two shares and the rest one, so one larger share each (6 sequences of 1024..4096 rows: 28.9 -> 25.3 us)
        if (nwg > (wmax + 3) / 4) nwg = (wmax + 3) / 4;
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
