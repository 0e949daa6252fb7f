// Beam-search top-K over fp32 logits for gfx950.
//
// Order of candidates (a total order, so the result does not depend on how the reduction tree is
// shaped): larger value first; equal values: smaller global flat index (row*V + token) first.
// A candidate is packed into one 64-bit key whose unsigned order IS that order:
//   high word = the float's bits made monotone (negative: all bits flipped, else sign bit set;
//               -0 is folded onto +0 first so the two zeros tie, as they do for floats),
//   low word  = 0xFFFFFFFF - index  (smaller index -> larger key);
// key 0 is the empty slot and loses against everything.  Values are read back from the logits by
// index when results are stored, so the stored bits are the input's bits.
//
// Stage 1: each (row, block) pair scans the tokens it owns.  A wave takes its values in batches (one
// to sixteen per lane, all requested from memory at once) and keeps one sorted K-slot list for the whole wave in
// registers every lane agrees on.  Of a batch it first takes a floor no member of the wave's top K can be
// below - the lanes are cut into 2K groups, each group's largest value is found with lane exchanges, and the
// K-th largest of those is the floor: K values at least that large exist - so one float compare per value
// rejects all but a handful; the survivors rank themselves against each other (each one's key is read out
// of its lane and compared in all lanes), the K best are merged into the wave's list, and that raises the
// floor for what follows.  (Once a batch leaves survivors in more than sixteen lanes, or four in one lane -
// ties, sorted input - the wave goes over to per-lane lists and a bitonic merge across the wave at the
// end, which cost the same whatever the data; lists of eight always do.)  The four waves of a workgroup combine their lists through LDS with a bitonic
// top-K merge (max of a[i] and b[K-1-i], then a bitonic sort).  Stage 2: the beam*nblk*K survivors of a
// batch entry go through the same scan, in the stage-1 workgroup of that entry that finishes last (one
// launch), or in a second launch with one workgroup per batch entry.  Traffic: the logits are read once
// (rows*V*4 bytes).
//
// The one-launch form counts the workgroups of a batch entry that have stored their survivors in an arrival
// counter.  The caller's workspace has no room for counters and is not zeroed, so they live in a file-scope
// device array (zero when the module is loaded; the workgroup that merges sets its counter back to zero, so
// every launch leaves them zero).  Launches that may overlap need counters of their own: a launch uses the
// set its (device, workspace pointer) owns (counter_sets.hpp: owned from the first launch until the caller
// gives it back with onellm_release_workspace, never reassigned in between) - two launches that share a
// workspace may not overlap anyway, they would overwrite each other's survivors.  A workspace that finds
// every set owned, or a batch beyond the set's size, takes the two-launch form, and
// onellm_beam_topk_last_path says which of the two it was.
#include <limits.h>
#include <math.h>
#include <mutex>
#include "common.hpp"
#include "counter_sets.hpp"

namespace onellm {
int tune_get(const char* key);
namespace {

typedef unsigned long long Key;

constexpr int kArrivalSets = 64;        // workspaces that can run the one-launch form (per process)
constexpr int kArrivalEntries = 1024;   // batch entries per launch of the one-launch form
__device__ unsigned g_arrivals[kArrivalSets * kArrivalEntries];

thread_local int g_last_launches = 0;
thread_local int g_last_path = 0;

CounterSets g_arrival_sets("onellm_beam_topk", kArrivalSets);

__device__ __forceinline__ Key make_key(float v, int id)
{
    v += 0.0f;                                              // -0 -> +0
    unsigned u = __float_as_uint(v);
    u ^= (u & 0x80000000u) ? 0xFFFFFFFFu : 0x80000000u;
    return ((Key)u << 32) | (Key)(0xFFFFFFFFu - (unsigned)id);
}
__device__ __forceinline__ int key_id(Key k) { return k == 0 ? -1 : (int)(0xFFFFFFFFu - (unsigned)(k & 0xFFFFFFFFu)); }

// The value a key was made from.  The key's high word is an invertible map of the float's bits, except that -0 was
// folded onto +0: a zero is therefore read back from the logits (the stored bits must be the input's bits); every
// other value is decoded from the key, which spares the kernels a dependent memory round trip before their stores.
__device__ __forceinline__ float key_value(Key k, int id, const float* __restrict__ logits)
{
    if (id < 0) return -INFINITY;
    unsigned u = (unsigned)(k >> 32);
    u ^= (u & 0x80000000u) ? 0x80000000u : 0xFFFFFFFFu;
    const float v = __uint_as_float(u);
    return v == 0.0f ? logits[id] : v;
}

__device__ __forceinline__ void cmp_exchange(Key& hi, Key& lo)
{
    const bool sw = lo > hi;
    const Key a = sw ? lo : hi, b = sw ? hi : lo;
    hi = a;
    lo = b;
}

// KP = list length, a power of two (K is rounded up to it; the surplus slots are real slots, the
// caller just stores fewer)
template <int KP>
struct TopList {
    Key k[KP];

    __device__ __forceinline__ void clear()
    {
#pragma unroll
        for (int i = 0; i < KP; ++i) k[i] = 0;
    }
    // sorted best-first; one bubble pass from the tail (fully unrolled, no dynamic indexing)
    __device__ __forceinline__ void insert(Key c)
    {
        if (c <= k[KP - 1]) return;
        k[KP - 1] = c;
#pragma unroll
        for (int s = KP - 2; s >= 0; --s) cmp_exchange(k[s], k[s + 1]);
    }
    // keep the KP best of this list and another sorted list: c[i] = max(a[i], b[KP-1-i]) holds
    // them as a bitonic sequence, which log2(KP) compare-exchange stages sort
    __device__ __forceinline__ void merge(const TopList<KP>& o)
    {
#pragma unroll
        for (int i = 0; i < KP; ++i) {
            const Key b = o.k[KP - 1 - i];
            k[i] = b > k[i] ? b : k[i];
        }
#pragma unroll
        for (int stride = KP / 2; stride >= 1; stride /= 2)
#pragma unroll
            for (int i = 0; i < KP; ++i)
                if ((i & stride) == 0) cmp_exchange(k[i], k[i + stride]);
    }
};

__device__ __forceinline__ Key shfl_xor_key(Key v, int mask)
{
    const unsigned lo = __shfl_xor((unsigned)(v & 0xFFFFFFFFu), mask, kWave);
    const unsigned hi = __shfl_xor((unsigned)(v >> 32), mask, kWave);
    return ((Key)hi << 32) | lo;
}
template <int CTRL>
__device__ __forceinline__ Key dpp_key(Key v)
{
    const unsigned lo = (unsigned)dpp_i32<CTRL>((int)(unsigned)(v & 0xFFFFFFFFu));
    const unsigned hi = (unsigned)dpp_i32<CTRL>((int)(unsigned)(v >> 32));
    return ((Key)hi << 32) | lo;
}

template <int KP, int CTRL>
__device__ __forceinline__ void merge_dpp(TopList<KP>& t)
{
    TopList<KP> o;
#pragma unroll
    for (int i = 0; i < KP; ++i) o.k[i] = dpp_key<CTRL>(t.k[i]);
    t.merge(o);
}
template <int KP>
__device__ __forceinline__ void merge_xor(TopList<KP>& t, int mask)
{
    TopList<KP> o;
#pragma unroll
    for (int i = 0; i < KP; ++i) o.k[i] = shfl_xor_key(t.k[i], mask);
    t.merge(o);
}

// after this every lane of the wave holds the wave's KP best
template <int KP>
__device__ __forceinline__ void wave_merge(TopList<KP>& t)
{
    merge_dpp<KP, kDppQuadXor1>(t);
    merge_dpp<KP, kDppQuadXor2>(t);
    merge_dpp<KP, kDppRowHalfMirror>(t);
    merge_dpp<KP, kDppRowMirror>(t);
    merge_xor<KP>(t, 16);
    merge_xor<KP>(t, 32);
}

__device__ __forceinline__ float key_float(Key k)
{
    unsigned u = (unsigned)(k >> 32);
    u ^= (u & 0x80000000u) ? 0x80000000u : 0xFFFFFFFFu;
    return __uint_as_float(u);
}

__device__ __forceinline__ Key readlane_key(Key v, int lane)
{
    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(v & 0xFFFFFFFFu), lane);
    const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(v >> 32), lane);
    return ((Key)hi << 32) | lo;
}

__device__ __forceinline__ float readlane_f32(float v, int lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// A value that at least KP of the wave's 64 values m reach: the lanes are cut into 2*KP groups, each group's
// largest value is found with lane exchanges (NaN never wins against a number; a group of nothing but NaN counts
// as -inf), and the KP-th largest of the group maxima is returned: every group counts the maxima above its own,
// and a group that counts the most without exceeding KP-1 holds it.  The same in every lane.
template <int KP>
__device__ __forceinline__ float kth_group_maximum(float m)
{
    constexpr int NG = 2 * KP, G = 64 / NG;
    m = fmaxf(m, dpp_f32<kDppQuadXor1>(m));
    m = fmaxf(m, dpp_f32<kDppQuadXor2>(m));
    if (G >= 8) m = fmaxf(m, dpp_f32<kDppRowHalfMirror>(m));
    if (G >= 16) m = fmaxf(m, dpp_f32<kDppRowMirror>(m));
    if (G >= 32) m = fmaxf(m, __shfl_xor(m, 16, kWave));
    m = (m == m) ? m : -INFINITY;
    int above = 0;
#pragma unroll
    for (int g = 0; g < NG; ++g) above += readlane_f32(m, g * G) > m ? 1 : 0;
#pragma unroll
    for (int i = KP - 1; i > 0; --i) {
        const unsigned long long who = __builtin_amdgcn_ballot_w64(above == i);
        if (who) return readlane_f32(m, __builtin_ctzll(who));
    }
    return readlane_f32(m, __builtin_ctzll(__builtin_amdgcn_ballot_w64(above == 0)));
}

// One wave's running top KP.  `top` holds the same values in every lane (it is only ever updated from values read
// out of one lane, under control flow the whole wave takes); `lanes` is the per-lane list the wave goes over to, for
// good, once a batch leaves too many survivors to rank (lists of eight use nothing else).
template <int KP>
struct WaveTop {
    static constexpr int kRankAtMost = 16;
    static constexpr bool kPerLaneOnly = KP > 4;   // lists of eight: ranking and merging them costs more than the per-lane road
    TopList<KP> top, lanes;
    float floor;
    bool used_lanes;

    __device__ __forceinline__ void clear()
    {
        top.clear();
        lanes.clear();
        floor = -INFINITY;
        used_lanes = kPerLaneOnly;
    }
    // true: the wave has gone over to the per-lane lists for good; the caller inserts its values into `lanes` itself
    __device__ __forceinline__ bool per_lane_road() const { return kPerLaneOnly || used_lanes; }
    // before a batch: lane_max = the largest valid value this lane holds in the batch (-inf if none)
    __device__ __forceinline__ void raise_floor(float lane_max)
    {
        if (kPerLaneOnly || used_lanes) return;
        floor = fmaxf(floor, kth_group_maximum<KP>(lane_max));
    }
    // One candidate key per lane (0: none), in at most kRankAtMost lanes.  The lanes whose key beats the wave's K-th
    // are the contenders: every contender counts the contenders' keys above its own (they are read out of their
    // lanes one by one), the ones that count 0 .. KP-1 form a sorted list, and that list is merged into `top`.
    __device__ __forceinline__ void offer(Key k)
    {
        const bool contends = k > top.k[KP - 1];
        const unsigned long long m = __builtin_amdgcn_ballot_w64(contends);
        if (m == 0) return;
        if ((m & (m - 1)) == 0) {
            top.insert(readlane_key(k, __builtin_ctzll(m)));
        } else {
            int above = 0;
            for (unsigned long long mm = m; mm; mm &= mm - 1) above += readlane_key(k, __builtin_ctzll(mm)) > k ? 1 : 0;
            TopList<KP> best;
#pragma unroll
            for (int i = 0; i < KP; ++i) {
                const unsigned long long who = __builtin_amdgcn_ballot_w64(contends && above == i);
                best.k[i] = who ? readlane_key(k, __builtin_ctzll(who)) : (Key)0;
            }
            if (top.k[0] == 0) top = best;
            else top.merge(best);
        }
        if (top.k[KP - 1] != 0) floor = fmaxf(floor, key_float(top.k[KP - 1]));
    }
    // A batch of NV values per lane; bit j of `valid` says whether x[j] exists, and its flat index is
    // id0 + (j / E) * id_step + j % E.  One compare per value marks what the floor does not reject (`!(x < floor)`
    // keeps NaN, which the key order places); then each round offers every lane's next marked value, until no lane
    // has one left - one or two rounds on ordinary data, NV on data that is all ties.
    template <int NV, int E>
    __device__ __forceinline__ void take(const float (&x)[NV], unsigned valid, int id0, int id_step)
    {
        take_with<NV>(x, valid, [&](int j) { return id0 + (j / E) * id_step + j % E; });
    }
    // the same with the flat indices in an array (the survivors of an earlier stage carry theirs)
    template <int NV>
    __device__ __forceinline__ void take(const float (&x)[NV], unsigned valid, const int (&id)[NV])
    {
        take_with<NV>(x, valid, [&](int j) {
            int pick[NV];
#pragma unroll
            for (int i = 0; i < NV; ++i) pick[i] = id[i];
#pragma unroll
            for (int bit = 0; (NV >> bit) > 1; ++bit) {
                const bool odd = (j >> bit) & 1;
#pragma unroll
                for (int i = 0; i < (NV >> (bit + 1)); ++i) pick[i] = odd ? pick[2 * i + 1] : pick[2 * i];
            }
            return pick[0];
        });
    }
    template <int NV, class IdOf>
    __device__ __forceinline__ void take_with(const float (&x)[NV], unsigned valid, IdOf id_of)
    {
        if (kPerLaneOnly) {
#pragma unroll
            for (int j = 0; j < NV; ++j)
                if ((valid >> j) & 1) lanes.insert(make_key(x[j], id_of(j)));
            return;
        }
        unsigned marked = valid;
        if (!used_lanes) {
            marked = 0;
#pragma unroll
            for (int j = 0; j < NV; ++j) marked |= !(x[j] < floor) ? (1u << j) : 0u;
            marked &= valid;
            // Ties and sorted input leave many values marked.  The rounds below cost about a hundred instructions
            // each and a lane offers one value per round, so once a batch has a lane with four or more, or more
            // lanes with one than can rank themselves, the wave takes the road whose cost does not depend on the
            // data, for this batch and every later one: each value into the per-lane lists.
            const unsigned long long holders = __builtin_amdgcn_ballot_w64(marked != 0);
            if (holders == 0) return;
            used_lanes = __builtin_popcountll(holders) > kRankAtMost ||
                         __builtin_amdgcn_ballot_w64(__builtin_popcount(marked) >= 4) != 0;
        }
        if (used_lanes) {
#pragma unroll
            for (int j = 0; j < NV; ++j)
                if ((marked >> j) & 1) lanes.insert(make_key(x[j], id_of(j)));
            return;
        }
        while (__builtin_amdgcn_ballot_w64(marked != 0) != 0) {
            const int j = marked ? __builtin_ctz(marked) : 0;
            float pick[NV];      // x[j] for a j that differs from lane to lane: halve the choice once per bit of j
#pragma unroll
            for (int i = 0; i < NV; ++i) pick[i] = x[i];
#pragma unroll
            for (int bit = 0; (NV >> bit) > 1; ++bit) {
                const bool odd = (j >> bit) & 1;
#pragma unroll
                for (int i = 0; i < (NV >> (bit + 1)); ++i) pick[i] = odd ? pick[2 * i + 1] : pick[2 * i];
            }
            const float xv = pick[0];
            const Key k = marked ? make_key(xv, id_of(j)) : (Key)0;
            marked &= marked - 1;
            offer(k);
        }
    }
    // after the last batch: every lane holds the wave's KP best in `top`
    __device__ __forceinline__ void finish()
    {
        if (used_lanes) {
            wave_merge<KP>(lanes);
            top.merge(lanes);
        }
    }
};

// workgroup of NWV waves, `t` the finished list of each wave -> the lanes of wave 0 return the workgroup's KP best
template <int KP, int NWV>
__device__ __forceinline__ void block_merge(TopList<KP>& t, Key* skey)
{
    const int tid = threadIdx.x, wave = tid / kWave;
    if ((tid & (kWave - 1)) == 0) {
#pragma unroll
        for (int i = 0; i < KP; ++i) skey[wave * KP + i] = t.k[i];
    }
    __syncthreads();
    if (wave == 0) {
        for (int w = 1; w < NWV; ++w) {
            TopList<KP> o;
#pragma unroll
            for (int i = 0; i < KP; ++i) o.k[i] = skey[w * KP + i];
            t.merge(o);
        }
    }
}

// One wave merges the n survivors (value, flat index; index -1 = empty slot) of a batch entry, four per lane and
// batch, and its lane 0 stores the K best.  DEVICE_SCOPE: the survivors were stored by other workgroups of this
// launch, so they are read with device-scope loads.
template <int KP, bool DEVICE_SCOPE>
__device__ __forceinline__ void merge_survivors(const float* __restrict__ logits, const float* vals, const int* ids, int n, int K,
                                                float* __restrict__ fvals, int* __restrict__ fids)
{
    constexpr int NV = 4;
    const int lane = threadIdx.x & (kWave - 1);
    WaveTop<KP> w;
    w.clear();
    for (int base = 0; base < n; base += NV * kWave) {
        float x[NV];
        int id[NV];
        unsigned valid = 0;
        float lane_max = -INFINITY;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int i = base + j * kWave + lane;
            x[j] = -INFINITY;
            id[j] = -1;
            if (i < n) {
                if (DEVICE_SCOPE) {
                    id[j] = __hip_atomic_load(&ids[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    x[j] = __hip_atomic_load(&vals[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                } else {
                    id[j] = ids[i];
                    x[j] = vals[i];
                }
            }
            if (id[j] != -1) {
                valid |= 1u << j;
                lane_max = fmaxf(lane_max, x[j]);
            }
        }
        w.raise_floor(lane_max);
        w.template take<NV>(x, valid, id);
    }
    w.finish();
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < KP; ++i) {
            if (i < K) {
                const int id = key_id(w.top.k[i]);
                fvals[i] = key_value(w.top.k[i], id, logits);
                fids[i] = id;
            }
        }
    }
}

// grid = rows * nblk.  Block `lane_blk` of a row owns the 256-token chunks lane_blk, lane_blk + nblk,
// ... (the reference's ownership: token tid + lane_blk*256 + m*nblk*256).  On the vector path a
// thread reads 4 consecutive tokens of a chunk with one 16-byte load and four such loads are issued
// before any candidate is inserted, so a block has its whole slice of the row in flight at once.
//
// FUSED: `set` >= 0 names the arrival counters; the workgroup that finds the other beam*nblk - 1 workgroups of its
// batch entry arrived merges the entry's survivors and stores the final K.  Ordering: thread 0 stores the
// workgroup's survivors, then adds to the counter with release order at device scope; the add of the last
// arriver has acquire order and the barrier after it extends that to the workgroup, whose loads of the
// survivors are device-scope loads (they do not take a line an earlier launch left in this compute unit's cache).
//
// NWV waves per workgroup: four take a row slice's chunks in turns of four, eight in turns of eight (every SIMD then
// has a second chain of dependent instructions to run while the first waits, and each chain has half the values to
// look at; it pays for long rows only, see launch_topk).
template <int KP, bool FUSED, int NWV>
__global__ __launch_bounds__(NWV * kWave)
void topk_stage1_kernel(const float* __restrict__ logits, int V, int nblk, int vec_ok, int K,
                        float* __restrict__ vals, int* __restrict__ ids, int set, int beam,
                        float* __restrict__ fvals, int* __restrict__ fids)
{
    __shared__ Key skey[NWV * KP];
    __shared__ int s_last;
    const int row = blockIdx.x / nblk, lane_blk = blockIdx.x % nblk;
    const float* p = logits + (size_t)row * V;
    const int flat0 = row * V;
    WaveTop<KP> w;
    w.clear();
    if (vec_ok) {
        constexpr int PASSES = NWV == 4 ? 4 : 2;                  // (a 32000-token row is one batch per wave either way)
        const int nchunks = (V + 255) / 256;
        const int sub = threadIdx.x / 64, l4 = (threadIdx.x % 64) * 4;
        for (int c0 = lane_blk + nblk * sub; c0 < nchunks; c0 += nblk * NWV * PASSES) {
            f32x4 v[PASSES];
            int tok[PASSES];
#pragma unroll
            for (int q = 0; q < PASSES; ++q) {
                tok[q] = (c0 + nblk * NWV * q) * 256 + l4;
                v[q] = f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
                if (tok[q] < V) v[q] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p + tok[q]));
            }
            if (w.per_lane_road()) {
#pragma unroll
                for (int q = 0; q < PASSES; ++q) {
                    if (tok[q] < V) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) w.lanes.insert(make_key(v[q][e], flat0 + tok[q] + e));
                    }
                }
                continue;
            }
            float x[4 * PASSES];
            float lane_max = -INFINITY;
            unsigned valid = 0;
#pragma unroll
            for (int q = 0; q < PASSES; ++q) {
#pragma unroll
                for (int e = 0; e < 4; ++e) x[4 * q + e] = v[q][e];
                if (tok[q] < V) {      // V % 4 == 0 here, so tok < V means tok + 3 < V
                    valid |= 0xFu << (4 * q);
                    lane_max = fmaxf(fmaxf(lane_max, fmaxf(v[q][0], v[q][1])), fmaxf(v[q][2], v[q][3]));
                }
            }
            w.raise_floor(lane_max);
            w.template take<4 * PASSES, 4>(x, valid, flat0 + tok[0], nblk * NWV * 256);
        }
    } else {
        // (a thread looks at token `threadIdx.x % 256` of the 256-token chunks lane_blk + nblk * (threadIdx.x / 256 + j * NWV / 4))
        constexpr int PASSES = 8;
        constexpr int STEP = NWV / 4;                               // chunks of the slice the workgroup covers at a time
        const int first = (int)(threadIdx.x % 256) + (lane_blk + nblk * (int)(threadIdx.x / 256)) * 256;
        for (int tok0 = first; tok0 - (int)(threadIdx.x % 256) < V; tok0 += nblk * 256 * STEP * PASSES) {
            float x[PASSES];
            unsigned valid = 0;
#pragma unroll
            for (int q = 0; q < PASSES; ++q) {
                const int tok = tok0 + q * nblk * 256 * STEP;
                x[q] = -INFINITY;
                if (tok < V) {
                    x[q] = p[tok];
                    valid |= 1u << q;
                }
            }
            if (w.per_lane_road()) {
#pragma unroll
                for (int q = 0; q < PASSES; ++q)
                    if ((valid >> q) & 1) w.lanes.insert(make_key(x[q], flat0 + tok0 + q * nblk * 256 * STEP));
                continue;
            }
            float lane_max = -INFINITY;
#pragma unroll
            for (int q = 0; q < PASSES; ++q) lane_max = fmaxf(lane_max, x[q]);
            w.raise_floor(lane_max);
            w.template take<PASSES, 1>(x, valid, flat0 + tok0, nblk * 256 * STEP);
        }
    }
    w.finish();
    TopList<KP>& t = w.top;
    block_merge<KP, NWV>(t, skey);
    if (threadIdx.x == 0) {
#pragma unroll
        for (int i = 0; i < KP; ++i) {
            if (i < K) {
                const int id = key_id(t.k[i]);
                const float v = key_value(t.k[i], id, logits);
                if (FUSED) {
                    __hip_atomic_store(&vals[(size_t)blockIdx.x * K + i], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(&ids[(size_t)blockIdx.x * K + i], id, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                } else {
                    vals[(size_t)blockIdx.x * K + i] = v;
                    ids[(size_t)blockIdx.x * K + i] = id;
                }
            }
        }
    }
    if (!FUSED) return;
    const int b = row / beam, pieces = beam * nblk;
    if (threadIdx.x == 0) {
        unsigned* ctr = &g_arrivals[set * kArrivalEntries + b];
        const unsigned before = __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        const int last = before == (unsigned)(pieces - 1);
        if (last) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = last;
    }
    __syncthreads();
    if (!s_last) return;
    if (threadIdx.x >= kWave) return;
    const int n = pieces * K;
    merge_survivors<KP, true>(logits, vals + (size_t)b * n, ids + (size_t)b * n, n, K, fvals + (size_t)b * K, fids + (size_t)b * K);
}

// grid = B, one wave each; merges the n = beam*nblk*K stage-1 survivors of one batch entry
template <int KP>
__global__ __launch_bounds__(kWave)
void topk_stage2_kernel(const float* __restrict__ logits, const float* __restrict__ vals, const int* __restrict__ ids,
                        int n, int K, float* __restrict__ fvals, int* __restrict__ fids)
{
    const int b = blockIdx.x;
    merge_survivors<KP, false>(logits, vals + (size_t)b * n, ids + (size_t)b * n, n, K, fvals + (size_t)b * K, fids + (size_t)b * K);
}

template <int KP>
int launch_topk(const float* logits, int B, int beam, int V, int K, int nblk, float* ws, hipStream_t st)
{
    const size_t n1 = (size_t)B * beam * nblk * K;
    float* vals = ws;
    int* ids = reinterpret_cast<int*>(vals + n1);
    float* fvals = reinterpret_cast<float*>(ids + n1);
    int* fids = reinterpret_cast<int*>(fvals + (size_t)B * K);
    const int vec_ok = (V % 4 == 0) && aligned16(logits);
    // One launch costs the host a launch less and the device about 1.5 us more (the store - count - load chain
    // of the last workgroup is longer than a second launch's start-up): it is the form of a stream that runs
    // launch by launch, where the host is the limit; a stream under capture, whose launches will be replayed
    // without the host, gets the two-launch form.
    int two = tune_get("topk_two_launches");
    if (two < 0) {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &cs) != hipSuccess) {
            (void)hipGetLastError();
            cs = hipStreamCaptureStatusNone;
        }
        two = cs != hipStreamCaptureStatusNone;
    }
    // Eight waves per workgroup (512 threads: two dependent chains per SIMD, half the values per wave) pay only where a
    // wave's per-value work is heavy - the per-lane lists of K > 4 - and its row slice long: graph replay, batch 8 x beam
    // 4, V = 128256: K = 8 26.1 -> 24.5 us (K = 5: 25.0 -> 23.4; V = 65536: 19.6 -> 20.3; batch 16: 29.5 -> 30.0), but K = 4
    // 14.06 -> 14.01, V = 65536 9.68 -> 10.07 (batch 16: 10.66 -> 11.77), V = 32000 7.73 -> 8.00 - a wave's fixed work (floor, marks, ranking) does not shrink with its share of the row, and
    // the workgroup merges eight lists instead of four.  Tuning key topk_waves = 4 / 8 forces either.
    const int want_waves = tune_get("topk_waves");
    const bool eight = want_waves == 8 || (want_waves != 4 && KP > 4 && (long)B * beam * nblk <= 256 && V >= nblk * 8 * 256 * 6);
    int set = -1;
    g_last_path = ONELLM_TOPK_PATH_TWO_LAUNCHES;
    if (B <= kArrivalEntries && !two) {
        int dev = 0;
        const hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return (int)e;
        set = g_arrival_sets.acquire(dev, ws);
        if (set < 0) g_last_path = ONELLM_TOPK_PATH_NO_COUNTER_SET;
    }
    if (set >= 0) {
        g_last_path = ONELLM_TOPK_PATH_ONE_LAUNCH;
        if (eight) hipLaunchKernelGGL((topk_stage1_kernel<KP, true, 8>), dim3(B * beam * nblk), dim3(512), 0, st, logits, V, nblk, vec_ok, K,
                                      vals, ids, set, beam, fvals, fids);
        else hipLaunchKernelGGL((topk_stage1_kernel<KP, true, 4>), dim3(B * beam * nblk), dim3(256), 0, st, logits, V, nblk, vec_ok, K,
                                vals, ids, set, beam, fvals, fids);
        g_last_launches = 1;
        return launch_status();
    }
    if (eight) hipLaunchKernelGGL((topk_stage1_kernel<KP, false, 8>), dim3(B * beam * nblk), dim3(512), 0, st, logits, V, nblk, vec_ok, K,
                                  vals, ids, -1, beam, fvals, fids);
    else hipLaunchKernelGGL((topk_stage1_kernel<KP, false, 4>), dim3(B * beam * nblk), dim3(256), 0, st, logits, V, nblk, vec_ok, K,
                            vals, ids, -1, beam, fvals, fids);
    int rc = launch_status();
    if (rc) return rc;
    hipLaunchKernelGGL((topk_stage2_kernel<KP>), dim3(B), dim3(kWave), 0, st, logits, vals, ids, beam * nblk * K, K, fvals, fids);
    g_last_launches = 2;
    return launch_status();
}

}  // namespace
}  // namespace onellm

extern "C" size_t onellm_beam_topk_workspace_bytes(int B, int beam, int K)
{
    if (B <= 0 || beam <= 0 || K <= 0) return 0;
    const size_t nblk = ONELLM_TOPK_BLOCKS_PER_ROW;
    return sizeof(float) * (2 * (size_t)B * beam * nblk * K + 2 * (size_t)B * K);
}

extern "C" int onellm_beam_topk(const float* logits, int B, int beam, int V, int K, float* workspace,
                                onellm_stream_t stream)
{
    using namespace onellm;
    g_last_launches = 0;
    g_last_path = 0;
    if (!logits || !workspace || B <= 0 || beam <= 0 || V <= 0) return ONELLM_EINVAL;
    if (K < 1 || K > 8) return ONELLM_EUNSUPPORTED;
    if ((long)B * beam * V > (long)INT_MAX - 1) return ONELLM_EUNSUPPORTED;   // ids are int32 flat indices
    const int nblk = ONELLM_TOPK_BLOCKS_PER_ROW;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (K == 1) return launch_topk<1>(logits, B, beam, V, K, nblk, workspace, st);
    if (K == 2) return launch_topk<2>(logits, B, beam, V, K, nblk, workspace, st);
    if (K <= 4) return launch_topk<4>(logits, B, beam, V, K, nblk, workspace, st);
    return launch_topk<8>(logits, B, beam, V, K, nblk, workspace, st);
}

extern "C" int onellm_beam_topk_last_launches(void) { return onellm::g_last_launches; }

extern "C" int onellm_beam_topk_last_path(void) { return onellm::g_last_path; }
