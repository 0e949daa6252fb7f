// Decode attention: launch arguments, what a workgroup works on, the grid and the balanced workgroup schedules.
// (part of decode_attn.hip, which is the only file that includes it: everything here sits in its anonymous namespace)
#pragma once
#include "common.hpp"

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
    int unit_cost;        // what starting on another unit costs a workgroup, in items (set-up, finish, an emptied load queue)
    int turns;            // co-resident workgroups take turns at wave priority (take_turns below); 0: they do not
    int gt;               // query heads per tile
    int on_mfma;          // the step runs on the matrix-core kernels (host-side choice)
    // fused finish (counters != NULL): one arrival counter per unit, zero between calls; the piece
    // that arrives last merges the unit's partial states itself and no merge kernel is launched
    int* counters;
    int early_look;       // 1: a piece that finds all the others arrived merges the unit from its registers, unpublished
    int ordered;          // 1: the counter add is a release and the merging piece takes an acquire fence (agent scope)
#ifdef ONELLM_ATTN_STAMPS
    long long* stamps;    // timeline build only: four words per workgroup (entry, end, XCC id, HW_ID)
#endif
};

// Timeline build (-DONELLM_ATTN_STAMPS, a separate test-side library): thread 0 of every workgroup records the
// chip-wide 100 MHz clock at entry and after its last store was acknowledged, the id of the XCD and of the compute
// unit (shader engine, array, unit) it runs on.
#ifdef ONELLM_ATTN_STAMPS
__device__ __forceinline__ void stamp_entry(const AttnArgs& a)
{
    if (a.stamps && threadIdx.x == 0) {
        const long long wg = ((long long)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
        a.stamps[wg * 4 + 0] = wall_clock64();
        a.stamps[wg * 4 + 2] = __builtin_amdgcn_s_getreg(20 | (0 << 6) | ((4 - 1) << 11));   // HW_REG_XCC_ID, bits 3:0
        a.stamps[wg * 4 + 3] = __builtin_amdgcn_s_getreg(4 | (0 << 6) | ((32 - 1) << 11));   // HW_REG_HW_ID: cu 11:8, sh 12, se 15:13
    }
}
__device__ __forceinline__ void stamp_end(const AttnArgs& a)
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (a.stamps && threadIdx.x == 0) {
        const long long wg = ((long long)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
        a.stamps[wg * 4 + 1] = wall_clock64();
    }
}
// phase stamps of the matrix-core kernels: behind the four words per workgroup, kStampEvents words per workgroup -
// four per unit piece in the order it meets them (piece begun, set-up done, last row consumed, piece finished)
constexpr int kStampEvents = 16;
__device__ __forceinline__ void stamp_event(const AttnArgs& a, int& next)
{
    if (a.stamps && threadIdx.x == 0 && next < kStampEvents) {
        const long long total = (long long)gridDim.x * gridDim.y * gridDim.z;
        const long long wg = ((long long)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
        a.stamps[total * 4 + wg * kStampEvents + next] = wall_clock64();
    }
    ++next;
}
#else
__device__ __forceinline__ void stamp_entry(const AttnArgs&) {}
__device__ __forceinline__ void stamp_end(const AttnArgs&) {}
__device__ __forceinline__ void stamp_event(const AttnArgs&, int&) {}
#endif

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
//
// Changing units is not free for a workgroup (the finish of one, the set-up of the next and a load queue that
// runs empty in between cost about as much as three items), so the shares are equal in cost rather than in
// rows: every unit is preceded by unit_cost items that stand for that overhead and hold no rows.  A workgroup
// whose share only touches those has nothing to do for the unit; the one whose share crosses into the rows
// pays the overhead and gets correspondingly fewer rows.
__device__ __forceinline__ int seq_items(const AttnArgs& a, int t)
{
    if (t < 1 || t > a.S) return 0;               // out-of-contract length: no work, nothing touched
    const int n = (t - 1 + a.item_rows - 1) / a.item_rows;
    return (n < 1 ? 1 : n) + a.unit_cost;
}

// The schedule is the same in every lane; saying so keeps it in scalar registers (the kernels that
// walk it are short of vector registers).
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ unsigned uniform(unsigned v) { return (unsigned)__builtin_amdgcn_readfirstlane((int)v); }

// Thread index as a value the compiler takes as new each time it is asked for: everything a unit
// derives from it (addresses, masks, lane roles) is then recomputed per unit instead of being
// hoisted out of the loop over units and held in registers across the streaming loop.
__device__ __forceinline__ int lane_id_per_unit()
{
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    return tid;
}

// Item numbers are 32-bit: the host takes the balanced schedule only for steps whose item count, times the
// workgroups that share it, stays below 2^31 (kBalancedMaxItemsTimesWorkgroups), so every product below fits.
// The walk sits on every workgroup's path before its first load (and again at each change of unit), which is why it
// is written for latency: one load of the lengths, sums across the wave on the DPP row operations (no trips
// through the LDS crossbar), 32-bit divisions.
constexpr unsigned kBalancedMaxItemsTimesWorkgroups = 0x7FFFFFFFu;

// inclusive prefix sum over the wave's 64 lanes; lane 63 ends up with the total
__device__ __forceinline__ unsigned wave_inclusive_scan(unsigned v)
{
    constexpr int kRowShr1 = 0x111, kRowShr2 = 0x112, kRowShr4 = 0x114, kRowShr8 = 0x118, kRowBcast15 = 0x142, kRowBcast31 = 0x143;
    int x = (int)v;
    x += __builtin_amdgcn_update_dpp(0, x, kRowShr1, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0, x, kRowShr2, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0, x, kRowShr4, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0, x, kRowShr8, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0, x, kRowBcast15, 0xA, 0xF, false);     // rows 1 and 3 take the total of the row before
    x += __builtin_amdgcn_update_dpp(0, x, kRowBcast31, 0xC, 0xF, false);     // rows 2 and 3 take the total of the first half
    return (unsigned)x;
}
__device__ __forceinline__ unsigned lane_value(unsigned v, int lane) { return (unsigned)__builtin_amdgcn_readlane((int)v, lane); }

// items of all sequences, and of the sequences before `before` (every lane gets both)
__device__ __forceinline__ void count_items(const AttnArgs& a, int before, unsigned& total, unsigned& prefix)
{
    if (!a.t_dev) {
        const unsigned it = (unsigned)seq_items(a, a.t_host);
        total = (unsigned)a.B * it;
        prefix = (unsigned)before * it;
        return;
    }
    const int lane = threadIdx.x & (kWave - 1);
    unsigned tot = 0, pre = 0;
    for (int c = 0; c < a.B; c += kWave) {
        const int bb = c + lane;
        const unsigned it = bb < a.B ? (unsigned)seq_items(a, a.t_dev[bb]) : 0u;
        const unsigned inc = wave_inclusive_scan(it);
        tot += lane_value(inc, kWave - 1);
        // sequences of this block before `before`: the inclusive sum of lane before - c - 1
        const int last = before - c - 1;
        if (last >= kWave - 1) pre += lane_value(inc, kWave - 1);
        else if (last >= 0) pre += lane_value(inc, uniform(last));
    }
    total = tot;
    prefix = pre;
}

// workgroup that owns item x when W items are dealt to N workgroups as [i*W/N, (i+1)*W/N)
__device__ __forceinline__ int item_owner(unsigned x, unsigned W, int N)
{
    return (int)(((x + 1u) * (unsigned)N - 1u) / W);
}

// Workgroups that take part: never more than there are items, so that no share is empty and the
// workgroups of a unit are consecutive - and, as the host sizes the grid for the longest length it
// was given while the real lengths may be much shorter: no workgroup for fewer than four items, and
// not between one and two workgroups per compute unit (some units would get two shares, the rest one:
// better one larger share each).  The launch has one workgroup per compute unit or two (or what a sweep
// asked for, taken as it is).
__device__ __forceinline__ int balanced_workgroups(const AttnArgs& a, unsigned W)
{
    unsigned n = (W + 3u) / 4u;
    if (n > (unsigned)a.bal_nwg) n = (unsigned)a.bal_nwg;
    if (a.bal_nwg == kBalancedWorkgroups && n > kBalancedWorkgroups / 2 && n < kBalancedWorkgroups) n = kBalancedWorkgroups / 2;
    return (int)n;
}

struct Walk {
    unsigned W;            // items of the whole step
    int N;                 // workgroups that share them
    unsigned cur, hi;      // next item of this workgroup, end of its share
    unsigned base;         // first item of sequence b
    int b, items;          // current sequence and its items per unit
    int nunits;            // units per sequence
};

// Positions the walk at the first item of workgroup blockIdx.x; false when its share is empty.
__device__ __forceinline__ bool walk_begin(const AttnArgs& a, int nunits, Walk& w)
{
    const int lane = threadIdx.x & (kWave - 1);
    w.nunits = nunits;
    if (!a.t_dev) {
        w.items = seq_items(a, a.t_host);
        const unsigned W = (unsigned)a.B * (unsigned)w.items * (unsigned)nunits;
        const int N = balanced_workgroups(a, W);
        if ((int)blockIdx.x >= N) return false;
        w.W = W;
        w.N = N;
        w.cur = uniform(blockIdx.x * W / (unsigned)N);
        w.hi = uniform((blockIdx.x + 1u) * W / (unsigned)N);       // > cur, because N <= W
        w.b = uniform((int)(w.cur / ((unsigned)w.items * (unsigned)nunits)));
        w.base = (unsigned)w.b * (unsigned)w.items * (unsigned)nunits;
        return true;
    }
    // up to 64 sequences (the usual case): their lengths are loaded once and stay in the lanes
    const int first_bb = lane;
    const unsigned it0 = first_bb < a.B ? (unsigned)seq_items(a, a.t_dev[first_bb]) : 0u;
    const unsigned inc0 = wave_inclusive_scan(it0);
    unsigned total = lane_value(inc0, kWave - 1);
    for (int c = kWave; c < a.B; c += kWave) {
        const int bb = c + lane;
        const unsigned it = bb < a.B ? (unsigned)seq_items(a, a.t_dev[bb]) : 0u;
        total += lane_value(wave_inclusive_scan(it), kWave - 1);
    }
    const unsigned W = total * (unsigned)nunits;
    const int N = balanced_workgroups(a, W);
    if ((int)blockIdx.x >= N) return false;
    w.W = W;
    w.N = N;
    w.cur = uniform(blockIdx.x * W / (unsigned)N);
    w.hi = uniform((blockIdx.x + 1u) * W / (unsigned)N);           // > cur, because N <= W
    const unsigned target = w.cur / (unsigned)nunits;   // the sequence that holds item `cur` holds per-unit item `target`
    unsigned run = 0;
    for (int c = 0; c < a.B; c += kWave) {
        unsigned it = it0, inc = inc0;
        if (c > 0) {
            const int bb = c + lane;
            it = bb < a.B ? (unsigned)seq_items(a, a.t_dev[bb]) : 0u;
            inc = wave_inclusive_scan(it);
        }
        const unsigned tot = lane_value(inc, kWave - 1);
        if (run + tot > target) {
            const unsigned long long hit = __builtin_amdgcn_ballot_w64(run + inc > target);
            const int f = __builtin_ctzll(hit);
            w.b = c + f;
            w.items = (int)lane_value(it, f);
            w.base = (run + lane_value(inc, f) - (unsigned)w.items) * (unsigned)nunits;
            return true;
        }
        run += tot;
    }
    return false;                                   // not reached: target < total
}

// The unit piece at the walk's position (as many of the unit's remaining items as the share allows).
// (false: this piece lies inside the unit's overhead items - no rows, nothing to do)
template <int GT>
__device__ __forceinline__ bool walk_unit(const AttnArgs& a, const Walk& w, Unit& u, int& nitems)
{
    const int ngt = (a.G + GT - 1) / GT;
    const unsigned rel = w.cur - w.base;
    const int uib = uniform((int)(rel / (unsigned)w.items));
    const int item = uniform((int)(rel - (unsigned)uib * (unsigned)w.items));
    const unsigned left = w.hi - w.cur;
    nitems = w.items - item;
    if (left < (unsigned)nitems) nitems = (int)left;
    nitems = uniform(nitems);
    u.b = w.b;
    u.kvh = uib / ngt;
    u.g0 = (uib % ngt) * GT;
    u.t = uniform(a.t_dev ? a.t_dev[w.b] : a.t_host);
    u.pos = u.t + a.pos_offset;
    u.split = 0;
    u.last = 0;
    const int c0 = a.unit_cost;
    const int lo = item > c0 ? item - c0 : 0, hi = item + nitems > c0 ? item + nitems - c0 : 0;   // items that hold rows
    u.r0 = lo * a.item_rows;
    u.r1 = min(hi * a.item_rows, u.t - 1);
    u.is_last = item + nitems == w.items;
    u.direct = item <= c0 && u.is_last;          // every item that holds rows is here
    const size_t unit_index = (size_t)w.b * w.nunits + uib;
    u.pbase = ((size_t)blockIdx.x + unit_index) * GT;
    u.pstride = 1;
    u.p0 = 0;
    u.sstride = GT;
    u.npieces = 1;
    u.counter = (int)unit_index;
    if (!u.direct && a.counters) {
        const unsigned first = w.base + (unsigned)uib * (unsigned)w.items;
        const int i0 = uniform(item_owner(first + (unsigned)c0, w.W, w.N)), i1 = uniform(item_owner(first + (unsigned)w.items - 1u, w.W, w.N));
        u.p0 = ((size_t)i0 + unit_index) * GT;
        u.npieces = i1 - i0 + 1;
    }
    return hi > 0;
}

// Moves past nitems items; steps to the next sequence that has work when the current one is done.
__device__ __forceinline__ void walk_advance(const AttnArgs& a, Walk& w, int nitems)
{
    w.cur += (unsigned)nitems;
    if (w.cur >= w.hi) return;
    if (w.cur == w.base + (unsigned)w.items * (unsigned)w.nunits) {
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

// Workgroups that share a compute unit do not share it fairly: the one that came first gets its instructions issued
// first whenever several are ready, runs faster and leaves the others to finish alone, at a fraction of the unit's
// memory parallelism.  Measured finish times: 80 / 90 us for the first / second 256 workgroups of the balanced
// schedule's 512 matrix-core workgroups in a 101 us step (raising the wave priority of the second 256 flips it to
// 92 / 80).  So they take turns: wave priority follows the chip-wide constant-rate clock (~5 us per turn), shifted
// by the place the workgroup probably has among the co-resident ones of its unit - workgroups i, i + 256, i + 512,
// ... land on the same compute unit.  Called once per iteration of the matrix-core kernels' streaming loops (86 / 88
// us afterwards, 1-2 % per step).  Not in the vector-ALU kernel: its two workgroups per unit at config 2 finish
// together as it is, and with four per unit (1024 workgroups: 96 / 130 us for the first / last 256 of a 159 us step)
// taking turns made the step 1-3 % slower - there the staggered finish does no harm.
__device__ __forceinline__ void take_turns(const AttnArgs& a)
{
    const unsigned total = gridDim.x * gridDim.y * gridDim.z;
    if (total <= 256 || !a.turns) return;
    const unsigned places = total > 768 ? 4 : (total + 255) / 256;
    const unsigned id = (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
    const unsigned turn = ((unsigned)(wall_clock64() >> 9) + id / 256) % places;
    switch (turn) {
        case 0: __builtin_amdgcn_s_setprio(0); break;
        case 1: __builtin_amdgcn_s_setprio(1); break;
        case 2: __builtin_amdgcn_s_setprio(2); break;
        default: __builtin_amdgcn_s_setprio(3); break;
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
            const bool rows = walk_unit<GT>(a, w, u, nitems);
            if (rows) body(u);
            walk_advance(a, w, nitems);
            if (rows && w.cur < w.hi) __syncthreads();   // the next unit reuses the LDS staging
        }
    }
}

}  // namespace
}  // namespace onellm
