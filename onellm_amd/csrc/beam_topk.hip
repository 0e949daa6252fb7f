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
// Stage 1: each (row, block) pair scans the tokens it owns with a sorted K-slot list per lane in
// registers, merges the 64 lists of a wave with lane exchanges (DPP inside 16 lanes, the crossbar
// beyond) using a bitonic top-K merge (max of a[i] and b[K-1-i], then a bitonic sort), then the
// waves of the workgroup through LDS.  Stage 2: one workgroup per batch entry merges the
// beam*nblk*K survivors.  Traffic: the logits are read once (rows*V*4 bytes).
#include <limits.h>
#include <math.h>
#include "common.hpp"

namespace onellm {
namespace {

typedef unsigned long long Key;

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

// workgroup of 256 lanes -> the lanes of wave 0 return the workgroup's KP best
template <int KP>
__device__ __forceinline__ void block_merge(TopList<KP>& t, Key* skey)
{
    wave_merge<KP>(t);
    const int tid = threadIdx.x, wave = tid / kWave;
    if ((tid & (kWave - 1)) == 0) {
#pragma unroll
        for (int i = 0; i < KP; ++i) skey[wave * KP + i] = t.k[i];
    }
    __syncthreads();
    if (wave == 0) {
        for (int w = 1; w < 4; ++w) {
            TopList<KP> o;
#pragma unroll
            for (int i = 0; i < KP; ++i) o.k[i] = skey[w * KP + i];
            t.merge(o);
        }
    }
}

// grid = rows * nblk.  Block `lane_blk` of a row owns the 256-token chunks lane_blk, lane_blk + nblk,
// ... (the reference's ownership: token tid + lane_blk*256 + m*nblk*256).  On the vector path a
// thread reads 4 consecutive tokens of a chunk with one 16-byte load and four such loads are issued
// before any candidate is inserted, so a block has its whole slice of the row in flight at once.
template <int KP>
__global__ __launch_bounds__(256)
void topk_stage1_kernel(const float* __restrict__ logits, int V, int nblk, int vec_ok, int K,
                        float* __restrict__ vals, int* __restrict__ ids)
{
    __shared__ Key skey[4 * KP];
    const int row = blockIdx.x / nblk, lane_blk = blockIdx.x % nblk;
    const float* p = logits + (size_t)row * V;
    const int flat0 = row * V;
    TopList<KP> t;
    t.clear();
    if (vec_ok) {
        constexpr int PASSES = 4;
        const int nchunks = (V + 255) / 256;
        const int sub = threadIdx.x / 64, l4 = (threadIdx.x % 64) * 4;
        for (int c0 = lane_blk + nblk * sub; c0 < nchunks; c0 += nblk * 4 * PASSES) {
            f32x4 v[PASSES];
            int tok[PASSES];
#pragma unroll
            for (int q = 0; q < PASSES; ++q) {
                tok[q] = (c0 + nblk * 4 * q) * 256 + l4;
                if (tok[q] < V) v[q] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p + tok[q]));
            }
#pragma unroll
            for (int q = 0; q < PASSES; ++q) {
                if (tok[q] < V) {          // V % 4 == 0 here, so tok < V means tok + 3 < V
#pragma unroll
                    for (int e = 0; e < 4; ++e) t.insert(make_key(v[q][e], flat0 + tok[q] + e));
                }
            }
        }
    } else {
        for (int tok = threadIdx.x + lane_blk * 256; tok < V; tok += nblk * 256) t.insert(make_key(p[tok], flat0 + tok));
    }
    block_merge<KP>(t, skey);
    if (threadIdx.x == 0) {
#pragma unroll
        for (int i = 0; i < KP; ++i) {
            if (i < K) {
                const int id = key_id(t.k[i]);
                vals[(size_t)blockIdx.x * K + i] = key_value(t.k[i], id, logits);
                ids[(size_t)blockIdx.x * K + i] = id;
            }
        }
    }
}

// grid = B; merges the n = beam*nblk*K stage-1 survivors of one batch entry
template <int KP>
__global__ __launch_bounds__(256)
void topk_stage2_kernel(const float* __restrict__ logits, const float* __restrict__ vals, const int* __restrict__ ids,
                        int n, int K, float* __restrict__ fvals, int* __restrict__ fids)
{
    __shared__ Key skey[4 * KP];
    const int b = blockIdx.x;
    TopList<KP> t;
    t.clear();
    for (int i = threadIdx.x; i < n; i += 256) {
        const int id = ids[(size_t)b * n + i];
        if (id != -1) t.insert(make_key(vals[(size_t)b * n + i], id));
    }
    block_merge<KP>(t, skey);
    if (threadIdx.x == 0) {
#pragma unroll
        for (int i = 0; i < KP; ++i) {
            if (i < K) {
                const int id = key_id(t.k[i]);
                fvals[(size_t)b * K + i] = key_value(t.k[i], id, logits);
                fids[(size_t)b * K + i] = id;
            }
        }
    }
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
    hipLaunchKernelGGL((topk_stage1_kernel<KP>), dim3(B * beam * nblk), dim3(256), 0, st, logits, V, nblk, vec_ok, K, vals, ids);
    int rc = launch_status();
    if (rc) return rc;
    hipLaunchKernelGGL((topk_stage2_kernel<KP>), dim3(B), dim3(256), 0, st, logits, vals, ids, beam * nblk * K, K, fvals, fids);
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
