// Beam-search top-K over fp32 logits for gfx950.
//
// Order of candidates (a total order, so the result does not depend on how the reduction tree is
// shaped): larger value first; equal values: smaller global flat index (row*V + token) first.
// Stage 1: each (row, block) pair scans the tokens it owns with a K-slot sorted list per lane in
// registers, merges the 64 lists of a wave with lane exchanges (DPP inside 16 lanes, the crossbar
// beyond), then the waves of the workgroup through LDS.  Stage 2: one workgroup per batch entry
// merges the beam*nblk*K survivors.  Traffic: the logits are read once (rows*V*4 bytes).
#include <limits.h>
#include <math.h>
#include "common.hpp"

namespace onellm {
namespace {

constexpr int kEmptyId = INT_MAX;   // internal marker of a free slot: loses against every real candidate

__device__ __forceinline__ bool better(float v1, int i1, float v2, int i2)
{
    return v1 > v2 || (v1 == v2 && i1 < i2);
}

template <int K>
struct TopList {
    float val[K];
    int id[K];

    __device__ __forceinline__ void clear()
    {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            val[k] = -INFINITY;
            id[k] = kEmptyId;
        }
    }
    // keep the list sorted best-first; fully unrolled compare-exchange chain, no dynamic indexing
    __device__ __forceinline__ void insert(float v, int i)
    {
        if (!better(v, i, val[K - 1], id[K - 1])) return;
        val[K - 1] = v;
        id[K - 1] = i;
#pragma unroll
        for (int s = K - 2; s >= 0; --s) {
            const bool sw = better(val[s + 1], id[s + 1], val[s], id[s]);
            const float hv = sw ? val[s + 1] : val[s], lv = sw ? val[s] : val[s + 1];
            const int hi = sw ? id[s + 1] : id[s], li = sw ? id[s] : id[s + 1];
            val[s] = hv; val[s + 1] = lv;
            id[s] = hi; id[s + 1] = li;
        }
    }
};

template <int K, int CTRL>
__device__ __forceinline__ void merge_dpp(TopList<K>& t)
{
    TopList<K> o;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        o.val[k] = dpp_f32<CTRL>(t.val[k]);
        o.id[k] = dpp_i32<CTRL>(t.id[k]);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) t.insert(o.val[k], o.id[k]);
}

template <int K>
__device__ __forceinline__ void merge_xor(TopList<K>& t, int mask)
{
    TopList<K> o;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        o.val[k] = __shfl_xor(t.val[k], mask, kWave);
        o.id[k] = __shfl_xor(t.id[k], mask, kWave);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) t.insert(o.val[k], o.id[k]);
}

// after this every lane of the wave holds the wave's K best
template <int K>
__device__ __forceinline__ void wave_merge(TopList<K>& t)
{
    merge_dpp<K, kDppQuadXor1>(t);
    merge_dpp<K, kDppQuadXor2>(t);
    merge_dpp<K, kDppRowHalfMirror>(t);
    merge_dpp<K, kDppRowMirror>(t);
    merge_xor<K>(t, 16);
    merge_xor<K>(t, 32);
}

// workgroup of 256 lanes -> thread 0 returns the workgroup's K best
template <int K>
__device__ __forceinline__ void block_merge(TopList<K>& t, float* sval, int* sid)
{
    wave_merge<K>(t);
    const int tid = threadIdx.x, wave = tid / kWave;
    if ((tid & (kWave - 1)) == 0) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            sval[wave * K + k] = t.val[k];
            sid[wave * K + k] = t.id[k];
        }
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 4; ++w)
#pragma unroll
            for (int k = 0; k < K; ++k) t.insert(sval[w * K + k], sid[w * K + k]);
    }
}

// grid = rows * nblk; block `lane` of a row owns tokens tid + lane*256 + m*nblk*256
template <int K>
__global__ __launch_bounds__(256)
void topk_stage1_kernel(const float* __restrict__ logits, int V, int nblk, float* __restrict__ vals, int* __restrict__ ids)
{
    __shared__ float sval[4 * K];
    __shared__ int sid[4 * K];
    const int row = blockIdx.x / nblk, lane_blk = blockIdx.x % nblk;
    const float* p = logits + (size_t)row * V;
    const int flat0 = row * V;
    TopList<K> t;
    t.clear();
    for (int tok = threadIdx.x + lane_blk * 256; tok < V; tok += nblk * 256) t.insert(p[tok], flat0 + tok);
    block_merge<K>(t, sval, sid);
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            vals[(size_t)blockIdx.x * K + k] = t.val[k];
            ids[(size_t)blockIdx.x * K + k] = t.id[k] == kEmptyId ? -1 : t.id[k];
        }
    }
}

// grid = B; merges the n = beam*nblk*K stage-1 survivors of one batch entry
template <int K>
__global__ __launch_bounds__(256)
void topk_stage2_kernel(const float* __restrict__ vals, const int* __restrict__ ids, int n,
                        float* __restrict__ fvals, int* __restrict__ fids)
{
    __shared__ float sval[4 * K];
    __shared__ int sid[4 * K];
    const int b = blockIdx.x;
    TopList<K> t;
    t.clear();
    for (int i = threadIdx.x; i < n; i += 256) {
        const int id = ids[(size_t)b * n + i];
        if (id != -1) t.insert(vals[(size_t)b * n + i], id);
    }
    block_merge<K>(t, sval, sid);
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            fvals[(size_t)b * K + k] = t.val[k];
            fids[(size_t)b * K + k] = t.id[k] == kEmptyId ? -1 : t.id[k];
        }
    }
}

template <int K>
int launch_topk(const float* logits, int B, int beam, int V, int nblk, float* ws, hipStream_t st)
{
    const size_t n1 = (size_t)B * beam * nblk * K;
    float* vals = ws;
    int* ids = reinterpret_cast<int*>(vals + n1);
    float* fvals = reinterpret_cast<float*>(ids + n1);
    int* fids = reinterpret_cast<int*>(fvals + (size_t)B * K);
    hipLaunchKernelGGL((topk_stage1_kernel<K>), dim3(B * beam * nblk), dim3(256), 0, st, logits, V, nblk, vals, ids);
    int rc = launch_status();
    if (rc) return rc;
    hipLaunchKernelGGL((topk_stage2_kernel<K>), dim3(B), dim3(256), 0, st, vals, ids, beam * nblk * K, fvals, fids);
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
    switch (K) {
        case 1: return launch_topk<1>(logits, B, beam, V, nblk, workspace, st);
        case 2: return launch_topk<2>(logits, B, beam, V, nblk, workspace, st);
        case 3: return launch_topk<3>(logits, B, beam, V, nblk, workspace, st);
        case 4: return launch_topk<4>(logits, B, beam, V, nblk, workspace, st);
        case 5: return launch_topk<5>(logits, B, beam, V, nblk, workspace, st);
        case 6: return launch_topk<6>(logits, B, beam, V, nblk, workspace, st);
        case 7: return launch_topk<7>(logits, B, beam, V, nblk, workspace, st);
        default: return launch_topk<8>(logits, B, beam, V, nblk, workspace, st);
    }
}
