// KV-cache concat (append new rows at each sequence's history offset) and KV repeat (broadcast
// of KV heads to query heads) for gfx950.  Both are pure copies, bit-exact, HBM-bound:
// every thread moves one 16-byte piece of a cache row; the repeat kernel reads a source piece
// once and stores it to each of the G query heads of its group (algorithmic traffic:
// (1 + G) * bytes of the valid source rows, instead of 2*G for a gather per destination).
#include "common.hpp"

namespace onellm {
namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// COPY is the access type: 16 bytes on the normal path, the element itself otherwise.
// a piece stored for a reader that comes much later: 16-byte pieces written through, smaller ones non-temporal
template <bool NT, typename COPY>
__device__ __forceinline__ void store_piece(COPY* p, const COPY& v)
{
    if constexpr (sizeof(COPY) == 16) store16_write_through<NT>(p, __builtin_bit_cast(stream_f32x4, v));
    else __builtin_nontemporal_store(v, p);
}

template <typename COPY>
__global__ __launch_bounds__(256)
void kv_append_kernel(const COPY* __restrict__ k_src, const COPY* __restrict__ v_src,
                      COPY* __restrict__ k_cache, COPY* __restrict__ v_cache,
                      const int* __restrict__ cur_len, const int* __restrict__ history_len,
                      int Hkv, int max_q_len, int S, int rowv, size_t slab)
{
    // grid: x over (tau, piece) of one (b, kvh); y = b*Hkv + kvh; z = 0 (K) / 1 (V)
    const int i = blockIdx.x * 256 + threadIdx.x;
    const int tau = i / rowv, c = i % rowv;
    const int bh = blockIdx.y;
    const int b = bh / Hkv;
    if (tau >= max_q_len || tau >= cur_len[b]) return;
    const long drow = (long)history_len[b] + tau;
    if (drow < 0 || drow >= S) return;
    const COPY* src = blockIdx.z ? v_src : k_src;
    COPY* dst = blockIdx.z ? v_cache : k_cache;
    // streamed once in, once out: keep it out of the way of reusable cache lines
    store_piece<false>(&dst[slab + ((size_t)bh * S + (size_t)drow) * rowv + c],
                __builtin_nontemporal_load(&src[((size_t)bh * max_q_len + tau) * rowv + c]));
}

template <typename COPY>
__global__ __launch_bounds__(256)
void kv_repeat_kernel(const COPY* __restrict__ k_cache, const COPY* __restrict__ v_cache,
                      COPY* __restrict__ k_dst, COPY* __restrict__ v_dst,
                      const int* __restrict__ context_len,
                      int Hkv, int G, int S, int max_k_len, int rowv, size_t slab)
{
    // grid: x over (s, piece) of one (b, kvh); y = b*Hkv + kvh; z = 0 (K) / 1 (V)
    const int i = blockIdx.x * 256 + threadIdx.x;
    const int s = i / rowv, c = i % rowv;
    const int bh = blockIdx.y;
    const int b = bh / Hkv, kvh = bh % Hkv;
    int len = context_len[b];
    len = len < max_k_len ? len : max_k_len;
    len = len < S ? len : S;
    if (s >= len) return;
    const COPY* src = blockIdx.z ? v_cache : k_cache;
    COPY* dst = blockIdx.z ? v_dst : k_dst;
    const COPY val = __builtin_nontemporal_load(&src[slab + ((size_t)bh * S + s) * rowv + c]);
    const size_t Hq = (size_t)Hkv * G;
    size_t o = (((size_t)b * Hq + (size_t)kvh * G) * max_k_len + s) * rowv + c;
    for (int g = 0; g < G; ++g, o += (size_t)max_k_len * rowv) store_piece<true>(&dst[o], val);
}

struct CopyPlan {
    int access;   // bytes per thread access: 16, 4 or 2
    int rowv;     // accesses per row
};

CopyPlan plan(int row_bytes, int esz, std::initializer_list<const void*> ptrs)
{
    bool ok16 = row_bytes % 16 == 0;
    for (const void* p : ptrs) ok16 = ok16 && aligned16(p);
    if (ok16) return {16, row_bytes / 16};
    return {esz, row_bytes / esz};
}

}  // namespace
}  // namespace onellm

extern "C" int onellm_kv_append(int dtype, const void* k_src, const void* v_src, void* k_cache, void* v_cache,
                                const int* cur_len, const int* history_len, int B, int Hkv, int max_q_len, int S,
                                int D, int layer, int num_layers, onellm_stream_t stream)
{
    using namespace onellm;
    if (!k_src || !v_src || !k_cache || !v_cache || !cur_len || !history_len) return ONELLM_EINVAL;
    if (B <= 0 || Hkv <= 0 || max_q_len <= 0 || S <= 0 || D <= 0 || num_layers <= 0) return ONELLM_EINVAL;
    if (layer < 0 || layer >= num_layers) return ONELLM_EINVAL;
    if (dtype != ONELLM_FP32 && dtype != ONELLM_FP16) return ONELLM_EINVAL;
    const int esz = dtype == ONELLM_FP16 ? 2 : 4;
    const CopyPlan p = plan(D * esz, esz, {k_src, v_src, k_cache, v_cache});
    const size_t slab = (size_t)layer * B * Hkv * (size_t)S * p.rowv;
    const long per_head = (long)max_q_len * p.rowv;
    if ((long)B * Hkv > 65535 || (per_head + 255) / 256 > 0x7fffffffL) return ONELLM_EUNSUPPORTED;
    const dim3 grid((unsigned)((per_head + 255) / 256), B * Hkv, 2), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define ONELLM_APPEND(CT)                                                                                            \
    hipLaunchKernelGGL((kv_append_kernel<CT>), grid, block, 0, st, (const CT*)k_src, (const CT*)v_src, (CT*)k_cache, \
                       (CT*)v_cache, cur_len, history_len, Hkv, max_q_len, S, p.rowv, slab)
    if (p.access == 16) ONELLM_APPEND(u32x4);
    else if (p.access == 4) ONELLM_APPEND(uint32_t);
    else ONELLM_APPEND(uint16_t);
#undef ONELLM_APPEND
    return launch_status();
}

extern "C" int onellm_kv_repeat(int dtype, const void* k_cache, const void* v_cache, void* k_dst, void* v_dst,
                                const int* context_len, int B, int Hq, int Hkv, int S, int max_k_len, int D,
                                int layer, int num_layers, onellm_stream_t stream)
{
    using namespace onellm;
    if (!k_cache || !v_cache || !k_dst || !v_dst || !context_len) return ONELLM_EINVAL;
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || S <= 0 || max_k_len <= 0 || D <= 0 || num_layers <= 0) return ONELLM_EINVAL;
    if (layer < 0 || layer >= num_layers) return ONELLM_EINVAL;
    if (dtype != ONELLM_FP32 && dtype != ONELLM_FP16) return ONELLM_EINVAL;
    const int esz = dtype == ONELLM_FP16 ? 2 : 4;
    const CopyPlan p = plan(D * esz, esz, {k_cache, v_cache, k_dst, v_dst});
    const size_t slab = (size_t)layer * B * Hkv * (size_t)S * p.rowv;
    const int rows = max_k_len < S ? max_k_len : S;
    const long per_head = (long)rows * p.rowv;
    if ((long)B * Hkv > 65535 || (per_head + 255) / 256 > 0x7fffffffL) return ONELLM_EUNSUPPORTED;
    const dim3 grid((unsigned)((per_head + 255) / 256), B * Hkv, 2), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define ONELLM_REPEAT(CT)                                                                                         \
    hipLaunchKernelGGL((kv_repeat_kernel<CT>), grid, block, 0, st, (const CT*)k_cache, (const CT*)v_cache,        \
                       (CT*)k_dst, (CT*)v_dst, context_len, Hkv, Hq / Hkv, S, max_k_len, p.rowv, slab)
    if (p.access == 16) ONELLM_REPEAT(u32x4);
    else if (p.access == 4) ONELLM_REPEAT(uint32_t);
    else ONELLM_REPEAT(uint16_t);
#undef ONELLM_REPEAT
    return launch_status();
}
