// Bare access-pattern kernels for gfx950: what the memory system of the GPU at hand delivers for the access mix of
// each product kernel, with no arithmetic to speak of.  Test-side only (bench.py times them next to the kernels whose
// mix they share and prints both; tests/test_access_ceilings.py checks that each moves the bytes it claims to).
// Nothing in the product links or loads this.
//
// Every kernel moves 16 bytes per lane per access through raw buffer instructions, so that the cache policy of
// each access is a parameter: `aux` is the instruction's policy field on gfx950 (bit 0 = sc0, bit 1 = nt,
// bit 4 = sc1; 0 = plain, 2 = non-temporal, 18 = non-temporal + written through ...).
//
//   read    : a pure read stream (each workgroup reads 16 KiB and keeps one checksum word)
//   fill    : a pure write stream
//   copy    : one stream in, one stream out, separate buffers
//   rows    : per row: read the row (of STREAMS buffers), reduce over the row, barrier, write the row back in place -
//             the shape of RMSNorm (1 buffer) and of the fused add-residual norm (2 buffers); optionally every
//             workgroup also reads a row-sized vector shared by all rows (gamma)
//   fanout  : one stream in, G streams out (the KV repeat)
//   regroup : rows of 256 bytes stored token-major [tokens][heads] copied to head-major [sequences][heads][tokens of
//             the sequence] - the transposing copy of the prefill QKV kernel, eight tokens per workgroup, a head's
//             eight rows leaving as one 2 KiB store
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t descriptor(const void* p, unsigned bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
template <int AUX>
__device__ __forceinline__ f32x4 load16(__amdgpu_buffer_rsrc_t r, unsigned off)
{
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, AUX));
}
template <int AUX>
__device__ __forceinline__ void store16(__amdgpu_buffer_rsrc_t r, unsigned off, f32x4 v)
{
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, v), r, (int)off, 0, AUX);
}

constexpr int kChunk = 16 * 1024;      // bytes per workgroup of the flat kernels: 256 threads x 4 accesses

template <int LA>
__global__ __launch_bounds__(256) void read_kernel(const char* __restrict__ src, float* __restrict__ sink)
{
    const __amdgpu_buffer_rsrc_t d = descriptor(src + (size_t)blockIdx.x * kChunk, kChunk);
    f32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = load16<LA>(d, (threadIdx.x + u * 256) * 16);
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) s += v[u][0] + v[u][1] + v[u][2] + v[u][3];
    if (s == 12345.678f) sink[blockIdx.x] = s;         // (keeps the loads alive; practically never taken)
}

template <int SA>
__global__ __launch_bounds__(256) void fill_kernel(char* __restrict__ dst, float value)
{
    const __amdgpu_buffer_rsrc_t d = descriptor(dst + (size_t)blockIdx.x * kChunk, kChunk);
    const f32x4 v = {value, value, value, value};
#pragma unroll
    for (int u = 0; u < 4; ++u) store16<SA>(d, (threadIdx.x + u * 256) * 16, v);
}

template <int LA, int SA>
__global__ __launch_bounds__(256) void copy_kernel(char* __restrict__ dst, const char* __restrict__ src)
{
    const __amdgpu_buffer_rsrc_t ds = descriptor(src + (size_t)blockIdx.x * kChunk, kChunk);
    const __amdgpu_buffer_rsrc_t dd = descriptor(dst + (size_t)blockIdx.x * kChunk, kChunk);
    f32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = load16<LA>(ds, (threadIdx.x + u * 256) * 16);
#pragma unroll
    for (int u = 0; u < 4; ++u) store16<SA>(dd, (threadIdx.x + u * 256) * 16, v[u]);
}

// one workgroup of 512 threads per row, NV accesses per thread and buffer
template <int LA, int SA, int NV, int STREAMS, bool SHARED>
__global__ __launch_bounds__(512) void rows_kernel(char* __restrict__ a, char* __restrict__ b, const char* __restrict__ shared,
                                                   unsigned row_bytes)
{
    __shared__ float part[8];
    const __amdgpu_buffer_rsrc_t da = descriptor(a + (size_t)blockIdx.x * row_bytes, row_bytes);
    const __amdgpu_buffer_rsrc_t db = descriptor(STREAMS > 1 ? b + (size_t)blockIdx.x * row_bytes : nullptr, STREAMS > 1 ? row_bytes : 0u);
    const __amdgpu_buffer_rsrc_t dg = descriptor(shared, SHARED ? row_bytes : 0u);
    f32x4 x[NV], y[NV], g[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) x[j] = load16<LA>(da, (threadIdx.x + j * 512) * 16);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        if (STREAMS > 1) y[j] = load16<LA>(db, (threadIdx.x + j * 512) * 16);
        if (SHARED) g[j] = load16<0>(dg, (threadIdx.x + j * 512) * 16);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        if (STREAMS > 1) x[j] += y[j];
        s += x[j][0] + x[j][1] + x[j][2] + x[j][3];
    }
#pragma unroll
    for (int off = 32; off; off >>= 1) s += __shfl_xor(s, off, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    s = part[0] + part[1] + part[2] + part[3] + part[4] + part[5] + part[6] + part[7];
    const float keep = s == 12345.678f ? 2.f : 1.f;      // the stores depend on the whole row, as a norm's do
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        f32x4 o = x[j] * keep;
        if (SHARED) o += g[j] * (keep - 1.f);
        store16<SA>(da, (threadIdx.x + j * 512) * 16, o);
        if (STREAMS > 1) store16<SA>(db, (threadIdx.x + j * 512) * 16, o);
    }
}

// chunk == 0: copy g of the whole source starts at dst + g * dst_stride.  chunk > 0: the source is a row of chunks and
// the G copies of a chunk follow each other (chunk c, copy g at (c * G + g) * chunk) - how the KV repeat lays out the
// query heads of one kv head.
template <int LA, int SA>
__global__ __launch_bounds__(256) void fanout_kernel(char* __restrict__ dst, const char* __restrict__ src, int G, size_t dst_stride,
                                                     size_t chunk)
{
    const size_t off = (size_t)blockIdx.x * 4096;
    const __amdgpu_buffer_rsrc_t ds = descriptor(src + off, 4096);
    const f32x4 v = load16<LA>(ds, threadIdx.x * 16);
    const size_t base = chunk ? (off / chunk) * chunk * G + off % chunk : off;
    const size_t step = chunk ? chunk : dst_stride;
    for (int g = 0; g < G; ++g) {
        const __amdgpu_buffer_rsrc_t dd = descriptor(dst + (size_t)g * step + base, 4096);
        store16<SA>(dd, threadIdx.x * 16, v);
    }
}

// 256 threads: 16-byte piece tid % 16 of the row, token (tid / 16) % 8 of the workgroup's eight, heads tid / 128 + 2 k;
// eight heads in flight per thread, as in the product kernel
template <int LA, int SA>
__global__ __launch_bounds__(256) void regroup_kernel(char* __restrict__ dst, const char* __restrict__ src, unsigned bytes,
                                                      int heads, int seq_tokens)
{
    const __amdgpu_buffer_rsrc_t ds = descriptor(src, bytes), dd = descriptor(dst, bytes);
    const unsigned piece = threadIdx.x & 15, tl = (threadIdx.x >> 4) & 7, h0 = threadIdx.x >> 7;
    const unsigned tok = blockIdx.x * 8 + tl;
    const unsigned b = tok / seq_tokens, sq = tok % seq_tokens;
    const unsigned in = tok * heads * 256u + piece * 16u;
    const unsigned out = (b * heads * seq_tokens + sq) * 256u + piece * 16u, head_step = (unsigned)seq_tokens * 256u;
    for (unsigned hb = h0; hb < (unsigned)heads; hb += 16) {
        f32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (hb + 2 * u < (unsigned)heads) v[u] = load16<LA>(ds, in + (hb + 2 * u) * 256u);
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (hb + 2 * u < (unsigned)heads) store16<SA>(dd, out + (hb + 2 * u) * head_step, v[u]);
    }
}

inline int status() { return (int)hipGetLastError(); }

// policy pairs the library is built for: index -> (load aux, store aux)
//   0: plain / plain      1: nt / nt      2: nt / nt+sc1      3: nt / sc1      4: nt / sc0+sc1
#define CEILING_POLICIES(X) X(0, 0, 0) X(1, 2, 2) X(2, 2, 18) X(3, 2, 16) X(4, 2, 17)

}  // namespace

extern "C" {

int ceiling_policy_count(void) { return 5; }

const char* ceiling_policy_name(int policy)
{
    switch (policy) {
        case 0: return "plain loads, plain stores";
        case 1: return "nt loads, nt stores";
        case 2: return "nt loads, nt+sc1 stores";
        case 3: return "nt loads, sc1 stores";
        case 4: return "nt loads, sc0+sc1 stores";
        default: return "?";
    }
}

// bytes must be a multiple of 16 KiB for read / fill / copy and of 4 KiB for fanout; -1 = bad argument
int ceiling_read(const void* src, size_t bytes, void* sink, int policy, void* stream)
{
    if (!src || !sink || bytes == 0 || bytes % kChunk) return -1;
    const dim3 grid((unsigned)(bytes / kChunk));
    hipStream_t st = (hipStream_t)stream;
    if (policy == 0) hipLaunchKernelGGL(read_kernel<0>, grid, dim3(256), 0, st, (const char*)src, (float*)sink);
    else hipLaunchKernelGGL(read_kernel<2>, grid, dim3(256), 0, st, (const char*)src, (float*)sink);
    return status();
}

int ceiling_fill(void* dst, size_t bytes, float value, int policy, void* stream)
{
    if (!dst || bytes == 0 || bytes % kChunk) return -1;
    const dim3 grid((unsigned)(bytes / kChunk));
    hipStream_t st = (hipStream_t)stream;
    switch (policy) {
#define X(i, la, sa) case i: hipLaunchKernelGGL(fill_kernel<sa>, grid, dim3(256), 0, st, (char*)dst, value); break;
        CEILING_POLICIES(X)
#undef X
        default: return -1;
    }
    return status();
}

int ceiling_copy(void* dst, const void* src, size_t bytes, int policy, void* stream)
{
    if (!dst || !src || bytes == 0 || bytes % kChunk) return -1;
    const dim3 grid((unsigned)(bytes / kChunk));
    hipStream_t st = (hipStream_t)stream;
    switch (policy) {
#define X(i, la, sa) case i: hipLaunchKernelGGL((copy_kernel<la, sa>), grid, dim3(256), 0, st, (char*)dst, (const char*)src); break;
        CEILING_POLICIES(X)
#undef X
        default: return -1;
    }
    return status();
}

// rows x row_bytes in place; row_bytes = 8192, 16384 or 32768 (512 threads x 1, 2 or 4 accesses); b == NULL: one buffer;
// shared == NULL: no row-sized vector read by every workgroup
int ceiling_rows(void* a, void* b, const void* shared, int rows, int row_bytes, int policy, void* stream)
{
    if (!a || rows <= 0 || (row_bytes != 8192 && row_bytes != 16384 && row_bytes != 32768)) return -1;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid(rows), block(512);
#define ROWS_LAUNCH(la, sa, nv)                                                                                                   \
    do {                                                                                                                          \
        if (b && shared) hipLaunchKernelGGL((rows_kernel<la, sa, nv, 2, true>), grid, block, 0, st, (char*)a, (char*)b, (const char*)shared, (unsigned)row_bytes);   \
        else if (b) hipLaunchKernelGGL((rows_kernel<la, sa, nv, 2, false>), grid, block, 0, st, (char*)a, (char*)b, (const char*)shared, (unsigned)row_bytes);      \
        else if (shared) hipLaunchKernelGGL((rows_kernel<la, sa, nv, 1, true>), grid, block, 0, st, (char*)a, (char*)b, (const char*)shared, (unsigned)row_bytes);  \
        else hipLaunchKernelGGL((rows_kernel<la, sa, nv, 1, false>), grid, block, 0, st, (char*)a, (char*)b, (const char*)shared, (unsigned)row_bytes);             \
    } while (0)
    switch (policy) {
#define X(i, la, sa)                                                       \
    case i:                                                                \
        if (row_bytes == 8192) ROWS_LAUNCH(la, sa, 1);                     \
        else if (row_bytes == 16384) ROWS_LAUNCH(la, sa, 2);               \
        else ROWS_LAUNCH(la, sa, 4);                                       \
        break;
        CEILING_POLICIES(X)
#undef X
        default: return -1;
    }
#undef ROWS_LAUNCH
    return status();
}

// src_bytes of src copied to G destinations dst, dst + dst_stride, ... (chunk == 0), or chunk by chunk with the G
// copies of a chunk side by side (chunk > 0, a multiple of 4 KiB that divides src_bytes; dst_stride is not used)
int ceiling_fanout(void* dst, const void* src, size_t src_bytes, int G, size_t dst_stride, size_t chunk, int policy, void* stream)
{
    if (!dst || !src || src_bytes == 0 || src_bytes % 4096 || G < 1) return -1;
    if (chunk ? (chunk % 4096 || src_bytes % chunk) : dst_stride < src_bytes) return -1;
    const dim3 grid((unsigned)(src_bytes / 4096));
    hipStream_t st = (hipStream_t)stream;
    switch (policy) {
#define X(i, la, sa) case i: hipLaunchKernelGGL((fanout_kernel<la, sa>), grid, dim3(256), 0, st, (char*)dst, (const char*)src, G, dst_stride, chunk); break;
        CEILING_POLICIES(X)
#undef X
        default: return -1;
    }
    return status();
}

// tokens * heads rows of 256 bytes, token-major in src, head-major per sequence of seq_tokens tokens in dst
// (tokens a multiple of 8 and of seq_tokens; the whole buffer below 4 GiB)
int ceiling_regroup(void* dst, const void* src, int tokens, int heads, int seq_tokens, int policy, void* stream)
{
    if (!dst || !src || tokens <= 0 || heads <= 0 || seq_tokens <= 0 || tokens % 8 || tokens % seq_tokens) return -1;
    const size_t bytes = (size_t)tokens * heads * 256;
    if (bytes >= (1ull << 32)) return -1;
    const dim3 grid((unsigned)(tokens / 8));
    hipStream_t st = (hipStream_t)stream;
    switch (policy) {
#define X(i, la, sa) case i: hipLaunchKernelGGL((regroup_kernel<la, sa>), grid, dim3(256), 0, st, (char*)dst, (const char*)src, (unsigned)bytes, heads, seq_tokens); break;
        CEILING_POLICIES(X)
#undef X
        default: return -1;
    }
    return status();
}

}  // extern "C"
