// y[M, N] = x[M, K] . W[K, N] with M <= 32: the projections of a decode step.  fp16 operands (fp32 ones further
// down), fp32 accumulation.
//
// With so few rows the multiplication is a stream over the weights: every byte of W is read once and meets all M rows
// of x, so the kernel is bound by how fast the compute units can pull W, and everything else is arranged around that.
//   * A workgroup owns a panel of NT = 16 * CPL columns (64 or 128) and, when the problem is cut along K, one slice of
//     the rows; its waves take super-blocks of 64 rows of the panel in turn.  A lane (column group nl = lane % 16, row
//     group kg = lane / 16) loads CPL consecutive columns of the 16 rows 16 kg .. 16 kg + 15: the sixteen lanes of a
//     row group read 128 or 256 contiguous bytes of a weight row per instruction, and a wave has 16 such
//     instructions per super-block in flight, twice that with two stages.
//   * x[16, 64] of the same super-block comes in the A-operand layout of v_mfma_f32_16x16x16_f16 straight from memory
//     (lane (nl, kg): row nl, columns 16 kg .. 16 kg + 15; x is small and stays in cache).  Product j of a super-block
//     takes rows 16 kg + 4 j + {0..3} from every row group, so the B operand of column c is the c-th half of four
//     of the lane's weight registers, gathered with two byte-permutes; the result tile leaves lane (nl, kg) with rows
//     4 kg + {0..3} of column CPL * nl + c.
//   * The waves' tiles meet in LDS.  A run cut along K writes its slice's sums to the workspace with device-scope
//     stores and bumps the panel's arrival counter; the slice that finds all others there adds them up in slice order
//     (the result does not depend on who came last) and writes y.  The counters live in this library (one set per
//     (device, workspace), owned until the workspace is released), are zero between calls and are reset by the slice
//     that reads them last.
// Alignment and shape rules are in skinny_shape_ok / skinny_launch; whatever they decline goes to the library GEMM.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include "onellm_gemm.h"
#include "counter_sets.hpp"
#include "device_symbol.hpp"
#include "skinny_gemm.hpp"

namespace onellm {
int tune_get(const char* key);
namespace {

typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kSuperBlock = 64;              // rows of W one wave multiplies per step
constexpr int kCounterSets = 128;            // workspaces that can run sliced at the same time
constexpr int kCounterPanels = 2048;         // column panels per call
__device__ unsigned g_slice_arrivals[kCounterSets * kCounterPanels];

constexpr int kStream = 2;                   // nt: the weights are read once
constexpr int kDeviceScope = 16;             // sc1: partial sums cross between compute units of different chip quarters
constexpr unsigned kNowhere = 0xFFFFFFF0u;   // an offset past every buffer: the load returns zeros

struct SkinnyArgs {
    const void* x;
    const void* w;
    void* y;
    const void* w_second;                    // a launch of two problems that share x and shape (grid.z = 2): the other W and y
    void* y_second;
    float* partial;                          // [panels][splits][rows][NT]
    unsigned* counters;                      // [panels]
    int M, K, N, ldy, splits;
    int ordered;                             // 1: the counter add is a release and the reading slice takes an acquire fence
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t window(const void* p, unsigned bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

// CPL consecutive fp16 columns of one weight row
template <int CPL> struct WeightPiece;
template <> struct WeightPiece<4> {
    u32x2 v;
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, unsigned off) { v = __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, kStream); }
    __device__ __forceinline__ unsigned pair(int i) const { return v[i]; }
};
template <> struct WeightPiece<8> {
    u32x4 v;
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, unsigned off) { v = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, kStream); }
    __device__ __forceinline__ unsigned pair(int i) const { return v[i]; }
};

// What follows the waves' tiles in LDS (lds[wave][row][column], ROWS x NT floats per wave): their sum, the hand-over
// between the slices of a cut run, and the rows of y.  OUT is the element type of y.
template <typename OUT, int ROWS, int NT, int NW>
__device__ __forceinline__ void finish_tile(const SkinnyArgs& a, const float* lds, int tid, int n0, int slot, int split, bool second)
{
    constexpr int NTHR = NW * kWave;
    __syncthreads();
    // a thread owns pieces of four consecutive columns of one row
    constexpr int PIECES = ROWS * NT / 4, PER = (PIECES + NTHR - 1) / NTHR;
    f32x4 sum[PER];
#pragma unroll
    for (int p = 0; p < PER; ++p) {
        const int piece = p * NTHR + tid;
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
        if (piece < PIECES) {
#pragma unroll
            for (int wv = 0; wv < NW; ++wv) s = s + *reinterpret_cast<const f32x4*>(&lds[wv * ROWS * NT + piece * 4]);
        }
        sum[p] = s;
    }

    if (a.splits > 1) {
        // Every slice writes its sums with device-scope stores, waits until they are acknowledged and adds one to the
        // panel's counter; the one that finds all others there reads them back with device-scope loads.  The stores
        // are written through to memory before the wait ends and the add executes at memory, so the reader's loads
        // come after every other slice's sums; nobody waits for anybody.
        __shared__ int s_last;
        const __amdgpu_buffer_rsrc_t rp = window(a.partial, 0x7FFFFFFFu);
        const unsigned panel_bytes = (unsigned)(ROWS * NT * 4);
        const unsigned mine = ((unsigned)slot * a.splits + split) * panel_bytes;
#pragma unroll
        for (int p = 0; p < PER; ++p) {
            const int piece = p * NTHR + tid;
            if (piece < PIECES)
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, sum[p]), rp, mine + piece * 16, 0, kDeviceScope);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            // (the formally ordered form - tuning key gemm_ordered_finish - makes the add a release and has the reading
            // slice take an acquire fence: the compiler then adds the write-back / invalidate of this chip quarter's L2,
            // which the written-through stores and the memory-served loads do not need; kept for the soak test)
            const unsigned before = a.ordered
                ? __hip_atomic_fetch_add(&a.counters[slot], 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT)
                : __hip_atomic_fetch_add(&a.counters[slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int last = before == (unsigned)(a.splits - 1);
            if (last) {
                __hip_atomic_store(&a.counters[slot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // zero for the next call
                if (a.ordered) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            }
            s_last = last;
        }
        __syncthreads();
        if (!s_last) return;
        const unsigned all = (unsigned)slot * a.splits * panel_bytes;
#pragma unroll
        for (int p = 0; p < PER; ++p) {
            const int piece = p * NTHR + tid;
            f32x4 s = {0.f, 0.f, 0.f, 0.f};
            if (piece < PIECES) {
                for (int s0 = 0; s0 < a.splits; s0 += 4) {
                    f32x4 t[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int sp = min(s0 + j, a.splits - 1);
                        t[j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rp, all + sp * panel_bytes + piece * 16, 0, kDeviceScope));
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (s0 + j < a.splits) s = s + t[j];
                }
            }
            sum[p] = s;
        }
    }
#pragma unroll
    for (int p = 0; p < PER; ++p) {
        const int piece = p * NTHR + tid;
        const int m = piece / (NT / 4), n = n0 + 4 * (piece % (NT / 4));
        if (piece < PIECES && m < a.M && n < a.N) {
            void* y = second ? a.y_second : a.y;
            if constexpr (sizeof(OUT) == 2) {
                const f16x4 o = {(_Float16)sum[p][0], (_Float16)sum[p][1], (_Float16)sum[p][2], (_Float16)sum[p][3]};
                *reinterpret_cast<f16x4*>(static_cast<_Float16*>(y) + (size_t)m * a.ldy + n) = o;
            } else {
                *reinterpret_cast<f32x4*>(static_cast<float*>(y) + (size_t)m * a.ldy + n) = sum[p];
            }
        }
    }
}

// MT: tiles of 16 rows of x; U: super-blocks a wave has in flight; NW: waves; CPL: columns per lane
template <int MT, int U, int NW, int CPL>
__global__ __launch_bounds__(NW * kWave)
void skinny_gemm_kernel(const SkinnyArgs a)
{
    extern __shared__ float lds[];
    constexpr int NT = 16 * CPL;
    constexpr int ROWS = MT * 16;
    const int panel = blockIdx.x, split = blockIdx.y;
    const bool second = blockIdx.z != 0;
    const int slot = second ? gridDim.x + panel : panel;         // where this panel's partial sums and counter are
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int nl = lane & 15, kg = lane >> 4;
    const int n0 = panel * NT;
    const int nsb = a.K / kSuperBlock;
    const int sb0 = (int)((long long)nsb * split / a.splits), sb1 = (int)((long long)nsb * (split + 1) / a.splits);
    const __amdgpu_buffer_rsrc_t rw = window(second ? a.w_second : a.w, (unsigned)((size_t)a.K * a.N * 2));
    const __amdgpu_buffer_rsrc_t rx = window(a.x, (unsigned)((size_t)a.M * a.K * 2));
    // byte offsets of this lane inside super-block 0; a column past N reads the next row's start (or nothing, in the
    // last row) and its sums are dropped at the end, a row of x past M reads past the buffer, i.e. zeros
    const unsigned w_lane = (unsigned)((16 * kg) * a.N + n0 + CPL * nl) * 2u;
    const unsigned w_row = (unsigned)a.N * 2u, w_sb = (unsigned)a.N * (2u * kSuperBlock);
    const unsigned x_lane = (unsigned)(nl * a.K + 16 * kg) * 2u, x_tile = (unsigned)a.K * 32u;

    f32x4 acc[MT][CPL];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int c = 0; c < CPL; ++c) acc[mt][c] = f32x4{0.f, 0.f, 0.f, 0.f};

    WeightPiece<CPL> wr[U][16];
    u32x4 xr[U][MT][2];
    auto request = [&](int u, int sb) {
        const bool in = sb < sb1;
        const unsigned wo = w_lane + (unsigned)sb * w_sb;
        const unsigned xo = x_lane + (unsigned)sb * (2u * kSuperBlock);
#pragma unroll
        for (int t = 0; t < 16; ++t) wr[u][t].load(rw, in ? wo + t * w_row : kNowhere);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int h = 0; h < 2; ++h) xr[u][mt][h] = __builtin_amdgcn_raw_buffer_load_b128(rx, in ? xo + mt * x_tile + h * 16 : kNowhere, 0, 0);
    };
    int sb = sb0 + wave;
#pragma unroll
    for (int u = 0; u < U; ++u) request(u, sb + NW * u);
    for (; sb < sb1; sb += NW * U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            // (the stage's registers are copied so that its next super-block can be requested before this one is used)
            WeightPiece<CPL> wc[16];
            u32x4 xc[MT][2];
#pragma unroll
            for (int t = 0; t < 16; ++t) wc[t] = wr[u][t];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                xc[mt][0] = xr[u][mt][0];
                xc[mt][1] = xr[u][mt][1];
            }
            request(u, sb + NW * u + NW * U);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int c = 0; c < CPL; ++c) {
                    constexpr unsigned kLow = 0x05040100u, kHigh = 0x07060302u;
                    const unsigned sel = (c & 1) ? kHigh : kLow;
                    const u32x2 b = {__builtin_amdgcn_perm(wc[4 * j + 1].pair(c / 2), wc[4 * j].pair(c / 2), sel),
                                     __builtin_amdgcn_perm(wc[4 * j + 3].pair(c / 2), wc[4 * j + 2].pair(c / 2), sel)};
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        const u32x2 av = {xc[mt][j / 2][2 * (j % 2)], xc[mt][j / 2][2 * (j % 2) + 1]};
                        acc[mt][c] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, av), __builtin_bit_cast(f16x4, b),
                                                                           acc[mt][c], 0, 0, 0);
                    }
                }
            }
        }
    }

    // ---- the waves' tiles meet in LDS: lds[wave][row][column]
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c4 = 0; c4 < CPL / 4; ++c4) {
                const f32x4 v = {acc[mt][4 * c4 + 0][r], acc[mt][4 * c4 + 1][r], acc[mt][4 * c4 + 2][r], acc[mt][4 * c4 + 3][r]};
                *reinterpret_cast<f32x4*>(&lds[(wave * ROWS + mt * 16 + 4 * kg + r) * NT + CPL * nl + 4 * c4]) = v;
            }
    finish_tile<_Float16, ROWS, NT, NW>(a, lds, tid, n0, slot, split, second);
}

// The same stream for fp32 weights (the reference's own element type) on v_mfma_f32_16x16x4_f32.  A lane loads CPL = 2
// or 4 consecutive fp32 columns of the rows 16 kg .. 16 kg + 15 of a 64-row super-block (panels of 32 or 64 columns,
// 128 or 256 contiguous bytes per row group); product t of a super-block takes row 16 kg + t from every row group as
// its four k-values, so both operands are registers as loaded - x comes as row nl, columns 16 kg .. 16 kg + 15 - and
// no gather is needed.  Sums, hand-over and output are the fp16 kernel's.
// (The loaded registers are kept as float vectors and indexed as such: bit-casting one element of an integer vector to
// float - __builtin_bit_cast(float, v[i]) - gave element 0 for every i with this compiler.)
template <int CPL> struct WeightPiece32;
typedef float f32x2 __attribute__((ext_vector_type(2)));
template <> struct WeightPiece32<2> {
    f32x2 v;
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, unsigned off)
    {
        v = __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, kStream));
    }
    __device__ __forceinline__ float column(int i) const { return v[i]; }
};
template <> struct WeightPiece32<4> {
    f32x4 v;
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, unsigned off)
    {
        v = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, kStream));
    }
    __device__ __forceinline__ float column(int i) const { return v[i]; }
};

template <int MT, int U, int NW, int CPL>
__global__ __launch_bounds__(NW * kWave)
void skinny_gemm_f32_kernel(const SkinnyArgs a)
{
    extern __shared__ float lds[];
    constexpr int NT = 16 * CPL;
    constexpr int ROWS = MT * 16;
    const int panel = blockIdx.x, split = blockIdx.y;
    const bool second = blockIdx.z != 0;
    const int slot = second ? gridDim.x + panel : panel;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int nl = lane & 15, kg = lane >> 4;
    const int n0 = panel * NT;
    const int nsb = a.K / kSuperBlock;
    const int sb0 = (int)((long long)nsb * split / a.splits), sb1 = (int)((long long)nsb * (split + 1) / a.splits);
    const __amdgpu_buffer_rsrc_t rw = window(second ? a.w_second : a.w, (unsigned)((size_t)a.K * a.N * 4));
    const __amdgpu_buffer_rsrc_t rx = window(a.x, (unsigned)((size_t)a.M * a.K * 4));
    const unsigned w_lane = (unsigned)((16 * kg) * a.N + n0 + CPL * nl) * 4u;
    const unsigned w_row = (unsigned)a.N * 4u, w_sb = (unsigned)a.N * (4u * kSuperBlock);
    const unsigned x_lane = (unsigned)(nl * a.K + 16 * kg) * 4u, x_tile = (unsigned)a.K * 64u;

    f32x4 acc[MT][CPL];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int c = 0; c < CPL; ++c) acc[mt][c] = f32x4{0.f, 0.f, 0.f, 0.f};

    WeightPiece32<CPL> wr[U][16];
    f32x4 xr[U][MT][4];
    auto request = [&](int u, int sb) {
        const bool in = sb < sb1;
        const unsigned wo = w_lane + (unsigned)sb * w_sb;
        const unsigned xo = x_lane + (unsigned)sb * (4u * kSuperBlock);
#pragma unroll
        for (int t = 0; t < 16; ++t) wr[u][t].load(rw, in ? wo + t * w_row : kNowhere);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int q = 0; q < 4; ++q)
                xr[u][mt][q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, in ? xo + mt * x_tile + q * 16 : kNowhere, 0, 0));
    };
    int sb = sb0 + wave;
#pragma unroll
    for (int u = 0; u < U; ++u) request(u, sb + NW * u);
    for (; sb < sb1; sb += NW * U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            WeightPiece32<CPL> wc[16];
            f32x4 xc[MT][4];
#pragma unroll
            for (int t = 0; t < 16; ++t) wc[t] = wr[u][t];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int q = 0; q < 4; ++q) xc[mt][q] = xr[u][mt][q];
            request(u, sb + NW * u + NW * U);
#pragma unroll
            for (int t = 0; t < 16; ++t)
#pragma unroll
                for (int c = 0; c < CPL; ++c)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[mt][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(xc[mt][t / 4][t % 4], wc[t].column(c), acc[mt][c], 0, 0, 0);
        }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c = 0; c < CPL; ++c) lds[(wave * ROWS + mt * 16 + 4 * kg + r) * NT + CPL * nl + c] = acc[mt][c][r];
    finish_tile<float, ROWS, NT, NW>(a, lds, tid, n0, slot, split, second);
}

struct Variant {
    int dtype, mt, nt, nw;
    void (*launch)(const SkinnyArgs&, dim3, hipStream_t);
};

template <int MT, int U, int NW, int CPL>
void launch_variant(const SkinnyArgs& a, dim3 grid, hipStream_t st)
{
    constexpr size_t lds_bytes = sizeof(float) * NW * MT * 16 * 16 * CPL;
    hipLaunchKernelGGL((skinny_gemm_kernel<MT, U, NW, CPL>), grid, dim3(NW * kWave), lds_bytes, st, a);
}

template <int MT, int U, int NW, int CPL>
void launch_variant_f32(const SkinnyArgs& a, dim3 grid, hipStream_t st)
{
    constexpr size_t lds_bytes = sizeof(float) * NW * MT * 16 * 16 * CPL;
    hipLaunchKernelGGL((skinny_gemm_f32_kernel<MT, U, NW, CPL>), grid, dim3(NW * kWave), lds_bytes, st, a);
}

// up to 16 rows: 64-column panels with two super-blocks in flight or one, 128-column panels with one or two;
// 17..32 rows: the same panels with two row tiles
// fp32: 64-column panels with one super-block in flight, 32-column panels with two or one; the same with two row tiles
const Variant g_variants[] = {
    {ONELLM_FP16, 1, 64, 4, launch_variant<1, 2, 4, 4>},  {ONELLM_FP16, 1, 128, 4, launch_variant<1, 1, 4, 8>},
    {ONELLM_FP16, 1, 64, 4, launch_variant<1, 1, 4, 4>},  {ONELLM_FP16, 1, 128, 4, launch_variant<1, 2, 4, 8>},
    {ONELLM_FP16, 2, 64, 4, launch_variant<2, 2, 4, 4>},  {ONELLM_FP16, 2, 128, 4, launch_variant<2, 1, 4, 8>},
    {ONELLM_FP16, 2, 64, 4, launch_variant<2, 1, 4, 4>},
    {ONELLM_FP32, 1, 64, 4, launch_variant_f32<1, 1, 4, 4>}, {ONELLM_FP32, 1, 32, 4, launch_variant_f32<1, 2, 4, 2>},
    {ONELLM_FP32, 1, 32, 4, launch_variant_f32<1, 1, 4, 2>}, {ONELLM_FP32, 2, 64, 4, launch_variant_f32<2, 1, 4, 4>},
    {ONELLM_FP32, 2, 32, 4, launch_variant_f32<2, 2, 4, 2>},
};
constexpr int kVariants = (int)(sizeof(g_variants) / sizeof(g_variants[0]));

int panels_of(const Variant& v, int N) { return (N + v.nt - 1) / v.nt; }
size_t partial_bytes(const Variant& v, int splits, int N, int problems)
{
    return splits > 1 ? (size_t)problems * panels_of(v, N) * splits * v.mt * 16 * v.nt * sizeof(float) : 0;
}
bool config_fits(const Variant& v, int dtype, int splits, int M, int K, int N, size_t ws_bytes, int problems)
{
    if (v.dtype != dtype) return false;
    if (M > v.mt * 16 || (v.mt == 2 && M <= 16)) return false;
    if (splits < 1 || splits > K / kSuperBlock) return false;
    if (problems * panels_of(v, N) > kCounterPanels) return false;
    const size_t need = partial_bytes(v, splits, N, problems);
    return need <= ws_bytes && need < (1u << 30);
}

// The counter set of a (device, workspace): owned from the workspace's first cut run until the caller releases
// the workspace, never handed to another one in between (counter_sets.hpp).
CounterSets g_slice_sets("onellm_linear (few-row kernel cut along K)", kCounterSets);

// this device's copy of the counters (every device has its own, at its own address)
DeviceSymbol g_slice_arrivals_address;

bool aligned(const void* p, size_t a) { return (reinterpret_cast<size_t>(p) & (a - 1)) == 0; }

}  // namespace

bool skinny_shape_ok(int dtype, int M, int K, int N, int ldy, int w_is_nk)
{
    if ((dtype != ONELLM_FP16 && dtype != ONELLM_FP32) || w_is_nk) return false;
    const unsigned long long esz = dtype == ONELLM_FP16 ? 2 : 4;
    if (M < 1 || M > kSkinnyMaxRows) return false;
    if (K < kSuperBlock || K % kSuperBlock != 0) return false;       // whole super-blocks (a ragged one would multiply stray x by zero)
    if (N < 8 || (N * esz) % 16 != 0) return false;                  // 16-byte pieces of a weight row start aligned
    if (ldy == 0) ldy = N;
    if (ldy < N || ldy % 4 != 0) return false;                       // y is stored four columns at a time
    if ((unsigned long long)K * N * esz >= (1ull << 32) || (unsigned long long)M * K * esz >= (1ull << 32)) return false;
    return true;
}

int skinny_candidates(int dtype, int M, int K, int N, size_t ws_bytes, int problems, SkinnyConfig* out, int max)
{
    static const int kSplits[] = {1, 2, 3, 4, 6, 8, 12, 16};
    int n = 0;
    for (int v = 0; v < kVariants; ++v)
        for (int s : kSplits) {
            if (!config_fits(g_variants[v], dtype, s, M, K, N, ws_bytes, problems)) continue;
            const long long panels = (long long)problems * panels_of(g_variants[v], N);
            if (s > 1 && (panels * s > 2048 || panels >= 1024)) continue;   // slicing is for problems that do not fill the chip
            if (n < max) out[n++] = SkinnyConfig{v, s};
        }
    return n;
}

SkinnyConfig skinny_default(int dtype, int M, int K, int N, size_t ws_bytes, int problems)
{
    SkinnyConfig best;
    long long best_gap = 0;
    SkinnyConfig cand[96];
    const int n = skinny_candidates(dtype, M, K, N, ws_bytes, problems, cand, 96);
    for (int i = 0; i < n; ++i) {
        const Variant& v = g_variants[cand[i].variant];
        if (v.nt != 64) continue;                                        // the 64-column forms
        long long gap = (long long)problems * panels_of(v, N) * cand[i].splits - 256;
        if (gap < 0) gap = -gap;
        if (best.variant < 0 || gap < best_gap) {
            best = cand[i];
            best_gap = gap;
        }
    }
    if (best.variant < 0 && n > 0) best = cand[0];
    return best;
}

int skinny_launch(SkinnyConfig c, int dtype, const void* x, const void* w, void* y, const void* w_second, void* y_second, int M, int K,
                  int N, int ldy, void* workspace, size_t workspace_bytes, hipStream_t stream)
{
    if (ldy == 0) ldy = N;
    if (c.variant < 0 || c.variant >= kVariants || !skinny_shape_ok(dtype, M, K, N, ldy, 0)) return ONELLM_EUNSUPPORTED;
    const Variant& v = g_variants[c.variant];
    const int problems = w_second ? 2 : 1;
    if (!workspace) workspace_bytes = 0;
    if (!config_fits(v, dtype, c.splits, M, K, N, workspace_bytes, problems)) return ONELLM_EUNSUPPORTED;
    const size_t y_align = dtype == ONELLM_FP16 ? 8 : 16;                 // four columns per store
    if (!aligned(x, 16) || !aligned(w, 16) || !aligned(y, y_align)) return ONELLM_EUNSUPPORTED;
    if (w_second && (!y_second || !aligned(w_second, 16) || !aligned(y_second, y_align))) return ONELLM_EUNSUPPORTED;
    SkinnyArgs a{};
    a.x = x; a.w = w; a.y = y;
    a.w_second = w_second; a.y_second = y_second;
    a.M = M; a.K = K; a.N = N; a.ldy = ldy; a.splits = c.splits;
    if (c.splits > 1) {
        if (!aligned(workspace, 16)) return ONELLM_EUNSUPPORTED;
        int dev = 0;
        const hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return (int)e;
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
            (void)hipGetLastError();
            capturing = hipStreamCaptureStatusNone;
        }
        const int set = g_slice_sets.acquire(dev, workspace, capturing != hipStreamCaptureStatusNone);
        if (set < 0) return kSkinnyNoCounterSet;
        void* counters = nullptr;
        const int rc = g_slice_arrivals_address.address(HIP_SYMBOL(g_slice_arrivals), &counters);
        if (rc != 0) return rc;
        a.partial = static_cast<float*>(workspace);
        a.counters = static_cast<unsigned*>(counters) + (size_t)set * kCounterPanels;
        a.ordered = tune_get("gemm_ordered_finish") == 1;
    }
    v.launch(a, dim3(panels_of(v, N), c.splits, problems), stream);
    return (int)hipGetLastError();
}

}  // namespace onellm
