// Shared device helpers for the gfx950 decode-path kernels: wave64 reductions on DPP,
// 16-byte vector access, storage-type conversion, and the host-side argument checks.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include "onellm_hip.h"

namespace onellm {

constexpr int kWave = 64;

// ---------------------------------------------------------------- DPP lane exchange (wave64)

// dpp_ctrl encodings (GCN3+/CDNA ISA): quad_perm = 0x00..0xFF, row_shr:n = 0x110+n,
// row_mirror = 0x140, row_half_mirror = 0x141.
constexpr int kDppQuadXor1 = 0xB1;     // quad_perm [1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;     // quad_perm [2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}

// Sum over aligned groups of LANES consecutive lanes; every lane of a group gets the group's sum.
// Up to 16 lanes it is pure DPP (no LDS traffic); beyond that the crossbar (ds_bpermute) is used.
template <int LANES>
__device__ __forceinline__ float group_sum(float v)
{
    static_assert(LANES == 1 || LANES == 2 || LANES == 4 || LANES == 8 || LANES == 16 || LANES == 32 || LANES == 64, "");
    if constexpr (LANES >= 2) v += dpp_f32<kDppQuadXor1>(v);
    if constexpr (LANES >= 4) v += dpp_f32<kDppQuadXor2>(v);
    if constexpr (LANES >= 8) v += dpp_f32<kDppRowHalfMirror>(v);
    if constexpr (LANES >= 16) v += dpp_f32<kDppRowMirror>(v);
    if constexpr (LANES >= 32) v += __shfl_xor(v, 16, kWave);
    if constexpr (LANES >= 64) v += __shfl_xor(v, 32, kWave);
    return v;
}

__device__ __forceinline__ float wave_sum(float v) { return group_sum<64>(v); }

// ---------------------------------------------------------------- storage types

template <typename T> struct Elt;
template <> struct Elt<float> {
    static constexpr int kVec = 4;            // elements in 16 bytes
    static constexpr int kDtype = ONELLM_FP32;
};
template <> struct Elt<__half> {
    static constexpr int kVec = 8;
    static constexpr int kDtype = ONELLM_FP16;
};

// 16 bytes of storage seen as fp32 values.  The raw member is a clang vector so that a widening
// read is an fpext of an extracted element, which the backend folds into v_fma_mix_f32.
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

template <typename T> struct Vec16;
template <> struct Vec16<float> {
    f32x4 raw;
    __device__ __forceinline__ float get(int i) const { return raw[i]; }
    __device__ __forceinline__ void set(int i, float v) { raw[i] = v; }
};
template <> struct Vec16<__half> {
    f16x8 raw;
    __device__ __forceinline__ float get(int i) const { return (float)raw[i]; }
    __device__ __forceinline__ void set(int i, float v) { raw[i] = (_Float16)v; }   // round-to-nearest-even
};

template <typename T>
__device__ __forceinline__ Vec16<T> load16(const T* p)
{
    Vec16<T> v;
    v.raw = *reinterpret_cast<const decltype(v.raw)*>(p);
    return v;
}
template <typename T>
__device__ __forceinline__ void store16(T* p, const Vec16<T>& v)
{
    *reinterpret_cast<decltype(v.raw)*>(p) = v.raw;
}

// Streaming variants: data that is touched once (cache rows, activation rows) is moved with the
// non-temporal hint so that it does not displace reusable lines in L2 / Infinity Cache; on
// MI355X this alone lifts a pure read stream from ~6.2 to ~7.0 TB/s.
template <typename T>
__device__ __forceinline__ Vec16<T> load16_stream(const T* p)
{
    Vec16<T> v;
    v.raw = __builtin_nontemporal_load(reinterpret_cast<const decltype(v.raw)*>(p));
    return v;
}
template <typename T>
__device__ __forceinline__ void store16_stream(T* p, const Vec16<T>& v)
{
    __builtin_nontemporal_store(v.raw, reinterpret_cast<decltype(v.raw)*>(p));
}
// 16 bytes written through to memory (the sc1 bit), with or without the non-temporal hint.  Pays where stores
// dominate - measured on MI355X against the non-temporal hint alone: the KV repeat (one load, G stores) 8 % faster
// with sc1 + nt (sc1 alone: 2 %), a prefill-sized KV append 12 % faster with sc1 alone (sc1 + nt: 7 %), an in-place
// read-modify-write stream 2 % with sc1 + nt.  Kernels that read two streams per stream written (SwiGLU, the
// prefill transpose) are 0.5-2 % slower with either and keep the plain non-temporal store.
typedef float stream_f32x4 __attribute__((ext_vector_type(4)));
template <bool NT>
__device__ __forceinline__ void store16_write_through(void* p, stream_f32x4 v)
{
    if constexpr (NT) asm volatile("global_store_dwordx4 %0, %1, off sc1 nt" : : "v"(p), "v"(v) : "memory");
    else asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(__half v) { return __half2float(v); }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ __half from_f32<__half>(float v) { return __float2half_rn(v); }
// value after one trip through the storage type
template <typename T> __device__ __forceinline__ float round_to(float v) { return to_f32(from_f32<T>(v)); }

// ---------------------------------------------------------------- host side

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Launch status: a failed launch is reported through hipGetLastError (which also clears it).
inline int launch_status() { return static_cast<int>(hipGetLastError()); }

// Internal tuning knobs (see tuning.cpp); -1 = choose automatically.
int tune_get(const char* key);

}  // namespace onellm
