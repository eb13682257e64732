// Shared device helpers for the gfx950 kernels: 128-bit vector types, dtype
// conversion, wavefront (64-lane) and workgroup reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <set>
#include <type_traits>
#include <utility>

#include "../../include/xpu_graph_amd.h"

namespace xg {

constexpr int kWave = 64;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16_t;
typedef _Float16 f16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

// Per-dtype traits: a 16-byte vector of VEC elements and conversion to / from fp32.
template <typename T>
struct VecOf;
template <>
struct VecOf<float> {
  static constexpr int N = 4;
  typedef f32x4 type;
};
template <>
struct VecOf<bf16_t> {
  static constexpr int N = 8;
  typedef bf16x8 type;
};
template <>
struct VecOf<f16_t> {
  static constexpr int N = 8;
  typedef f16x8 type;
};

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }
__device__ __forceinline__ float to_f32(f16_t v) { return (float)v; }

template <typename T>
__device__ __forceinline__ T from_f32(float v) {
  return (T)v;  // round-to-nearest-even; gfx950 has native f32->bf16 conversion
}

// sigmoid and SiLU in fp32 from the hardware's exp2 and reciprocal (each within 1 ulp): four instructions instead of
// the dozen of an IEEE division.  Every kernel that applies them uses these two, so fused and unfused paths round
// identically.  t = -inf gives NaN for SiLU, as x * sigmoid(x) does in eager.
__device__ __forceinline__ float sigmoid_f32(float t) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(t * -1.44269504088896340736f));
}
__device__ __forceinline__ float silu_f32(float t) { return t * sigmoid_f32(t); }

// 16-byte global load / store.  The NT variants mark the access as streaming
// (data that is touched once), which keeps it from displacing reused lines.
template <typename V>
__device__ __forceinline__ V load_vec(const V* p) {
  return *p;
}
template <typename V>
__device__ __forceinline__ V load_vec_nt(const V* p) {
  return __builtin_nontemporal_load(p);
}
template <typename V>
__device__ __forceinline__ void store_vec(V* p, V v) {
  *p = v;
}
template <typename V>
__device__ __forceinline__ void store_vec_nt(V* p, V v) {
  __builtin_nontemporal_store(v, p);
}

// Sum over the low `width` lanes of each aligned lane group (width a power of
// two <= 64); every lane of the group ends with the total.  Inside a row of 16
// lanes the exchange is done by the DPP modifiers of the adds themselves (quad
// permutes, then the two row mirrors); only the steps across rows go through
// the LDS crossbar.
template <int WIDTH = kWave>
__device__ __forceinline__ float wave_sum(float v) {
  auto dpp = [](float x, auto CTRL) {
    constexpr int ctrl = decltype(CTRL)::value;
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), ctrl, 0xF, 0xF, true));
  };
  if constexpr (WIDTH >= 2) v += dpp(v, std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]: lane ^ 1
  if constexpr (WIDTH >= 4) v += dpp(v, std::integral_constant<int, 0x4E>{});   // quad_perm [2,3,0,1]: lane ^ 2
  if constexpr (WIDTH >= 8) v += dpp(v, std::integral_constant<int, 0x141>{});  // row_half_mirror: 7 - lane within 8
  if constexpr (WIDTH >= 16) v += dpp(v, std::integral_constant<int, 0x140>{}); // row_mirror: 15 - lane within 16
#pragma unroll
  for (int off = 16; off < WIDTH; off <<= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
template <int WIDTH = kWave>
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = WIDTH / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over the THREADS lanes that share one row.  THREADS <= 64: shuffle only.
// THREADS > 64: per-wave shuffle, then the NW = THREADS/64 partial sums meet in
// LDS (`red` holds NW floats per row group and is reused after a barrier).
// FRESH: `red` has not been read since the last barrier (first use, or a buffer of its own), so the
// barrier that protects an earlier reader can be left out.
template <int THREADS, bool FRESH = false>
__device__ __forceinline__ float group_sum(float v, float* red, int lane_in_row) {
  if constexpr (THREADS <= kWave) {
    return wave_sum<THREADS>(v);
  } else {
    constexpr int NW = THREADS / kWave;
    v = wave_sum<kWave>(v);
    if constexpr (!FRESH) __syncthreads();  // previous use of `red` is over
    if ((lane_in_row & (kWave - 1)) == 0) red[lane_in_row / kWave] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NW; ++i) t += red[i];
    return t;
  }
}

// 16 bytes per lane from global memory straight into LDS: lane i's data lands at lds_base + 16 i.  `base` and
// `lds_base` are wave-uniform.  Issued as inline asm so that the compiler does not know of LDS writes in flight:
// it would otherwise hold back LDS reads it cannot prove disjoint (the transposing reads) until every direct load
// in flight has landed.  The caller orders loads and reads with s_waitcnt vmcnt and a barrier.
__device__ __forceinline__ void load_to_lds16(const void* base, uint32_t lane_off, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(lane_off), "s"(base) : "memory", "m0");
}

inline int status_from_hip(hipError_t e) { return e == hipSuccess ? XG_OK : XG_ERR_LAUNCH; }

// Raise the dynamic-LDS limit of `kernel` to `bytes` on the current device, once per (kernel, device).  Keyed by the
// kernel's address, not by its type: many kernels here share one signature.
inline int allow_dynamic_lds(const void* kernel, int bytes) {
  static std::mutex mu;
  static std::set<std::pair<const void*, int>> done;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return XG_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(mu);
  if (done.count({kernel, dev})) return XG_OK;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return XG_ERR_LAUNCH;
  done.insert({kernel, dev});
  return XG_OK;
}

inline bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

}  // namespace xg
