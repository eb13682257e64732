// Pieces shared by the attention forward and backward kernels: vector types, the compile-time loop, the MFMA
// wrappers and the LDS chunk swizzles.
#pragma once
#include "xg_common.hpp"

#include <math.h>
#include <stdlib.h>

#include <type_traits>
#include <utility>

namespace xg {
namespace sdpa {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(1))) void gvoid;
typedef __attribute__((address_space(3))) void lvoid;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

constexpr int BQ = 128;   // query rows per workgroup
constexpr int BKV = 64;   // key rows per step
constexpr int kThreads = 256;

template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

template <typename T>
struct Vec8;
template <>
struct Vec8<bf16_t> {
  typedef bf16x8 type;
};
template <>
struct Vec8<f16_t> {
  typedef f16x8 type;
};

__device__ __forceinline__ f32x16 mma(bf16x8 a, bf16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
__device__ __forceinline__ f32x16 mma(f16x8 a, f16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }

// Chunk swizzles (16-byte chunks within a row of D elements).
template <int D>
__device__ __forceinline__ int swz_k(int r) {
  if constexpr (D == 128) return r & 15;  // 256-byte rows: 16 rows x one chunk -> 16 distinct bank groups
  else return (r >> 1) & 7;               // 128-byte rows: two rows per 256 bytes
}
template <int D>
__device__ __forceinline__ int swz_v(int r) {
  // the transposing read touches 8 consecutive rows x 4 aligned chunks: rows must move the GROUP of four
  if constexpr (D == 128) return ((r & 3) << 2) | ((r >> 2) & 3);
  else return (((r >> 1) & 1) << 2) | ((r >> 2) & 3);
}

}  // namespace sdpa
}  // namespace xg
