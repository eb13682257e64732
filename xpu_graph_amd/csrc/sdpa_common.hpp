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

// Which problem (batch x head) and which of its blocks a workgroup takes, rank 0 being the heaviest block.  Workgroup
// ids are dealt to the 8 XCDs round-robin; with `group` >= 2 (and a problem count that is a multiple of 8) every XCD
// walks its own problems `group` at a time, their blocks interleaved heaviest first: the blocks in flight on an XCD then
// belong to few problems and find each other's tiles in its L2.  Otherwise: the heaviest blocks of all problems first.
__device__ __forceinline__ void grouped_block_order(int id, int n_prob, int n_blk, int group, int& prob, int& rank) {
  if (group >= 2 && (n_prob & 7) == 0) {
    const int xcd = id & 7, slot = id >> 3;
    const int per = group * n_blk;
    const int g = slot / per, r = slot % per;
    const int left = (n_prob >> 3) - g * group;
    const int gsz = left < group ? left : group;
    prob = (g * group + r % gsz) * 8 + xcd;
    rank = r / gsz;
  } else {
    prob = id % n_prob;
    rank = id / n_prob;
  }
}
// Problems per XCD taken at a time by grouped_block_order: all of them up to eight (0: no grouping).
inline int block_order_group(int64_t n_prob) {
  if (n_prob % 8 != 0 || n_prob / 8 < 2) return 0;
  return (int)(n_prob / 8 < 8 ? n_prob / 8 : 8);
}

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
