// Shared implementation of the dense-layer kernels (included by gemm_bf16.hip, gemm_f16.hip and
// gemm_fp8.hip, one translation unit per operand type so that they compile in parallel).
//
// Dense layer for gfx950: out = act(A @ B(+T) * scales + bias + residual) on the
// matrix cores.
//
// Tiling: one 256-thread workgroup (4 wavefronts, 2 x 2) owns a 256 x 256 output
// tile; each wavefront owns 128 x 128 of it as 4 x 4 MFMA tiles of 32 x 32, i.e.
// 256 fp32 accumulators per lane -- the whole accumulator file at one wavefront
// per SIMD.  K advances in slabs of 128 BYTES per row (64 bf16/f16 or 128 fp8
// elements), double-buffered in 128 KiB of LDS.
//
// Problems whose 256 x 256 tiles would fill at most a quarter of the compute units
// (small batches: a decode step, a short prefill) go to gemm_small_kernel instead:
// 64 x 64 tiles with K split between the four wavefronts of a workgroup; its
// description sits with its code below.  Grids in between that would leave much
// of a round empty run as 128 x 256 tiles throughout (half_height_wins).
//
// Two large-tile kernels share everything but the way a slab reaches LDS:
//  * gemm_dma_kernel (K a multiple of the slab): `global_load_lds_dwordx4` moves
//    memory straight into LDS, 1 KiB per wavefront instruction.  The source is
//    written in issue order: exactly one direct load and / or one LDS fragment
//    read sits in front of each MFMA, so the matrix pipe never waits for the
//    wavefront to finish issuing memory instructions.  The pipeline is rotated by
//    one k-step: the wait-and-barrier that hands slab t+1 over sits in front of
//    the LAST k-step of slab t (whose fragments are already in registers), so the
//    first fragments of slab t+1 and the loads of slab t+2 go out under that
//    step's MFMAs.  Every memory wait of the loop is explicit: the direct loads
//    are issued as inline asm, because the compiler would otherwise wait for ALL
//    loads in flight in front of every transposing read (which it cannot prove
//    disjoint from the stage being loaded), and the hand-over barrier is a bare
//    s_barrier, without the fence of __syncthreads().  Nothing prefetches into
//    L2 beyond that: 4-byte "touch" loads one to four slabs ahead, from one
//    tile per group or from every tile, all measured slower than no touches
//    (8192 x 4096 x 11008 bf16: 616 / 648-659 / 593 us) -- the loop is limited
//    by memory requests in flight, and every touch is one more.
//  * gemm_staged_kernel (any K % 8 == 0): slabs pass through registers, which
//    lets the last, partial slab be zero-filled.
//
// LDS layout (K-contiguous operands): row r of a slab is 128 bytes = 8 chunks of
// 16 bytes; chunk c is stored at c ^ (r & 7) ^ ((r >> 3) & 1), which makes the
// 16-byte fragment reads of 16 consecutive rows and the row-wise writes conflict
// free.  Direct-to-LDS loads write 64 lanes x 16 bytes consecutively, so there
// the permutation is applied on the global side: the lane that lands on
// physical chunk pc of row r fetches logical chunk pc ^ swz(r).  A [K, N]
// (N-contiguous) B operand is kept [k][n] in LDS and read with the transposing
// LDS load of gfx950 (ds_read_b64_tr_b16), so no transpose pass is needed.
//
// The MFMA is issued with B's fragment as the first operand, so each lane ends
// up with 4 CONSECUTIVE output columns of one row, which makes the accumulators
// cheap to park in LDS; the epilogue (scales, bias, residual, activation,
// rounding) then runs as a short rolled loop over row-major data and stores
// 16 bytes per lane, whole 128-byte lines per row.
//
// Workgroups are dealt to the 8 XCDs round-robin by the hardware; the block id
// is remapped so that each XCD works through one contiguous, grouped run of
// tiles and its L2 sees each operand slab a few times instead of once per CU.
#pragma once
#include "xg_common.hpp"

#include <stdlib.h>

#include <type_traits>
#include <utility>

namespace xg {
namespace gemm {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) void gvoid;
typedef __attribute__((address_space(3))) void lvoid;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

constexpr int BM = 256, BN = 256;
constexpr int ROW_BYTES = 128;               // bytes of K per tile row and slab
constexpr int SLAB_BYTES = BM * ROW_BYTES;   // 32 KiB per operand per stage
constexpr int STAGE_BYTES = 2 * SLAB_BYTES;  // A slab, then B slab
constexpr int SMEM_BYTES = 2 * STAGE_BYTES;
constexpr int kThreads = 256;
constexpr int kXcds = 8;
constexpr int kGroupM = 8;

enum class BLayout { KMajor, NMajor };  // B stored [N, K] (K contiguous) or [K, N] (N contiguous)
// A stored [M, K] (K contiguous) or [K, M] (M contiguous: the left operand arrives transposed, as in a weight
// gradient dW = X^T dY).  An M-contiguous A slab is laid out and read exactly like an N-contiguous B slab --
// [64 k][256 m] in LDS, fetched with the transposing LDS read -- and is wired for 16-bit elements, N-contiguous B
// and full-height (256-row) tiles only.
enum class ALayout { KMajor, MMajor };

struct GemmParams {
  const void* A;
  const void* B;
  const void* B2;  // gated layer only: the second ("up") weight; B is then the gate weight
  void* gate_out;  // gated layer only, optional: where the two rounded projections go as well ([M, N] each, row
  void* up_out;    // stride ldc), for a backward pass that would otherwise recompute them
  const void* bias;
  const void* res;
  void* out;
  const float* a_scale;  // fp8 only
  const float* b_scale;  // fp8 only
  int M, N, K;
  int64_t lda, ldb, ldr, ldc;  // row strides in elements of A, B, the residual and the output
  int act;
  int bias_f32;
  int tiles_m, tiles_n;
  // Batched layer: grid.y entries, each a dense layer of its own on operands `*_batch` BYTES apart (0: shared by
  // every entry).  Every kernel starts with for_batch_entry(), so tiles, heuristics and limits are per entry.
  int batch;
  int64_t a_batch, b_batch, bias_batch, res_batch, out_batch;
};

// The parameters of batch entry blockIdx.y.
__device__ __forceinline__ GemmParams for_batch_entry(const GemmParams& p) {
  GemmParams q = p;
  if (p.batch > 1) {
    const int64_t z = blockIdx.y;
    q.A = reinterpret_cast<const char*>(p.A) + z * p.a_batch;
    q.B = reinterpret_cast<const char*>(p.B) + z * p.b_batch;
    if (p.bias) q.bias = reinterpret_cast<const char*>(p.bias) + z * p.bias_batch;
    if (p.res) q.res = reinterpret_cast<const char*>(p.res) + z * p.res_batch;
    q.out = reinterpret_cast<char*>(p.out) + z * p.out_batch;
  }
  return q;
}

// Compile-time loop: the body receives std::integral_constant indices, so every
// accumulator access has a constant index and the accumulators stay in registers.
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

template <typename T>
struct Elem;
template <>
struct Elem<bf16_t> {
  static constexpr int BYTES = 2;
  static constexpr int KSTEPS = 4;  // 4 x (32x32x16) per 64-element slab
};
template <>
struct Elem<f16_t> {
  static constexpr int BYTES = 2;
  static constexpr int KSTEPS = 4;
};
template <>
struct Elem<float> {
  static constexpr int BYTES = 4;
  static constexpr int KSTEPS = 4;  // a k-step is 8 elements (two 16-byte chunks): 4 x (32x32x2) per lane chunk
};
template <>
struct Elem<uint8_t> {  // OCP e4m3
  static constexpr int BYTES = 1;
  static constexpr int KSTEPS = 2;  // 2 x (32x32x64) per 128-element slab
};

// One k-step's operand fragment of a 32-row MFMA tile: 16 bytes per lane for the
// 16-bit types, 32 bytes per lane for fp8.
template <typename T>
struct Frag {
  u32x4 v;
};
template <>
struct Frag<uint8_t> {
  u32x4 lo, hi;
};

__device__ __forceinline__ f32x16 mma(const Frag<bf16_t>& a, const Frag<bf16_t>& b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a.v), __builtin_bit_cast(bf16x8, b.v), c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mma(const Frag<f16_t>& a, const Frag<f16_t>& b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a.v), __builtin_bit_cast(f16x8, b.v), c, 0, 0, 0);
}
// fp32: a lane's 16-byte chunk holds 4 consecutive k of its row; MFMA m of the four takes element m from both
// operands (lane half h supplies k slot h), so a k-step covers k = 8 ks + 4 h + m.
__device__ __forceinline__ f32x16 mma(const Frag<float>& a, const Frag<float>& b, f32x16 c) {
  // the whole vector is reinterpreted first: a bit cast of a single swizzled element (a.v.y) reads element 0
  const f32x4 x = __builtin_bit_cast(f32x4, a.v), y = __builtin_bit_cast(f32x4, b.v);
  c = __builtin_amdgcn_mfma_f32_32x32x2f32(x[0], y[0], c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_32x32x2f32(x[1], y[1], c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_32x32x2f32(x[2], y[2], c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_32x32x2f32(x[3], y[3], c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mma(const Frag<uint8_t>& a, const Frag<uint8_t>& b, f32x16 c) {
  const i32x8 x = {(int)a.lo.x, (int)a.lo.y, (int)a.lo.z, (int)a.lo.w, (int)a.hi.x, (int)a.hi.y, (int)a.hi.z, (int)a.hi.w};
  const i32x8 y = {(int)b.lo.x, (int)b.lo.y, (int)b.lo.z, (int)b.lo.w, (int)b.hi.x, (int)b.hi.y, (int)b.hi.z, (int)b.hi.w};
  // format 0 = e4m3 for both operands; scale exponents 127 = 2^0
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(x, y, c, 0, 0, 0, 127, 0, 127);
}

// 16 x 16 x 32 (16-bit types): lane = 16 q + l16 supplies row (or column) l16 and the 8 k of chunk q; the accumulator holds
// output rows 4 q .. 4 q + 3 (rows of a) at column l16 (row of b).
__device__ __forceinline__ f32x4 mma16(const Frag<bf16_t>& a, const Frag<bf16_t>& b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a.v), __builtin_bit_cast(bf16x8, b.v), c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mma16(const Frag<f16_t>& a, const Frag<f16_t>& b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a.v), __builtin_bit_cast(f16x8, b.v), c, 0, 0, 0);
}

// Workgroup barrier without the memory fence of __syncthreads(), which waits for EVERY outstanding memory
// operation.  The caller waits for what it needs with explicit s_waitcnt.
__device__ __forceinline__ void barrier_only() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// s_waitcnt as a real instruction rather than inline asm, so that the compiler's own wait insertion knows about it.
// gfx9 encoding: vmcnt = bits 3:0 and 15:14, expcnt = 6:4, lgkmcnt = 11:8; a field at its maximum does not wait.
template <int N>
__device__ __forceinline__ void wait_vm() {
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}
__device__ __forceinline__ void wait_lgkm0() { __builtin_amdgcn_s_waitcnt(0xC07F); }

__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// XCD-aware, grouped tile order.
__device__ __forceinline__ void tile_of_block(const GemmParams& p, int bid, int nb, int& tm, int& tn) {
  const int xcd = bid % kXcds, local = bid / kXcds;
  const int base = nb / kXcds, extra = nb % kXcds;
  const int tile = xcd * base + (xcd < extra ? xcd : extra) + local;
  const int per_group = kGroupM * p.tiles_n;
  const int group = tile / per_group;
  const int first_m = group * kGroupM;
  const int gsz = (p.tiles_m - first_m) < kGroupM ? (p.tiles_m - first_m) : kGroupM;
  const int in_group = tile % per_group;
  tm = first_m + in_group % gsz;
  tn = in_group / gsz;
}

// Lane coordinates shared by the fragment reads and the epilogue.
struct Lane {
  int tid, lane, wave, wm, wn, l32, half, p16, blk;
  int fsw;    // swz() of this lane's fragment row
  int tr_sw;  // granule permutation of the transposing read
  int a_row[4], b_row[4];
  // ni: 32-row A units per wave (4: 256-row tile, 2: 128-row tile)
  __device__ __forceinline__ explicit Lane(int ni = 4) {
    tid = threadIdx.x;
    lane = tid & 63;
    wave = tid >> 6;
    wm = wave >> 1;
    wn = wave & 1;
    l32 = lane & 31;
    half = lane >> 5;
    p16 = lane & 15;
    blk = (lane >> 4) & 1;
    fsw = swz(l32);
    tr_sw = (p16 >> 2) | (half << 2);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a_row[i] = (wm * ni * 32 + i * 32 + l32) * ROW_BYTES;
      b_row[i] = (wn * 128 + i * 32 + l32) * ROW_BYTES;
    }
  }
};

// Unit U (0..3: A tile row U, 4..7: B tile column U-4) of the fragments of k-step ks from the slabs at a_s / b_s.
template <typename T, BLayout BL, int U, ALayout AL = ALayout::KMajor>
__device__ __forceinline__ void read_unit(const Lane& L, const char* a_s, const char* b_s, int ks, Frag<T> (&fa)[4],
                                          Frag<T> (&fb)[4]) {
  if constexpr (Elem<T>::BYTES >= 2) {
    const int ch = ((ks * 2 + L.half) ^ L.fsw) << 4;
    if constexpr (U < 4 && AL == ALayout::MMajor) {
      // slab is [64 k][256 m]: the same transposing read as for an N-contiguous B, with this wave's row units
      const int gran = ((L.wm * 4 + U) ^ L.tr_sw) & 7;
      const int col = (gran << 6) + (L.blk << 5) + ((L.p16 & 3) << 3);
      const int row0 = ks * 16 + L.half * 8 + (L.p16 >> 2);
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(a_s + row0 * (BM * 2) + col));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(a_s + (row0 + 4) * (BM * 2) + col));
      const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
      fa[U].v = u32x4{l2.x, l2.y, h2.x, h2.y};
    } else if constexpr (U < 4) {
      fa[U].v = *reinterpret_cast<const u32x4*>(a_s + L.a_row[U] + ch);
    } else if constexpr (BL == BLayout::KMajor) {
      fb[U - 4].v = *reinterpret_cast<const u32x4*>(b_s + L.b_row[U - 4] + ch);
    } else if constexpr (Elem<T>::BYTES == 4) {
      // fp32 slab is [32 k][256 n], 1 KiB per k row, the two 128-byte halves of every 256 bytes swapped on k rows
      // with bit 2 set, so that the two lane halves (k rows 4 apart) read different banks.  Four 4-byte reads:
      // k = 8 ks + 4 half + m at column n.
      constexpr int j = U - 4;
      const int n4 = ((L.wn * 128 + j * 32 + L.l32) * 4) ^ (L.half << 7);
      const char* at = b_s + (ks * 8 + L.half * 4) * 1024 + n4;
      fb[j].v = u32x4{*reinterpret_cast<const uint32_t*>(at), *reinterpret_cast<const uint32_t*>(at + 1024),
                      *reinterpret_cast<const uint32_t*>(at + 2048), *reinterpret_cast<const uint32_t*>(at + 3072)};
    } else {
      // slab is [64 k][256 n]: a 16-lane group reads a 4(k) x 16(n) block and gets it back transposed
      constexpr int j = U - 4;
      const int gran = ((L.wn * 4 + j) ^ L.tr_sw) & 7;
      const int col = (gran << 6) + (L.blk << 5) + ((L.p16 & 3) << 3);
      const int row0 = ks * 16 + L.half * 8 + (L.p16 >> 2);
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(b_s + row0 * (BN * 2) + col));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(b_s + (row0 + 4) * (BN * 2) + col));
      const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
      fb[j].v = u32x4{l2.x, l2.y, h2.x, h2.y};
    }
  } else {
    // fp8: a k-step is 64 elements; each lane half supplies 32 consecutive bytes (2 chunks)
    const int ch0 = ((ks * 4 + L.half * 2) ^ L.fsw) << 4, ch1 = ((ks * 4 + L.half * 2 + 1) ^ L.fsw) << 4;
    if constexpr (U < 4) {
      fa[U].lo = *reinterpret_cast<const u32x4*>(a_s + L.a_row[U] + ch0);
      fa[U].hi = *reinterpret_cast<const u32x4*>(a_s + L.a_row[U] + ch1);
    } else {
      fb[U - 4].lo = *reinterpret_cast<const u32x4*>(b_s + L.b_row[U - 4] + ch0);
      fb[U - 4].hi = *reinterpret_cast<const u32x4*>(b_s + L.b_row[U - 4] + ch1);
    }
  }
}

// All fragments of k-step ks (NI A units, 4 B units).
template <typename T, BLayout BL, int NI = 4, ALayout AL = ALayout::KMajor>
__device__ __forceinline__ void read_frags(const Lane& L, const char* a_s, const char* b_s, int ks, Frag<T> (&fa)[4],
                                           Frag<T> (&fb)[4]) {
  static_for<8>([&](auto U) {
    constexpr int u = decltype(U)::value;
    if constexpr (u >= 4 || u < NI) read_unit<T, BL, u, AL>(L, a_s, b_s, ks, fa, fb);
  });
}

template <typename T, int NI = 4>
__device__ __forceinline__ void mma_step(f32x16 (&acc)[4][4], const Frag<T> (&fa)[4], const Frag<T> (&fb)[4]) {
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = mma(fb[j], fa[i], acc[i][j]);
}

// ---- epilogue -------------------------------------------------------------------------
// Runs per wavefront, in two halves of 64 output columns, through the wavefront's own 32 KiB of
// LDS (the slabs are dead by then):
//   1. park the raw fp32 accumulators of the half (16-byte stores, constant register indices);
//   2. a ROLLED loop re-reads them row-major -- 8 lanes x 8 columns cover a 64-column row
//      segment, 8 rows per pass -- applies scale, bias, residual and activation, rounds, and
//      writes 16 bytes per lane (one full 128-byte line per row).
// All the arithmetic therefore exists once, in a loop a few dozen instructions long, instead of
// 256 unrolled copies; the per-lane bias and scale values are loop invariant.
template <typename OT, int ACT>
__device__ __forceinline__ void epilogue_one_row(const GemmParams& p, const f32x4 lo, const f32x4 hi, const float (&sv)[8],
                                                 const float (&bv)[8], const OT* res_at, OT* out_at) {
  typedef OT O8 __attribute__((ext_vector_type(8)));
  float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = v[e] * sv[e] + bv[e];
  if (p.res) {
    const O8 r = *reinterpret_cast<const O8*>(res_at);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] += to_f32(r[e]);
  }
  O8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float t = v[e];
    if constexpr (ACT == XG_ACT_RELU) t = fmaxf(t, 0.f);
    if constexpr (ACT == XG_ACT_GELU) t = 0.5f * t * (1.f + erff(t * 0.70710678118654752f));
    if constexpr (ACT == XG_ACT_SILU) t = silu_f32(t);
    if constexpr (ACT == XG_ACT_SIGMOID) t = sigmoid_f32(t);
    o[e] = from_f32<OT>(t);
  }
  store_vec_nt(reinterpret_cast<O8*>(out_at), o);  // written once, read by another kernel
}

template <typename OT, int ACT>
__device__ __forceinline__ void epilogue_rows(const GemmParams& p, const char* park, int lane, int m_base, int n, bool n_ok,
                                              const float (&sv)[8], const float (&bv)[8], int passes) {
  const int c = lane & 7, rr = lane >> 3;
  // Pass `it` handles row it * 8 + rr, whose chunk permutation (row & 15) alternates between rr and rr | 8: the LDS
  // addresses of an even and of an odd pass are formed once and only advanced, and the output / residual pointers
  // step by eight rows -- the loop then holds the arithmetic and little else (it is issue-bound: one wave per SIMD).
  const char* pk = park + rr * 256;
  const int lo_e = ((2 * c) ^ rr) << 4, hi_e = ((2 * c + 1) ^ rr) << 4, lo_o = lo_e ^ 128, hi_o = hi_e ^ 128;
  OT* out_at = reinterpret_cast<OT*>(p.out) + (int64_t)(m_base + rr) * p.ldc + n;
  const OT* res_at = p.res ? reinterpret_cast<const OT*>(p.res) + (int64_t)(m_base + rr) * p.ldr + n : nullptr;
  const int64_t out_step = 8 * p.ldc, res_step = 8 * p.ldr;
  // whole wave inside the matrix (uniform): no per-lane predicates
  const bool inside = __builtin_amdgcn_ballot_w64(!n_ok) == 0 && m_base + passes * 8 <= p.M;
  if (inside && (passes & 1) == 0) {
    for (int it = 0; it < passes; it += 2) {
      const f32x4 lo0 = *reinterpret_cast<const f32x4*>(pk + lo_e), hi0 = *reinterpret_cast<const f32x4*>(pk + hi_e);
      const f32x4 lo1 = *reinterpret_cast<const f32x4*>(pk + 2048 + lo_o), hi1 = *reinterpret_cast<const f32x4*>(pk + 2048 + hi_o);
      epilogue_one_row<OT, ACT>(p, lo0, hi0, sv, bv, res_at, out_at);
      epilogue_one_row<OT, ACT>(p, lo1, hi1, sv, bv, res_at + res_step, out_at + out_step);
      pk += 4096;
      out_at += 2 * out_step;
      res_at += 2 * res_step;
    }
    return;
  }
  for (int it = 0; it < passes; ++it) {
    const bool odd = it & 1;
    const f32x4 lo = *reinterpret_cast<const f32x4*>(pk + (odd ? lo_o : lo_e)), hi = *reinterpret_cast<const f32x4*>(pk + (odd ? hi_o : hi_e));
    if (n_ok && m_base + it * 8 + rr < p.M) epilogue_one_row<OT, ACT>(p, lo, hi, sv, bv, res_at, out_at);
    pk += 2048;
    out_at += out_step;
    res_at += res_step;
  }
}

// Scale and bias of 8 consecutive output columns starting at n (loop invariant over the rows of a tile).
template <typename OT>
__device__ __forceinline__ void column_terms(const GemmParams& p, int n, bool n_ok, float a_sc, float (&sv)[8], float (&bv)[8]) {
  typedef OT O8 __attribute__((ext_vector_type(8)));
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    sv[e] = a_sc;
    bv[e] = 0.f;
  }
  if (n_ok && p.b_scale) {
#pragma unroll
    for (int e = 0; e < 8; ++e) sv[e] = a_sc * p.b_scale[n + e];
  }
  if (n_ok && p.bias) {
    if (p.bias_f32) {
#pragma unroll
      for (int e = 0; e < 8; ++e) bv[e] = reinterpret_cast<const float*>(p.bias)[n + e];
    } else {
      const O8 t = *reinterpret_cast<const O8*>(reinterpret_cast<const OT*>(p.bias) + n);
#pragma unroll
      for (int e = 0; e < 8; ++e) bv[e] = to_f32(t[e]);
    }
  }
}

// epilogue_rows with the (uniform) activation of the call: each case is the same short loop with one activation inlined.
template <typename OT>
__device__ __forceinline__ void epilogue_rows_act(const GemmParams& p, const char* park, int lane, int m_base, int n, bool n_ok,
                                                  const float (&sv)[8], const float (&bv)[8], int passes) {
  switch (p.act) {
    case XG_ACT_RELU:
      epilogue_rows<OT, XG_ACT_RELU>(p, park, lane, m_base, n, n_ok, sv, bv, passes);
      break;
    case XG_ACT_GELU:
      epilogue_rows<OT, XG_ACT_GELU>(p, park, lane, m_base, n, n_ok, sv, bv, passes);
      break;
    case XG_ACT_SILU:
      epilogue_rows<OT, XG_ACT_SILU>(p, park, lane, m_base, n, n_ok, sv, bv, passes);
      break;
    case XG_ACT_SIGMOID:
      epilogue_rows<OT, XG_ACT_SIGMOID>(p, park, lane, m_base, n, n_ok, sv, bv, passes);
      break;
    default:
      epilogue_rows<OT, XG_ACT_NONE>(p, park, lane, m_base, n, n_ok, sv, bv, passes);
      break;
  }
}

template <typename OT, int NI = 4>
__device__ __forceinline__ void epilogue(const GemmParams& p, const Lane& L, f32x16 (&acc)[4][4], char* smem, int m0,
                                         int n0) {
  char* park = smem + L.wave * (128 * 64 * 4);
  const float a_sc = p.a_scale ? *p.a_scale : 1.f;
  const int m_base = m0 + L.wm * (NI * 32);
  static_for<2>([&](auto H) {
    constexpr int h = decltype(H)::value;
    // 1. park: row = i*32 + l32, 16-byte chunk = jj*8 + g*2 + half, xor-ed with the row to spread the banks
    static_for<2>([&](auto JJ) {
      static_for<4>([&](auto G) {
        static_for<NI>([&](auto I) {
          constexpr int jj = decltype(JJ)::value, g = decltype(G)::value, i = decltype(I)::value;
          const int row = i * 32 + L.l32;
          const int chunk = (jj * 8 + g * 2 + L.half) ^ (row & 15);
          const f32x16& a = acc[i][h * 2 + jj];
          *reinterpret_cast<f32x4*>(park + row * 256 + (chunk << 4)) = f32x4{a[4 * g], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
        });
      });
    });
    // 2. this lane's 8 columns of the half, and their scale / bias
    const int n = n0 + L.wn * 128 + h * 64 + (L.lane & 7) * 8;
    const bool n_ok = n < p.N;  // N % 8 == 0: the 8 columns are in or out together
    float sv[8], bv[8];
    column_terms<OT>(p, n, n_ok, a_sc, sv, bv);
    // The bias and scale loads are waited for HERE.  Left pending into the row loop, the compiler's wait (it counts
    // loads and stores with one counter) would sit inside the loop and also wait, in every pass, for the previous
    // pass's output store to be acknowledged by memory.
    wait_vm<0>();
    epilogue_rows_act<OT>(p, park, L.lane, m_base, n, n_ok, sv, bv, NI * 4);
  });
}

// Gated layer: waves (wm, 0) hold the gate and waves (wm, 1) the up projection of the same NI*32 rows x 128
// columns.  Per half of 64 columns: all waves park (as above), a barrier, then each wave of the pair combines HALF of
// the rows -- silu(gate) * up, one rounding, 16-byte stores -- reading the gate from its partner's or its own park.
template <typename OT, int NI>
__device__ __forceinline__ void epilogue_glu(const GemmParams& p, const Lane& L, f32x16 (&acc)[4][4], char* smem, int m0,
                                             int n0) {
  typedef OT O8 __attribute__((ext_vector_type(8)));
  constexpr int PARK = 128 * 64 * 4;
  char* park = smem + L.wave * PARK;
  const char* gate = smem + (L.wm * 2) * PARK;
  const char* up = smem + (L.wm * 2 + 1) * PARK;
  const int m_base = m0 + L.wm * (NI * 32);
  const int c = L.lane & 7, rr = L.lane >> 3;
  static_for<2>([&](auto H) {
    constexpr int h = decltype(H)::value;
    static_for<2>([&](auto JJ) {
      static_for<4>([&](auto G) {
        static_for<NI>([&](auto I) {
          constexpr int jj = decltype(JJ)::value, g = decltype(G)::value, i = decltype(I)::value;
          const int row = i * 32 + L.l32;
          const int chunk = (jj * 8 + g * 2 + L.half) ^ (row & 15);
          const f32x16& a = acc[i][h * 2 + jj];
          *reinterpret_cast<f32x4*>(park + row * 256 + (chunk << 4)) = f32x4{a[4 * g], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
        });
      });
    });
    __syncthreads();  // both parks of the pair are complete
    const int n = n0 + h * 64 + c * 8;
    const bool n_ok = n < p.N;  // N % 8 == 0: the 8 columns are in or out together
    // One row of the pair's result: each projection is rounded to the storage type first, as the two separate
    // layers would do.
    auto one_row = [&](const f32x4 g0, const f32x4 g1, const f32x4 u0, const f32x4 u1, int64_t at) {
      const float gv[8] = {g0[0], g0[1], g0[2], g0[3], g1[0], g1[1], g1[2], g1[3]};
      const float uv[8] = {u0[0], u0[1], u0[2], u0[3], u1[0], u1[1], u1[2], u1[3]};
      O8 o, go, uo;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const OT g16 = from_f32<OT>(gv[e]), u16 = from_f32<OT>(uv[e]);
        const float gr = to_f32(g16), ur = to_f32(u16);
        o[e] = from_f32<OT>(silu_f32(gr) * ur);
        go[e] = g16;
        uo[e] = u16;
      }
      store_vec_nt(reinterpret_cast<O8*>(reinterpret_cast<OT*>(p.out) + at), o);  // written once, read by another kernel
      if (p.gate_out != nullptr) {
        store_vec_nt(reinterpret_cast<O8*>(reinterpret_cast<OT*>(p.gate_out) + at), go);
        store_vec_nt(reinterpret_cast<O8*>(reinterpret_cast<OT*>(p.up_out) + at), uo);
      }
    };
    // Pass `it` handles row r0 + it * 8, whose chunk permutation (row & 15) alternates between rr and rr | 8: the
    // LDS offsets of an even and of an odd pass are formed once and advanced, as is the output offset.
    const int r0 = L.wn * (NI * 16) + rr;
    int off = r0 * 256;
    const int lo_e = ((2 * c) ^ rr) << 4, hi_e = ((2 * c + 1) ^ rr) << 4, lo_o = lo_e ^ 128, hi_o = hi_e ^ 128;
    int64_t at = (int64_t)(m_base + r0) * p.ldc + n;
    const int64_t step = 8 * p.ldc;
    const bool inside = __builtin_amdgcn_ballot_w64(!n_ok) == 0 && m_base + L.wn * (NI * 16) + NI * 16 <= p.M;  // uniform
    if (inside) {
      for (int it = 0; it < NI * 2; it += 2) {
        const f32x4 g0 = *reinterpret_cast<const f32x4*>(gate + off + lo_e), g1 = *reinterpret_cast<const f32x4*>(gate + off + hi_e);
        const f32x4 u0 = *reinterpret_cast<const f32x4*>(up + off + lo_e), u1 = *reinterpret_cast<const f32x4*>(up + off + hi_e);
        const f32x4 g2 = *reinterpret_cast<const f32x4*>(gate + off + 2048 + lo_o), g3 = *reinterpret_cast<const f32x4*>(gate + off + 2048 + hi_o);
        const f32x4 u2 = *reinterpret_cast<const f32x4*>(up + off + 2048 + lo_o), u3 = *reinterpret_cast<const f32x4*>(up + off + 2048 + hi_o);
        one_row(g0, g1, u0, u1, at);
        one_row(g2, g3, u2, u3, at + step);
        off += 4096;
        at += 2 * step;
      }
    } else {
      for (int it = 0; it < NI * 2; ++it) {
        const bool odd = it & 1;
        const int o0 = off + (odd ? lo_o : lo_e), o1 = off + (odd ? hi_o : hi_e);
        const f32x4 g0 = *reinterpret_cast<const f32x4*>(gate + o0), g1 = *reinterpret_cast<const f32x4*>(gate + o1);
        const f32x4 u0 = *reinterpret_cast<const f32x4*>(up + o0), u1 = *reinterpret_cast<const f32x4*>(up + o1);
        if (n_ok && m_base + r0 + it * 8 < p.M) one_row(g0, g1, u0, u1, at);
        off += 2048;
        at += step;
      }
    }
    __syncthreads();  // the parks are free for the next half
  });
}

__device__ __forceinline__ void zero_acc(f32x16 (&acc)[4][4]) {
  const f32x16 zero = {};
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = zero;
}

// ---- kernel 1: direct global -> LDS ------------------------------------------------------
// T: operand element type (bf16_t, f16_t, or uint8_t for OCP e4m3); OT: output / bias / residual type.
// NI: 32-row A units per wave: 4 = 256 x 256 tile, 2 = 128 x 256 tile (used for the last, partial round of tiles).
// bid / nb: this workgroup's index among the nb workgroups that share the tile grid of p.
// GLU (gated layer, K-contiguous weights only): the 256 B rows of a tile are 128 rows of the gate weight followed by
// the same 128 rows of the up weight, so waves with wn = 0 accumulate x Wg^T and waves with wn = 1 accumulate
// x Wu^T for the SAME 128 output columns; the epilogue writes silu(gate) * up.  A slabs are shared, so the
// operand traffic per output element is that of two separate layers minus one read of x.
template <typename T, typename OT, BLayout BL, int NI, bool GLU = false, ALayout AL = ALayout::KMajor>
__device__ __forceinline__ void gemm_dma_tile(const GemmParams& p, int bid, int nb, char* smem) {
  static_assert(!GLU || BL == BLayout::KMajor, "the gated layer is wired for K-contiguous weights");
  static_assert(AL == ALayout::KMajor || (BL == BLayout::NMajor && NI == 4 && !GLU), "M-contiguous A: N-contiguous B, full tiles");
  constexpr int EB = Elem<T>::BYTES;
  constexpr int KSTEPS = Elem<T>::KSTEPS;
  constexpr int SLAB_K = ROW_BYTES / EB;
  static_assert(BL == BLayout::KMajor || EB >= 2, "N-contiguous weights: 16-bit (transposing LDS read) or fp32 (4-byte reads)");
  static_assert(AL == ALayout::KMajor || EB == 2, "M-contiguous A is wired for 16-bit elements only");

  int tm, tn;
  tile_of_block(p, bid, nb, tm, tn);
  const int m0 = tm * (NI * 64), n0 = tn * (GLU ? BN / 2 : BN);
  const Lane L(NI);

  // Per-lane byte offsets of the 8 + 8 direct loads of a slab, relative to the slab's
  // (uniform) base address; the host guarantees they fit in 31 bits.
  uint32_t a_off[8], b_off[8];
  {
    const int lrow = L.lane >> 3;
    const int lc = (L.lane & 7) ^ lrow ^ (L.wave & 1);  // logical chunk this lane fetches (see header)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int r = j * 32 + L.wave * 8 + lrow;
      if constexpr (AL == ALayout::KMajor) {
        int gr = m0 + r;
        gr = gr < p.M ? gr : p.M - 1;  // rows past the edge re-read the last row; their results are never stored
        a_off[j] = (uint32_t)(((int64_t)gr * p.lda) * EB + lc * 16);
      } else {
        const int kr = j * 8 + L.wave * 2 + L.half;
        const int pc32 = L.lane & 31;
        const int sw = ((L.wave * 2 + L.half) & 3) | ((j & 1) << 2);
        const int gran = ((pc32 >> 2) ^ sw) & 7;
        int gc = m0 + (gran * 4 + (pc32 & 3)) * 8;
        gc = gc < p.M ? gc : (p.M - 8);  // M % 8 == 0 is checked on the host
        a_off[j] = (uint32_t)(((int64_t)kr * p.lda + gc) * EB);
      }
      if constexpr (BL == BLayout::KMajor) {
        int gn = n0 + (GLU ? (r & 127) : r);  // gated: tile rows 128..255 are rows 0..127 again, of the up weight
        gn = gn < p.N ? gn : p.N - 1;
        b_off[j] = (uint32_t)(((int64_t)gn * p.ldb) * EB + lc * 16);
      } else if constexpr (EB == 4) {
        // load j of this wave fills k row 4 j + wave (1 KiB); lane i lands at chunk i, which holds column chunk
        // i ^ 8 on k rows with bit 2 set (see read_unit)
        const int kr = j * 4 + L.wave;
        int gc = n0 + ((L.lane ^ (((kr >> 2) & 1) << 3)) << 2);
        gc = gc < p.N ? gc : (p.N - 4);  // N % 8 == 0 is checked on the host
        b_off[j] = (uint32_t)(((int64_t)kr * p.ldb + gc) * EB);
      } else {
        const int kr = j * 8 + L.wave * 2 + L.half;
        const int pc32 = L.lane & 31;
        const int sw = ((L.wave * 2 + L.half) & 3) | ((j & 1) << 2);
        const int gran = ((pc32 >> 2) ^ sw) & 7;
        int gc = n0 + (gran * 4 + (pc32 & 3)) * 8;
        gc = gc < p.N ? gc : (p.N - 8);  // N % 8 == 0 is checked on the host
        b_off[j] = (uint32_t)(((int64_t)kr * p.ldb + gc) * EB);
      }
    }
  }
  const int64_t a_step = AL == ALayout::KMajor ? (int64_t)ROW_BYTES : (int64_t)SLAB_K * p.lda * EB;
  const int64_t b_step = BL == BLayout::KMajor ? (int64_t)ROW_BYTES : (int64_t)SLAB_K * p.ldb * EB;
  const int wave_u = __builtin_amdgcn_readfirstlane(L.wave);  // LDS destinations of direct loads are wavefront-uniform
  const char* const a_base = reinterpret_cast<const char*>(p.A);
  const char* const b_base = reinterpret_cast<const char*>(p.B);
  const char* const b2_base = reinterpret_cast<const char*>(GLU ? p.B2 : p.B);

  // load number Q (0..15) of slab kt into `stage`: uniform slab base + 32-bit lane offset
  auto issue = [&](auto Q, int kt, int stage) {
    constexpr int q = decltype(Q)::value;
    if constexpr (q < 8 && q >= 2 * NI) return;  // a 128-row tile has only 4 A loads per wave
    char* dst = smem + stage * STAGE_BYTES + wave_u * 1024 + (q & 7) * 4096 + (q < 8 ? 0 : SLAB_BYTES);
    const uint32_t off = q < 8 ? a_off[q & 7] : b_off[q & 7];
    // B loads 8..11 fill tile rows 0..127, loads 12..15 rows 128..255 (the up weight of a gated layer)
    const char* base = q < 8 ? a_base + kt * a_step : ((GLU && q >= 12) ? b2_base : b_base) + kt * b_step;
    load_to_lds16(base, off, (uint32_t)(size_t)(lvoid*)dst);
  };

  f32x16 acc[4][4];
  zero_acc(acc);
  Frag<T> fa[2][4], fb[2][4];
  static_assert(KSTEPS % 2 == 0, "the fragment double buffer assumes that a slab starts in buffer 0");

  const int KT = p.K / SLAB_K;
  // Issue plan of the 16 direct loads of a slab.  The instruction stream of a wave is in order and the CU's
  // address unit moves 64 bytes per clock, so a direct load holds up the MFMAs behind it for a few clocks; the
  // loads are spread out, one in front of every second MFMA: the first half in the last k-step of slab t-2
  // (right after the barrier that frees the stage), the rest in the first k-step of slab t-1, so that at least
  // one k-step of math (16-bit types) separates the last load from the barrier that needs it.
  struct Plan {
    int early[16];  // load to issue in front of MFMA idx of the LAST k-step (of slab t-2), or -1
    int late[16];   // same for k-step 0 (of slab t-1)
    int n_early;
  };
  constexpr Plan plan = []() constexpr {
    Plan P{};
    for (int i = 0; i < 16; ++i) P.early[i] = P.late[i] = -1;
    int q = 0;
    for (int i = 0; i < 16; i += 2) P.early[i] = q++;
    for (int i = 0; i < 16; i += 2) P.late[i] = q++;
    P.n_early = 8;
    return P;
  }();
  static_assert(KSTEPS >= 2, "the late loads need a k-step that is not the last");
  static_for<16>([&](auto Q) { issue(Q, 0, 0); });
  if (KT > 1) {
    static_for<plan.n_early>([&](auto Q) { issue(Q, 1, 1); });
    // slab 0 has landed when only the early loads of slab 1 (the A loads that exist for this tile height) are in flight
    static_assert(plan.n_early == 8, "the waits below count the early loads of slab 1");
    if constexpr (NI == 4) {
      wait_vm<8>();
    } else {
      wait_vm<4>();
    }
  } else {
    wait_vm<0>();
  }
  barrier_only();
  read_frags<T, BL, NI, AL>(L, smem, smem + SLAB_BYTES, 0, fa[0], fb[0]);

  // One slab of math, written in issue order.  NEXT: slab kt+1 exists (hand it over in front of the last
  // k-step and fetch its first fragments under that step); NEXT2: slab kt+2 exists (its direct loads go
  // into this slab's stage, which is free once every wavefront is past the barrier).
  auto slab = [&](auto NEXT, auto NEXT2, int kt) {
    constexpr bool next = decltype(NEXT)::value, next2 = decltype(NEXT2)::value;
    const int stage = kt & 1;
    const char* a_s = smem + stage * STAGE_BYTES;
    const char* b_s = a_s + SLAB_BYTES;
    const char* a_n = smem + (stage ^ 1) * STAGE_BYTES;
    const char* b_n = a_n + SLAB_BYTES;
    static_for<KSTEPS>([&](auto KS) {
      constexpr int ks = decltype(KS)::value;
      constexpr bool last_step = ks + 1 == KSTEPS;
      // the transposing reads are not tracked by the compiler: this step's fragments, read under the previous
      // step, are in registers once the LDS queue is empty (it has had at least eight MFMAs to drain)
      if constexpr (last_step && next) {
        // This step's fragments are in registers, so nothing of slab kt is read from LDS any more, and
        // every direct load of slab kt+1 must have landed.
        wait_lgkm0();
        wait_vm<0>();
        barrier_only();
      }
      static_for<16>([&](auto IDX) {
        constexpr int idx = decltype(IDX)::value;
        constexpr int i = idx / 4, j = idx % 4;
        if constexpr (idx < 8 && (idx >= 4 || idx < NI)) {  // units 0..3 are A tile rows: a 128-row tile has two
          if constexpr (!last_step) read_unit<T, BL, idx, AL>(L, a_s, b_s, ks + 1, fa[(ks + 1) & 1], fb[(ks + 1) & 1]);
          else if constexpr (next) read_unit<T, BL, idx, AL>(L, a_n, b_n, 0, fa[0], fb[0]);
        }
        // direct loads: the rest of slab kt+1 early in this slab, the head of slab kt+2 after the barrier
        if constexpr (next && ks == 0 && !last_step) {
          constexpr int q = plan.late[idx];
          if constexpr (q >= 0) issue(std::integral_constant<int, (q >= 0 ? q : 0)>{}, kt + 1, stage ^ 1);
        }
        if constexpr (next2 && last_step) {
          constexpr int q = plan.early[idx];
          if constexpr (q >= 0) issue(std::integral_constant<int, (q >= 0 ? q : 0)>{}, kt + 2, stage);
        }
        if constexpr (i < NI) acc[i][j] = mma(fb[ks & 1][j], fa[ks & 1][i], acc[i][j]);
        __builtin_amdgcn_sched_barrier(0);  // keep the issue order of the source
      });
    });
  };

  for (int kt = 0; kt + 2 < KT; ++kt) slab(std::true_type{}, std::true_type{}, kt);
  if (KT > 1) slab(std::true_type{}, std::false_type{}, KT - 2);
  slab(std::false_type{}, std::false_type{}, KT - 1);
  __syncthreads();  // the slabs are dead: the epilogue reuses LDS

  if constexpr (GLU) epilogue_glu<OT, NI>(p, L, acc, smem, m0, n0);
  else epilogue<OT, NI>(p, L, acc, smem, m0, n0);
}

template <typename T, typename OT, BLayout BL, ALayout AL = ALayout::KMajor>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_dma_kernel(GemmParams p) {
  extern __shared__ __align__(16) char smem[];
  gemm_dma_tile<T, OT, BL, 4, false, AL>(for_batch_entry(p), blockIdx.x, gridDim.x, smem);
}

// One launch for two tile grids: the first n_full workgroups compute the 256 x 256 tiles of `full`, the others the
// 128 x 256 tiles of `rest` (the tile columns past the last full round), which start as soon as compute units free up.
template <typename T, typename OT, BLayout BL>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_dma_split_kernel(GemmParams full, GemmParams rest,
                                                                                                                    int n_full) {
  extern __shared__ __align__(16) char smem[];
  const int bid = blockIdx.x;  // uniform
  if (bid < n_full) {
    gemm_dma_tile<T, OT, BL, 4>(for_batch_entry(full), bid, n_full, smem);
  } else {
    gemm_dma_tile<T, OT, BL, 2>(for_batch_entry(rest), bid - n_full, (int)gridDim.x - n_full, smem);
  }
}

// Every tile half height: for grids whose full-size tiles would leave a large part of a round empty.
template <typename T, typename OT, BLayout BL>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_dma_half_kernel(GemmParams p) {
  extern __shared__ __align__(16) char smem[];
  gemm_dma_tile<T, OT, BL, 2>(for_batch_entry(p), blockIdx.x, gridDim.x, smem);
}

// The gated layer: same launch shapes as above.
template <typename T, typename OT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_glu_kernel(GemmParams p) {
  extern __shared__ __align__(16) char smem[];
  gemm_dma_tile<T, OT, BLayout::KMajor, 4, true>(p, blockIdx.x, gridDim.x, smem);
}

template <typename T, typename OT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_glu_split_kernel(GemmParams full, GemmParams rest,
                                                                                                               int n_full) {
  extern __shared__ __align__(16) char smem[];
  const int bid = blockIdx.x;  // uniform
  if (bid < n_full) {
    gemm_dma_tile<T, OT, BLayout::KMajor, 4, true>(full, bid, n_full, smem);
  } else {
    gemm_dma_tile<T, OT, BLayout::KMajor, 2, true>(rest, bid - n_full, (int)gridDim.x - n_full, smem);
  }
}

// ---- kernel 2: slabs staged through registers (any K) --------------------------------------
template <typename T, typename OT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_glu_half_kernel(GemmParams p) {
  extern __shared__ __align__(16) char smem[];
  gemm_dma_tile<T, OT, BLayout::KMajor, 2, true>(p, blockIdx.x, gridDim.x, smem);
}

template <typename T, typename OT, BLayout BL, ALayout AL = ALayout::KMajor>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_staged_kernel(GemmParams p_all) {
  extern __shared__ __align__(16) char smem[];
  const GemmParams p = for_batch_entry(p_all);
  constexpr int EB = Elem<T>::BYTES;
  constexpr int KSTEPS = Elem<T>::KSTEPS;
  constexpr int SLAB_K = ROW_BYTES / EB;
  static_assert(BL == BLayout::KMajor || EB >= 2, "N-contiguous weights: 16-bit or fp32");
  static_assert(AL == ALayout::KMajor || (BL == BLayout::NMajor && EB == 2), "M-contiguous A goes with N-contiguous B, 16-bit");

  int tm, tn;
  tile_of_block(p, blockIdx.x, gridDim.x, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const Lane L;
  const int tid = L.tid;

  // K-major operand: thread covers chunk c8 of rows r0 + 32 j (8 threads = one 128-byte row).
  const int c8 = tid & 7, r0 = tid >> 3;
  const char* a_ptr[8];
  const char* b_ptr[8];
  int a_lds[8], b_lds[8];
  if constexpr (AL == ALayout::KMajor) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int r = r0 + 32 * j;
      int gr = m0 + r;
      gr = gr < p.M ? gr : p.M - 1;
      a_ptr[j] = reinterpret_cast<const char*>(p.A) + ((int64_t)gr * p.lda) * EB + c8 * 16;
      a_lds[j] = r * ROW_BYTES + ((c8 ^ swz(r)) << 4);
    }
  } else {
    // M-major operand: slab is [64 k][256 m], covered like the N-major B slab below
    const int c32 = tid & 31, kr0 = tid >> 5;
    int gc = m0 + c32 * 8;
    gc = gc < p.M ? gc : (p.M - 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int kr = kr0 + 8 * j;
      a_ptr[j] = reinterpret_cast<const char*>(p.A) + ((int64_t)kr * p.lda + gc) * EB;
      const int sw = (kr & 3) | (((kr >> 3) & 1) << 2);
      a_lds[j] = kr * (BM * EB) + ((((c32 >> 2) ^ sw) & 7) << 6) + ((c32 & 3) << 4);
    }
  }
  if constexpr (BL == BLayout::KMajor) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int r = r0 + 32 * j;
      int gr = n0 + r;
      gr = gr < p.N ? gr : p.N - 1;
      b_ptr[j] = reinterpret_cast<const char*>(p.B) + ((int64_t)gr * p.ldb) * EB + c8 * 16;
      b_lds[j] = r * ROW_BYTES + ((c8 ^ swz(r)) << 4);
    }
  } else if constexpr (EB == 4) {
    // fp32 N-major operand: slab is [32 k][256 n]; thread covers 16-byte chunk c64 (4 columns) of k rows kr0 + 4 j.
    const int c64 = tid & 63, kr0 = tid >> 6;
    int gc = n0 + c64 * 4;
    gc = gc < p.N ? gc : (p.N - 4);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int kr = kr0 + 4 * j;
      b_ptr[j] = reinterpret_cast<const char*>(p.B) + ((int64_t)kr * p.ldb + gc) * EB;
      b_lds[j] = kr * 1024 + ((c64 ^ (((kr >> 2) & 1) << 3)) << 4);
    }
  } else {
    // N-major operand: slab is [64 k][256 n]; thread covers 16-byte chunk c32 (8 columns) of k rows kr0 + 8 j.
    const int c32 = tid & 31, kr0 = tid >> 5;
    int gc = n0 + c32 * 8;
    gc = gc < p.N ? gc : (p.N - 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int kr = kr0 + 8 * j;
      b_ptr[j] = reinterpret_cast<const char*>(p.B) + ((int64_t)kr * p.ldb + gc) * EB;
      const int sw = (kr & 3) | (((kr >> 3) & 1) << 2);
      b_lds[j] = kr * (BN * EB) + ((((c32 >> 2) ^ sw) & 7) << 6) + ((c32 & 3) << 4);
    }
  }

  u32x4 ga[8], gb[8];
  auto load_slab = [&](int kt) {
    const int k_left = p.K - kt * SLAB_K;  // elements of K still valid from this slab's start
    const int64_t koff = AL == ALayout::KMajor ? (int64_t)kt * ROW_BYTES : (int64_t)kt * SLAB_K * p.lda * EB;
    const int64_t boff = BL == BLayout::KMajor ? koff : (int64_t)kt * SLAB_K * p.ldb * EB;
    if (k_left >= SLAB_K) {  // uniform: a whole slab, no per-load predicate
#pragma unroll
      for (int j = 0; j < 8; ++j) ga[j] = *reinterpret_cast<const u32x4*>(a_ptr[j] + koff);
#pragma unroll
      for (int j = 0; j < 8; ++j) gb[j] = *reinterpret_cast<const u32x4*>(b_ptr[j] + boff);
    } else {  // the last, partial slab: chunks past K read as zero
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const bool ok = AL == ALayout::KMajor ? (c8 * (16 / EB) < k_left) : ((tid >> 5) + 8 * j < k_left);
        ga[j] = ok ? *reinterpret_cast<const u32x4*>(a_ptr[j] + koff) : u32x4{0, 0, 0, 0};
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const bool ok = BL == BLayout::KMajor ? (c8 * (16 / EB) < k_left) : (EB == 4 ? (tid >> 6) + 4 * j < k_left : (tid >> 5) + 8 * j < k_left);
        gb[j] = ok ? *reinterpret_cast<const u32x4*>(b_ptr[j] + boff) : u32x4{0, 0, 0, 0};
      }
    }
  };
  auto store_slab = [&](int stage) {
#pragma unroll
    for (int j = 0; j < 8; ++j) *reinterpret_cast<u32x4*>(smem + stage * STAGE_BYTES + a_lds[j]) = ga[j];
#pragma unroll
    for (int j = 0; j < 8; ++j) *reinterpret_cast<u32x4*>(smem + stage * STAGE_BYTES + SLAB_BYTES + b_lds[j]) = gb[j];
  };

  f32x16 acc[4][4];
  zero_acc(acc);

  const int KT = (p.K + SLAB_K - 1) / SLAB_K;
  load_slab(0);
  store_slab(0);
  __syncthreads();
  if (KT > 1) load_slab(1);

  for (int kt = 0; kt < KT; ++kt) {
    const int stage = kt & 1;
    const char* a_s = smem + stage * STAGE_BYTES;
    const char* b_s = a_s + SLAB_BYTES;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      Frag<T> fa[4], fb[4];
      read_frags<T, BL, 4, AL>(L, a_s, b_s, ks, fa, fb);
      mma_step<T>(acc, fa, fb);
      if (ks == 0 && kt + 1 < KT) store_slab(stage ^ 1);  // slab kt+1: registers -> the idle LDS stage
      if (ks == 1 && kt + 2 < KT) load_slab(kt + 2);      // slab kt+2: memory -> registers
    }
    __syncthreads();
  }

  epilogue<OT>(p, L, acc, smem, m0, n0);
}

// ---- Problems too small to fill the machine with 256 x 256 tiles -------------------------------------------
// 64 x 64 output tiles, and the four wavefronts of a workgroup split K between them: every wavefront accumulates
// the WHOLE tile over its own quarter of each 64-element slab (k-step = wavefront index: 2 + 2 fragment reads and
// 4 MFMAs per slab), and the four partial tiles are summed through LDS in the epilogue.  A 4096 x 4096 weight
// against 256 rows is then 256 workgroups instead of 16, and the per-workgroup work is short enough that two
// workgroups share a compute unit (64 KiB of LDS each).  Slabs reach LDS by direct loads, four stages deep
// (three slabs in flight per workgroup: one slab of math is far shorter than the memory latency).
// LDS layout: A, and B when K-contiguous, as in the large kernels (128-byte rows, chunk c of row r at slot
// c ^ swz(r)); an N-contiguous B slab is [64 k][64 n], 128 bytes per k row, chunk c of row k at slot
// c ^ (4 * bit 1 of k): the eight k rows a half-wavefront's transposing read touches then fall on distinct banks.
constexpr int S_TILE = 64;
constexpr int S_STAGES = 4;
constexpr int S_SLAB_BYTES = S_TILE * ROW_BYTES;  // 8 KiB per operand per stage
constexpr int S_STAGE_BYTES = 2 * S_SLAB_BYTES;
constexpr int S_SMEM_BYTES = S_STAGES * S_STAGE_BYTES;  // 64 KiB; the epilogue parks 4 x (64 x 64 fp32) in the same space
static_assert(S_SMEM_BYTES >= 4 * S_TILE * S_TILE * 4, "the four partial tiles must fit where the slabs were");

// GLU (gated layer, K-contiguous weights): the 64 B rows of a tile are 32 rows of the gate weight (p.B) followed
// by the same 32 rows of the up weight (p.B2); the output tile is 64 x 32 and p.tiles_n counts 32-column tiles.
template <typename T, typename OT, BLayout BL, bool GLU = false>
__global__ __launch_bounds__(kThreads) void gemm_small_kernel(GemmParams p_all) {
  extern __shared__ __align__(16) char smem[];
  const GemmParams p = for_batch_entry(p_all);
  constexpr int EB = Elem<T>::BYTES;
  constexpr bool F8 = EB == 1;
  static_assert(!F8 || (BL == BLayout::KMajor && !GLU), "fp8: K-contiguous weights, plain layer");
  static_assert(!GLU || BL == BLayout::KMajor, "the gated layer is wired for K-contiguous weights");
  constexpr int SLAB_K = ROW_BYTES / EB;
  // fp8 slabs have two k-steps (of 64 elements): wavefront w takes k-step w & 1 and the 32 output columns w >> 1,
  // so two partial tiles are summed instead of four.  NJ: 32-column units a wavefront accumulates.
  constexpr int NJ = F8 ? 1 : 2;
  constexpr int PARTS = F8 ? 2 : 4;

  int tm, tn;
  tile_of_block(p, blockIdx.x, gridDim.x, tm, tn);
  const int m0 = tm * S_TILE, n0 = tn * (GLU ? S_TILE / 2 : S_TILE);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, half = lane >> 5, p16 = lane & 15, blk = (lane >> 4) & 1;

  // direct loads: per slab and operand 8 wavefront loads of 1 KiB (8 rows), two per wavefront
  uint32_t a_off[2], b_off[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int r = (q * 4 + wave) * 8 + (lane >> 3);
    const int slot = lane & 7;
    int gr = m0 + r;
    gr = gr < p.M ? gr : p.M - 1;  // rows past the edge re-read the last row; their results are never stored
    a_off[q] = (uint32_t)(((int64_t)gr * p.lda) * EB + ((slot ^ swz(r)) << 4));
    if constexpr (BL == BLayout::KMajor) {
      int gn = n0 + (GLU ? (r & 31) : r);  // gated: load 0 of a wavefront fills gate rows, load 1 the same rows of up
      gn = gn < p.N ? gn : p.N - 1;
      b_off[q] = (uint32_t)(((int64_t)gn * p.ldb) * EB + ((slot ^ swz(r)) << 4));
    } else if constexpr (EB == 4) {
      // fp32 slab is [32 k][64 n], 256 bytes per k row: a 1 KiB load covers k rows 4 L .. 4 L + 3 (L = q * 4 + wave),
      // lane i lands at chunk i & 15 of row i >> 4; on the loads with odd L (k bit 2 set) the two 128-byte halves of a
      // row are swapped so that the lane halves of a fragment read (k rows 4 apart) fall on different banks
      const int load = q * 4 + wave;
      const int kr = load * 4 + (lane >> 4);
      int gc = n0 + (((lane & 15) ^ ((load & 1) << 3)) << 2);
      gc = gc < p.N ? gc : p.N - 4;  // N % 8 == 0 is checked on the host
      b_off[q] = (uint32_t)(((int64_t)kr * p.ldb + gc) * EB);
    } else {
      int gc = n0 + ((slot ^ (((r >> 1) & 1) << 2)) << 3);  // r is the k row here
      gc = gc < p.N ? gc : p.N - 8;                          // N % 8 == 0 is checked on the host
      b_off[q] = (uint32_t)(((int64_t)r * p.ldb + gc) * EB);
    }
  }
  const char* const a_base = reinterpret_cast<const char*>(p.A);
  const char* const b_base = reinterpret_cast<const char*>(p.B);
  const char* const b2_base = reinterpret_cast<const char*>(GLU ? p.B2 : p.B);
  const int64_t b_step = BL == BLayout::KMajor ? (int64_t)ROW_BYTES : (int64_t)SLAB_K * p.ldb * EB;
  auto issue = [&](int kt) {
    char* dst = smem + (kt % S_STAGES) * S_STAGE_BYTES + wave * 1024;
#pragma unroll
    for (int q = 0; q < 2; ++q) load_to_lds16(a_base + (int64_t)kt * ROW_BYTES, a_off[q], (uint32_t)(size_t)(lvoid*)(dst + q * 4096));
#pragma unroll
    for (int q = 0; q < 2; ++q)
      load_to_lds16((q == 0 ? b_base : b2_base) + kt * b_step, b_off[q], (uint32_t)(size_t)(lvoid*)(dst + S_SLAB_BYTES + q * 4096));
  };

  // fragment addresses of this wavefront's k-step inside a stage
  const int ks = F8 ? (wave & 1) : wave;
  const int jbase = F8 ? (wave >> 1) : 0;  // first 32-column unit of this wavefront
  int a_frag[2], b_frag[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int row = u * 32 + l32;
    // 16-bit: chunk 2 ks + half; fp8: chunks 4 ks + 2 half and the next one (read as frag + 16 ^ ... below)
    a_frag[u] = row * ROW_BYTES + (((F8 ? ks * 4 + half * 2 : ks * 2 + half) ^ swz(row)) << 4);
    if constexpr (F8) {
      const int brow = (jbase + u) * 32 + l32;  // only u = 0 is used
      b_frag[u] = S_SLAB_BYTES + brow * ROW_BYTES + (((ks * 4 + half * 2) ^ swz(brow)) << 4);
    } else if constexpr (BL == BLayout::KMajor) {
      b_frag[u] = S_SLAB_BYTES + a_frag[u];
    } else if constexpr (EB == 4) {
      // k = 8 ks + 4 half + m (m = 0..3: four 4-byte reads 256 bytes apart) at column 32 u + l32
      b_frag[u] = S_SLAB_BYTES + (ks * 8 + half * 4) * 256 + (((u * 32 + l32) * 4) ^ (half << 7));
    } else {
      const int kr = wave * 16 + half * 8 + (p16 >> 2);
      const int chunk = u * 4 + blk * 2 + ((p16 & 3) >> 1);
      b_frag[u] = S_SLAB_BYTES + kr * ROW_BYTES + ((chunk ^ (((kr >> 1) & 1) << 2)) << 4) + ((p16 & 1) << 3);
    }
  }

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int KT = p.K / SLAB_K;
  for (int s = 0; s < S_STAGES - 1 && s < KT; ++s) issue(s);
  for (int kt = 0; kt < KT; ++kt) {
    // slab kt has landed when only the (at most two) slabs issued after it are in flight: 4 loads each
    const int after = KT - 1 - kt;
    if (after >= 2) {
      wait_vm<8>();
    } else if (after == 1) {
      wait_vm<4>();
    } else {
      wait_vm<0>();
    }
    barrier_only();  // slab kt is visible to all, and all are done with slab kt-1 ...
    if (kt + S_STAGES - 1 < KT) issue(kt + S_STAGES - 1);  // ... whose stage takes the next slab
    const char* st = smem + (kt % S_STAGES) * S_STAGE_BYTES;
    Frag<T> fa[2], fb[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      if constexpr (F8) {
        // the second 16-byte chunk of a lane's 32 bytes is the neighbour chunk: slot ^ 1 (the xor of the layout
        // only touches the chunk index, and chunk + 1 == chunk ^ 1 for the even chunk the lane starts at)
        fa[u].lo = *reinterpret_cast<const u32x4*>(st + a_frag[u]);
        fa[u].hi = *reinterpret_cast<const u32x4*>(st + (a_frag[u] ^ 16));
        if (u < NJ) {
          fb[u].lo = *reinterpret_cast<const u32x4*>(st + b_frag[u]);
          fb[u].hi = *reinterpret_cast<const u32x4*>(st + (b_frag[u] ^ 16));
        }
      } else if constexpr (BL == BLayout::KMajor) {
        fa[u].v = *reinterpret_cast<const u32x4*>(st + a_frag[u]);
        fb[u].v = *reinterpret_cast<const u32x4*>(st + b_frag[u]);
      } else if constexpr (EB == 4) {
        fa[u].v = *reinterpret_cast<const u32x4*>(st + a_frag[u]);
        const char* at = st + b_frag[u];
        fb[u].v = u32x4{*reinterpret_cast<const uint32_t*>(at), *reinterpret_cast<const uint32_t*>(at + 256),
                        *reinterpret_cast<const uint32_t*>(at + 512), *reinterpret_cast<const uint32_t*>(at + 768)};
      } else {
        fa[u].v = *reinterpret_cast<const u32x4*>(st + a_frag[u]);
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(st + b_frag[u]));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(st + b_frag[u] + 4 * ROW_BYTES));
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        fb[u].v = u32x4{l2.x, l2.y, h2.x, h2.y};
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) acc[i][j] = mma(fb[j], fa[i], acc[i][j]);
  }
  __syncthreads();  // the slabs are dead: the partial tiles take their place

  // park this wavefront's partial tile (fp8: its 32 columns of partial tile ks): row r at r * 256, 16-byte chunk
  // (4 columns) c at slot c ^ (r & 15)
  char* park = smem + (F8 ? ks : wave) * (S_TILE * S_TILE * 4);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int row = i * 32 + l32;
        const int chunk = ((jbase + j) * 8 + g * 2 + half) ^ (row & 15);
        const f32x16& a = acc[i][j];
        *reinterpret_cast<f32x4*>(park + row * 256 + (chunk << 4)) = f32x4{a[4 * g], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
      }
  __syncthreads();
  // Sum the partial tiles (four; fp8: two) into the first one.  A thread sums exactly the (row, 8 columns) pieces it finishes
  // below -- rows wave * 16 + pass * 8 + lane / 8, columns (lane & 7) * 8 -- so no barrier is needed in between.
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int row = wave * 16 + it * 8 + (lane >> 3);
    const int c = lane & 7;
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      char* at = smem + row * 256 + (((2 * c + hh) ^ (row & 15)) << 4);
      f32x4 v = *reinterpret_cast<const f32x4*>(at);
#pragma unroll
      for (int w = 1; w < PARTS; ++w) v += *reinterpret_cast<const f32x4*>(at + w * (S_TILE * S_TILE * 4));
      *reinterpret_cast<f32x4*>(at) = v;
    }
  }
  if constexpr (!GLU) {
    const int n = n0 + (lane & 7) * 8;
    const bool n_ok = n < p.N;
    float sv[8], bv[8];
    column_terms<OT>(p, n, n_ok, p.a_scale ? *p.a_scale : 1.f, sv, bv);
    epilogue_rows_act<OT>(p, smem + wave * 16 * 256, lane, m0 + wave * 16, n, n_ok, sv, bv, 2);
  } else {
    // columns 0..31 of the summed tile are the gate, 32..63 the up projection of the same outputs: the lanes that
    // summed gate pieces combine them with the up pieces other lanes of the wavefront summed
    typedef OT O8 __attribute__((ext_vector_type(8)));
    __syncthreads();
    const int c = lane & 7;
    const int n = n0 + c * 8;
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int row = wave * 16 + it * 8 + (lane >> 3);
      const int m = m0 + row;
      if (!(c < 4 && n < p.N && m < p.M)) continue;
      const char* at = smem + row * 256;
      const f32x4 g0 = *reinterpret_cast<const f32x4*>(at + (((2 * c) ^ (row & 15)) << 4));
      const f32x4 g1 = *reinterpret_cast<const f32x4*>(at + (((2 * c + 1) ^ (row & 15)) << 4));
      const f32x4 u0 = *reinterpret_cast<const f32x4*>(at + (((8 + 2 * c) ^ (row & 15)) << 4));
      const f32x4 u1 = *reinterpret_cast<const f32x4*>(at + (((9 + 2 * c) ^ (row & 15)) << 4));
      const float gv[8] = {g0[0], g0[1], g0[2], g0[3], g1[0], g1[1], g1[2], g1[3]};
      const float uv[8] = {u0[0], u0[1], u0[2], u0[3], u1[0], u1[1], u1[2], u1[3]};
      O8 o, go, uo;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        // each projection is rounded to the storage type first, as the two separate layers would do
        const OT g16 = from_f32<OT>(gv[e]), u16 = from_f32<OT>(uv[e]);
        const float gr = to_f32(g16), ur = to_f32(u16);
        o[e] = from_f32<OT>(silu_f32(gr) * ur);
        go[e] = g16;
        uo[e] = u16;
      }
      store_vec_nt(reinterpret_cast<O8*>(reinterpret_cast<OT*>(p.out) + (int64_t)m * p.ldc + n), o);  // written once, read by another kernel
      if (p.gate_out != nullptr) {
        store_vec_nt(reinterpret_cast<O8*>(reinterpret_cast<OT*>(p.gate_out) + (int64_t)m * p.ldc + n), go);
        store_vec_nt(reinterpret_cast<O8*>(reinterpret_cast<OT*>(p.up_out) + (int64_t)m * p.ldc + n), uo);
      }
    }
  }
}

// ---- at most 32 rows: a decode step ---------------------------------------------------------------------------
// out[M <= 32, N] = A W^T with K-contiguous 16-bit W is weight streaming: every weight is used M times.  A workgroup owns 16
// output columns, i.e. 16 whole rows of W, and its four wavefronts a quarter of K each, so a wavefront walks its 16 rows
// front to back in 64-byte steps -- sequential in memory, where the 64 x 64 kernel's slabs take 128 bytes of each of 64 rows
// 2 K bytes apart.  Fragments go from global memory straight to registers in 16 x 16 x 32 MFMA layout (lane = 16 q + l16:
// row l16, k chunk q), U k-steps of loads in flight behind U k-steps of math; the four partial tiles meet in LDS.
// The accumulation order is this kernel's own, as the 64 x 64 kernel's is.
// GLU (gated layer): the workgroup walks the same 16 rows of the gate weight (p.B) and of the up weight (p.B2) against one
// set of activation fragments; each projection is summed and rounded exactly as the plain kernel does it, so the gated
// layer equals two plain layers and the gate kernel bit for bit.
template <typename T, typename OT, int MT, bool GLU = false>
__global__ __launch_bounds__(kThreads) void gemm_skinny_kernel(GemmParams p_all) {
  static_assert(Elem<T>::BYTES == 2, "16-bit operands");
  constexpr int U = (MT == 1 ? 8 : 4) / (GLU ? 2 : 1);
  constexpr int NW = GLU ? 2 : 1;  // weights walked
  __shared__ float part[4][NW][MT][16][16];
  const GemmParams p = GLU ? p_all : for_batch_entry(p_all);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, q = lane >> 4;
  const int n0 = blockIdx.x * 16;
  int n = n0 + l16;
  n = n < p.N ? n : p.N - 1;  // columns past the edge re-read the last row of W; their results are never stored
  const int kq = p.K / 4;     // K % 128 == 0 is checked on the host: every quarter is a whole number of k-steps
  const T* w_at[NW];
  w_at[0] = reinterpret_cast<const T*>(p.B) + (int64_t)n * p.ldb + wave * kq + 8 * q;
  if constexpr (GLU) w_at[1] = reinterpret_cast<const T*>(p.B2) + (int64_t)n * p.ldb + wave * kq + 8 * q;
  const T* x_at[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    int m = 16 * t + l16;
    m = m < p.M ? m : p.M - 1;
    x_at[t] = reinterpret_cast<const T*>(p.A) + (int64_t)m * p.lda + wave * kq + 8 * q;
  }
  f32x4 acc[NW][MT];
#pragma unroll
  for (int w = 0; w < NW; ++w)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[w][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  Frag<T> fw[2][NW][U], fx[2][MT][U];
  auto load = [&](int buf, int k) {  // k-steps k .. k + U - 1 of this wavefront's quarter
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int w = 0; w < NW; ++w) fw[buf][w][u].v = *reinterpret_cast<const u32x4*>(w_at[w] + (k + u) * 32);
#pragma unroll
      for (int t = 0; t < MT; ++t) fx[buf][t][u].v = *reinterpret_cast<const u32x4*>(x_at[t] + (k + u) * 32);
    }
  };
  auto math = [&](int buf) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int w = 0; w < NW; ++w) acc[w][t] = mma16(fw[buf][w][u], fx[buf][t][u], acc[w][t]);
  };
  const int steps = kq / 32, groups = steps / U;
  if (groups > 0) load(0, 0);
  for (int g = 0; g + 1 < groups; g += 2) {  // two groups per trip: the buffer indices stay compile-time
    load(1, (g + 1) * U);
    math(0);
    if (g + 2 < groups) load(0, (g + 2) * U);
    math(1);
  }
  if (groups & 1) math(0);
  for (int k = groups * U; k < steps; ++k) {  // what does not fill a group
    Frag<T> a[NW], b;
#pragma unroll
    for (int w = 0; w < NW; ++w) a[w].v = *reinterpret_cast<const u32x4*>(w_at[w] + k * 32);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      b.v = *reinterpret_cast<const u32x4*>(x_at[t] + k * 32);
#pragma unroll
      for (int w = 0; w < NW; ++w) acc[w][t] = mma16(a[w], b, acc[w][t]);
    }
  }

  // accumulator t of a lane: output rows 16 t + l16 (A rows), columns n0 + 4 q .. + 3
#pragma unroll
  for (int w = 0; w < NW; ++w)
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) part[wave][w][t][4 * q + e][l16] = acc[w][t][e];
  __syncthreads();
  for (int idx = tid; idx < MT * 256; idx += kThreads) {
    const int nl = idx & 15, ml = (idx >> 4) & 15, t = idx >> 8;
    const int m = 16 * t + ml, nn = n0 + nl;
    if (m >= p.M || nn >= p.N) continue;
    float v = (part[0][0][t][nl][ml] + part[1][0][t][nl][ml]) + (part[2][0][t][nl][ml] + part[3][0][t][nl][ml]);
    if constexpr (GLU) {
      const float u = (part[0][1][t][nl][ml] + part[1][1][t][nl][ml]) + (part[2][1][t][nl][ml] + part[3][1][t][nl][ml]);
      // each projection is rounded to the storage type first, as the two separate layers would do
      const OT g16 = from_f32<OT>(v), u16 = from_f32<OT>(u);
      float gated = silu_f32(to_f32(g16)) * to_f32(u16);
      // the product exists in fp32 before it is rounded to the storage type, as in the gate kernel: left alone, the
      // compiler folds the multiplication and the conversion to fp16 into one mixed-precision instruction that rounds once
      asm volatile("" : "+v"(gated));
      reinterpret_cast<OT*>(p.out)[(int64_t)m * p.ldc + nn] = from_f32<OT>(gated);
      if (p.gate_out != nullptr) {
        reinterpret_cast<OT*>(p.gate_out)[(int64_t)m * p.ldc + nn] = g16;
        reinterpret_cast<OT*>(p.up_out)[(int64_t)m * p.ldc + nn] = u16;
      }
      continue;
    }
    if (p.bias) v += p.bias_f32 ? reinterpret_cast<const float*>(p.bias)[nn] : to_f32(reinterpret_cast<const OT*>(p.bias)[nn]);
    if (p.res) v += to_f32(reinterpret_cast<const OT*>(p.res)[(int64_t)m * p.ldr + nn]);
    switch (p.act) {
      case XG_ACT_RELU: v = fmaxf(v, 0.f); break;
      case XG_ACT_GELU: v = 0.5f * v * (1.f + erff(v * 0.70710678118654752f)); break;
      case XG_ACT_SILU: v = silu_f32(v); break;
      case XG_ACT_SIGMOID: v = sigmoid_f32(v); break;
      default: break;
    }
    reinterpret_cast<OT*>(p.out)[(int64_t)m * p.ldc + nn] = from_f32<OT>(v);
  }
}

// The same walk for e4m3 operands (the quantised weight is always K-contiguous): a lane's 16 bytes are 16 values of k, the
// low and the high eight feed one 16 x 16 x 32 MFMA each -- which 32 values of k meet in one instruction does not matter,
// as long as the weight and the activation fragment pair the same ones -- so a wavefront advances 64 values of k per step.
// Scales, bias and activation as in the other fp8 kernels: act(sum * a_scale * b_scale[n] + bias[n]).
template <typename OT, int MT>
__global__ __launch_bounds__(kThreads) void gemm_skinny_fp8_kernel(GemmParams p) {
  constexpr int U = MT == 1 ? 8 : 4;
  __shared__ float part[4][MT][16][16];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, q = lane >> 4;
  const int n0 = blockIdx.x * 16;
  int n = n0 + l16;
  n = n < p.N ? n : p.N - 1;  // columns past the edge re-read the last row of W; their results are never stored
  const int kq = p.K / 4;     // K % 256 == 0 is checked on the host: every quarter is a whole number of 64-byte steps
  const uint8_t* w_at = reinterpret_cast<const uint8_t*>(p.B) + (int64_t)n * p.ldb + wave * kq + 16 * q;
  const uint8_t* x_at[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    int m = 16 * t + l16;
    m = m < p.M ? m : p.M - 1;
    x_at[t] = reinterpret_cast<const uint8_t*>(p.A) + (int64_t)m * p.lda + wave * kq + 16 * q;
  }
  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  typedef long l64x2 __attribute__((ext_vector_type(2)));
  auto two = [](const l64x2 a, const l64x2 b, f32x4 c) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a[0], b[0], c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a[1], b[1], c, 0, 0, 0);
  };

  l64x2 fw[2][U], fx[2][MT][U];
  auto load = [&](int buf, int k) {  // steps k .. k + U - 1 of this wavefront's quarter
#pragma unroll
    for (int u = 0; u < U; ++u) {
      fw[buf][u] = *reinterpret_cast<const l64x2*>(w_at + (k + u) * 64);
#pragma unroll
      for (int t = 0; t < MT; ++t) fx[buf][t][u] = *reinterpret_cast<const l64x2*>(x_at[t] + (k + u) * 64);
    }
  };
  auto math = [&](int buf) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = two(fw[buf][u], fx[buf][t][u], acc[t]);
  };
  const int steps = kq / 64, groups = steps / U;
  if (groups > 0) load(0, 0);
  for (int g = 0; g + 1 < groups; g += 2) {  // two groups per trip: the buffer indices stay compile-time
    load(1, (g + 1) * U);
    math(0);
    if (g + 2 < groups) load(0, (g + 2) * U);
    math(1);
  }
  if (groups & 1) math(0);
  for (int k = groups * U; k < steps; ++k) {  // what does not fill a group
    const l64x2 a = *reinterpret_cast<const l64x2*>(w_at + k * 64);
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = two(a, *reinterpret_cast<const l64x2*>(x_at[t] + k * 64), acc[t]);
  }

  // accumulator t of a lane: output rows 16 t + l16 (A rows), columns n0 + 4 q .. + 3
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) part[wave][t][4 * q + e][l16] = acc[t][e];
  __syncthreads();
  const float a_sc = p.a_scale ? *p.a_scale : 1.f;
  for (int idx = tid; idx < MT * 256; idx += kThreads) {
    const int nl = idx & 15, ml = (idx >> 4) & 15, t = idx >> 8;
    const int m = 16 * t + ml, nn = n0 + nl;
    if (m >= p.M || nn >= p.N) continue;
    float v = (part[0][t][nl][ml] + part[1][t][nl][ml]) + (part[2][t][nl][ml] + part[3][t][nl][ml]);
    const float sc = p.b_scale ? a_sc * p.b_scale[nn] : a_sc;
    const float bias = !p.bias ? 0.f : p.bias_f32 ? reinterpret_cast<const float*>(p.bias)[nn] : to_f32(reinterpret_cast<const OT*>(p.bias)[nn]);
    v = v * sc + bias;
    switch (p.act) {
      case XG_ACT_RELU: v = fmaxf(v, 0.f); break;
      case XG_ACT_GELU: v = 0.5f * v * (1.f + erff(v * 0.70710678118654752f)); break;
      case XG_ACT_SILU: v = silu_f32(v); break;
      case XG_ACT_SIGMOID: v = sigmoid_f32(v); break;
      default: break;
    }
    reinterpret_cast<OT*>(p.out)[(int64_t)m * p.ldc + nn] = from_f32<OT>(v);
  }
}

// ---- 128 x 128 tiles: between the 64 x 64 kernel and the large tiles -------------------------------------------
// A problem whose 256 x 256 grid fills a fraction of the compute units, or just over a whole number of rounds, has four
// times as many 128 x 128 tiles: each of the four wavefronts owns a 64 x 64 quadrant (2 x 2 MFMA tiles) over the whole
// of K, so every output element sees the same sequence of MFMAs as in the large-tile kernels and the results are the
// same bits.  Slabs (128 rows x 128 bytes per operand) reach LDS by direct loads, four stages deep (three slabs in
// flight: a slab of math, 16 MFMAs per wavefront, is far shorter than the memory latency); one workgroup per compute unit.
// 16-bit types, both weight layouts, plain layer.
constexpr int MID_TILE = 128;
constexpr int MID_STAGES = 4;
constexpr int MID_SLAB_BYTES = MID_TILE * ROW_BYTES;  // 16 KiB per operand per stage
constexpr int MID_STAGE_BYTES = 2 * MID_SLAB_BYTES;
constexpr int MID_SMEM_BYTES = MID_STAGES * MID_STAGE_BYTES;  // 128 KiB; the epilogue parks 4 x (64 x 64 fp32) in the same space

template <typename T, typename OT, BLayout BL>
__global__ __launch_bounds__(kThreads) void gemm_mid_kernel(GemmParams p_all) {
  extern __shared__ __align__(16) char smem[];
  const GemmParams p = for_batch_entry(p_all);
  constexpr int EB = Elem<T>::BYTES;
  static_assert(EB == 2, "16-bit operands");
  constexpr int SLAB_K = ROW_BYTES / EB;

  int tm, tn;
  tile_of_block(p, blockIdx.x, gridDim.x, tm, tn);
  const int m0 = tm * MID_TILE, n0 = tn * MID_TILE;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, half = lane >> 5, p16 = lane & 15, blk = (lane >> 4) & 1;

  // direct loads: per slab and operand 16 wavefront loads of 1 KiB, four per wavefront.  A, and B when K-contiguous: 8
  // rows of 128 bytes per load.  An N-contiguous B slab is [64 k][128 n], 256 bytes per k row: a load covers 4 k rows,
  // lane i lands at chunk i & 15 of row i >> 4, and the four 64-byte granules of a row are XOR-ed with k & 3 so that
  // the four k rows a 16-lane group of the transposing read touches fall on different banks.
  uint32_t a_off[4], b_off[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int r = (q * 4 + wave) * 8 + (lane >> 3);
    const int slot = lane & 7;
    int gr = m0 + r;
    gr = gr < p.M ? gr : p.M - 1;  // rows past the edge re-read the last row; their results are never stored
    a_off[q] = (uint32_t)(((int64_t)gr * p.lda) * EB + ((slot ^ swz(r)) << 4));
    if constexpr (BL == BLayout::KMajor) {
      int gn = n0 + r;
      gn = gn < p.N ? gn : p.N - 1;
      b_off[q] = (uint32_t)(((int64_t)gn * p.ldb) * EB + ((slot ^ swz(r)) << 4));
    } else {
      const int kr = (q * 4 + wave) * 4 + (lane >> 4);
      const int chunk = (((p16 >> 2) ^ (kr & 3)) << 2) | (p16 & 3);  // logical 16-byte chunk (8 columns) this LDS slot holds
      int gc = n0 + chunk * 8;
      gc = gc < p.N ? gc : p.N - 8;  // N % 8 == 0 is checked on the host
      b_off[q] = (uint32_t)(((int64_t)kr * p.ldb + gc) * EB);
    }
  }
  const char* const a_base = reinterpret_cast<const char*>(p.A);
  const char* const b_base = reinterpret_cast<const char*>(p.B);
  const int64_t b_step = BL == BLayout::KMajor ? (int64_t)ROW_BYTES : (int64_t)SLAB_K * p.ldb * EB;
  auto issue = [&](int kt) {
    char* dst = smem + (kt % MID_STAGES) * MID_STAGE_BYTES + wave * 1024;
#pragma unroll
    for (int q = 0; q < 4; ++q) load_to_lds16(a_base + (int64_t)kt * ROW_BYTES, a_off[q], (uint32_t)(size_t)(lvoid*)(dst + q * 4096));
#pragma unroll
    for (int q = 0; q < 4; ++q)
      load_to_lds16(b_base + kt * b_step, b_off[q], (uint32_t)(size_t)(lvoid*)(dst + MID_SLAB_BYTES + q * 4096));
  };

  // fragment rows of this wavefront's quadrant inside a stage; the chunk of k-step ks is (2 ks + half) ^ swz(row)
  int a_row[2], b_row[2], sw[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    a_row[u] = (wm * 64 + u * 32 + l32) * ROW_BYTES;
    sw[u] = swz(u * 32 + l32);  // swz() looks at the low four bits of the row only: the same for both operands
    if constexpr (BL == BLayout::KMajor) {
      b_row[u] = MID_SLAB_BYTES + (wn * 64 + u * 32 + l32) * ROW_BYTES;
    } else {
      // transposing read of k-step 0: k row half * 8 + p16 / 4, granule (32 columns) 2 wn + u at slot granule ^ (k & 3),
      // inside it 32 bytes per 16-lane block and 8 bytes per lane; k-step ks is 16 rows (4 KiB) further, the upper four
      // k of a lane 4 rows (1 KiB) further (same k & 3, same slot)
      const int kr = half * 8 + (p16 >> 2);
      b_row[u] = MID_SLAB_BYTES + kr * 256 + ((((wn * 2 + u) ^ (kr & 3)) & 3) << 6) + (blk << 5) + ((p16 & 3) << 3);
    }
  }

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int KT = p.K / SLAB_K;
  for (int s = 0; s < MID_STAGES - 1 && s < KT; ++s) issue(s);
  for (int kt = 0; kt < KT; ++kt) {
    // slab kt has landed when only the (at most two) slabs issued after it are in flight: 8 loads each
    const int after = KT - 1 - kt;  // slabs issued after slab kt: at most MID_STAGES - 2 are in flight, 8 loads each
    if (after >= MID_STAGES - 2) {
      wait_vm<8 * (MID_STAGES - 2)>();
    } else if (after >= 3) {
      wait_vm<24>();
    } else if (after == 2) {
      wait_vm<16>();
    } else if (after == 1) {
      wait_vm<8>();
    } else {
      wait_vm<0>();
    }
    barrier_only();  // slab kt is visible to all, and all are done with slab kt-1 ...
    if (kt + MID_STAGES - 1 < KT) issue(kt + MID_STAGES - 1);  // ... whose stage takes the next slab
    const char* st = smem + (kt % MID_STAGES) * MID_STAGE_BYTES;
    // every fragment of the slab is requested before the first MFMA: one LDS round trip per slab is exposed instead of
    // one per k-step (one wavefront per SIMD: nobody else hides it)
    Frag<T> fa[4][2], fb[4][2];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int ch = ((ks * 2 + half) ^ sw[u]) << 4;
        fa[ks][u].v = *reinterpret_cast<const u32x4*>(st + a_row[u] + ch);
        if constexpr (BL == BLayout::KMajor) {
          fb[ks][u].v = *reinterpret_cast<const u32x4*>(st + b_row[u] + ch);
        } else {
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(st + b_row[u] + ks * 4096));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(st + b_row[u] + ks * 4096 + 1024));
          const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
          fb[ks][u].v = u32x4{l2.x, l2.y, h2.x, h2.y};
        }
      }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mma(fb[ks][j], fa[ks][i], acc[i][j]);
  }
  __syncthreads();  // the slabs are dead: the quadrants take their place

  // park this wavefront's quadrant in its own 16 KiB: row r at r * 256, 16-byte chunk (4 columns) c at slot c ^ (r & 15)
  char* park = smem + wave * (64 * 64 * 4);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int row = i * 32 + l32;
        const int chunk = (j * 8 + g * 2 + half) ^ (row & 15);
        const f32x16& a = acc[i][j];
        *reinterpret_cast<f32x4*>(park + row * 256 + (chunk << 4)) = f32x4{a[4 * g], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
      }
  __syncthreads();
  const int n = n0 + wn * 64 + (lane & 7) * 8;
  const bool n_ok = n < p.N;
  float sv[8], bv[8];
  column_terms<OT>(p, n, n_ok, 1.f, sv, bv);
  epilogue_rows_act<OT>(p, park, lane, m0 + wm * 64, n, n_ok, sv, bv, 8);
}

template <typename K>
int set_smem_once(K kernel) {
  return allow_dynamic_lds(reinterpret_cast<const void*>(kernel), SMEM_BYTES);
}

template <typename K>
int launch_kernel(K kernel, const GemmParams& p, hipStream_t stream) {
  if (int st = set_smem_once(kernel)) return st;
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  if (tiles > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)p.batch), dim3(kThreads), SMEM_BYTES, stream, p);
  return status_from_hip(hipGetLastError());
}

// The direct-to-LDS kernel needs whole slabs and 31-bit operand offsets.
template <typename T>
bool dma_ok(const GemmParams& p, BLayout bl, ALayout al = ALayout::KMajor) {
  constexpr int EB = Elem<T>::BYTES;
  constexpr int SLAB_K = ROW_BYTES / EB;
  if (p.K % SLAB_K != 0) return false;
  const int64_t lim = 0x7fffffffLL;
  const int64_t a_bytes = al == ALayout::KMajor ? ((int64_t)p.M * p.lda) * EB : ((int64_t)SLAB_K * p.lda + p.M) * EB;
  const int64_t b_bytes = bl == BLayout::KMajor ? ((int64_t)p.N * p.ldb) * EB : ((int64_t)SLAB_K * p.ldb + p.N) * EB;
  return a_bytes < lim && b_bytes < lim;
}

inline int cu_count() {
  static const int n = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    return cus;
  }();
  return n;
}

// A launch of tm x tn tiles on C compute units runs ceil(tm tn / C) rounds, and the last one may be mostly empty
// (C4: 1376 tiles on 256 CUs = 5.4 rounds, paid as 6).  When the tiles past the last full round are at most half a
// round, the tile columns they make up are computed as 128 x 256 tiles instead: twice as many workgroups of half
// the work fill the machine once, for about 0.55 of a round.  Returns how many tile columns the
// full-size tiles keep (tn: no split).
inline int full_tile_columns(int tm, int tn) {
  const int cus = cu_count();
  int g = tm, c = cus;  // gcd
  while (c) {
    const int t = g % c;
    g = c;
    c = t;
  }
  const int col_step = cus / g;  // tile columns per whole number of rounds
  const int keep = tn / col_step * col_step;
  const int tail_tiles = tm * (tn - keep);
  if (keep == 0 || keep == tn || 2 * tail_tiles > cus) return tn;
  return keep;
}

// Large tiles that would leave most compute units idle give way to the 64 x 64 kernel.  Measured crossover on
// 256 compute units (N = K = 4096, us, 64 x 64 kernel / half-height tiles / full tiles): 64 tiles 54 / 58 / 83,
// 80 tiles 71 / 62 / 86, 128 tiles 98 / 66 / 88.
inline int small_tile_limit() { return cu_count() / 4; }

template <typename T, typename OT, BLayout BL, bool GLU = false>
int launch_small(GemmParams p, hipStream_t stream) {
  auto kernel = gemm_small_kernel<T, OT, BL, GLU>;
  if (int st = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), S_SMEM_BYTES)) return st;
  constexpr int cols = GLU ? S_TILE / 2 : S_TILE;
  p.tiles_m = (p.M + S_TILE - 1) / S_TILE;
  p.tiles_n = (p.N + cols - 1) / cols;
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  if (tiles > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)p.batch), dim3(kThreads), S_SMEM_BYTES, stream, p);
  return status_from_hip(hipGetLastError());
}

// A half-height (128-row) tile takes 0.55 of a full tile's time for half of its work, so a grid of them pays when
// the full-size grid leaves much of its last round empty (128 full tiles on 256 units: one round of 256 half tiles,
// 0.55 instead of 1).  tn: tile columns; the tile rows follow from M.
inline bool half_height_wins(int M, int tn, int batch = 1) {
  const int64_t cus = cu_count();
  const int64_t full = (int64_t)((M + BM - 1) / BM) * tn * batch, half = (int64_t)((M + 127) / 128) * tn * batch;
  const double t_full = (double)((full + cus - 1) / cus), t_half = 0.55 * (double)((half + cus - 1) / cus);
  return t_half < 0.95 * t_full;
}

// Estimated time (us) of the single launch that launch_gemm picks without the 128 x 128 kernel: the 64 x 64 kernel for
// few tiles, full tiles with the last tile columns at half height, half-height tiles, or full tiles.
inline double single_launch_estimate(const GemmParams& p) {
  const double cus = cu_count();
  const double s = p.K / 64.0;
  const double t_full = 10.6 + 1.525 * s, t_half = 0.55 * t_full;
  const int64_t tm = p.tiles_m, tn = p.tiles_n, t256 = tm * tn;
  if (t256 <= small_tile_limit()) {
    const int64_t t64 = (int64_t)((p.M + 63) / 64) * ((p.N + 63) / 64);
    return 3.0 + 0.19 * s + (t64 > 256 ? (double)(t64 - 256) * 0.047 * s / 64.0 : 0.0);
  }
  const int keep = full_tile_columns((int)tm, (int)tn);
  if (keep != tn) return (double)(tm * keep) / cus * t_full + t_half;
  if (half_height_wins(p.M, (int)tn)) {
    const int64_t th = (int64_t)((p.M + 127) / 128) * tn;
    return (double)((th + (int64_t)cus - 1) / (int64_t)cus) * t_half;
  }
  return (double)((t256 + (int64_t)cus - 1) / (int64_t)cus) * t_full;
}

// Whether the 128 x 128 kernel beats what launch_gemm would otherwise pick, by measured times (us, bf16, 256 compute
// units; s = K / 64 slabs): a round of 256 x 256 tiles 10.6 + 1.525 s, of 128 x 256 tiles 0.55 of that, of 128 x 128
// tiles 4 + 0.57 s (bound by the operand stream: 32 KiB per slab and tile), the 64 x 64 kernel 3 + 0.19 s up to 256
// tiles and 0.047 s / 64 per tile beyond.  It wins where its grid fills a whole number of rounds and the others'
// do not: M = 1024, N = K = 4096 46 us against 53 (64 x 64), M = 1024, N = 4096, K = 11008 99 against 129,
// M = 4096, N = 1024, K = 8192 76 against 88.  Decided from M, N and K alone, never from the batch count: a layer gives
// the same bits alone and as one entry of a batch (the 64 x 64 kernel adds in another order).
inline bool mid_tiles_win(const GemmParams& p) {
  const double cus = cu_count();
  const double s = p.K / 64.0;
  const double t_mid = 4.0 + 0.57 * s;
  const int64_t t128 = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128);
  const double est_mid = (double)((t128 + (int64_t)cus - 1) / (int64_t)cus) * t_mid;
  return est_mid < 0.92 * single_launch_estimate(p);
}

// A decode step with K-contiguous weights streams them row by row where the 64 x 64 kernel's grid (N / 64 workgroups) is
// too small to pull the weights at memory speed.  Every workgroup re-reads the M activation rows, M / 16 of what it reads
// of W, so it pays for few rows and moderate N only.  Measured (us, bf16, this kernel / the 64 x 64 kernel): M = 1, N = K =
// 4096 11.2 / 14.9; M = 16 11.1 / 14.9; M = 32 12.8 / 15; M = 64 20.3 / 15.5; M = 16, N = 4096, K = 11008 21.7 / 33.7; M = 1,
// N = K = 8192 20.4 / 26.0; M = 16, N = 11008, K = 4096 23.0 / 15.9 (172 workgroups already stream at 5.6 TB/s).  Decided
// from M, N and K alone, like every choice between kernels that add in different orders.
inline bool skinny_fits(const GemmParams& p) {
  if (p.N < 512 || p.K < 512 || p.K % 128 != 0) return false;
  return p.M <= 4 || (p.M <= 16 && p.N <= 4608) || (p.M <= 32 && p.N <= 4096);
}

// Where the e4m3 walk beats the 64 x 64 kernel.  Measured (us, this kernel at M = 1 / 8 / 16 / 32, then the 64 x 64 kernel,
// which is flat in M here): N = K = 4096 5.6 / 6.2 / 6.8 / 9.0, 9.6; N = 11008, K = 4096 10.2 / 12.0 / 13.9 / 19.5, 13.1;
// N = 4096, K = 11008 10.6 / 12.0 / 13.6 / 18.8, 23.8; N = K = 8192 13.6 / 14.9 / 18.0 / 24.5, 21.2; N = 1024, K = 4096
// 4.8 / 5.6 / 6.3 / 8.4, 9.5.  Every workgroup re-reads the M activation rows (M / 16 of its weight bytes), which is
// what the limits on M follow.
inline bool skinny_fp8_fits(const GemmParams& p) {
  if (p.N < 512 || p.K < 1024 || p.K % 256 != 0 || p.batch != 1 || p.res != nullptr) return false;
  return p.M <= 8 || (p.M <= 16 && p.N <= 8192) || (p.M <= 32 && p.N <= 4096);
}
template <typename OT>
int launch_skinny_fp8(const GemmParams& p, hipStream_t stream) {
  const int64_t blocks = (p.N + 15) / 16;
  if (blocks > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  if (p.M <= 16) hipLaunchKernelGGL((gemm_skinny_fp8_kernel<OT, 1>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, p);
  else hipLaunchKernelGGL((gemm_skinny_fp8_kernel<OT, 2>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, p);
  return status_from_hip(hipGetLastError());
}

template <typename T, typename OT, bool GLU = false>
int launch_skinny(const GemmParams& p, hipStream_t stream) {
  const int64_t blocks = (p.N + 15) / 16;
  if (blocks > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  const dim3 grid((unsigned)blocks, GLU ? 1u : (unsigned)p.batch);
  if constexpr (GLU) {
    if (p.M <= 16) hipLaunchKernelGGL((gemm_skinny_kernel<T, OT, 1, true>), grid, dim3(kThreads), 0, stream, p);
    else hipLaunchKernelGGL((gemm_skinny_kernel<T, OT, 2, true>), grid, dim3(kThreads), 0, stream, p);
  } else {
    if (p.M <= 16) hipLaunchKernelGGL((gemm_skinny_kernel<T, OT, 1>), grid, dim3(kThreads), 0, stream, p);
    else hipLaunchKernelGGL((gemm_skinny_kernel<T, OT, 2>), grid, dim3(kThreads), 0, stream, p);
  }
  return status_from_hip(hipGetLastError());
}

template <typename T, typename OT, BLayout BL>
int launch_mid(GemmParams p, hipStream_t stream) {
  auto kernel = gemm_mid_kernel<T, OT, BL>;
  if (int st = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), MID_SMEM_BYTES)) return st;
  p.tiles_m = (p.M + MID_TILE - 1) / MID_TILE;
  p.tiles_n = (p.N + MID_TILE - 1) / MID_TILE;
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  if (tiles > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)p.batch), dim3(kThreads), MID_SMEM_BYTES, stream, p);
  return status_from_hip(hipGetLastError());
}

// ---- two launches for a grid of a whole number of rounds plus a little --------------------------------------------
// Measured round times as in mid_tiles_win (us; s = K / 64 slabs).
struct RoundTimes {
  double full, half, mid;
  explicit RoundTimes(int K) {
    const double s = K / 64.0;
    full = 10.6 + 1.525 * s;
    half = 0.55 * full;
    mid = 4.0 + 0.57 * s;
  }
};
enum class TileKind { Full, Half, Mid };

// Cheapest of the three kernels that add in the large-tile order for an M x N problem, and its estimated time.
inline double best_same_order_plan(int M, int N, const RoundTimes& t, TileKind& kind) {
  const int64_t cus = cu_count();
  auto rounds = [&](int64_t tiles) { return (double)((tiles + cus - 1) / cus); };
  const int64_t tn = (N + BN - 1) / BN;
  const double e_full = rounds((int64_t)((M + BM - 1) / BM) * tn) * t.full;
  const double e_half = rounds((int64_t)((M + 127) / 128) * tn) * t.half;
  const double e_mid = rounds((int64_t)((M + 127) / 128) * ((N + 127) / 128)) * t.mid;
  kind = TileKind::Full;
  double best = e_full;
  if (e_half < best) best = e_half, kind = TileKind::Half;
  if (e_mid < best) best = e_mid, kind = TileKind::Mid;
  return best;
}

// A grid of r whole rounds of full tiles and a few more pays a whole extra round for them (or runs on half-height tiles
// throughout, which quantise the same way).  Instead: full tiles on as many tile columns (or tile rows) as fill r rounds,
// then a second launch for the strip that is left, with whichever of the full / half-height / 128 x 128 kernels takes
// it fastest -- all three add in the same order, so the result is the same bits as one launch.  Taken when the estimate
// beats the single launch's by 8 %: M = 1536, N = 11008 169 -> 148 us, M = 3072, N = 6144 170 -> 150 us (K = 4096).
struct TwoPart {
  bool by_rows;   // the strip is the last rows (else the last columns)
  int split;      // first row / column of the strip
  TileKind rest;  // kernel of the strip
};
inline bool two_part_plan(const GemmParams& p, double est_single, TwoPart& out) {
  const int64_t cus = cu_count();
  const RoundTimes t(p.K);
  const int64_t tm = p.tiles_m, tn = p.tiles_n;
  const int64_t r = tm * tn / cus;
  if (r < 1 || tm * tn == r * cus) return false;
  double best = 0.92 * est_single;
  bool found = false;
  const double gap = 3.0;  // second launch
  const int64_t keep_c = r * cus / tm < tn - 1 ? r * cus / tm : tn - 1;
  if (keep_c >= 1) {
    TileKind k;
    const double e = (double)((tm * keep_c + cus - 1) / cus) * t.full + best_same_order_plan(p.M, p.N - (int)(keep_c * BN), t, k) + gap;
    if (e < best) best = e, found = true, out = TwoPart{false, (int)(keep_c * BN), k};
  }
  const int64_t keep_r = r * cus / tn < tm - 1 ? r * cus / tn : tm - 1;
  if (keep_r >= 1) {
    TileKind k;
    const double e = (double)((keep_r * tn + cus - 1) / cus) * t.full + best_same_order_plan(p.M - (int)(keep_r * BM), p.N, t, k) + gap;
    if (e < best) best = e, found = true, out = TwoPart{true, (int)(keep_r * BM), k};
  }
  return found;
}

template <typename T, typename OT, BLayout BL>
int launch_same_order(GemmParams p, TileKind kind, hipStream_t stream) {
  p.tiles_n = (p.N + BN - 1) / BN;
  if (kind == TileKind::Mid) return launch_mid<T, OT, BL>(p, stream);
  if (kind == TileKind::Half) {
    p.tiles_m = (p.M + 127) / 128;
    return launch_kernel(gemm_dma_half_kernel<T, OT, BL>, p, stream);
  }
  p.tiles_m = (p.M + BM - 1) / BM;
  return launch_kernel(gemm_dma_kernel<T, OT, BL>, p, stream);
}

template <typename T, typename OT, BLayout BL>
int launch_gemm(const GemmParams& p, hipStream_t stream) {
  if (!dma_ok<T>(p, BL)) return launch_kernel(gemm_staged_kernel<T, OT, BL>, p, stream);
  if constexpr (Elem<T>::BYTES == 2 && BL == BLayout::KMajor) {
    if (skinny_fits(p)) return launch_skinny<T, OT>(p, stream);
  }
  if constexpr (Elem<T>::BYTES == 1 && BL == BLayout::KMajor) {
    if (skinny_fp8_fits(p)) return launch_skinny_fp8<OT>(p, stream);
  }
  if constexpr (Elem<T>::BYTES == 2) {
    if (mid_tiles_win(p)) return launch_mid<T, OT, BL>(p, stream);
  }
  // decided per batch entry: the 64 x 64 kernel splits K between its waves and so adds in another order than the
  // large tiles; a layer must give the same bits whether it runs alone or as one entry of a batch
  if ((int64_t)p.tiles_m * p.tiles_n <= small_tile_limit()) return launch_small<T, OT, BL>(p, stream);
  // the split of the last, partial round is worked out for one tile grid: batched layers run whole tiles
  const int keep = p.batch > 1 ? p.tiles_n : full_tile_columns(p.tiles_m, p.tiles_n);
  if constexpr (Elem<T>::BYTES == 2) {
    TwoPart tp;
    if (p.batch == 1 && two_part_plan(p, single_launch_estimate(p), tp)) {
      constexpr int EB2 = Elem<T>::BYTES;
      GemmParams first = p, rest = p;
      if (tp.by_rows) {
        first.M = tp.split;
        rest.M = p.M - tp.split;
        rest.A = reinterpret_cast<const char*>(p.A) + (int64_t)tp.split * p.lda * EB2;
        if (p.res) rest.res = reinterpret_cast<const char*>(p.res) + (int64_t)tp.split * p.ldr * (int64_t)sizeof(OT);
        rest.out = reinterpret_cast<char*>(p.out) + (int64_t)tp.split * p.ldc * (int64_t)sizeof(OT);
      } else {
        const int64_t n_split = tp.split;
        first.N = tp.split;
        rest.N = p.N - tp.split;
        rest.B = reinterpret_cast<const char*>(p.B) + (BL == BLayout::KMajor ? n_split * p.ldb * EB2 : n_split * EB2);
        if (p.bias) rest.bias = reinterpret_cast<const char*>(p.bias) + n_split * (p.bias_f32 ? 4 : (int64_t)sizeof(OT));
        if (p.res) rest.res = reinterpret_cast<const char*>(p.res) + n_split * (int64_t)sizeof(OT);
        rest.out = reinterpret_cast<char*>(p.out) + n_split * (int64_t)sizeof(OT);
      }
      if (int st = launch_same_order<T, OT, BL>(first, TileKind::Full, stream)) return st;
      return launch_same_order<T, OT, BL>(rest, tp.rest, stream);
    }
  }
  if (keep == p.tiles_n) {
    if (half_height_wins(p.M, p.tiles_n, p.batch)) {
      GemmParams h = p;
      h.tiles_m = (p.M + 127) / 128;
      return launch_kernel(gemm_dma_half_kernel<T, OT, BL>, h, stream);
    }
    return launch_kernel(gemm_dma_kernel<T, OT, BL>, p, stream);
  }
  // columns [0, keep * BN): full tiles; the rest: 128-row tiles on operand pointers moved to the split column
  constexpr int EB = Elem<T>::BYTES;
  const int64_t n_split = (int64_t)keep * BN;
  GemmParams full = p;
  full.N = (int)n_split;
  full.tiles_n = keep;
  GemmParams rest = p;
  rest.N = p.N - (int)n_split;
  rest.tiles_n = p.tiles_n - keep;
  rest.tiles_m = (p.M + 127) / 128;
  rest.B = reinterpret_cast<const char*>(p.B) + (BL == BLayout::KMajor ? n_split * p.ldb * EB : n_split * EB);
  if (p.bias) rest.bias = reinterpret_cast<const char*>(p.bias) + n_split * (p.bias_f32 ? 4 : (int64_t)sizeof(OT));
  if (p.b_scale) rest.b_scale = p.b_scale + n_split;
  if (p.res) rest.res = reinterpret_cast<const char*>(p.res) + n_split * (int64_t)sizeof(OT);
  rest.out = reinterpret_cast<char*>(p.out) + n_split * (int64_t)sizeof(OT);
  auto kernel = gemm_dma_split_kernel<T, OT, BL>;
  if (int st = set_smem_once(kernel)) return st;
  const int64_t n_full = (int64_t)full.tiles_m * full.tiles_n, n_rest = (int64_t)rest.tiles_m * rest.tiles_n;
  if (n_full + n_rest > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  hipLaunchKernelGGL(kernel, dim3((unsigned)(n_full + n_rest), 1), dim3(kThreads), SMEM_BYTES, stream, full, rest, (int)n_full);
  return status_from_hip(hipGetLastError());
}

// Left operand transposed in memory: out[M, N] = At^T B with At [K, M] (row stride lda) and B [K, N], the shape of a
// weight gradient.  Full-height tiles only (whole slabs by direct loads, any K through registers).
template <typename T, typename OT>
int launch_gemm_at(const GemmParams& p, hipStream_t stream) {
  if (!dma_ok<T>(p, BLayout::NMajor, ALayout::MMajor))
    return launch_kernel(gemm_staged_kernel<T, OT, BLayout::NMajor, ALayout::MMajor>, p, stream);
  return launch_kernel(gemm_dma_kernel<T, OT, BLayout::NMajor, ALayout::MMajor>, p, stream);
}

// Gated layer: out[M, N] = silu(A Wg^T) * (A Wu^T), Wg = p.B and Wu = p.B2 both [N, K] with row stride ldb.
// Output tiles are 256 x 128 (p.tiles_n counts 128-column tiles).  Needs whole K slabs: the caller checks dma_ok.
template <typename T, typename OT>
int launch_glu(const GemmParams& p, hipStream_t stream) {
  constexpr int EB = Elem<T>::BYTES;
  // Up to 128 rows the row-streaming and the 64 x 64 kernel are taken exactly where the plain layer takes them for the same
  // M, N, K (its tiles are 256 columns wide, the gated layer's 128), so that the gated layer stays two plain layers and the
  // gate kernel bit for bit there.  A decode step (M = 1, K = 4096, N = 11008) took 74 us on the large tiles, 86 of them for
  // 256 compute units; 33 us row by row.  Measured at N = 11008, K = 4096 (us, 64 x 64 kernel / large tiles): M = 64 47 / 76,
  // M = 128 61 / 76, M = 256 101 / 80: beyond 128 rows the tile count of the gated layer's own tiles decides, as before.
  if (skinny_fits(p)) return launch_skinny<T, OT, true>(p, stream);
  const int64_t plain_tiles = (int64_t)p.tiles_m * ((p.N + BN - 1) / BN);
  if ((p.M <= 128 && plain_tiles <= small_tile_limit()) || (int64_t)p.tiles_m * p.tiles_n <= small_tile_limit())
    return launch_small<T, OT, BLayout::KMajor, true>(p, stream);
  const int keep = full_tile_columns(p.tiles_m, p.tiles_n);
  if (keep == p.tiles_n) {
    if (half_height_wins(p.M, p.tiles_n)) {
      GemmParams h = p;
      h.tiles_m = (p.M + 127) / 128;
      return launch_kernel(gemm_glu_half_kernel<T, OT>, h, stream);
    }
    return launch_kernel(gemm_glu_kernel<T, OT>, p, stream);
  }
  const int64_t n_split = (int64_t)keep * (BN / 2);
  GemmParams full = p;
  full.N = (int)n_split;
  full.tiles_n = keep;
  GemmParams rest = p;
  rest.N = p.N - (int)n_split;
  rest.tiles_n = p.tiles_n - keep;
  rest.tiles_m = (p.M + 127) / 128;
  rest.B = reinterpret_cast<const char*>(p.B) + n_split * p.ldb * EB;
  rest.B2 = reinterpret_cast<const char*>(p.B2) + n_split * p.ldb * EB;
  rest.out = reinterpret_cast<char*>(p.out) + n_split * (int64_t)sizeof(OT);
  if (p.gate_out) {
    rest.gate_out = reinterpret_cast<char*>(p.gate_out) + n_split * (int64_t)sizeof(OT);
    rest.up_out = reinterpret_cast<char*>(p.up_out) + n_split * (int64_t)sizeof(OT);
  }
  auto kernel = gemm_glu_split_kernel<T, OT>;
  if (int st = set_smem_once(kernel)) return st;
  const int64_t n_full = (int64_t)full.tiles_m * full.tiles_n, n_rest = (int64_t)rest.tiles_m * rest.tiles_n;
  if (n_full + n_rest > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  hipLaunchKernelGGL(kernel, dim3((unsigned)(n_full + n_rest)), dim3(kThreads), SMEM_BYTES, stream, full, rest, (int)n_full);
  return status_from_hip(hipGetLastError());
}

inline GemmParams make_params(const void* a, const void* b, const void* bias, const void* residual, void* out, int64_t M,
                       int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldr, int act, bool bias_f32) {
  GemmParams p{};
  p.A = a;
  p.B = b;
  p.B2 = nullptr;
  p.gate_out = p.up_out = nullptr;
  p.bias = bias;
  p.res = residual;
  p.out = out;
  p.a_scale = nullptr;
  p.b_scale = nullptr;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.lda = lda;
  p.ldb = ldb;
  p.ldr = ldr;
  p.ldc = N;
  p.act = act;
  p.bias_f32 = bias_f32 ? 1 : 0;
  p.tiles_m = (int)((M + BM - 1) / BM);
  p.tiles_n = (int)((N + BN - 1) / BN);
  p.batch = 1;
  p.a_batch = p.b_batch = p.bias_batch = p.res_batch = p.out_batch = 0;
  return p;
}

}  // namespace gemm
}  // namespace xg
