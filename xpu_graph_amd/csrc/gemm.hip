// Dense layer for gfx950: out = act(A @ B(+T) * scales + bias + residual) on the
// matrix cores.
//
// Tiling: one 256-thread workgroup (4 wavefronts, 2 x 2) owns a 256 x 256 output
// tile; each wavefront owns 128 x 128 of it as 4 x 4 MFMA tiles of 32 x 32, i.e.
// 256 fp32 accumulators per lane, the whole accumulator file at one wavefront per
// SIMD.  K advances in slabs of 128 BYTES per row (64 bf16/f16 or 128 fp8
// elements), double-buffered in 128 KiB of LDS: while the MFMAs of slab t run,
// slab t+1 moves from registers to LDS and slab t+2 is in flight from memory.
//
// LDS layout (K-contiguous operands): row r of a slab is 128 bytes = 8 chunks of
// 16 bytes; chunk c is stored at c ^ (r & 7) ^ ((r >> 3) & 1), which makes both
// the 16-byte fragment reads of 16 consecutive rows and the row-wise writes
// conflict free.  A [K, N] (N-contiguous) B operand is kept [k][n] in LDS and
// read with the transposing LDS load of gfx950 (ds_read_b64_tr_b16), so no
// separate transpose pass is needed.
//
// The MFMA is issued with B's fragment as the first operand, so each lane ends
// up with 4 CONSECUTIVE output columns of one row: the epilogue (scales, bias,
// residual, activation, rounding) works on those and stores 8 or 16 bytes.
//
// Workgroups are dealt to the 8 XCDs round-robin by the hardware; the block id
// is remapped so that each XCD works through one contiguous, grouped run of
// tiles and its L2 sees each operand slab a few times instead of once per CU.
#include "xg_common.hpp"

#include <stdlib.h>

#include <type_traits>
#include <utility>

namespace xg {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

constexpr int BM = 256, BN = 256;
constexpr int ROW_BYTES = 128;        // bytes of K per tile row and slab
constexpr int SLAB_BYTES = BM * ROW_BYTES;  // 32 KiB per operand per stage
constexpr int SMEM_BYTES = 4 * SLAB_BYTES;  // A, B x 2 stages
constexpr int kThreads = 256;
constexpr int kXcds = 8;
constexpr int kGroupM = 8;

enum class BLayout { KMajor, NMajor };  // B stored [N, K] (K contiguous) or [K, N] (N contiguous)

struct GemmParams {
  const void* A;
  const void* B;
  const void* bias;
  const void* res;
  void* out;
  const float* a_scale;  // fp8 only
  const float* b_scale;  // fp8 only
  int M, N, K;
  int64_t lda, ldb, ldr;
  int act;
  int bias_f32;
  int tiles_m, tiles_n;
};

__device__ __forceinline__ float apply_act(float v, int act) {
  switch (act) {
    case XG_ACT_RELU:
      return fmaxf(v, 0.f);
    case XG_ACT_GELU:
      return 0.5f * v * (1.f + erff(v * 0.70710678118654752f));
    case XG_ACT_SILU:
      return v / (1.f + __expf(-v));
    case XG_ACT_SIGMOID:
      return 1.f / (1.f + __expf(-v));
    default:
      return v;
  }
}

// Element traits: MFMA flavour, elements per 16-byte chunk, k-steps per slab.
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
struct Elem<uint8_t> {  // OCP e4m3
  static constexpr int BYTES = 1;
  static constexpr int KSTEPS = 2;  // 2 x (32x32x64) per 128-element slab
};

__device__ __forceinline__ f32x16 mfma_step(bf16_t, u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mfma_step(f16_t, u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
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

__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// XCD-aware, grouped tile order.
__device__ __forceinline__ void tile_of_block(const GemmParams& p, int& tm, int& tn) {
  const int nb = gridDim.x;
  const int bid = blockIdx.x;
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

// T: operand element type (bf16_t, f16_t, or uint8_t for OCP e4m3); OT: output / bias / residual type.
template <typename T, typename OT, BLayout BL>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_kernel(GemmParams p) {
  extern __shared__ __align__(16) char smem[];
  constexpr int EB = Elem<T>::BYTES;
  constexpr int KSTEPS = Elem<T>::KSTEPS;
  constexpr int SLAB_K = ROW_BYTES / EB;  // elements of K per slab
  static_assert(BL == BLayout::KMajor || EB == 2, "the transposing LDS read is wired for 16-bit elements only");

  int tm, tn;
  tile_of_block(p, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, half = lane >> 5;

  // stage s: A slab at smem + s * 2 * SLAB_BYTES, B slab right behind it

  // ---- global -> register staging ------------------------------------------------
  // K-major operand: thread covers chunk c of rows r0 + 32 j (8 threads = one 128-byte row).
  const int c8 = tid & 7, r0 = tid >> 3;
  const char* a_ptr[8];
  int a_lds[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int r = r0 + 32 * j;
    int gr = m0 + r;
    gr = gr < p.M ? gr : p.M - 1;  // rows past the edge re-read the last row; their results are never stored
    a_ptr[j] = reinterpret_cast<const char*>(p.A) + ((int64_t)gr * p.lda) * EB + c8 * 16;
    a_lds[j] = r * ROW_BYTES + ((c8 ^ swz(r)) << 4);
  }
  const char* b_ptr[8];
  int b_lds[8];
  if constexpr (BL == BLayout::KMajor) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int r = r0 + 32 * j;
      int gr = n0 + r;
      gr = gr < p.N ? gr : p.N - 1;
      b_ptr[j] = reinterpret_cast<const char*>(p.B) + ((int64_t)gr * p.ldb) * EB + c8 * 16;
      b_lds[j] = r * ROW_BYTES + ((c8 ^ swz(r)) << 4);
    }
  } else {
    // N-major operand: slab is [64 k][256 n]; thread covers 16-byte chunk c32 (8 columns) of k rows kr0 + 8 j.
    const int c32 = tid & 31, kr0 = tid >> 5;
    int gc = n0 + c32 * 8;
    gc = gc < p.N ? gc : (p.N - 8);  // N % 8 == 0 is checked on the host
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
    const int64_t koff = (int64_t)kt * ROW_BYTES;
    const int64_t boff = BL == BLayout::KMajor ? koff : (int64_t)kt * SLAB_K * p.ldb * EB;
    if (k_left >= SLAB_K) {  // uniform: a whole slab, no per-load predicate
#pragma unroll
      for (int j = 0; j < 8; ++j) ga[j] = *reinterpret_cast<const u32x4*>(a_ptr[j] + koff);
#pragma unroll
      for (int j = 0; j < 8; ++j) gb[j] = *reinterpret_cast<const u32x4*>(b_ptr[j] + boff);
    } else {  // the last, partial slab: chunks past K read as zero
#pragma unroll
      for (int j = 0; j < 8; ++j)
        ga[j] = (c8 * (16 / EB) < k_left) ? *reinterpret_cast<const u32x4*>(a_ptr[j] + koff) : u32x4{0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const bool ok = BL == BLayout::KMajor ? (c8 * (16 / EB) < k_left) : ((tid >> 5) + 8 * j < k_left);
        gb[j] = ok ? *reinterpret_cast<const u32x4*>(b_ptr[j] + boff) : u32x4{0, 0, 0, 0};
      }
    }
  };
  auto store_slab = [&](int stage) {
#pragma unroll
    for (int j = 0; j < 8; ++j) *reinterpret_cast<u32x4*>(smem + stage * (2 * SLAB_BYTES) + a_lds[j]) = ga[j];
#pragma unroll
    for (int j = 0; j < 8; ++j) *reinterpret_cast<u32x4*>(smem + stage * (2 * SLAB_BYTES) + SLAB_BYTES + b_lds[j]) = gb[j];
  };

  // ---- fragment addressing --------------------------------------------------------
  const int fsw = swz(l32);
  int a_row[4], b_row[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a_row[i] = (wm * 128 + i * 32 + l32) * ROW_BYTES;
    b_row[i] = (wn * 128 + i * 32 + l32) * ROW_BYTES;
  }
  // N-major B: per (n-tile j, k-step, part q) address pieces
  const int p16 = lane & 15, blk = (lane >> 4) & 1;
  const int tr_sw = (p16 >> 2) | (half << 2);

  f32x16 acc[4][4];
  {
    const f32x16 zero = {};
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = zero;
  }

  const int KT = (p.K + SLAB_K - 1) / SLAB_K;
  load_slab(0);
  store_slab(0);
  __syncthreads();
  if (KT > 1) load_slab(1);

  for (int kt = 0; kt < KT; ++kt) {
    const int stage = kt & 1;
    const char* a_s = smem + stage * (2 * SLAB_BYTES);
    const char* b_s = a_s + SLAB_BYTES;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      if constexpr (EB == 2) {
        u32x4 fa[4], fb[4];
        const int ch = ((ks * 2 + half) ^ fsw) << 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) fa[i] = *reinterpret_cast<const u32x4*>(a_s + a_row[i] + ch);
        if constexpr (BL == BLayout::KMajor) {
#pragma unroll
          for (int j = 0; j < 4; ++j) fb[j] = *reinterpret_cast<const u32x4*>(b_s + b_row[j] + ch);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int gran = ((wn * 4 + j) ^ tr_sw) & 7;
            const int col = (gran << 6) + (blk << 5) + ((p16 & 3) << 3);
            const int row0 = ks * 16 + half * 8 + (p16 >> 2);
            typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
            s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(b_s + row0 * (BN * 2) + col));
            s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(b_s + (row0 + 4) * (BN * 2) + col));
            u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
            fb[j] = u32x4{l2.x, l2.y, h2.x, h2.y};
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j] = mfma_step(T{}, fb[j], fa[i], acc[i][j]);
      } else {
        // fp8: a k-step is 64 elements; each lane half supplies 32 consecutive bytes (2 chunks)
        i32x8 fa[4], fb[4];
        const int ch0 = ((ks * 4 + half * 2) ^ fsw) << 4, ch1 = ((ks * 4 + half * 2 + 1) ^ fsw) << 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          u32x4 x = *reinterpret_cast<const u32x4*>(a_s + a_row[i] + ch0);
          u32x4 y = *reinterpret_cast<const u32x4*>(a_s + a_row[i] + ch1);
          fa[i] = i32x8{(int)x.x, (int)x.y, (int)x.z, (int)x.w, (int)y.x, (int)y.y, (int)y.z, (int)y.w};
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          u32x4 x = *reinterpret_cast<const u32x4*>(b_s + b_row[j] + ch0);
          u32x4 y = *reinterpret_cast<const u32x4*>(b_s + b_row[j] + ch1);
          fb[j] = i32x8{(int)x.x, (int)x.y, (int)x.z, (int)x.w, (int)y.x, (int)y.y, (int)y.z, (int)y.w};
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            // format 0 = e4m3 for both operands; scale exponents 127 = 2^0
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j], fa[i], acc[i][j], 0, 0, 0, 127, 0, 127);
      }
      if (ks == 0 && kt + 1 < KT) store_slab(stage ^ 1);  // slab kt+1: registers -> the idle LDS stage
      if (ks == 1 && kt + 2 < KT) load_slab(kt + 2);      // slab kt+2: memory -> registers
    }
    __syncthreads();
  }

  // ---- epilogue ---------------------------------------------------------------------
  const float a_sc = p.a_scale ? *p.a_scale : 1.f;
  typedef OT O4 __attribute__((ext_vector_type(4)));
  static_for<4>([&](auto J) {
    static_for<4>([&](auto G) {
      constexpr int j = decltype(J)::value, g = decltype(G)::value;
      const int n = n0 + wn * 128 + j * 32 + 8 * g + 4 * half;
      const bool n_ok = n < p.N;  // N % 4 == 0: the 4 columns are in or out together
      float bv[4] = {0.f, 0.f, 0.f, 0.f};
      float sv[4] = {a_sc, a_sc, a_sc, a_sc};
      if (n_ok && p.bias) {
        if (p.bias_f32) {
          const f32x4 t = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p.bias) + n);
#pragma unroll
          for (int e = 0; e < 4; ++e) bv[e] = t[e];
        } else {
          const O4 t = *reinterpret_cast<const O4*>(reinterpret_cast<const OT*>(p.bias) + n);
#pragma unroll
          for (int e = 0; e < 4; ++e) bv[e] = to_f32(t[e]);
        }
      }
      if (n_ok && p.b_scale) {
        const f32x4 t = *reinterpret_cast<const f32x4*>(p.b_scale + n);
#pragma unroll
        for (int e = 0; e < 4; ++e) sv[e] = a_sc * t[e];
      }
      static_for<4>([&](auto I) {
        constexpr int i = decltype(I)::value;
        const int m = m0 + wm * 128 + i * 32 + l32;
        if (n_ok && m < p.M) {
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * g + e] * sv[e] + bv[e];
          if (p.res) {
            const O4 r = *reinterpret_cast<const O4*>(reinterpret_cast<const OT*>(p.res) + (int64_t)m * p.ldr + n);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += to_f32(r[e]);
          }
          O4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = from_f32<OT>(apply_act(v[e], p.act));
          *reinterpret_cast<O4*>(reinterpret_cast<OT*>(p.out) + (int64_t)m * p.N + n) = o;
        }
      });
    });
  });
}

}  // namespace
}  // namespace xg

namespace xg {
namespace {

template <typename K>
int set_smem_once(K kernel) {
  static hipError_t st = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES);
  return st == hipSuccess ? XG_OK : XG_ERR_LAUNCH;
}

template <typename T, typename OT, BLayout BL>
int launch_gemm(const GemmParams& p, hipStream_t stream) {
  auto kernel = gemm_kernel<T, OT, BL>;
  if (int st = set_smem_once(kernel)) return st;
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  if (tiles > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles), dim3(kThreads), SMEM_BYTES, stream, p);
  return status_from_hip(hipGetLastError());
}

}  // namespace
}  // namespace xg

extern "C" {

int xg_dense(const void* a, const void* b, const void* bias, const void* residual, void* out, int64_t M, int64_t N,
             int64_t K, int64_t lda, int64_t ldb, int64_t ldr, int b_trans, int act, int dtype, int bias_dtype,
             xg_stream_t stream) {
  using namespace xg;
  if (a == nullptr || b == nullptr || out == nullptr) return XG_ERR_NULL_PTR;
  if (M < 0 || N <= 0 || K <= 0 || lda < K || (b_trans ? ldb < K : ldb < N) || (residual && ldr < N)) return XG_ERR_BAD_SHAPE;
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return XG_ERR_TOO_LARGE;
  if (dtype != XG_BF16 && dtype != XG_F16) return XG_ERR_BAD_DTYPE;
  if (bias && bias_dtype != dtype && bias_dtype != XG_F32) return XG_ERR_BAD_DTYPE;
  if (act < XG_ACT_NONE || act > XG_ACT_SIGMOID) return XG_ERR_BAD_ARG;
  // 16-byte operand loads and 8-byte output stores
  if (K % 8 != 0 || N % 8 != 0 || lda % 8 != 0 || ldb % 8 != 0 || (residual && ldr % 4 != 0)) return XG_ERR_BAD_ALIGN;
  if (!aligned_to(a, 16) || !aligned_to(b, 16) || !aligned_to(out, 16) || (bias && !aligned_to(bias, 16)) ||
      (residual && !aligned_to(residual, 8)))
    return XG_ERR_BAD_ALIGN;
  if (M == 0) return XG_OK;
  GemmParams p{};
  p.A = a;
  p.B = b;
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
  p.act = act;
  p.bias_f32 = (bias && bias_dtype == XG_F32) ? 1 : 0;
  p.tiles_m = (int)((M + BM - 1) / BM);
  p.tiles_n = (int)((N + BN - 1) / BN);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == XG_BF16)
    return b_trans ? launch_gemm<bf16_t, bf16_t, BLayout::KMajor>(p, st) : launch_gemm<bf16_t, bf16_t, BLayout::NMajor>(p, st);
  return b_trans ? launch_gemm<f16_t, f16_t, BLayout::KMajor>(p, st) : launch_gemm<f16_t, f16_t, BLayout::NMajor>(p, st);
}

int xg_dense_fp8(const void* a_q, const void* b_q, const float* a_scale_dev, const float* b_scale_dev, const void* bias,
                 void* out, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int b_trans, int act,
                 int out_dtype, int bias_dtype, xg_stream_t stream) {
  using namespace xg;
  if (a_q == nullptr || b_q == nullptr || out == nullptr || a_scale_dev == nullptr || b_scale_dev == nullptr)
    return XG_ERR_NULL_PTR;
  if (!b_trans) return XG_ERR_BAD_ARG;  // the quantised weight is stored [N, K] (K contiguous)
  if (M < 0 || N <= 0 || K <= 0 || lda < K || ldb < K) return XG_ERR_BAD_SHAPE;
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return XG_ERR_TOO_LARGE;
  if (out_dtype != XG_BF16 && out_dtype != XG_F16 && out_dtype != XG_F32) return XG_ERR_BAD_DTYPE;
  if (bias && bias_dtype != out_dtype && bias_dtype != XG_F32) return XG_ERR_BAD_DTYPE;
  if (act < XG_ACT_NONE || act > XG_ACT_SIGMOID) return XG_ERR_BAD_ARG;
  if (K % 16 != 0 || N % 8 != 0 || lda % 16 != 0 || ldb % 16 != 0) return XG_ERR_BAD_ALIGN;
  if (!aligned_to(a_q, 16) || !aligned_to(b_q, 16) || !aligned_to(out, 16) || (bias && !aligned_to(bias, 16)) ||
      !aligned_to(b_scale_dev, 16))
    return XG_ERR_BAD_ALIGN;
  if (M == 0) return XG_OK;
  GemmParams p{};
  p.A = a_q;
  p.B = b_q;
  p.bias = bias;
  p.res = nullptr;
  p.out = out;
  p.a_scale = a_scale_dev;
  p.b_scale = b_scale_dev;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.lda = lda;
  p.ldb = ldb;
  p.ldr = 0;
  p.act = act;
  p.bias_f32 = (bias && bias_dtype == XG_F32) ? 1 : 0;
  p.tiles_m = (int)((M + BM - 1) / BM);
  p.tiles_n = (int)((N + BN - 1) / BN);
  hipStream_t st = (hipStream_t)stream;
  switch (out_dtype) {
    case XG_BF16:
      return launch_gemm<uint8_t, bf16_t, BLayout::KMajor>(p, st);
    case XG_F16:
      return launch_gemm<uint8_t, f16_t, BLayout::KMajor>(p, st);
    default:
      return launch_gemm<uint8_t, float, BLayout::KMajor>(p, st);
  }
}

}  // extern "C"
