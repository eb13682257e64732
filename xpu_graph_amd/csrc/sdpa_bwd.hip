// Backward of scaled dot-product attention for gfx950 (flash-attention backward): the probabilities are
// recomputed tile by tile from the saved log-sum-exp of every query row, so nothing of size [Sq, Skv] is ever
// stored.  Two kernels, each the owner of the rows it writes (no atomics, results independent of scheduling):
//
//   dq kernel   workgroup = 128 query rows of one (batch, head), wave = 32 rows, lane = one query (lanes l and
//               l ^ 32 share it).  K and V tiles of 64 keys stream through LDS as in the forward kernel.
//                 S^T  = K Q^T          (K tile rows as the A operand, Q rows in registers as B)
//                 P    = exp2(S c - L)  (L = log-sum-exp of the row in base-2 units)
//                 dP^T = V dO^T         (V tile rows as A, dO rows in registers as B)
//                 dS   = P (dP - delta) (delta = <dO row, O row>, computed here and written for the other kernel)
//                 dQ^T += K^T dS^T      (K tile read with the transposing LDS read; dS stays in the lane)
//   dk/dv kernel workgroup = 128 keys of one (batch, key/value head), wave = 32 keys, lane = one key.  Q and dO
//               tiles of 64 queries (plus the 64 log-sum-exps and deltas) stream through LDS; with fewer key/value
//               heads than query heads the workgroup walks every query head of its group.
//                 S    = Q K^T          (Q tile rows as A, K rows in registers as B)
//                 dP   = dO V^T         (dO tile rows as A, V rows in registers as B)
//                 dV^T += dO^T P, dK^T += Q^T dS   (transposing reads of the dO / Q tiles)
//
// As in the forward kernel the k index of the second kind of product is permuted so that its slots are exactly
// the rows a lane already holds in its accumulator registers: P and dS never move between lanes.
// Every tile uses the swizzle of the transposing reads; 16 consecutive rows still land on 16 different chunk
// slots, so the row-wise (A operand) reads of the same tile stay conflict free.
#include "sdpa_common.hpp"

#include <map>
#include <mutex>

namespace xg {
namespace sdpa {

constexpr int KW = 8;          // waves per workgroup of the dk/dv kernel, 32 keys each
constexpr int BK = 32 * KW;   // keys per workgroup of the dk/dv kernel

struct BwdParams {
  const void* q;
  const void* k;
  const void* v;
  const void* o;
  const void* d_o;
  const float* lse;  // [B, H, Sq] natural log
  float* delta;      // [B, H, Sq] workspace: written by the dq kernel, read by the dk/dv kernel
  void* dq;          // [B, H, Sq, D]
  void* dk;          // [B, Hkv, Skv, D]
  void* dv;
  int B, H, Hkv, Sq, Skv;
  int64_t qs[3], ks[3], vs[3], os[3], dos[3];  // element strides of batch, head, sequence
  int64_t dqs[3], dks[3], dvs[3];              // ... of the three outputs (rows of D contiguous elements)
  float scale;
  const float* scale_dev;  // when set: the scale is read from this one-element device tensor instead
  const void* mask;        // additive mask (MASK kernels only), element [b, h, i, j] at ms[0] b + ms[1] h + ms[2] i + j
  int64_t ms[3];           // element strides of batch, head, query row (0: broadcast)
  int mask_f32;            // mask elements are fp32 (else the dtype of q)
  int mask_vec;            // rows of the mask can be read four elements at a time
  int causal;
  int n_qb, n_kb;
  int group_q, group_k;  // block order of the two kernels (grouped_block_order)
};

constexpr float kLog2e = 1.44269504088896340736f;

// 4 bytes per lane from global memory straight into LDS: lane i's word lands at lds_base + 4 i.
__device__ __forceinline__ void load_to_lds4(const void* base, uint32_t lane_off, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_base), "v"(lane_off), "s"(base) : "memory", "m0");
}

// acc[v] += <tile row 32 t + 8 (v / 4) + 4 h + v % 4, the row held by lane l32 in `regs`> over the D columns
template <typename T, int D>
__device__ __forceinline__ f32x16 rows_times_regs(const char* tile, int t, int l32, int h, int sx, const typename Vec8<T>::type* regs) {
  typedef typename Vec8<T>::type V8;
  constexpr int RB = D * 2, KK = D / 16;
  f32x16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  static_for<KK>([&](auto KI) {
    constexpr int kk = decltype(KI)::value;
    const int off = l32 * RB + (((2 * kk + h) ^ sx) << 4);
    const V8 f = *reinterpret_cast<const V8*>(tile + 32 * t * RB + off);
    acc = mma(f, regs[kk], acc);
  });
  return acc;
}

// The same product with the lane's row read from LDS as well: `held` points at the 32 rows of this wave (row l32 is
// the lane's), laid out like a tile block.
template <typename T, int D>
__device__ __forceinline__ f32x16 rows_times_rows(const char* tile, int t, int l32, int h, int sx, const char* held) {
  typedef typename Vec8<T>::type V8;
  constexpr int RB = D * 2, KK = D / 16;
  f32x16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  static_for<KK>([&](auto KI) {
    constexpr int kk = decltype(KI)::value;
    const int off = l32 * RB + (((2 * kk + h) ^ sx) << 4);
    const V8 a = *reinterpret_cast<const V8*>(tile + 32 * t * RB + off);
    const V8 b = *reinterpret_cast<const V8*>(held + off);
    acc = mma(a, b, acc);
  });
  return acc;
}

// Per-lane parts of the transposing-read addresses (see the forward kernel).
struct TrLane {
  int row, chunk, sub;
  __device__ __forceinline__ explicit TrLane(int lane) {
    const int h = lane >> 5, a16 = lane & 15, b16 = (lane >> 4) & 1;
    row = 4 * h + (a16 >> 2);
    chunk = 2 * b16 + ((a16 & 3) >> 1);
    sub = (a16 & 1) << 3;
  }
};

// acc[dt][4 g + e] += sum over the 32 rows of tile block t of tile[row][32 dt + 8 g + 4 h + e] * w[row], where
// w[8 (v / 4) + 4 h + v % 4] for v = 0..15 are the values this lane holds (rounded to T for the product).
// The held values come rounded and packed: wf[st][jj] = w[8 st + jj].
template <typename T, int D>
__device__ __forceinline__ void transposed_times_packed(const char* tile, int t, const TrLane& L, const typename Vec8<T>::type (&wfs)[2],
                                                        f32x16 (&acc)[D / 32]) {
  typedef typename Vec8<T>::type V8;
  constexpr int RB = D * 2, DT = D / 32;
  static_for<2>([&](auto SI) {
    constexpr int st = decltype(SI)::value;
    const V8 wf = wfs[st];
    static_for<DT>([&](auto DI) {
      constexpr int dt = decltype(DI)::value;
      const int off0 = L.row * RB + (((4 * dt + L.chunk) ^ swz_v<D>(L.row)) << 4) + L.sub;
      const int off1 = (L.row + 8) * RB + (((4 * dt + L.chunk) ^ swz_v<D>(L.row + 8)) << 4) + L.sub;
      const char* base = tile + (32 * t + 16 * st) * RB;
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(base + off0));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(base + off1));
      const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      acc[dt] = mma(__builtin_bit_cast(V8, both), wf, acc[dt]);
    });
  });
}

template <typename T, int D>
__device__ __forceinline__ void transposed_times_held(const char* tile, int t, const TrLane& L, const f32x16& w, f32x16 (&acc)[D / 32]) {
  typename Vec8<T>::type wfs[2];
  static_for<16>([&](auto VI) {
    constexpr int v = decltype(VI)::value;
    wfs[v / 8][v % 8] = (T)w[v];
  });
  transposed_times_packed<T, D>(tile, t, L, wfs, acc);
}

// Write acc^T (lane = row l32 of this wave's 32 rows, registers = columns) times `mul` as rows of D elements of T
// to dst + row * row_stride, for rows below rows_valid.  `park` is this wave's 32 x D x 2 bytes of LDS; every wave of the
// workgroup must make the call (it holds a barrier).
template <typename T, int D>
__device__ __forceinline__ void store_rows(char* park, const f32x16 (&acc)[D / 32], float mul, T* dst, int64_t row_stride, int rows_valid,
                                           int lane) {
  constexpr int RB = D * 2, DT = D / 32;
  const int l32 = lane & 31, h = lane >> 5;
  static_for<DT>([&](auto DI) {
    constexpr int dt = decltype(DI)::value;
    static_for<4>([&](auto GI) {
      constexpr int g = decltype(GI)::value;
      typedef T t4 __attribute__((ext_vector_type(4)));
      t4 w;
      static_for<4>([&](auto EI) {
        constexpr int e = decltype(EI)::value;
        w[e] = (T)(acc[dt][4 * g + e] * mul);
      });
      *reinterpret_cast<t4*>(park + l32 * RB + (((4 * dt + g) ^ swz_k<D>(l32)) << 4) + 8 * h) = w;
    });
  });
  __syncthreads();  // called by every wave of the workgroup: the parks are complete (and the compiler keeps the order)
  static_for<RB / 32>([&](auto I) {
    constexpr int i = decltype(I)::value;
    const int pos = i * 1024 + lane * 16;
    const int row = pos / RB, pc = (pos % RB) >> 4;
    const int c = pc ^ swz_k<D>(row);
    const u32x4 val = *reinterpret_cast<const u32x4*>(park + pos);
    if (row < rows_valid) *reinterpret_cast<u32x4*>(dst + (int64_t)row * row_stride + c * 8) = val;
  });
}

// ---------------------------------------------------------------------------------------------- dq
// MASK: the forward added an additive mask to the scaled scores; the probabilities are recomputed with it (the mask
// itself gets no gradient).
template <typename T, int D, bool MASK = false>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void sdpa_bwd_dq_kernel(BwdParams p) {
  typedef typename Vec8<T>::type V8;
  constexpr int RB = D * 2, CH = RB / 16, TILE = BKV * RB, STAGE = 2 * TILE, KK = D / 16, DT = D / 32, LPW = CH / 4;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, h = lane >> 5;
  const float scale = p.scale_dev ? *p.scale_dev : p.scale;
  const float c = scale * kLog2e;

  const int nbh = p.B * p.H;
  int bh, rank;
  grouped_block_order(blockIdx.x, nbh, p.n_qb, p.group_q, bh, rank);
  const int qb = p.n_qb - 1 - rank;  // causal: late query blocks have the most keys, start them first
  const int b = bh / p.H, head = bh % p.H, hkv = head / (p.H / p.Hkv);
  const int q0 = qb * BQ;
  const int qrow = q0 + 32 * wave + l32;
  const int qr = qrow < p.Sq ? qrow : p.Sq - 1;

  // Q and dO rows in B-operand order, delta = <dO row, O row>, L = log-sum-exp in base-2 units
  V8 qf[KK], dof[KK];
  float delta = 0.f;
  {
    const T* qg = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.qs[0] + (int64_t)head * p.qs[1] + (int64_t)qr * p.qs[2];
    const T* og = reinterpret_cast<const T*>(p.o) + (int64_t)b * p.os[0] + (int64_t)head * p.os[1] + (int64_t)qr * p.os[2];
    const T* dg = reinterpret_cast<const T*>(p.d_o) + (int64_t)b * p.dos[0] + (int64_t)head * p.dos[1] + (int64_t)qr * p.dos[2];
    static_for<KK>([&](auto KI) {
      constexpr int kk = decltype(KI)::value;
      qf[kk] = *reinterpret_cast<const V8*>(qg + 16 * kk + 8 * h);
      dof[kk] = *reinterpret_cast<const V8*>(dg + 16 * kk + 8 * h);
      const V8 of = *reinterpret_cast<const V8*>(og + 16 * kk + 8 * h);
      static_for<8>([&](auto EI) {
        constexpr int e = decltype(EI)::value;
        delta = __builtin_fmaf((float)dof[kk][e], (float)of[e], delta);
      });
    });
    delta += __shfl_xor(delta, 32, kWave);
    if (h == 0 && qrow < p.Sq) p.delta[(int64_t)bh * p.Sq + qrow] = delta;
  }
  float L = p.lse[(int64_t)bh * p.Sq + qr] * kLog2e;
  L = L == -INFINITY ? 0.f : L;  // a row without a visible key: every probability below is masked to zero anyway

  const char* kg = reinterpret_cast<const char*>(p.k) + ((int64_t)b * p.ks[0] + (int64_t)hkv * p.ks[1]) * 2;
  const char* vg = reinterpret_cast<const char*>(p.v) + ((int64_t)b * p.vs[0] + (int64_t)hkv * p.vs[1]) * 2;
  const uint32_t k_row_bytes = (uint32_t)(p.ks[2] * 2), v_row_bytes = (uint32_t)(p.vs[2] * 2);
  int ld_row[LPW], ld_chunk[LPW];
  static_for<LPW>([&](auto I) {
    constexpr int i = decltype(I)::value;
    const int pos = (wave * LPW + i) * 1024 + lane * 16;
    ld_row[i] = pos / RB;
    ld_chunk[i] = (((pos % RB) >> 4) ^ swz_v<D>(ld_row[i])) << 4;
  });
  const int n_tiles_all = (p.Skv + BKV - 1) / BKV;
  auto issue = [&](int j, auto STAGE_IDX) {
    constexpr int stage = decltype(STAGE_IDX)::value;
    const int rows_valid = min(BKV, p.Skv - j * BKV);  // rows past the end repeat the last valid row; they are masked below
    const char* kt = kg + (int64_t)j * BKV * k_row_bytes;
    const char* vt = vg + (int64_t)j * BKV * v_row_bytes;
    static_for<LPW>([&](auto I) {
      constexpr int i = decltype(I)::value;
      const uint32_t row = (uint32_t)min(ld_row[i], rows_valid - 1);
      char* kd = smem + stage * STAGE + (wave * LPW + i) * 1024;
      load_to_lds16(kt, row * k_row_bytes + ld_chunk[i], (uint32_t)(size_t)(lvoid*)kd);
      load_to_lds16(vt, row * v_row_bytes + ld_chunk[i], (uint32_t)(size_t)(lvoid*)(kd + TILE));
    });
  };

  int n_steps = n_tiles_all;
  if (p.causal) {
    int q_last = q0 + BQ - 1;
    q_last = q_last < p.Sq ? q_last : p.Sq - 1;
    const int lim = q_last / BKV + 1;
    n_steps = n_steps < lim ? n_steps : lim;
  }
  const int qw_max = q0 + 32 * wave + 31;
  const int sx = swz_v<D>(l32);
  const TrLane TL(lane);
  const int64_t mbase = MASK ? (int64_t)b * p.ms[0] + (int64_t)head * p.ms[1] + (int64_t)qr * p.ms[2] : 0;

  f32x16 dq_acc[DT];
  static_for<DT>([&](auto I) {
    dq_acc[decltype(I)::value] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  });

  auto step = [&](auto STAGE_IDX, int j) {
    constexpr int stage = decltype(STAGE_IDX)::value;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // this wave's part of tile j has landed ...
    __syncthreads();                     // ... everyone's has, and everyone is done with tile j-1
    if (j + 1 < n_steps) issue(j + 1, std::integral_constant<int, stage ^ 1>{});
    const int kv0 = j * BKV;
    if (p.causal && kv0 > qw_max) return;  // wave-uniform: none of these keys is visible to this wave's queries
    const char* k_s = smem + stage * STAGE;
    const char* v_s = k_s + TILE;
    int lim = p.Skv - 1;  // last visible key of this lane's query
    if (p.causal) lim = lim < qrow ? lim : qrow;
    const int rel = lim - kv0 - 4 * h;
    // only tiles that cross the diagonal or the end of the keys pay for the mask (wave-uniform)
    const bool need_mask = (p.causal && kv0 + BKV - 1 > qw_max - 31) || (kv0 + BKV > p.Skv);
    static_for<2>([&](auto TI) {
      constexpr int t = decltype(TI)::value;
      f32x16 s = rows_times_regs<T, D>(k_s, t, l32, h, sx, qf);
      const f32x16 dp = rows_times_regs<T, D>(v_s, t, l32, h, sx, dof);
      float cc = c;
      if constexpr (MASK) {
        // scores in the exponent's base-2 scale with the mask added, as the forward formed them; afterwards cc = 1.
        // Key indices are clamped for the loads; what lies past the end is masked by index below.
        static_for<4>([&](auto GI) {
          constexpr int g = decltype(GI)::value;
          const int key0 = kv0 + 32 * t + 8 * g + 4 * h;
          float m4[4];
          if (p.mask_vec && key0 + 3 < p.Skv) {
            if (p.mask_f32) {
              const f32x4 mv = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p.mask) + mbase + key0);
              m4[0] = mv[0], m4[1] = mv[1], m4[2] = mv[2], m4[3] = mv[3];
            } else {
              typedef T t4 __attribute__((ext_vector_type(4)));
              const t4 mv = *reinterpret_cast<const t4*>(reinterpret_cast<const T*>(p.mask) + mbase + key0);
              m4[0] = (float)mv[0], m4[1] = (float)mv[1], m4[2] = (float)mv[2], m4[3] = (float)mv[3];
            }
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int key = key0 + e < p.Skv ? key0 + e : p.Skv - 1;
              m4[e] = p.mask_f32 ? reinterpret_cast<const float*>(p.mask)[mbase + key] : (float)reinterpret_cast<const T*>(p.mask)[mbase + key];
            }
          }
          static_for<4>([&](auto EI) {
            constexpr int e = decltype(EI)::value;
            s[4 * g + e] = __builtin_fmaf(s[4 * g + e], cc, m4[e] * kLog2e);
          });
        });
        cc = 1.f;
      }
      if (need_mask) {
        static_for<16>([&](auto VI) {
          constexpr int v = decltype(VI)::value;
          constexpr int key = 32 * t + 8 * (v / 4) + (v % 4);
          s[v] = key > rel ? -INFINITY : s[v] * cc;  // scaled here so that a negative scale cannot turn -inf around
        });
        cc = 1.f;
      }
      f32x16 ds;
      static_for<16>([&](auto VI) {
        constexpr int v = decltype(VI)::value;
        const float pr = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], cc, -L));
        ds[v] = pr * (dp[v] - delta);
      });
      transposed_times_held<T, D>(k_s, t, TL, ds, dq_acc);
    });
  };

  if (n_steps > 0) issue(0, std::integral_constant<int, 0>{});
  for (int j = 0; j < n_steps; j += 2) {
    step(std::integral_constant<int, 0>{}, j);
    if (j + 1 < n_steps) step(std::integral_constant<int, 1>{}, j + 1);
  }
  __syncthreads();  // all waves are done reading tiles: the parks reuse the space
  T* dst = reinterpret_cast<T*>(p.dq) + (int64_t)b * p.dqs[0] + (int64_t)head * p.dqs[1] + (int64_t)(q0 + 32 * wave) * p.dqs[2];
  store_rows<T, D>(smem + wave * (32 * RB), dq_acc, scale, dst, p.dqs[2], p.Sq - (q0 + 32 * wave), lane);
}

// ---------------------------------------------------------------------------------------------- dk, dv
// Eight waves of 32 keys: two per SIMD, so one wave's exponentials run beside the other's MFMAs.  A lane's dk and
// dv rows take 128 accumulation registers at D = 128; to stay within the 256 a lane may have at that occupancy only
// the K row of the lane is held in registers, its V row is read from LDS (the workgroup's 256 V rows are loaded
// once, each wave its own 32).
template <typename T, int D, bool MASK = false>
__global__ __launch_bounds__(64 * KW) __attribute__((amdgpu_waves_per_eu(2, 2))) void sdpa_bwd_dkv_kernel(BwdParams p) {
  typedef typename Vec8<T>::type V8;
  constexpr int RB = D * 2, CH = RB / 16, TILE = BKV * RB, KK = D / 16, DT = D / 32, LPW = CH / KW;
  static_assert(LPW * KW == CH, "tile loads must divide evenly over the waves");
  constexpr int STAGE = 2 * TILE + 1024;  // Q tile, dO tile, 64 log-sum-exps, 64 deltas
  constexpr int V_ROWS = 2 * STAGE;       // byte offset of the V rows, behind the two stages
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, h = lane >> 5;
  const float scale = p.scale_dev ? *p.scale_dev : p.scale;
  const float c = scale * kLog2e;

  const int nbk = p.B * p.Hkv, rep = p.H / p.Hkv;
  int bk, kb;  // causal: early key blocks meet the most queries, start them first
  grouped_block_order(blockIdx.x, nbk, p.n_kb, p.group_k, bk, kb);
  const int b = bk / p.Hkv, hkv = bk % p.Hkv;
  const int k0 = kb * BK;
  const int krow = k0 + 32 * wave + l32;
  const int kr = krow < p.Skv ? krow : p.Skv - 1;

  V8 kf[KK];
  {
    const T* kg = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.ks[0] + (int64_t)hkv * p.ks[1] + (int64_t)kr * p.ks[2];
    static_for<KK>([&](auto KI) {
      constexpr int kk = decltype(KI)::value;
      kf[kk] = *reinterpret_cast<const V8*>(kg + 16 * kk + 8 * h);
    });
  }
  // this wave's 32 V rows into LDS, in the layout of a tile block (rows past the end repeat the last valid one);
  // the wait and barrier of the first step cover them
  char* v_rows = smem + V_ROWS + wave * (32 * RB);
  {
    const char* vb = reinterpret_cast<const char*>(p.v) + ((int64_t)b * p.vs[0] + (int64_t)hkv * p.vs[1]) * 2;
    const uint32_t v_row_bytes = (uint32_t)(p.vs[2] * 2);
    const int first = min(k0 + 32 * wave, p.Skv - 1);        // wave-uniform
    const int n_valid = max(p.Skv - (k0 + 32 * wave), 1);    // rows of this block that exist (the clamped one at least)
    const char* base = vb + (int64_t)first * v_row_bytes;
    static_for<32 * RB / 1024>([&](auto I) {
      constexpr int i = decltype(I)::value;
      const int pos = i * 1024 + lane * 16;
      const int row = pos / RB;
      const int chunk = (((pos % RB) >> 4) ^ swz_v<D>(row)) << 4;
      const uint32_t src_row = (uint32_t)min(row, n_valid - 1);
      load_to_lds16(base, src_row * v_row_bytes + chunk, (uint32_t)(size_t)(lvoid*)(v_rows + i * 1024));
    });
  }

  const uint32_t q_row_bytes = (uint32_t)(p.qs[2] * 2), do_row_bytes = (uint32_t)(p.dos[2] * 2);
  int ld_row[LPW], ld_chunk[LPW];
  static_for<LPW>([&](auto I) {
    constexpr int i = decltype(I)::value;
    const int pos = (wave * LPW + i) * 1024 + lane * 16;
    ld_row[i] = pos / RB;
    ld_chunk[i] = (((pos % RB) >> 4) ^ swz_v<D>(ld_row[i])) << 4;
  });
  const int n_qt = (p.Sq + BKV - 1) / BKV;       // query tiles of 64 rows
  const int j0 = p.causal ? k0 / BKV : 0;        // first query tile that sees a key of this block
  const int nj = n_qt > j0 ? n_qt - j0 : 0;
  const int n_iter = nj * rep;                   // (query head of the group, query tile) pairs
  auto issue = [&](int it, auto STAGE_IDX) {
    constexpr int stage = decltype(STAGE_IDX)::value;
    const int head = hkv * rep + it / nj, j = j0 + it % nj;
    const int rows_valid = min(BKV, p.Sq - j * BKV);
    const char* qt = reinterpret_cast<const char*>(p.q) + ((int64_t)b * p.qs[0] + (int64_t)head * p.qs[1] + (int64_t)j * BKV * p.qs[2]) * 2;
    const char* dt = reinterpret_cast<const char*>(p.d_o) + ((int64_t)b * p.dos[0] + (int64_t)head * p.dos[1] + (int64_t)j * BKV * p.dos[2]) * 2;
    static_for<LPW>([&](auto I) {
      constexpr int i = decltype(I)::value;
      const uint32_t row = (uint32_t)min(ld_row[i], rows_valid - 1);
      char* qd = smem + stage * STAGE + (wave * LPW + i) * 1024;
      load_to_lds16(qt, row * q_row_bytes + ld_chunk[i], (uint32_t)(size_t)(lvoid*)qd);
      load_to_lds16(dt, row * do_row_bytes + ld_chunk[i], (uint32_t)(size_t)(lvoid*)(qd + TILE));
    });
    if (wave < 2) {  // wave 0: the tile's log-sum-exps, wave 1: its deltas (one word per lane, clamped to the last row)
      const float* src = (wave == 0 ? p.lse : p.delta) + ((int64_t)b * p.H + head) * p.Sq + (int64_t)j * BKV;
      const uint32_t off = (uint32_t)min(lane, rows_valid - 1) * 4;
      load_to_lds4(src, off, (uint32_t)(size_t)(lvoid*)(smem + stage * STAGE + 2 * TILE + wave * 256));
    }
  };

  const int kw_min = k0 + 32 * wave;
  const int sx = swz_v<D>(l32);
  const TrLane TL(lane);
  f32x16 dk_acc[DT], dv_acc[DT];
  static_for<DT>([&](auto I) {
    dk_acc[decltype(I)::value] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    dv_acc[decltype(I)::value] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  });

  auto step = [&](auto STAGE_IDX, int it) {
    constexpr int stage = decltype(STAGE_IDX)::value;
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    if (it + 1 < n_iter) issue(it + 1, std::integral_constant<int, stage ^ 1>{});
    const int qt0 = (j0 + it % nj) * BKV;
    if (p.causal && qt0 + BKV - 1 < kw_min) return;  // wave-uniform: every query of the tile lies before this wave's keys
    const char* q_s = smem + stage * STAGE;
    const char* do_s = q_s + TILE;
    const char* st_s = do_s + TILE;
    // query 32 t + 8 g + 4 h + e of the tile is visible to this lane's key when it is a real row and not before the key
    const int q_lo = (p.causal ? krow : 0) - qt0 - 4 * h;  // masked when (tile-relative, h-free) index < q_lo
    const int q_hi = p.Sq - qt0 - 4 * h;                   // ... or >= q_hi
    // Probabilities and score gradients of sub-tile t from its scores and dP.  (Measured, not adopted: both
    // sub-tiles' products first and the exponentials of one woven between the MFMAs of the other with scheduling
    // groups -- 689-732 us against 691 us for dq + dk/dv at B4 H32 S2048 D128: with one wave per SIMD the scores sit
    // in accumulation registers, and the moves that hand them to the vector ALU queue behind the MFMAs.)
    // only tiles that cross the diagonal or the end of the queries pay for the mask (wave-uniform)
    const bool need_mask = (p.causal && qt0 < kw_min + 31) || (qt0 + BKV > p.Sq);
    // the probabilities and score gradients leave `soft` rounded and packed, eight per 16-byte fragment: four
    // registers each instead of sixteen, which is what lets two waves share a SIMD's register file
    auto soft = [&](auto TI, f32x16& s, const f32x16& dp, V8 (&prf)[2], V8 (&dsf)[2]) {
      constexpr int t = decltype(TI)::value;
      float cc = c;
      if constexpr (MASK) {
        // the mask element of (query, this lane's key), one load per score: lanes of a half-wave read neighbouring
        // keys of one mask row.  Rows and keys past the end are clamped for the load and masked by index below.
        const int head = hkv * rep + it / nj;
        const int64_t mb = (int64_t)b * p.ms[0] + (int64_t)head * p.ms[1] + kr;
        static_for<16>([&](auto VI) {
          constexpr int v = decltype(VI)::value;
          int qi = qt0 + 32 * t + 8 * (v / 4) + 4 * h + (v % 4);
          qi = qi < p.Sq ? qi : p.Sq - 1;
          const int64_t at = mb + (int64_t)qi * p.ms[2];
          const float m = p.mask_f32 ? reinterpret_cast<const float*>(p.mask)[at] : (float)reinterpret_cast<const T*>(p.mask)[at];
          s[v] = __builtin_fmaf(s[v], cc, m * kLog2e);
        });
        cc = 1.f;
      }
      if (need_mask) {
        static_for<16>([&](auto VI) {
          constexpr int v = decltype(VI)::value;
          constexpr int qi = 32 * t + 8 * (v / 4) + (v % 4);
          s[v] = (qi < q_lo || qi >= q_hi) ? -INFINITY : s[v] * cc;  // scaled here: a negative scale must not turn -inf around
        });
        cc = 1.f;
      }
      static_for<4>([&](auto GI) {
        constexpr int g = decltype(GI)::value;
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(st_s + (32 * t + 8 * g + 4 * h) * 4);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(st_s + 256 + (32 * t + 8 * g + 4 * h) * 4);
        static_for<4>([&](auto EI) {
          constexpr int e = decltype(EI)::value;
          constexpr int v = 4 * g + e;
          // l4 is finite when the row sees a key: a causal row sees at least key 0.  A row that an additive mask
          // hides completely has log-sum-exp -inf and gives NaN here (-inf - (-inf)), as its forward result already
          // is and as the unfused graph's gradients are.
          const float pr = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], cc, -l4[e] * kLog2e));
          prf[v / 8][v % 8] = (T)pr;
          dsf[v / 8][v % 8] = (T)(pr * (dp[v] - d4[e]));
        });
      });
    };
    static_for<2>([&](auto TI) {
      constexpr int t = decltype(TI)::value;
      f32x16 s = rows_times_regs<T, D>(q_s, t, l32, h, sx, kf);
      const f32x16 dp = rows_times_rows<T, D>(do_s, t, l32, h, sx, v_rows);
      V8 prf[2], dsf[2];
      soft(TI, s, dp, prf, dsf);
      // nothing of the products below is started before the fragments above exist, and the next sub-tile waits for
      // this one: what is in flight at once has to fit the 256 registers of a lane
      __builtin_amdgcn_sched_barrier(0);
      transposed_times_packed<T, D>(do_s, t, TL, prf, dv_acc);
      transposed_times_packed<T, D>(q_s, t, TL, dsf, dk_acc);
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  if (n_iter > 0) issue(0, std::integral_constant<int, 0>{});
  for (int it = 0; it < n_iter; it += 2) {
    step(std::integral_constant<int, 0>{}, it);
    if (it + 1 < n_iter) step(std::integral_constant<int, 1>{}, it + 1);
  }
  __syncthreads();
  const int row0 = k0 + 32 * wave;
  char* park = smem + wave * (32 * RB);
  T* dk_dst = reinterpret_cast<T*>(p.dk) + (int64_t)b * p.dks[0] + (int64_t)hkv * p.dks[1] + (int64_t)row0 * p.dks[2];
  T* dv_dst = reinterpret_cast<T*>(p.dv) + (int64_t)b * p.dvs[0] + (int64_t)hkv * p.dvs[1] + (int64_t)row0 * p.dvs[2];
  store_rows<T, D>(park, dk_acc, scale, dk_dst, p.dks[2], p.Skv - row0, lane);
  __syncthreads();  // the parks have been read back before they are written again
  store_rows<T, D>(park, dv_acc, 1.f, dv_dst, p.dvs[2], p.Skv - row0, lane);
}

template <typename T, int D, bool MASK = false>
int launch_bwd(const BwdParams& p, hipStream_t stream) {
  constexpr int SMEM_DQ = 2 * 2 * BKV * D * 2;
  constexpr int SMEM_DKV = 2 * (2 * BKV * D * 2 + 1024) + BK * D * 2;
  auto dq_kernel = sdpa_bwd_dq_kernel<T, D, MASK>;
  auto dkv_kernel = sdpa_bwd_dkv_kernel<T, D, MASK>;
  if (int st = allow_dynamic_lds(reinterpret_cast<const void*>(dq_kernel), SMEM_DQ)) return st;
  if (int st = allow_dynamic_lds(reinterpret_cast<const void*>(dkv_kernel), SMEM_DKV)) return st;
  hipLaunchKernelGGL(dq_kernel, dim3((unsigned)((int64_t)p.B * p.H * p.n_qb)), dim3(kThreads), SMEM_DQ, stream, p);
  if (hipGetLastError() != hipSuccess) return XG_ERR_LAUNCH;
  hipLaunchKernelGGL(dkv_kernel, dim3((unsigned)((int64_t)p.B * p.Hkv * p.n_kb)), dim3(64 * KW), SMEM_DKV, stream, p);
  return status_from_hip(hipGetLastError());
}

}  // namespace sdpa
}  // namespace xg

namespace {

int backward_entry(const void* q, const void* k, const void* v, const void* out, const void* d_out, const float* lse, const void* mask,
                   const int64_t* mask_strides, int mask_dtype, const float* scale_dev, void* dq, void* dk, void* dv, float* delta_ws, int64_t B, int64_t H, int64_t Hkv, int64_t Sq, int64_t Skv, int64_t D,
                   const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3],
                   const int64_t do_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3], const int64_t dv_strides[3],
                   float scale, int causal, int dtype, xg_stream_t stream) {
  using namespace xg;
  if (dtype != XG_BF16 && dtype != XG_F16) return XG_ERR_BAD_DTYPE;
  if (B < 0 || H < 0 || Hkv < 0 || Sq < 0 || Skv < 0) return XG_ERR_BAD_SHAPE;
  if (D != 64 && D != 128) return XG_ERR_BAD_SHAPE;
  if (B == 0 || H == 0) return XG_OK;
  if (Hkv == 0 || H % Hkv != 0 || Sq == 0 || Skv == 0) return XG_ERR_BAD_SHAPE;
  if (!q || !k || !v || !out || !d_out || !lse || !dq || !dk || !dv || !delta_ws) return XG_ERR_NULL_PTR;
  if (!q_strides || !k_strides || !v_strides || !o_strides || !do_strides || !dq_strides || !dk_strides || !dv_strides) return XG_ERR_NULL_PTR;
  if (!(scale == scale) || fabsf(scale) > 3.0e38f) return XG_ERR_BAD_ARG;
  if (Sq > (1 << 30) || Skv > (1 << 30)) return XG_ERR_TOO_LARGE;
  const int64_t n_qb = (Sq + sdpa::BQ - 1) / sdpa::BQ, n_kb = (Skv + sdpa::BK - 1) / sdpa::BK;
  if (B * H > (1 << 24) || B * H * n_qb > 0x7fffffffLL || B * Hkv * n_kb > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  const void* ptrs[] = {q, k, v, out, d_out, dq, dk, dv};
  for (const void* ptr : ptrs)
    if (!aligned_to(ptr, 16)) return XG_ERR_BAD_ALIGN;
  if (!aligned_to(lse, 4) || !aligned_to(delta_ws, 4)) return XG_ERR_BAD_ALIGN;
  sdpa::BwdParams p;
  for (int i = 0; i < 3; ++i) {
    const int64_t s8[] = {q_strides[i], k_strides[i], v_strides[i], o_strides[i], do_strides[i], dq_strides[i], dk_strides[i], dv_strides[i]};
    for (int64_t s : s8) {
      if (s < 0) return XG_ERR_BAD_SHAPE;
      if (s % 8) return XG_ERR_BAD_ALIGN;
    }
    p.qs[i] = q_strides[i];
    p.ks[i] = k_strides[i];
    p.vs[i] = v_strides[i];
    p.os[i] = o_strides[i];
    p.dos[i] = do_strides[i];
    p.dqs[i] = dq_strides[i];
    p.dks[i] = dk_strides[i];
    p.dvs[i] = dv_strides[i];
  }
  // the outputs are written, so their rows must not overlap: every row holds D elements
  if (dq_strides[2] < D || dk_strides[2] < D || dv_strides[2] < D) return XG_ERR_BAD_SHAPE;
  // per-lane tile offsets are 32-bit: 64 rows of a streamed operand must span less than 2 GiB
  if (k_strides[2] > (1 << 23) || v_strides[2] > (1 << 23) || q_strides[2] > (1 << 23) || do_strides[2] > (1 << 23)) return XG_ERR_TOO_LARGE;
  p.q = q;
  p.k = k;
  p.v = v;
  p.o = out;
  p.d_o = d_out;
  p.lse = lse;
  p.delta = delta_ws;
  p.dq = dq;
  p.dk = dk;
  p.dv = dv;
  p.B = (int)B;
  p.H = (int)H;
  p.Hkv = (int)Hkv;
  p.Sq = (int)Sq;
  p.Skv = (int)Skv;
  p.scale = scale;
  if (scale_dev && !aligned_to(scale_dev, 4)) return XG_ERR_BAD_ALIGN;
  p.scale_dev = scale_dev;
  p.mask = mask;
  p.mask_f32 = 0;
  p.mask_vec = 0;
  p.ms[0] = p.ms[1] = p.ms[2] = 0;
  if (mask) {  // the same conditions as the forward's
    if (!mask_strides) return XG_ERR_NULL_PTR;
    if (mask_dtype != dtype && mask_dtype != XG_F32) return XG_ERR_BAD_DTYPE;
    const size_t esz = mask_dtype == XG_F32 ? 4 : 2;
    if (!aligned_to(mask, esz)) return XG_ERR_BAD_ALIGN;
    bool vec = aligned_to(mask, 4 * esz);
    for (int i = 0; i < 3; ++i) {
      if (mask_strides[i] < 0) return XG_ERR_BAD_SHAPE;
      p.ms[i] = mask_strides[i];
      vec = vec && mask_strides[i] % 4 == 0;
    }
    if (Sq > 1 && mask_strides[2] != 0 && mask_strides[2] < Skv) return XG_ERR_BAD_SHAPE;  // rows would overlap
    p.mask_f32 = mask_dtype == XG_F32 ? 1 : 0;
    p.mask_vec = vec ? 1 : 0;
  }
  p.causal = causal ? 1 : 0;
  p.n_qb = (int)n_qb;
  p.n_kb = (int)n_kb;
  p.group_q = sdpa::block_order_group(B * H);
  p.group_k = sdpa::block_order_group(B * Hkv);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (mask) {
    if (dtype == XG_BF16) return D == 128 ? sdpa::launch_bwd<bf16_t, 128, true>(p, st) : sdpa::launch_bwd<bf16_t, 64, true>(p, st);
    return D == 128 ? sdpa::launch_bwd<f16_t, 128, true>(p, st) : sdpa::launch_bwd<f16_t, 64, true>(p, st);
  }
  if (dtype == XG_BF16) return D == 128 ? sdpa::launch_bwd<bf16_t, 128>(p, st) : sdpa::launch_bwd<bf16_t, 64>(p, st);
  return D == 128 ? sdpa::launch_bwd<f16_t, 128>(p, st) : sdpa::launch_bwd<f16_t, 64>(p, st);
}

}  // namespace

// The delta workspace of xg_sdpa_backward_static: one per GPU, held until the process ends.
constexpr int64_t kScratchFloats = int64_t(1) << 21;  // 8 MiB: B * H * Sq <= 2 097 152 query rows per call
static __device__ __align__(256) float scratch[kScratchFloats];

// Device address of `scratch` on the current GPU (every GPU holds its own copy of the array at its own address;
// the array's name is only a host-side handle).  Looked up once per device.
static int scratch_address(float** out) {
  static std::mutex mu;
  static std::map<int, float*> known;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return XG_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(mu);
  auto it = known.find(dev);
  if (it == known.end()) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) return XG_ERR_LAUNCH;
    it = known.emplace(dev, static_cast<float*>(ptr)).first;
  }
  *out = it->second;
  return XG_OK;
}

extern "C" int xg_sdpa_backward(const void* q, const void* k, const void* v, const void* out, const void* d_out, const float* lse,
                                void* dq, void* dk, void* dv, float* delta_ws, int64_t B, int64_t H, int64_t Hkv, int64_t Sq,
                                int64_t Skv, int64_t D, const int64_t q_strides[3], const int64_t k_strides[3],
                                const int64_t v_strides[3], const int64_t o_strides[3], const int64_t do_strides[3],
                                const int64_t dq_strides[3], const int64_t dk_strides[3], const int64_t dv_strides[3], float scale,
                                int causal, int dtype, xg_stream_t stream) {
  return backward_entry(q, k, v, out, d_out, lse, nullptr, nullptr, dtype, nullptr, dq, dk, dv, delta_ws, B, H, Hkv, Sq, Skv, D, q_strides,
                        k_strides, v_strides, o_strides, do_strides, dq_strides, dk_strides, dv_strides, scale, causal, dtype, stream);
}

extern "C" int xg_sdpa_backward_masked(const void* q, const void* k, const void* v, const void* out, const void* d_out, const float* lse,
                                       const void* mask, const int64_t mask_strides[3], int mask_dtype, const float* scale_dev, void* dq,
                                       void* dk, void* dv, float* delta_ws, int64_t B, int64_t H, int64_t Hkv, int64_t Sq, int64_t Skv,
                                       int64_t D, const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                                       const int64_t o_strides[3], const int64_t do_strides[3], const int64_t dq_strides[3],
                                       const int64_t dk_strides[3], const int64_t dv_strides[3], float scale, int causal, int dtype,
                                       xg_stream_t stream) {
  return backward_entry(q, k, v, out, d_out, lse, mask, mask_strides, mask_dtype, scale_dev, dq, dk, dv, delta_ws, B, H, Hkv, Sq, Skv, D,
                        q_strides, k_strides, v_strides, o_strides, do_strides, dq_strides, dk_strides, dv_strides, scale, causal, dtype,
                        stream);
}

extern "C" int xg_sdpa_backward_static(const void* q, const void* k, const void* v, const void* out, const void* d_out,
                                       const float* lse, void* dq, void* dk, void* dv, int64_t B, int64_t H, int64_t Hkv, int64_t Sq,
                                       int64_t Skv, int64_t D, const int64_t q_strides[3], const int64_t k_strides[3],
                                       const int64_t v_strides[3], const int64_t o_strides[3], const int64_t do_strides[3],
                                       const int64_t dq_strides[3], const int64_t dk_strides[3], const int64_t dv_strides[3],
                                       float scale, int causal, int dtype, xg_stream_t stream) {
  if (B < 0 || H < 0 || Sq < 0) return XG_ERR_BAD_SHAPE;
  if (B > kScratchFloats || H > kScratchFloats || Sq > kScratchFloats || B * H > kScratchFloats || B * H * Sq > kScratchFloats)
    return XG_ERR_TOO_LARGE;  // more query rows than the static workspace holds: use xg_sdpa_backward
  if (B == 0 || H == 0) return XG_OK;
  float* ws = nullptr;
  if (int st = scratch_address(&ws)) return st;
  return backward_entry(q, k, v, out, d_out, lse, nullptr, nullptr, dtype, nullptr, dq, dk, dv, ws, B, H, Hkv, Sq, Skv, D, q_strides, k_strides,
                        v_strides, o_strides, do_strides, dq_strides, dk_strides, dv_strides, scale, causal, dtype, stream);
}
