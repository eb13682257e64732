// Attention for a decode step on gfx950: at most 32 query rows per head, optional additive mask, no causal flag.
//
// The general forward kernel gives every workgroup 128 query rows and lets it walk all keys: with one query row per
// head that is B x H workgroups, each streaming a whole K and V through one compute unit.  Here the KEYS are split
// instead:
//   workgroup = one (batch, key/value head, key range); its query rows are the Sq rows of every query head of the
//     group (rep x Sq <= 32 rows, packed into one 32-column MFMA tile), so K and V are read once per key/value head;
//     when rep x Sq exceeds 32 the query heads go one per workgroup (Sq <= 32).
//   tile = 128 keys, moved by `global_load_lds_dwordx4` into two stages (K tile, then V tile); wave w owns keys
//     32 w .. 32 w + 31 of every tile: S^T = K Q^T (8 or 4 MFMAs), its own running maximum and sum, O^T += V^T P^T.
//   at the end the four waves' (maximum, sum, O) are merged through LDS; with several key ranges per head the merged
//     partial goes to the workspace and a second small kernel merges the ranges the same way.
// Fragment layouts, swizzles and the permuted k index of V^T P^T are those of the general kernel (sdpa.hip).
#include "sdpa_common.hpp"

namespace xg {
namespace sdpa {

constexpr int DKV = 128;      // keys per tile
constexpr int DROWS = 32;     // query rows a workgroup holds

struct DecodeParams {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  float* lse;  // optional [B, H, Sq]
  float* ws;   // n_split > 1: per (problem, split) 32 x D partial outputs, then 32 maxima, then 32 sums
  int B, H, Hkv, Sq, Skv;
  int64_t qs[3], ks[3], vs[3], os[3];
  float c;         // scale * log2(e)
  const float* scale_dev;  // when set: the scale is read from this one-element device tensor instead
  const void* mask;        // additive mask (MASK kernels only), element [b, h, i, j] at ms[0] b + ms[1] h + ms[2] i + j
  int64_t ms[3];           // element strides of batch, head, query row (0: broadcast)
  int mask_f32;            // mask elements are fp32 (else the dtype of q)
  int mask_vec;            // rows of the mask can be read four elements at a time
  int pack;        // query heads per workgroup (H / Hkv, or 1)
  int n_split;     // key ranges per problem
  int tiles_per_split;
};

// 16 bytes per lane from global memory straight into LDS: lane i's chunk lands at lds_base + 16 i.
__device__ __forceinline__ void decode_load16(const void* base, uint32_t lane_off, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(lane_off), "s"(base) : "memory", "m0");
}

template <int D>
constexpr int decode_ws_floats() {
  return DROWS * D + 2 * DROWS;
}

// Merge n partial results of one query row: out = sum_i 2^(m_i - M) o_i, L = sum_i 2^(m_i - M) l_i, M = max m_i.
// A partial without any visible key has m = -inf and weight 0; a row that a mask hides completely has sum 0 and comes
// out as NaN (0 / 0), as in eager.
template <typename T, int D>
__device__ __forceinline__ void store_row_part(const DecodeParams& p, int b, int head0, int r, int d0, const float (&acc)[D / 8], float M, float L) {
  const int rows = p.pack * p.Sq;
  if (r >= rows) return;
  const int head = head0 + r / p.Sq, sq = r % p.Sq;
  const float inv = 1.f / L;
  T* og = reinterpret_cast<T*>(p.o) + (int64_t)b * p.os[0] + (int64_t)head * p.os[1] + (int64_t)sq * p.os[2] + d0;
  typedef T t8 __attribute__((ext_vector_type(8)));
  static_for<D / 64>([&](auto I) {
    constexpr int i = decltype(I)::value;
    t8 w;
    static_for<8>([&](auto EI) {
      constexpr int e = decltype(EI)::value;
      w[e] = (T)(acc[8 * i + e] * inv);
    });
    *reinterpret_cast<t8*>(og + 8 * i) = w;
  });
  if (p.lse && d0 == 0) p.lse[((int64_t)b * p.H + head) * p.Sq + sq] = (M + log2f(L)) * 0.69314718055994530942f;
}

// MASK: an additive mask is added to the scaled scores, as in the general kernel; a row whose every key is masked with
// -inf comes out as NaN, as it does in eager.
template <typename T, int D, bool MASK = false>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 2))) void sdpa_decode_kernel(DecodeParams p) {
  typedef typename Vec8<T>::type V8;
  constexpr int RB = D * 2, TILE = DKV * RB, STAGE = 2 * TILE, KK = D / 16, DT = D / 32;
  constexpr int LPW = TILE / 1024 / 4;  // direct loads per wave per operand tile
  constexpr int PITCH = D + 4;          // floats per parked row
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, h = lane >> 5;

  const int n_hg = p.H / p.pack;  // workgroup problems per batch entry
  const int split = blockIdx.x % p.n_split, prob = blockIdx.x / p.n_split;
  const int b = prob / n_hg, hg = prob % n_hg;
  const int head0 = hg * p.pack, hkv = head0 / (p.H / p.Hkv);
  const int rows = p.pack * p.Sq;

  const float c_eff = p.scale_dev ? *p.scale_dev * 1.44269504088896340736f : p.c;

  // ---- this lane's query row (rows past the end repeat the last one; they are not stored)
  V8 qf[KK];
  int64_t mbase = 0;
  {
    const int r = l32 < rows ? l32 : rows - 1;
    const int head = head0 + r / p.Sq, sq = r % p.Sq;
    if constexpr (MASK) mbase = (int64_t)b * p.ms[0] + (int64_t)head * p.ms[1] + (int64_t)sq * p.ms[2];
    const T* qg = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.qs[0] + (int64_t)head * p.qs[1] + (int64_t)sq * p.qs[2];
    static_for<KK>([&](auto KI) {
      constexpr int kk = decltype(KI)::value;
      qf[kk] = *reinterpret_cast<const V8*>(qg + 16 * kk + 8 * h);
    });
  }

  const int n_tiles_all = (p.Skv + DKV - 1) / DKV;
  const int t0 = split * p.tiles_per_split;
  const int t1 = min(t0 + p.tiles_per_split, n_tiles_all);
  const char* kg = reinterpret_cast<const char*>(p.k) + ((int64_t)b * p.ks[0] + (int64_t)hkv * p.ks[1]) * 2;
  const char* vg = reinterpret_cast<const char*>(p.v) + ((int64_t)b * p.vs[0] + (int64_t)hkv * p.vs[1]) * 2;
  const uint32_t k_row_bytes = (uint32_t)(p.ks[2] * 2), v_row_bytes = (uint32_t)(p.vs[2] * 2);
  int ld_row[LPW], ld_kc[LPW], ld_vc[LPW];
  static_for<LPW>([&](auto I) {
    constexpr int i = decltype(I)::value;
    const int pos = (wave * LPW + i) * 1024 + lane * 16;
    ld_row[i] = pos / RB;
    const int pc = (pos % RB) >> 4;
    ld_kc[i] = (pc ^ swz_k<D>(ld_row[i])) << 4;
    ld_vc[i] = (pc ^ swz_v<D>(ld_row[i])) << 4;
  });
  auto issue = [&](int j, int stage) {
    const int rows_valid = min(DKV, p.Skv - j * DKV);  // rows past the end repeat the last valid row; they are masked below
    const char* kt = kg + (int64_t)j * DKV * k_row_bytes;
    const char* vt = vg + (int64_t)j * DKV * v_row_bytes;
    static_for<LPW>([&](auto I) {
      constexpr int i = decltype(I)::value;
      const uint32_t row = (uint32_t)min(ld_row[i], rows_valid - 1);
      char* kd = smem + stage * STAGE + (wave * LPW + i) * 1024;
      decode_load16(kt, row * k_row_bytes + ld_kc[i], (uint32_t)(size_t)(lvoid*)kd);
      decode_load16(vt, row * v_row_bytes + ld_vc[i], (uint32_t)(size_t)(lvoid*)(kd + TILE));
    });
  };

  // ---- per-lane parts of the fragment addresses (see the general kernel)
  const int a16 = lane & 15, b16 = (lane >> 4) & 1;
  const int v_row = 4 * h + (a16 >> 2);
  const int v_chunk = 2 * b16 + ((a16 & 3) >> 1), v_sub = (a16 & 1) << 3;
  const int k_lane = (32 * wave + l32) * RB, kx = swz_k<D>(l32);

  f32x16 o_acc[DT];
  static_for<DT>([&](auto I) {
    o_acc[decltype(I)::value] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  });
  float m_run = -INFINITY, l_run = 0.f;

  if (t0 < t1) issue(t0, 0);
  for (int j = t0; j < t1; ++j) {
    const int stage = (j - t0) & 1;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // this wave's part of tile j has landed ...
    __syncthreads();                     // ... everyone's has, and everyone is done with tile j - 1
    if (j + 1 < t1) issue(j + 1, stage ^ 1);
    const char* k_s = smem + stage * STAGE;
    const char* v_s = k_s + TILE;
    const int key0 = j * DKV + 32 * wave;  // first key of this wave's block
    if (key0 >= p.Skv) continue;           // wave-uniform: the block lies past the end (the barrier above was reached)

    f32x16 s = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    static_for<KK>([&](auto KI) {
      constexpr int kk = decltype(KI)::value;
      const V8 kf = *reinterpret_cast<const V8*>(k_s + k_lane + (((2 * kk + h) ^ kx) << 4));
      s = mma(kf, qf[kk], s);
    });
    // s[v] = <key key0 + 8 (v / 4) + 4 h + v % 4, query row l32>, scaled to the exponent's base 2; keys past the end -> -inf
    const int rel = p.Skv - 1 - key0 - 4 * h;
    if constexpr (MASK) {
      // key indices are clamped for the loads; what lies past the end is masked by index below
      constexpr float kLog2e = 1.44269504088896340736f;
      static_for<4>([&](auto GI) {
        constexpr int g = decltype(GI)::value;
        const int kfirst = key0 + 8 * g + 4 * h;
        float m4[4];
        if (p.mask_vec && kfirst + 3 < p.Skv) {
          if (p.mask_f32) {
            const f32x4 mv = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p.mask) + mbase + kfirst);
            m4[0] = mv[0], m4[1] = mv[1], m4[2] = mv[2], m4[3] = mv[3];
          } else {
            typedef T t4 __attribute__((ext_vector_type(4)));
            const t4 mv = *reinterpret_cast<const t4*>(reinterpret_cast<const T*>(p.mask) + mbase + kfirst);
            m4[0] = (float)mv[0], m4[1] = (float)mv[1], m4[2] = (float)mv[2], m4[3] = (float)mv[3];
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int key = kfirst + e < p.Skv ? kfirst + e : p.Skv - 1;
            m4[e] = p.mask_f32 ? reinterpret_cast<const float*>(p.mask)[mbase + key] : (float)reinterpret_cast<const T*>(p.mask)[mbase + key];
          }
        }
        static_for<4>([&](auto EI) {
          constexpr int e = decltype(EI)::value;
          s[4 * g + e] = __builtin_fmaf(s[4 * g + e], c_eff, m4[e] * kLog2e);
        });
      });
    }
    float mx = -INFINITY;
    static_for<16>([&](auto VI) {
      constexpr int v = decltype(VI)::value;
      constexpr int key = 8 * (v / 4) + (v % 4);
      s[v] = key > rel ? -INFINITY : (MASK ? s[v] : s[v] * c_eff);
      mx = fmaxf(mx, s[v]);
    });
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));  // lanes l and l ^ 32 share a query row
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a row that a mask has hidden completely so far
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
    float psum = 0.f;
    static_for<16>([&](auto VI) {
      constexpr int v = decltype(VI)::value;
      const float e = __builtin_amdgcn_exp2f(s[v] - m_use);
      s[v] = e;
      psum += e;
    });
    l_run = __builtin_fmaf(l_run, alpha, psum);
    static_for<DT>([&](auto I) { o_acc[decltype(I)::value] *= alpha; });
    m_run = m_new;

    static_for<2>([&](auto SI) {
      constexpr int st = decltype(SI)::value;
      V8 pf;
      static_for<8>([&](auto JI) {
        constexpr int jj = decltype(JI)::value;
        pf[jj] = (T)s[8 * st + jj];
      });
      static_for<DT>([&](auto DI) {
        constexpr int dt = decltype(DI)::value;
        const int r0 = 32 * wave + 16 * st + v_row, r1 = r0 + 8;
        const char* a0 = v_s + r0 * RB + (((4 * dt + v_chunk) ^ swz_v<D>(v_row)) << 4) + v_sub;
        const char* a1 = v_s + r1 * RB + (((4 * dt + v_chunk) ^ swz_v<D>(v_row + 8)) << 4) + v_sub;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)a0);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)a1);
        const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        o_acc[dt] = mma(__builtin_bit_cast(V8, both), pf, o_acc[dt]);
      });
    });
  }

  // ---- merge the four waves: park O^T as [wave][row][D] fp32, maxima and sums behind it
  const float l_tot = l_run + __shfl_xor(l_run, 32, kWave);
  __syncthreads();  // all waves are done reading tiles
  float* park = reinterpret_cast<float*>(smem);
  float* stat = park + 4 * DROWS * PITCH;  // [wave][2][32]
  static_for<DT>([&](auto DI) {
    constexpr int dt = decltype(DI)::value;
    static_for<4>([&](auto GI) {
      constexpr int g = decltype(GI)::value;
      const f32x4 w = {o_acc[dt][4 * g], o_acc[dt][4 * g + 1], o_acc[dt][4 * g + 2], o_acc[dt][4 * g + 3]};
      *reinterpret_cast<f32x4*>(park + (wave * DROWS + l32) * PITCH + 32 * dt + 8 * g + 4 * h) = w;
    });
  });
  if (h == 0) {
    stat[wave * 64 + l32] = m_run;
    stat[wave * 64 + 32 + l32] = l_tot;
  }
  __syncthreads();
  constexpr int PER = D / 8;  // output columns per thread: 256 threads cover 32 rows x D
  const int r = tid >> 3, d0 = (tid & 7) * PER;
  if (r >= rows) return;  // no barrier follows
  float M = -INFINITY;
#pragma unroll
  for (int w = 0; w < 4; ++w) M = fmaxf(M, stat[w * 64 + r]);
  float L = 0.f, acc[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) acc[e] = 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const float mw = stat[w * 64 + r];
    const float f = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - M);  // a wave that saw no visible key adds nothing
    L = __builtin_fmaf(stat[w * 64 + 32 + r], f, L);
#pragma unroll
    for (int e = 0; e < PER; e += 4) {
      const f32x4 o4 = *reinterpret_cast<const f32x4*>(park + (w * DROWS + r) * PITCH + d0 + e);
      acc[e] = __builtin_fmaf(o4[0], f, acc[e]);
      acc[e + 1] = __builtin_fmaf(o4[1], f, acc[e + 1]);
      acc[e + 2] = __builtin_fmaf(o4[2], f, acc[e + 2]);
      acc[e + 3] = __builtin_fmaf(o4[3], f, acc[e + 3]);
    }
  }
  if (p.n_split == 1) {
    store_row_part<T, D>(p, b, head0, r, d0, acc, M, L);
  } else {
    float* dst = p.ws + (int64_t)blockIdx.x * decode_ws_floats<D>();
#pragma unroll
    for (int e = 0; e < PER; e += 4) *reinterpret_cast<f32x4*>(dst + r * D + d0 + e) = f32x4{acc[e], acc[e + 1], acc[e + 2], acc[e + 3]};
    if ((tid & 7) == 0) {
      dst[DROWS * D + r] = M;
      dst[DROWS * D + DROWS + r] = L;
    }
  }
}

// Merge the key ranges of one problem.  A thread owns four output columns of one query row (the rows that exist are
// dealt over the 256 threads) and walks the ranges with a running maximum, sixteen at a time so that their loads are in
// flight together: the kernel is a chain of memory round trips and nothing else.
template <typename T, int D>
__global__ __launch_bounds__(kThreads) void sdpa_decode_merge_kernel(DecodeParams p) {
  constexpr int WS = decode_ws_floats<D>(), G = 16, CPR = D / 4;  // four-column chunks per row
  const int prob = blockIdx.x, n_hg = p.H / p.pack;
  const int b = prob / n_hg, head0 = (prob % n_hg) * p.pack;
  const int rows = p.pack * p.Sq;
  const float* src = p.ws + (int64_t)prob * p.n_split * WS;
  for (int item = threadIdx.x; item < rows * CPR; item += kThreads) {
    const int r = item / CPR, d0 = (item % CPR) * 4;
    float M = -INFINITY, L = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < p.n_split; s0 += G) {
      float m[G], l[G];
      f32x4 o4[G];
#pragma unroll
      for (int u = 0; u < G; ++u) {
        const int s = s0 + u < p.n_split ? s0 + u : p.n_split - 1;  // a repeated range gets weight 0 below
        const float* part = src + (int64_t)s * WS;
        m[u] = part[DROWS * D + r];
        l[u] = part[DROWS * D + DROWS + r];
        o4[u] = *reinterpret_cast<const f32x4*>(part + r * D + d0);
      }
      float Mg = M;
#pragma unroll
      for (int u = 0; u < G; ++u) Mg = fmaxf(Mg, s0 + u < p.n_split ? m[u] : -INFINITY);
      const float keep = M == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(M - Mg);  // what was summed so far, at the new reference
      L *= keep;
      acc *= keep;
#pragma unroll
      for (int u = 0; u < G; ++u) {
        const float w = (s0 + u < p.n_split && m[u] != -INFINITY) ? __builtin_amdgcn_exp2f(m[u] - Mg) : 0.f;  // a range without a visible key adds nothing
        L = __builtin_fmaf(l[u], w, L);
        acc += o4[u] * w;
      }
      M = Mg;
    }
    const int head = head0 + r / p.Sq, sq = r % p.Sq;
    const float inv = 1.f / L;
    typedef T t4 __attribute__((ext_vector_type(4)));
    const t4 w4 = {(T)(acc[0] * inv), (T)(acc[1] * inv), (T)(acc[2] * inv), (T)(acc[3] * inv)};
    *reinterpret_cast<t4*>(reinterpret_cast<T*>(p.o) + (int64_t)b * p.os[0] + (int64_t)head * p.os[1] + (int64_t)sq * p.os[2] + d0) = w4;
    if (p.lse && d0 == 0) p.lse[((int64_t)b * p.H + head) * p.Sq + sq] = (M + log2f(L)) * 0.69314718055994530942f;
  }
}

// How the keys of one problem are split: one workgroup per compute unit, whole tiles per range.  A workgroup pays
// ~5 us before its first tile and after its last that nothing hides (it has the CU's LDS to itself), so more, shorter
// workgroups lose: B8 H32 Hkv8 Skv8192 53.8 us at 256 workgroups, 57.2 at 512, 60.4 at 768, 68.4 at 128.  Without a GPU
// (argument checks on a host) the published 256 compute units stand in.
inline int decode_cu_count() {
  static const int n = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    return cus;
  }();
  return n;
}
inline void decode_split(int64_t problems, int64_t Skv, int& n_split, int& tiles_per_split) {
  const int64_t n_tiles = (Skv + DKV - 1) / DKV;
  int64_t want = (decode_cu_count() + problems - 1) / problems;
  want = want < 1 ? 1 : (want > n_tiles ? n_tiles : want);
  const int64_t tps = (n_tiles + want - 1) / want;
  tiles_per_split = (int)tps;
  n_split = (int)((n_tiles + tps - 1) / tps);
}

template <typename T, int D, bool MASK = false>
int launch_decode(const DecodeParams& p, hipStream_t stream) {
  constexpr int STAGES = 2 * 2 * DKV * D * 2;
  constexpr int PARK = (4 * DROWS * (D + 4) + 4 * 64) * 4;
  constexpr int SMEM = STAGES > PARK ? STAGES : PARK;
  auto kernel = sdpa_decode_kernel<T, D, MASK>;
  if (int st = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), SMEM)) return st;
  const int64_t problems = (int64_t)p.B * (p.H / p.pack);
  hipLaunchKernelGGL(kernel, dim3((unsigned)(problems * p.n_split)), dim3(kThreads), SMEM, stream, p);
  if (hipGetLastError() != hipSuccess) return XG_ERR_LAUNCH;
  if (p.n_split > 1) hipLaunchKernelGGL((sdpa_decode_merge_kernel<T, D>), dim3((unsigned)problems), dim3(kThreads), 0, stream, p);
  return status_from_hip(hipGetLastError());
}

}  // namespace sdpa
}  // namespace xg

namespace {

// Query heads per workgroup: the whole group when its rows fit the tile, else one head.
int decode_pack(int64_t H, int64_t Hkv, int64_t Sq) {
  const int64_t rep = H / Hkv;
  return rep * Sq <= xg::sdpa::DROWS ? (int)rep : 1;
}

}  // namespace

extern "C" int64_t xg_sdpa_decode_workspace_floats(int64_t B, int64_t H, int64_t Hkv, int64_t Sq, int64_t Skv, int64_t D) {
  using namespace xg;
  if (B <= 0 || H <= 0 || Hkv <= 0 || Sq <= 0 || Skv <= 0 || H % Hkv != 0 || Sq > sdpa::DROWS || (D != 64 && D != 128)) return 0;
  const int64_t problems = B * (H / decode_pack(H, Hkv, Sq));
  int n_split = 1, tps = 1;
  sdpa::decode_split(problems, Skv, n_split, tps);
  if (n_split <= 1) return 0;
  return problems * n_split * (D == 128 ? sdpa::decode_ws_floats<128>() : sdpa::decode_ws_floats<64>());
}

extern "C" int xg_sdpa_decode(const void* q, const void* k, const void* v, void* out, float* lse, const void* mask,
                              const int64_t mask_strides[3], int mask_dtype, const float* scale_dev, float* workspace, int64_t workspace_floats,
                              int64_t B, int64_t H, int64_t Hkv, int64_t Sq, int64_t Skv, int64_t D, const int64_t q_strides[3],
                              const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3], float scale, int dtype,
                              xg_stream_t stream) {
  using namespace xg;
  if (dtype != XG_BF16 && dtype != XG_F16) return XG_ERR_BAD_DTYPE;
  if (B < 0 || H < 0 || Hkv < 0 || Sq < 0 || Skv < 0 || workspace_floats < 0) return XG_ERR_BAD_SHAPE;
  if (D != 64 && D != 128) return XG_ERR_BAD_SHAPE;
  if (Sq > sdpa::DROWS) return XG_ERR_BAD_SHAPE;  // more query rows than a workgroup holds: use xg_sdpa
  if (B == 0 || H == 0 || Sq == 0) return XG_OK;
  if (Hkv == 0 || H % Hkv != 0 || Skv == 0) return XG_ERR_BAD_SHAPE;
  if (!q || !k || !v || !out || !q_strides || !k_strides || !v_strides || !o_strides) return XG_ERR_NULL_PTR;
  if (!(scale == scale) || fabsf(scale) > 3.0e38f) return XG_ERR_BAD_ARG;
  if (Skv > (1 << 30) || B * H > (1 << 24)) return XG_ERR_TOO_LARGE;
  if (!aligned_to(q, 16) || !aligned_to(k, 16) || !aligned_to(v, 16) || !aligned_to(out, 16)) return XG_ERR_BAD_ALIGN;
  if ((lse && !aligned_to(lse, 4)) || (workspace && !aligned_to(workspace, 16))) return XG_ERR_BAD_ALIGN;
  sdpa::DecodeParams p;
  for (int i = 0; i < 3; ++i) {
    if (q_strides[i] < 0 || k_strides[i] < 0 || v_strides[i] < 0 || o_strides[i] < 0) return XG_ERR_BAD_SHAPE;
    if (q_strides[i] % 8 || k_strides[i] % 8 || v_strides[i] % 8 || o_strides[i] % 8) return XG_ERR_BAD_ALIGN;
    p.qs[i] = q_strides[i];
    p.ks[i] = k_strides[i];
    p.vs[i] = v_strides[i];
    p.os[i] = o_strides[i];
  }
  if (Sq > 1 && o_strides[2] < D) return XG_ERR_BAD_SHAPE;  // output rows would overlap
  // per-lane tile offsets are 32-bit: 128 rows of K / V must span less than 2 GiB
  if (k_strides[2] > (1 << 22) || v_strides[2] > (1 << 22)) return XG_ERR_TOO_LARGE;
  p.q = q;
  p.k = k;
  p.v = v;
  p.o = out;
  p.lse = lse;
  p.ws = workspace;
  p.B = (int)B;
  p.H = (int)H;
  p.Hkv = (int)Hkv;
  p.Sq = (int)Sq;
  p.Skv = (int)Skv;
  p.c = scale * 1.44269504088896340736f;
  if (scale_dev && !aligned_to(scale_dev, 4)) return XG_ERR_BAD_ALIGN;
  p.scale_dev = scale_dev;
  p.mask = mask;
  p.mask_f32 = 0;
  p.mask_vec = 0;
  p.ms[0] = p.ms[1] = p.ms[2] = 0;
  if (mask) {  // the same conditions as xg_sdpa_masked
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
  p.pack = decode_pack(H, Hkv, Sq);
  const int64_t problems = B * (H / p.pack);
  sdpa::decode_split(problems, Skv, p.n_split, p.tiles_per_split);
  const int64_t per = D == 128 ? sdpa::decode_ws_floats<128>() : sdpa::decode_ws_floats<64>();
  if (p.n_split > 1 && (!workspace || workspace_floats < problems * p.n_split * per)) {
    // too little workspace: as many key ranges as it holds (one needs none)
    const int64_t fit = workspace ? workspace_floats / (problems * per) : 0;
    const int64_t n_tiles = (Skv + sdpa::DKV - 1) / sdpa::DKV;
    const int64_t want = fit < 2 ? 1 : fit;
    p.tiles_per_split = (int)((n_tiles + want - 1) / want);
    p.n_split = (int)((n_tiles + p.tiles_per_split - 1) / p.tiles_per_split);
  }
  if (problems * p.n_split > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (mask) {
    if (dtype == XG_BF16) return D == 128 ? sdpa::launch_decode<bf16_t, 128, true>(p, st) : sdpa::launch_decode<bf16_t, 64, true>(p, st);
    return D == 128 ? sdpa::launch_decode<f16_t, 128, true>(p, st) : sdpa::launch_decode<f16_t, 64, true>(p, st);
  }
  if (dtype == XG_BF16) return D == 128 ? sdpa::launch_decode<bf16_t, 128>(p, st) : sdpa::launch_decode<bf16_t, 64>(p, st);
  return D == 128 ? sdpa::launch_decode<f16_t, 128>(p, st) : sdpa::launch_decode<f16_t, 64>(p, st);
}
