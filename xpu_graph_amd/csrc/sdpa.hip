// Scaled dot-product attention for gfx950: one pass over the keys with a running
// maximum (flash-attention forward), optional causal mask, no dropout.
//
// Work split
//   workgroup = 4 waves = 128 query rows of one (batch, head); wave w owns rows
//   32w..32w+31.  Keys / values stream through LDS in tiles of 64 rows, moved by
//   `global_load_lds_dwordx4` (no register staging) into two stages, so the tile
//   of step j+1 lands while step j is computed; one barrier per step.
//
// Transposed products: everything a query row needs stays in one lane
//   S^T = K Q^T   : MFMA 32x32x16 with the K tile as the A operand and the
//                   register-resident Q rows as B.  The result puts query
//                   (lane % 32) in the lane and 16 of a tile's 32 keys in its 16
//                   accumulator registers; lanes l and l^32 share a query.
//   softmax       : row maximum = per-lane max + ONE cross-lane exchange; the
//                   correction factor and the row sum are per-lane scalars.
//   O^T += V^T P^T: V^T tile as A, the probabilities as B.  The k index of an
//                   MFMA may be permuted freely as long as A and B agree, so the
//                   k slots are chosen to be exactly the keys a lane already
//                   holds: P never moves between lanes and never touches LDS.
//                   The matching V^T fragment (8 keys x 1 head-dim column per
//                   lane) comes from two `ds_read_b64_tr_b16` reads.
//
// LDS layout: row-major [64 keys][D] per tile, 16-byte chunks XOR-swizzled by a
// function of the row so that the 16-lane groups of the K reads (same chunk, 16
// rows) and the 8-row x 64-byte footprints of the transposing V reads spread over
// all banks.  The swizzle is applied to the GLOBAL address of each lane of the
// direct load, since its LDS side is fixed (lane i -> base + 16 i).
#include "sdpa_common.hpp"

namespace xg {
namespace sdpa {

struct Params {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  float* lse;  // when set: the natural-log sum of exponentials of every query row, [B, H, Sq] (what a backward pass recomputes the probabilities from)
  int B, H, Hkv, Sq, Skv;
  int64_t qs[3], ks[3], vs[3], os[3];  // element strides of batch, head, sequence
  float c;                             // scale * log2(e)
  const float* scale_dev;              // when set: the scale is read from this one-element device tensor instead
  const void* mask;                    // additive mask (MASK kernels only), element [b, h, i, j] at ms[0] b + ms[1] h + ms[2] i + j
  int64_t ms[3];                       // element strides of batch, head, query row (0: broadcast)
  int mask_f32;                        // mask elements are fp32 (else the dtype of q)
  int mask_vec;                        // rows of the mask can be read four elements at a time
  int causal;
  int n_qb;   // query blocks per (batch, head)
  int order;  // 0: heaviest query blocks of ALL heads first; 1: head after head inside each XCD; n >= 2: n heads at a time inside each XCD, heaviest blocks first
};

// MASK: an additive mask [B | 1, H | 1, Sq, Skv] is added to the scaled scores (aten.scaled_dot_product_attention's
// attn_mask); rows whose every key is masked with -inf come out as NaN, as they do in eager.
template <typename T, int D, bool MASK = false>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void sdpa_fwd_kernel(Params p) {
  typedef typename Vec8<T>::type V8;
  typedef __attribute__((address_space(3))) const V8 lds_V8;
  constexpr int RB = D * 2;          // bytes per tile row
  constexpr int CH = RB / 16;        // chunks per row
  constexpr int TILE = BKV * RB;     // one K or V tile
  constexpr int STAGE = 2 * TILE;    // K tile, then V tile
  constexpr int KK = D / 16;         // k-steps of Q K^T
  constexpr int DT = D / 32;         // 32-row tiles of O^T
  constexpr int LPW = CH / 4;        // direct loads per wave per tile (1 KiB each)
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, h = lane >> 5;
  // scale * log2(e): by value, or from a one-element device tensor (a scale that is only known on the device)
  const float c_eff = p.scale_dev ? *p.scale_dev * 1.44269504088896340736f : p.c;

  // ---- which (batch, head, query block).  Blocks are dealt round-robin to the 8 XCDs, so with the
  // number of heads a multiple of 8 both orders keep all query blocks of a head on ONE XCD (one L2).
  int bh, qb;
  {
    const int id = blockIdx.x, nbh = p.B * p.H;
    if (p.order == 1 && (nbh & 7) == 0) {
      const int xcd = id & 7, slot = id >> 3;
      bh = (slot / p.n_qb) * 8 + xcd;
      qb = p.n_qb - 1 - slot % p.n_qb;
    } else {
      int rank;
      grouped_block_order(id, nbh, p.n_qb, p.order, bh, rank);  // causal: late query blocks have the most keys, start them first
      qb = p.n_qb - 1 - rank;
    }
  }
  const int b = bh / p.H, head = bh % p.H, hkv = head / (p.H / p.Hkv);
  const int q0 = qb * BQ;
  const int qrow = q0 + 32 * wave + l32;  // this lane's query

  // ---- Q rows into registers, in B-operand order: lane holds Q[q][16 kk + 8 h .. +8]
  V8 qf[KK];
  {
    const int qr = qrow < p.Sq ? qrow : p.Sq - 1;
    const T* qg = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.qs[0] + (int64_t)head * p.qs[1] + (int64_t)qr * p.qs[2];
    static_for<KK>([&](auto KI) {
      constexpr int kk = decltype(KI)::value;
      qf[kk] = *reinterpret_cast<const V8*>(qg + 16 * kk + 8 * h);
    });
  }

  // ---- direct-load bookkeeping: load i of this wave fills LDS bytes [(wave*LPW+i)*1024, +1024) of a tile.
  // The global address is a workgroup-uniform tile base plus a 32-bit per-lane offset that does not change
  // from tile to tile (row within the tile x row stride + swizzled chunk), so a step costs no address math.
  const char* kg = reinterpret_cast<const char*>(p.k) + ((int64_t)b * p.ks[0] + (int64_t)hkv * p.ks[1]) * 2;
  const char* vg = reinterpret_cast<const char*>(p.v) + ((int64_t)b * p.vs[0] + (int64_t)hkv * p.vs[1]) * 2;
  const uint32_t k_row_bytes = (uint32_t)(p.ks[2] * 2), v_row_bytes = (uint32_t)(p.vs[2] * 2);
  uint32_t k_off[LPW], v_off[LPW];
  auto lane_offsets = [&](int rows_valid) {  // rows at or past rows_valid repeat the last valid row; they are masked below
    static_for<LPW>([&](auto I) {
      constexpr int i = decltype(I)::value;
      const int pos = (wave * LPW + i) * 1024 + lane * 16;
      int row = pos / RB;
      const int pc = (pos % RB) >> 4;
      const int kc = (pc ^ swz_k<D>(row)) << 4, vc = (pc ^ swz_v<D>(row)) << 4;
      row = row < rows_valid ? row : rows_valid - 1;
      k_off[i] = (uint32_t)row * k_row_bytes + kc;
      v_off[i] = (uint32_t)row * v_row_bytes + vc;
    });
  };
  lane_offsets(BKV);
  const int n_tiles_all = (p.Skv + BKV - 1) / BKV;
  const int rows_last = p.Skv - (n_tiles_all - 1) * BKV;  // valid rows of the last key tile
  auto issue = [&](int j, auto STAGE_IDX) {
    constexpr int stage = decltype(STAGE_IDX)::value;
    if (j == n_tiles_all - 1 && rows_last < BKV) lane_offsets(rows_last);  // at most once: it is the last tile
    const char* kt = kg + (int64_t)j * BKV * k_row_bytes;
    const char* vt = vg + (int64_t)j * BKV * v_row_bytes;
    static_for<LPW>([&](auto I) {
      constexpr int i = decltype(I)::value;
      char* kd = smem + stage * STAGE + (wave * LPW + i) * 1024;
      // inline-asm loads: the compiler must not know of LDS writes in flight, or it holds the transposing V reads
      // of THIS tile back until the loads of the next one have landed
      load_to_lds16(kt, k_off[i], (uint32_t)(size_t)(lvoid*)kd);
      load_to_lds16(vt, v_off[i], (uint32_t)(size_t)(lvoid*)(kd + TILE));
    });
  };

  // ---- number of key tiles this workgroup visits
  int n_steps = n_tiles_all;
  if (p.causal) {
    int q_last = q0 + BQ - 1;
    q_last = q_last < p.Sq ? q_last : p.Sq - 1;
    const int lim = q_last / BKV + 1;
    n_steps = n_steps < lim ? n_steps : lim;
  }
  const int qw_min = q0 + 32 * wave, qw_max = qw_min + 31;

  // ---- per-lane parts of the LDS read addresses (everything else is a compile-time offset)
  const int kx = swz_k<D>(l32);  // same for both 32-row tiles of a K tile
  const int a16 = lane & 15, b16 = (lane >> 4) & 1;
  const int v_row = 4 * h + (a16 >> 2);                          // key row (mod 16) this lane addresses for the V^T fragments
  const int v_chunk = 2 * b16 + ((a16 & 3) >> 1), v_sub = (a16 & 1) << 3;

  // The per-lane LDS byte addresses of every fragment read, formed once and held in registers (the empty asm keeps
  // the compiler from splitting them up again and redoing the additions in every step).
  int k_addr[KK], v_addr0[DT], v_addr1[DT];
  const int lds_base = (int)(uint32_t)(size_t)(lvoid*)smem;
  static_for<KK>([&](auto KI) {
    constexpr int kk = decltype(KI)::value;
    k_addr[kk] = lds_base + l32 * RB + (((2 * kk + h) ^ kx) << 4);
    asm volatile("" : "+v"(k_addr[kk]));
  });
  static_for<DT>([&](auto DI) {
    constexpr int dt = decltype(DI)::value;
    // lane a16 of a 16-lane group addresses key row (a16/4), head-dim columns 4(a16%4)..+3 of the group's
    // 16 columns; the transposing read returns, for result slot e, key row e at column a16.
    v_addr0[dt] = lds_base + v_row * RB + (((4 * dt + v_chunk) ^ swz_v<D>(v_row)) << 4) + v_sub;
    v_addr1[dt] = lds_base + (v_row + 8) * RB + (((4 * dt + v_chunk) ^ swz_v<D>(v_row + 8)) << 4) + v_sub;
    asm volatile("" : "+v"(v_addr0[dt]), "+v"(v_addr1[dt]));
  });

  f32x16 o_acc[DT];
  static_for<DT>([&](auto I) {
    o_acc[decltype(I)::value] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  });
  // m_run is the exponent reference of the running sums, not necessarily the true running maximum: it is
  // moved only when a row's maximum exceeds it by more than kSlack (in log2 units), so probabilities stay
  // below 2^kSlack and the accumulator rescale is skipped on most tiles.  The result is the same quotient.
  constexpr float kSlack = 8.f;
  float m_run = -INFINITY, l_run = 0.f;

  auto step = [&](auto STAGE_IDX, int j) {
    constexpr int stage = decltype(STAGE_IDX)::value;
    // this wave's part of tile j has landed.  A real s_waitcnt (vmcnt(0), the other counters at their maximum)
    // rather than inline asm: the compiler then knows that the Q rows loaded above have arrived too, and does
    // not count them down against the (untracked) direct loads inside the loop
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();                                  // ... everyone's has, and everyone is done with tile j-1
    if (j + 1 < n_steps) issue(j + 1, std::integral_constant<int, stage ^ 1>{});
    const int kv0 = j * BKV;
    if (p.causal && kv0 > qw_max) return;  // this wave's queries see none of these keys (wave-uniform)


    // S^T tile: s[t][v] = <key 32t + 8(v/4) + 4h + v%4 , query l32>
    // The two 32-key halves alternate MFMA by MFMA: a dependent MFMA cannot issue until its predecessor has
    // left the pipe (a chain of eight ran at one MFMA per ~80 clocks in a probe kernel), two interleaved chains can.
    f32x16 s[2];
    s[0] = s[1] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // K fragments are read PF k-steps ahead of the MFMAs that use them, so an LDS round trip hides behind MFMAs.
    constexpr int PF = 2;
    V8 kf[KK][2];
    auto read_k = [&](auto KI) {
      constexpr int kk = decltype(KI)::value;
      static_for<2>([&](auto TI) {
        constexpr int t = decltype(TI)::value;
        kf[kk][t] = *(lds_V8*)(uint32_t)(k_addr[kk] + stage * STAGE + 32 * t * RB);
      });
    };
    static_for<PF>([&](auto KI) { read_k(KI); });
    static_for<KK>([&](auto KI) {
      constexpr int kk = decltype(KI)::value;
      if constexpr (kk + PF < KK) read_k(std::integral_constant<int, kk + PF>{});
      __builtin_amdgcn_sched_barrier(0);  // the reads above are issued before the MFMAs below
      static_for<2>([&](auto TI) {
        constexpr int t = decltype(TI)::value;
        s[t] = mma(kf[kk][t], qf[kk], s[t]);
        __builtin_amdgcn_sched_barrier(0x7F7);  // everything but MFMAs may move across: the MFMA order stays as written
      });
    });

    // scores are s * c in the exponent's base-2 scale.  Tiles that cross the diagonal or the end of
    // the keys are scaled and masked explicitly (cc = 1 afterwards); all others fold c into the FMA.
    float cc = c_eff;
    if constexpr (MASK) {
      // scores in the exponent's base-2 scale with the mask added: s * c + m * log2(e); afterwards cc = 1.
      // Row and key indices are clamped for the loads; what lies past the end is masked by index below.
      const int mrow = qrow < p.Sq ? qrow : p.Sq - 1;
      const int64_t mbase = (int64_t)b * p.ms[0] + (int64_t)head * p.ms[1] + (int64_t)mrow * p.ms[2];
      constexpr float kLog2e = 1.44269504088896340736f;
      static_for<2>([&](auto TI) {
        constexpr int t = decltype(TI)::value;
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
            s[t][4 * g + e] = __builtin_fmaf(s[t][4 * g + e], cc, m4[e] * kLog2e);
          });
        });
      });
      cc = 1.f;
    }
    const bool need_mask = (p.causal && kv0 + BKV - 1 > qw_min) || (kv0 + BKV > p.Skv);
    if (need_mask) {
      int lim = p.Skv - 1;  // last visible key of this lane's query
      if (p.causal) lim = lim < qrow ? lim : qrow;
      const int rel = lim - kv0 - 4 * h;
      static_for<2>([&](auto TI) {
        constexpr int t = decltype(TI)::value;
        static_for<16>([&](auto VI) {
          constexpr int v = decltype(VI)::value;
          constexpr int key = 32 * t + 8 * (v / 4) + (v % 4);
          s[t][v] = key > rel ? -INFINITY : s[t][v] * cc;
        });
      });
      cc = 1.f;
    }
    float mx = s[0][0];
    if (cc >= 0.f) {
      static_for<2>([&](auto TI) { static_for<16>([&](auto VI) { mx = fmaxf(mx, s[decltype(TI)::value][decltype(VI)::value]); }); });
    } else {
      static_for<2>([&](auto TI) { static_for<16>([&](auto VI) { mx = fminf(mx, s[decltype(TI)::value][decltype(VI)::value]); }); });
    }
    float mt = mx * cc;
    {
      // lanes l and l ^ 32 share a query: one swap of the two register halves hands both partial maxima to both
      // lanes without a trip through the LDS crossbar.  Written as asm because the compiler folds the two results
      // of the builtin into one when both inputs are the same value.
      float lo = mt, hi = mt;
      asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
      mt = fmaxf(lo, hi);
    }
    const float m_new = mt > m_run + kSlack ? mt : m_run;  // -inf + slack = -inf: the first visible key always moves it
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a row with no visible key yet
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
    float psum = 0.f;
    static_for<2>([&](auto TI) {
      constexpr int t = decltype(TI)::value;
      static_for<16>([&](auto VI) {
        constexpr int v = decltype(VI)::value;
        const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][v], cc, -m_use));
        s[t][v] = e;
        psum += e;
      });
    });
    if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
      l_run *= alpha;
      static_for<DT>([&](auto I) { o_acc[decltype(I)::value] *= alpha; });
    }
    l_run += psum;
    m_run = m_new;

    // O^T += V^T P^T.  k-step (t, st) uses keys 32t + 16st + {4h..4h+3} and 32t + 16st + 8 + {4h..4h+3}:
    // exactly registers 8st..8st+7 of s[t] in this lane.
    // This phase issues two transposing reads per MFMA; with the wave's priority raised its reads and MFMAs go
    // ahead of the vector work of the other wave on the SIMD (B4 H32 S2048 D128 under sustained load: causal
    // 160.8 -> 157.2 us, unmasked 274.5 -> 263.3 us; the same priority on the score MFMAs as well takes it back).
    __builtin_amdgcn_s_setprio(1);
    static_for<2>([&](auto TI) {
      constexpr int t = decltype(TI)::value;
      static_for<2>([&](auto SI) {
        constexpr int st = decltype(SI)::value;
        V8 pf;
        static_for<8>([&](auto JI) {
          constexpr int jj = decltype(JI)::value;
          pf[jj] = (T)s[t][8 * st + jj];
        });
        static_for<DT>([&](auto DI) {
          constexpr int dt = decltype(DI)::value;
          constexpr int base = stage * STAGE + TILE + (32 * t + 16 * st) * RB;
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(uint32_t)(v_addr0[dt] + base));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(uint32_t)(v_addr1[dt] + base));
          const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          o_acc[dt] = mma(__builtin_bit_cast(V8, both), pf, o_acc[dt]);
        });
      });
    });
    __builtin_amdgcn_s_setprio(0);
  };

  issue(0, std::integral_constant<int, 0>{});
  for (int j = 0; j < n_steps; j += 2) {
    step(std::integral_constant<int, 0>{}, j);
    if (j + 1 < n_steps) step(std::integral_constant<int, 1>{}, j + 1);
  }

  // ---- normalise and write: O[q][d] = O^T[d][q] / l.  The tile is parked in LDS (per wave) so that
  // global stores are 16 bytes per lane and whole rows per 16 lanes.
  const float l_tot = l_run + __shfl_xor(l_run, 32, kWave);
  const float inv = 1.f / l_tot;
  if (p.lse && h == 0 && qrow < p.Sq)  // m_run is in base-2 units; a row without a visible key gives -inf
    p.lse[(int64_t)bh * p.Sq + qrow] = (m_run + log2f(l_tot)) * 0.69314718055994530942f;
  __syncthreads();  // all waves are done reading K / V tiles
  char* park = smem + wave * (32 * RB);
  static_for<DT>([&](auto DI) {
    constexpr int dt = decltype(DI)::value;
    static_for<4>([&](auto GI) {
      constexpr int g = decltype(GI)::value;
      typedef T t4 __attribute__((ext_vector_type(4)));
      t4 w;
      static_for<4>([&](auto EI) {
        constexpr int e = decltype(EI)::value;
        w[e] = (T)(o_acc[dt][4 * g + e] * inv);
      });
      // columns 32dt + 8g + 4h .. +3 of row l32: chunk 4dt + g, upper or lower 8 bytes
      *reinterpret_cast<t4*>(park + l32 * RB + (((4 * dt + g) ^ swz_k<D>(l32)) << 4) + 8 * h) = w;
    });
  });
  __syncthreads();
  T* og = reinterpret_cast<T*>(p.o) + (int64_t)b * p.os[0] + (int64_t)head * p.os[1];
  static_for<RB / 32>([&](auto I) {
    constexpr int i = decltype(I)::value;
    const int pos = i * 1024 + lane * 16;
    const int row = pos / RB, pc = (pos % RB) >> 4;
    const int c = pc ^ swz_k<D>(row);
    const u32x4 val = *reinterpret_cast<const u32x4*>(park + pos);
    const int qr = q0 + 32 * wave + row;
    if (qr < p.Sq) *reinterpret_cast<u32x4*>(og + (int64_t)qr * p.os[2] + c * 8) = val;
  });
}

template <typename T, int D, bool MASK = false>
int launch(const Params& p, hipStream_t stream) {
  constexpr int SMEM = 2 * 2 * BKV * D * 2;
  auto kernel = sdpa_fwd_kernel<T, D, MASK>;
  if (int st = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), SMEM)) return st;
  const int64_t blocks = (int64_t)p.B * p.H * p.n_qb;
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(kThreads), SMEM, stream, p);
  return status_from_hip(hipGetLastError());
}

}  // namespace sdpa
}  // namespace xg

namespace {

int sdpa_entry(const void* q, const void* k, const void* v, void* out, float* lse, const void* mask, const int64_t* mask_strides, int mask_dtype,
               const float* scale_dev, int64_t B, int64_t H, int64_t Hkv, int64_t Sq, int64_t Skv, int64_t D, const int64_t q_strides[3],
               const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3], float scale, int causal, int dtype,
               xg_stream_t stream) {
  using namespace xg;
  if (dtype != XG_BF16 && dtype != XG_F16) return XG_ERR_BAD_DTYPE;
  if (B < 0 || H < 0 || Hkv < 0 || Sq < 0 || Skv < 0) return XG_ERR_BAD_SHAPE;
  if (D != 64 && D != 128) return XG_ERR_BAD_SHAPE;
  if (B == 0 || H == 0 || Sq == 0) return XG_OK;
  if (Hkv == 0 || H % Hkv != 0 || Skv == 0) return XG_ERR_BAD_SHAPE;
  if (!q || !k || !v || !out || !q_strides || !k_strides || !v_strides || !o_strides) return XG_ERR_NULL_PTR;
  if (!(scale == scale) || fabsf(scale) > 3.0e38f) return XG_ERR_BAD_ARG;
  if (Sq > (1 << 30) || Skv > (1 << 30)) return XG_ERR_TOO_LARGE;
  const int64_t n_qb = (Sq + sdpa::BQ - 1) / sdpa::BQ;
  if (B * H > (1 << 24) || B * H * n_qb > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  if (!aligned_to(q, 16) || !aligned_to(k, 16) || !aligned_to(v, 16) || !aligned_to(out, 16)) return XG_ERR_BAD_ALIGN;
  sdpa::Params p;
  for (int i = 0; i < 3; ++i) {
    if (q_strides[i] < 0 || k_strides[i] < 0 || v_strides[i] < 0 || o_strides[i] < 0) return XG_ERR_BAD_SHAPE;
    if (q_strides[i] % 8 || k_strides[i] % 8 || v_strides[i] % 8 || o_strides[i] % 8) return XG_ERR_BAD_ALIGN;
    p.qs[i] = q_strides[i];
    p.ks[i] = k_strides[i];
    p.vs[i] = v_strides[i];
    p.os[i] = o_strides[i];
  }
  // per-lane tile offsets are 32-bit: 64 rows of K / V must span less than 2 GiB
  if (k_strides[2] > (1 << 23) || v_strides[2] > (1 << 23)) return XG_ERR_TOO_LARGE;
  p.mask = mask;
  p.mask_f32 = 0;
  p.mask_vec = 0;
  p.ms[0] = p.ms[1] = p.ms[2] = 0;
  if (mask) {
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
  if (scale_dev && !aligned_to(scale_dev, 4)) return XG_ERR_BAD_ALIGN;
  p.scale_dev = scale_dev;
  if (lse && !aligned_to(lse, 4)) return XG_ERR_BAD_ALIGN;
  p.lse = lse;
  p.q = q;
  p.k = k;
  p.v = v;
  p.o = out;
  p.B = (int)B;
  p.H = (int)H;
  p.Hkv = (int)Hkv;
  p.Sq = (int)Sq;
  p.Skv = (int)Skv;
  p.c = scale * 1.44269504088896340736f;
  p.causal = causal ? 1 : 0;
  p.n_qb = (int)n_qb;
  // Measured (D128): without a mask, walking head after head inside each XCD is faster (B4 H32 S2048 290 vs 315 us).
  // Causal problems want the heaviest query blocks first (S2048: 176 vs 205 us head after head), over at most eight
  // heads at a time per XCD, so that the blocks in flight share their keys in L2 (a CU streams 117 GB/s from L2, 27 GB/s
  // from the last-level cache): B4 H32 S2048 163 -> 158 us against all sixteen heads of an XCD at once, B2 H16 S8192
  // 533 (head after head) -> 511 us.
  p.order = p.causal ? sdpa::block_order_group(B * H) : 1;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (mask) {
    if (dtype == XG_BF16) return D == 128 ? sdpa::launch<bf16_t, 128, true>(p, st) : sdpa::launch<bf16_t, 64, true>(p, st);
    return D == 128 ? sdpa::launch<f16_t, 128, true>(p, st) : sdpa::launch<f16_t, 64, true>(p, st);
  }
  if (dtype == XG_BF16) return D == 128 ? sdpa::launch<bf16_t, 128>(p, st) : sdpa::launch<bf16_t, 64>(p, st);
  return D == 128 ? sdpa::launch<f16_t, 128>(p, st) : sdpa::launch<f16_t, 64>(p, st);
}

}  // namespace

extern "C" int xg_sdpa(const void* q, const void* k, const void* v, void* out, int64_t B, int64_t H, int64_t Hkv, int64_t Sq,
                       int64_t Skv, int64_t D, const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                       const int64_t o_strides[3], float scale, int causal, int dtype, xg_stream_t stream) {
  return sdpa_entry(q, k, v, out, nullptr, nullptr, nullptr, dtype, nullptr, B, H, Hkv, Sq, Skv, D, q_strides, k_strides, v_strides, o_strides, scale,
                    causal, dtype, stream);
}

extern "C" int xg_sdpa_masked(const void* q, const void* k, const void* v, void* out, const void* mask, const int64_t mask_strides[3],
                              int mask_dtype, const float* scale_dev, int64_t B, int64_t H, int64_t Hkv, int64_t Sq, int64_t Skv,
                              int64_t D, const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                              const int64_t o_strides[3], float scale, int causal, int dtype, xg_stream_t stream) {
  return sdpa_entry(q, k, v, out, nullptr, mask, mask_strides, mask_dtype, scale_dev, B, H, Hkv, Sq, Skv, D, q_strides, k_strides, v_strides,
                    o_strides, scale, causal, dtype, stream);
}

extern "C" int xg_sdpa_lse(const void* q, const void* k, const void* v, void* out, float* lse, int64_t B, int64_t H, int64_t Hkv,
                           int64_t Sq, int64_t Skv, int64_t D, const int64_t q_strides[3], const int64_t k_strides[3],
                           const int64_t v_strides[3], const int64_t o_strides[3], float scale, int causal, int dtype,
                           xg_stream_t stream) {
  if (lse == nullptr && B > 0 && H > 0 && Sq > 0) return XG_ERR_NULL_PTR;
  return sdpa_entry(q, k, v, out, lse, nullptr, nullptr, dtype, nullptr, B, H, Hkv, Sq, Skv, D, q_strides, k_strides, v_strides, o_strides,
                    scale, causal, dtype, stream);
}

extern "C" int xg_sdpa_masked_lse(const void* q, const void* k, const void* v, void* out, float* lse, const void* mask,
                                  const int64_t mask_strides[3], int mask_dtype, const float* scale_dev, int64_t B, int64_t H,
                                  int64_t Hkv, int64_t Sq, int64_t Skv, int64_t D, const int64_t q_strides[3],
                                  const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3], float scale,
                                  int causal, int dtype, xg_stream_t stream) {
  if (lse == nullptr && B > 0 && H > 0 && Sq > 0) return XG_ERR_NULL_PTR;
  return sdpa_entry(q, k, v, out, lse, mask, mask_strides, mask_dtype, scale_dev, B, H, Hkv, Sq, Skv, D, q_strides, k_strides, v_strides,
                    o_strides, scale, causal, dtype, stream);
}
