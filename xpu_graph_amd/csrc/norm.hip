// Row normalisation kernels for gfx950: RMSNorm / LayerNorm with optional
// fused residual add and optional second output (the pre-norm sum).
//
// Layout: a row of `cols` elements is split into 16-byte vectors.  TPR threads
// share one row and each keeps VPT vectors of it in registers in the storage
// dtype, so HBM is read exactly once and written exactly once per element.
// Statistics are two-pass over the registers (mean, then centred second
// moment) in fp32; lanes combine with wavefront shuffles and, when a row spans
// several wavefronts, a few floats of LDS.
#include "xg_common.hpp"

#include <stdlib.h>

namespace xg {
namespace {

template <typename T, int N>
struct Pack {
  typedef typename VecOf<T>::type V;
  static constexpr int NV = N / VecOf<T>::N;  // 16-byte vectors in a pack of N elements
  V v[NV > 0 ? NV : 1];
};

// Load N consecutive elements of WT (N a multiple of the 16-byte vector width of WT) as fp32.
template <typename WT, int N>
__device__ __forceinline__ void load_row_params(const WT* p, float (&out)[N]) {
  typedef typename VecOf<WT>::type V;
  constexpr int VN = VecOf<WT>::N;
  static_assert(N % VN == 0, "vector width mismatch");
#pragma unroll
  for (int i = 0; i < N / VN; ++i) {
    V t = *reinterpret_cast<const V*>(p + i * VN);
#pragma unroll
    for (int j = 0; j < VN; ++j) out[i * VN + j] = to_f32(t[j]);
  }
}

template <typename T, typename WT, int TPR, int VPT, bool LAYER>
__global__ __launch_bounds__((TPR > 256 ? TPR : 256)) void norm_rows_kernel(
    const T* __restrict__ x, const T* __restrict__ res, const WT* __restrict__ w, const WT* __restrict__ b,
    T* __restrict__ y, T* __restrict__ h_out, int64_t rows, int nvec, int64_t x_stride, int64_t res_stride,
    float eps, float inv_cols) {
  typedef typename VecOf<T>::type V;
  constexpr int VN = VecOf<T>::N;
  constexpr int BLOCK = TPR > 256 ? TPR : 256;
  constexpr int RPB = BLOCK / TPR;  // rows per block
  constexpr int NW = TPR > kWave ? TPR / kWave : 1;
  __shared__ float red_all[2 * RPB * NW];  // one buffer per reduction: each is written and read once

  const int group = threadIdx.x / TPR;
  const int lir = threadIdx.x % TPR;  // lane in row
  float* red = red_all + group * NW;
  float* red2 = red_all + (RPB + group) * NW;
  int64_t row = (int64_t)blockIdx.x * RPB + group;
  const bool row_ok = row < rows;
  if (!row_ok) row = rows - 1;  // keep every lane alive for the barriers; stores are masked below

  const V* xr = reinterpret_cast<const V*>(x + row * x_stride);
  V hv[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = lir + i * TPR;
    if (c < nvec) hv[i] = load_vec_nt(xr + c);
  }
  if (res != nullptr) {
    const V* rr = reinterpret_cast<const V*>(res + row * res_stride);
    V rv[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int c = lir + i * TPR;
      if (c < nvec) rv[i] = load_vec_nt(rr + c);
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int c = lir + i * TPR;
      if (c < nvec) {
#pragma unroll
        for (int j = 0; j < VN; ++j) hv[i][j] = from_f32<T>(to_f32(hv[i][j]) + to_f32(rv[i][j]));
      }
    }
    if (h_out != nullptr && row_ok) {
      V* hr = reinterpret_cast<V*>(h_out + row * (int64_t)nvec * VN);
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int c = lir + i * TPR;
        if (c < nvec) store_vec_nt(hr + c, hv[i]);
      }
    }
  }

  float mean = 0.f;
  if constexpr (LAYER) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      if (lir + i * TPR < nvec) {
#pragma unroll
        for (int j = 0; j < VN; ++j) s += to_f32(hv[i][j]);
      }
    }
    mean = group_sum<TPR, true>(s, red, lir) * inv_cols;
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    if (lir + i * TPR < nvec) {
#pragma unroll
      for (int j = 0; j < VN; ++j) {
        const float d = to_f32(hv[i][j]) - mean;
        ss += d * d;
      }
    }
  }
  const float rstd = rsqrtf(group_sum<TPR, true>(ss, red2, lir) * inv_cols + eps);

  if (!row_ok) return;
  V* yr = reinterpret_cast<V*>(y + row * (int64_t)nvec * VN);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = lir + i * TPR;
    if (c < nvec) {
      float wv[VN], bv[VN];
      if (w != nullptr) {
        load_row_params<WT, VN>(w + (int64_t)c * VN, wv);
      } else {
#pragma unroll
        for (int j = 0; j < VN; ++j) wv[j] = 1.f;
      }
      if (LAYER && b != nullptr) {
        load_row_params<WT, VN>(b + (int64_t)c * VN, bv);
      } else {
#pragma unroll
        for (int j = 0; j < VN; ++j) bv[j] = 0.f;
      }
      V o;
#pragma unroll
      for (int j = 0; j < VN; ++j) o[j] = from_f32<T>((to_f32(hv[i][j]) - mean) * rstd * wv[j] + bv[j]);
      store_vec_nt(yr + c, o);
    }
  }
}

// Any shape / alignment: one 256-thread block per row, three strided passes over
// the row (the re-reads come from cache).  Correctness net for odd column
// counts and unaligned views; the vector kernel above is the fast path.
template <typename T, typename WT, bool LAYER>
__global__ __launch_bounds__(256) void norm_rows_generic_kernel(const T* __restrict__ x, const T* __restrict__ res,
                                                                 const WT* __restrict__ w, const WT* __restrict__ b,
                                                                 T* __restrict__ y, T* __restrict__ h_out,
                                                                 int64_t cols, int64_t x_stride, int64_t res_stride,
                                                                 float eps, float inv_cols) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const T* xr = x + row * x_stride;
  const T* rr = res ? res + row * res_stride : nullptr;
  auto elem = [&](int64_t c) -> float {
    if (rr) return to_f32(from_f32<T>(to_f32(xr[c]) + to_f32(rr[c])));
    return to_f32(xr[c]);
  };
  float mean = 0.f;
  if constexpr (LAYER) {
    float s = 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += 256) s += elem(c);
    mean = group_sum<256>(s, red, threadIdx.x) * inv_cols;
  }
  float ss = 0.f;
  for (int64_t c = threadIdx.x; c < cols; c += 256) {
    const float d = elem(c) - mean;
    ss += d * d;
  }
  const float rstd = rsqrtf(group_sum<256>(ss, red, threadIdx.x) * inv_cols + eps);
  for (int64_t c = threadIdx.x; c < cols; c += 256) {
    const float hval = elem(c);
    if (rr && h_out) h_out[row * cols + c] = from_f32<T>(hval);
    const float wv = w ? to_f32(w[c]) : 1.f;
    const float bv = (LAYER && b) ? to_f32(b[c]) : 0.f;
    y[row * cols + c] = from_f32<T>((hval - mean) * rstd * wv + bv);
  }
}

struct NormArgs {
  const void* x;
  const void* res;
  const void* w;
  const void* b;
  void* y;
  void* h_out;
  int64_t rows, cols, x_stride, res_stride;
  float eps;
  hipStream_t stream;
};

template <typename T, typename WT, int TPR, int VPT, bool LAYER>
int launch_vec(const NormArgs& a, int nvec) {
  constexpr int BLOCK = TPR > 256 ? TPR : 256;
  constexpr int RPB = BLOCK / TPR;
  const int64_t blocks = (a.rows + RPB - 1) / RPB;
  if (blocks > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  hipLaunchKernelGGL((norm_rows_kernel<T, WT, TPR, VPT, LAYER>), dim3((unsigned)blocks), dim3(BLOCK), 0, a.stream,
                     (const T*)a.x, (const T*)a.res, (const WT*)a.w, (const WT*)a.b, (T*)a.y, (T*)a.h_out, a.rows, nvec,
                     a.x_stride, a.res_stride, a.eps, 1.0f / (float)a.cols);
  return status_from_hip(hipGetLastError());
}

template <typename T, typename WT, int TPR, bool LAYER>
int launch_tpr(const NormArgs& a, int nvec) {
  const int per = (nvec + TPR - 1) / TPR;
  if (per <= 1) return launch_vec<T, WT, TPR, 1, LAYER>(a, nvec);
  if (per <= 2) return launch_vec<T, WT, TPR, 2, LAYER>(a, nvec);
  if (per <= 4) return launch_vec<T, WT, TPR, 4, LAYER>(a, nvec);
  if (per <= 8) return launch_vec<T, WT, TPR, 8, LAYER>(a, nvec);
  return XG_ERR_TOO_LARGE;
}

template <typename T, typename WT, bool LAYER>
int launch_typed(const NormArgs& a) {
  constexpr int VN = VecOf<T>::N;
  const bool vec_ok = a.cols % VN == 0 && a.x_stride % VN == 0 && aligned_to(a.x, 16) && aligned_to(a.y, 16) &&
                      (a.res == nullptr || (a.res_stride % VN == 0 && aligned_to(a.res, 16))) &&
                      (a.h_out == nullptr || aligned_to(a.h_out, 16)) && (a.w == nullptr || aligned_to(a.w, 16)) &&
                      (a.b == nullptr || aligned_to(a.b, 16)) && a.cols / VN <= 1024 * 8;
  if (vec_ok) {
    const int nvec = (int)(a.cols / VN);
    // Heuristic from measurement on MI355X: short rows stay inside one wavefront
    // (no LDS, no barrier); from 256 vectors up a 256-thread row with few
    // vectors per thread streams better than one wavefront with many.
    int tpr;
    {
      if (nvec <= 16 * 2)
        tpr = 16;
      else if (nvec <= 64 * 4)
        tpr = 64;
      else if (nvec <= 256 * 8)
        tpr = 256;
      else
        tpr = 1024;
    }
    if (tpr * 8 < nvec) tpr = nvec <= 64 * 8 ? 64 : (nvec <= 256 * 8 ? 256 : 1024);
    switch (tpr) {
      case 16:
        return launch_tpr<T, WT, 16, LAYER>(a, nvec);
      case 64:
        return launch_tpr<T, WT, 64, LAYER>(a, nvec);
      case 128:
        return launch_tpr<T, WT, 128, LAYER>(a, nvec);
      case 256:
        return launch_tpr<T, WT, 256, LAYER>(a, nvec);
      case 1024:
        return launch_tpr<T, WT, 1024, LAYER>(a, nvec);
      default:
        return XG_ERR_BAD_ARG;
    }
  }
  if (a.rows > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  hipLaunchKernelGGL((norm_rows_generic_kernel<T, WT, LAYER>), dim3((unsigned)a.rows), dim3(256), 0, a.stream,
                     (const T*)a.x, (const T*)a.res, (const WT*)a.w, (const WT*)a.b, (T*)a.y, (T*)a.h_out, a.cols,
                     a.x_stride, a.res_stride, a.eps, 1.0f / (float)a.cols);
  return status_from_hip(hipGetLastError());
}

template <bool LAYER>
int dispatch(const NormArgs& a, int dtype, int wb_dtype) {
  if (a.x == nullptr || a.y == nullptr) return XG_ERR_NULL_PTR;
  if (a.rows < 0 || a.cols <= 0 || a.x_stride < a.cols || (a.res != nullptr && a.res_stride < a.cols))
    return XG_ERR_BAD_SHAPE;
  if (a.rows == 0) return XG_OK;
  const size_t esz = dtype == XG_F32 ? 4 : 2;
  if (!aligned_to(a.x, esz) || !aligned_to(a.y, esz)) return XG_ERR_BAD_ALIGN;
  if (dtype == XG_F32 && wb_dtype == XG_F32) return launch_typed<float, float, LAYER>(a);
  if (dtype == XG_BF16 && wb_dtype == XG_BF16) return launch_typed<bf16_t, bf16_t, LAYER>(a);
  if (dtype == XG_BF16 && wb_dtype == XG_F32) return launch_typed<bf16_t, float, LAYER>(a);
  if (dtype == XG_F16 && wb_dtype == XG_F16) return launch_typed<f16_t, f16_t, LAYER>(a);
  if (dtype == XG_F16 && wb_dtype == XG_F32) return launch_typed<f16_t, float, LAYER>(a);
  return XG_ERR_BAD_DTYPE;
}


// ---- backward of RMSNorm / LayerNorm with optional residual add -------------------------------------
// h = x (+ res, rounded to the storage type as the forward does), ghat = gy w
//   RMSNorm:    r = rsqrt(mean(h^2) + eps), hhat = h r
//               g_sum = r (ghat - hhat mean(ghat hhat)) (+ gh)
//   LayerNorm:  mu = mean(h), r = rsqrt(mean((h - mu)^2) + eps), hhat = (h - mu) r
//               g_sum = r (ghat - mean(ghat) - hhat mean(ghat hhat)) (+ gh)
//   g_sum is the gradient of x (and of res);  gw = sum over rows of gy hhat,  gb = sum over rows of gy (LayerNorm),
//   each written as one fp32 partial row per block.
// One block of 256 threads walks a strip of rows; a lane keeps the same CH chunks of 16 bytes of every row, so its
// share of gw / gb stays in registers across the strip.  One pass over h and gy per row.  RMSNorm needs one round of
// row sums (sum h^2 and sum ghat h do not depend on r); LayerNorm two, the mean first and the centred sums after it,
// as its forward does.
template <typename T, typename WT, int CH, bool LAYER>
__global__ __launch_bounds__(256) void norm_bwd_kernel(const T* __restrict__ x, const T* __restrict__ res, const WT* __restrict__ w,
                                                       const T* __restrict__ gy, const T* __restrict__ gh, T* __restrict__ gx,
                                                       float* __restrict__ gw_part, float* __restrict__ gb_part, int64_t rows, int nvec,
                                                       int64_t x_stride, int64_t res_stride, int64_t gy_stride, int64_t gh_stride,
                                                       float eps, float inv_cols, int rows_per_block) {
  typedef typename VecOf<T>::type V;
  constexpr int VN = VecOf<T>::N;
  __shared__ float red_a[4], red_b[4], red_c[4], red_m[4];
  const int lane = threadIdx.x;
  float wv[CH][VN], gw_acc[CH][VN], gb_acc[LAYER ? CH : 1][VN];
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = lane + i * 256;
#pragma unroll
    for (int j = 0; j < VN; ++j) {
      gw_acc[i][j] = 0.f;
      if constexpr (LAYER) gb_acc[i][j] = 0.f;
      wv[i][j] = (w != nullptr && c < nvec) ? to_f32(w[(int64_t)c * VN + j]) : 1.f;
    }
  }
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
  const int64_t r1 = r0 + rows_per_block < rows ? r0 + rows_per_block : rows;
  for (int64_t row = r0; row < r1; ++row) {
    float hf[CH][VN], gf[CH][VN];
    float s0 = 0.f;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c = lane + i * 256;
      if (c < nvec) {
        V hv = load_vec_nt(reinterpret_cast<const V*>(x + row * x_stride) + c);
        if (res != nullptr) {
          const V rv = load_vec_nt(reinterpret_cast<const V*>(res + row * res_stride) + c);
#pragma unroll
          for (int j = 0; j < VN; ++j) hv[j] = from_f32<T>(to_f32(hv[j]) + to_f32(rv[j]));
        }
        const V gv = load_vec_nt(reinterpret_cast<const V*>(gy + row * gy_stride) + c);
#pragma unroll
        for (int j = 0; j < VN; ++j) {
          hf[i][j] = to_f32(hv[j]);
          gf[i][j] = to_f32(gv[j]);
          s0 += hf[i][j];
        }
      } else {
#pragma unroll
        for (int j = 0; j < VN; ++j) hf[i][j] = gf[i][j] = 0.f;
      }
    }
    float mean = 0.f;
    if constexpr (LAYER) {
      s0 = wave_sum<kWave>(s0);
      if ((lane & 63) == 0) red_m[lane >> 6] = s0;  // its readers of the previous row passed two barriers since
      __syncthreads();
      mean = (red_m[0] + red_m[1] + red_m[2] + red_m[3]) * inv_cols;
    }
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      if (lane + i * 256 < nvec) {
#pragma unroll
        for (int j = 0; j < VN; ++j) {
          if constexpr (LAYER) hf[i][j] -= mean;
          const float ghat = gf[i][j] * wv[i][j];
          s1 = __builtin_fmaf(hf[i][j], hf[i][j], s1);
          s2 = __builtin_fmaf(ghat, hf[i][j], s2);
          if constexpr (LAYER) s3 += ghat;
        }
      }
    }
    s1 = wave_sum<kWave>(s1);
    s2 = wave_sum<kWave>(s2);
    if constexpr (LAYER) s3 = wave_sum<kWave>(s3);
    __syncthreads();  // the previous row's readers are done with red_a / red_b / red_c
    if ((lane & 63) == 0) {
      red_a[lane >> 6] = s1;
      red_b[lane >> 6] = s2;
      if constexpr (LAYER) red_c[lane >> 6] = s3;
    }
    __syncthreads();
    s1 = red_a[0] + red_a[1] + red_a[2] + red_a[3];
    s2 = red_b[0] + red_b[1] + red_b[2] + red_b[3];
    const float r = rsqrtf(s1 * inv_cols + eps);
    const float dot = r * s2 * inv_cols;  // mean(ghat * hhat)
    float gmean = 0.f;
    if constexpr (LAYER) gmean = (red_c[0] + red_c[1] + red_c[2] + red_c[3]) * inv_cols;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c = lane + i * 256;
      if (c < nvec) {
        V out;
        V ghv;
        if (gh != nullptr) ghv = load_vec_nt(reinterpret_cast<const V*>(gh + row * gh_stride) + c);
#pragma unroll
        for (int j = 0; j < VN; ++j) {
          const float hhat = hf[i][j] * r;
          float g = r * (gf[i][j] * wv[i][j] - gmean - hhat * dot);
          if (gh != nullptr) g += to_f32(ghv[j]);
          out[j] = from_f32<T>(g);
          gw_acc[i][j] = __builtin_fmaf(gf[i][j], hhat, gw_acc[i][j]);
          if constexpr (LAYER) gb_acc[i][j] += gf[i][j];
        }
        store_vec_nt(reinterpret_cast<V*>(gx + row * (int64_t)nvec * VN) + c, out);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = lane + i * 256;
    if (c < nvec) {
#pragma unroll
      for (int j = 0; j < VN; ++j) {
        if (gw_part != nullptr) gw_part[((int64_t)blockIdx.x * nvec + c) * VN + j] = gw_acc[i][j];
        if constexpr (LAYER) {
          if (gb_part != nullptr) gb_part[((int64_t)blockIdx.x * nvec + c) * VN + j] = gb_acc[i][j];
        }
      }
    }
  }
}

struct NormBwdArgs {
  const void *x, *res, *w, *gy, *gh;
  void* gx;
  float *gw_part, *gb_part;
  int64_t rows, cols, x_stride, res_stride, gy_stride, gh_stride;
  float eps;
  int n_blocks;
  hipStream_t stream;
};

template <typename T, typename WT, bool LAYER>
int norm_bwd_typed(const NormBwdArgs& a) {
  constexpr int VN = VecOf<T>::N;
  const int nvec = (int)(a.cols / VN);
  const int chunks = (nvec + 255) / 256;
  const int rpb = (int)((a.rows + a.n_blocks - 1) / a.n_blocks);
  const float inv_cols = 1.f / (float)a.cols;
#define XG_NORM_BWD(CH)                                                                                                              \
  hipLaunchKernelGGL((norm_bwd_kernel<T, WT, CH, LAYER>), dim3((unsigned)a.n_blocks), dim3(256), 0, a.stream, (const T*)a.x,          \
                     (const T*)a.res, (const WT*)a.w, (const T*)a.gy, (const T*)a.gh, (T*)a.gx, a.gw_part, a.gb_part, a.rows, nvec,   \
                     a.x_stride, a.res_stride, a.gy_stride, a.gh_stride, a.eps, inv_cols, rpb)
  if (chunks <= 1) XG_NORM_BWD(1);
  else if (chunks <= 2) XG_NORM_BWD(2);
  else if (chunks <= 4) XG_NORM_BWD(4);
  else if (chunks <= 8) XG_NORM_BWD(8);
  else return XG_ERR_TOO_LARGE;
#undef XG_NORM_BWD
  return status_from_hip(hipGetLastError());
}

// Argument checks and type dispatch shared by xg_rms_norm_bwd and xg_layer_norm_bwd.
template <bool LAYER>
int norm_bwd_entry(const void* x, const void* res, const void* w, const void* gy, const void* gh, void* gx, float* gw_part, float* gb_part,
                   int64_t rows, int64_t cols, int64_t x_stride, int64_t res_stride, int64_t gy_stride, int64_t gh_stride, float eps,
                   int dtype, int w_dtype, int n_blocks, xg_stream_t stream) {
  if (!x || !gy || !gx) return XG_ERR_NULL_PTR;
  if (rows < 0 || cols <= 0 || x_stride < cols || gy_stride < cols || (res && res_stride < cols) || (gh && gh_stride < cols)) return XG_ERR_BAD_SHAPE;
  if (n_blocks < 1 || n_blocks > 65535 || (gw_part && !w)) return XG_ERR_BAD_ARG;
  if (dtype != XG_F32 && dtype != XG_BF16 && dtype != XG_F16) return XG_ERR_BAD_DTYPE;
  if (w && w_dtype != dtype && w_dtype != XG_F32) return XG_ERR_BAD_DTYPE;
  const int64_t per16 = dtype == XG_F32 ? 4 : 8;
  if (cols % per16 || x_stride % per16 || gy_stride % per16 || (res && res_stride % per16) || (gh && gh_stride % per16)) return XG_ERR_BAD_ALIGN;
  const void* ptrs[] = {x, res, gy, gh, gx};
  for (const void* q : ptrs)
    if (q && !aligned_to(q, 16)) return XG_ERR_BAD_ALIGN;
  if ((w && !aligned_to(w, 4)) || (gw_part && !aligned_to(gw_part, 4)) || (gb_part && !aligned_to(gb_part, 4))) return XG_ERR_BAD_ALIGN;
  if (cols / per16 > 8 * 256) return XG_ERR_TOO_LARGE;  // a lane keeps at most eight 16-byte chunks of a row
  if (rows == 0) return XG_OK;
  if (n_blocks > rows) n_blocks = (int)rows;
  NormBwdArgs a{x, res, w, gy, gh, gx, gw_part, gb_part, rows, cols, x_stride, res_stride, gy_stride, gh_stride, eps, n_blocks, (hipStream_t)stream};
  const bool wf32 = w && w_dtype == XG_F32;
  if (dtype == XG_F32) return norm_bwd_typed<float, float, LAYER>(a);
  if (dtype == XG_BF16) return wf32 ? norm_bwd_typed<bf16_t, float, LAYER>(a) : norm_bwd_typed<bf16_t, bf16_t, LAYER>(a);
  return wf32 ? norm_bwd_typed<f16_t, float, LAYER>(a) : norm_bwd_typed<f16_t, f16_t, LAYER>(a);
}

}  // namespace
}  // namespace xg

extern "C" {

int xg_rms_norm(const void* x, const void* w, void* y, int64_t rows, int64_t cols, int64_t x_stride, float eps,
                int dtype, int wb_dtype, xg_stream_t stream) {
  xg::NormArgs a{x, nullptr, w, nullptr, y, nullptr, rows, cols, x_stride, 0, eps, (hipStream_t)stream};
  return xg::dispatch<false>(a, dtype, wb_dtype);
}

int xg_layer_norm(const void* x, const void* w, const void* b, void* y, int64_t rows, int64_t cols,
                  int64_t x_stride, float eps, int dtype, int wb_dtype, xg_stream_t stream) {
  xg::NormArgs a{x, nullptr, w, b, y, nullptr, rows, cols, x_stride, 0, eps, (hipStream_t)stream};
  return xg::dispatch<true>(a, dtype, wb_dtype);
}

int xg_add_rms_norm(const void* x, const void* res, const void* w, void* y, void* h_out, int64_t rows,
                    int64_t cols, int64_t x_stride, int64_t res_stride, float eps, int dtype, int wb_dtype,
                    xg_stream_t stream) {
  if (res == nullptr) return XG_ERR_NULL_PTR;
  xg::NormArgs a{x, res, w, nullptr, y, h_out, rows, cols, x_stride, res_stride, eps, (hipStream_t)stream};
  return xg::dispatch<false>(a, dtype, wb_dtype);
}

int xg_add_layer_norm(const void* x, const void* res, const void* w, const void* b, void* y, void* h_out,
                      int64_t rows, int64_t cols, int64_t x_stride, int64_t res_stride, float eps, int dtype,
                      int wb_dtype, xg_stream_t stream) {
  if (res == nullptr) return XG_ERR_NULL_PTR;
  xg::NormArgs a{x, res, w, b, y, h_out, rows, cols, x_stride, res_stride, eps, (hipStream_t)stream};
  return xg::dispatch<true>(a, dtype, wb_dtype);
}

int xg_rms_norm_bwd(const void* x, const void* res, const void* w, const void* gy, const void* gh, void* gx, float* gw_part,
                    int64_t rows, int64_t cols, int64_t x_stride, int64_t res_stride, int64_t gy_stride, int64_t gh_stride,
                    float eps, int dtype, int w_dtype, int n_blocks, xg_stream_t stream) {
  return xg::norm_bwd_entry<false>(x, res, w, gy, gh, gx, gw_part, nullptr, rows, cols, x_stride, res_stride, gy_stride, gh_stride, eps, dtype,
                                   w_dtype, n_blocks, stream);
}

int xg_layer_norm_bwd(const void* x, const void* res, const void* w, const void* gy, const void* gh, void* gx, float* gw_part,
                      float* gb_part, int64_t rows, int64_t cols, int64_t x_stride, int64_t res_stride, int64_t gy_stride,
                      int64_t gh_stride, float eps, int dtype, int w_dtype, int n_blocks, xg_stream_t stream) {
  return xg::norm_bwd_entry<true>(x, res, w, gy, gh, gx, gw_part, gb_part, rows, cols, x_stride, res_stride, gy_stride, gh_stride, eps, dtype,
                                  w_dtype, n_blocks, stream);
}

}  // extern "C"
