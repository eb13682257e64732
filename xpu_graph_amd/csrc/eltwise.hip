// Elementwise kernels for gfx950: the SwiGLU gate silu(a) * b, and the plain
// copy used as the known-size yardstick for the memory-traffic counters.
#include "xg_common.hpp"

namespace xg {
namespace {


// gate/up are [rows, d] views with row strides in elements; nvec = d / VW.
template <typename T, int VW>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                                       T* __restrict__ y, int64_t rows, int64_t nvec,
                                                       int64_t gate_stride, int64_t up_stride) {
  typedef T VT __attribute__((ext_vector_type(VW)));
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * nvec) return;
  const int64_t r = i / nvec, c = i % nvec;
  const VT g = __builtin_nontemporal_load(reinterpret_cast<const VT*>(gate + r * gate_stride) + c);
  const VT u = __builtin_nontemporal_load(reinterpret_cast<const VT*>(up + r * up_stride) + c);
  VT o;
#pragma unroll
  for (int j = 0; j < VW; ++j) o[j] = from_f32<T>(silu_f32(to_f32(g[j])) * to_f32(u[j]));
  __builtin_nontemporal_store(o, reinterpret_cast<VT*>(y) + i);
}

template <typename T>
__global__ __launch_bounds__(256) void silu_mul_scalar_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                                              T* __restrict__ y, int64_t rows, int64_t d,
                                                              int64_t gate_stride, int64_t up_stride) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * d) return;
  const int64_t r = i / d, c = i % d;
  y[i] = from_f32<T>(silu_f32(to_f32(gate[r * gate_stride + c])) * to_f32(up[r * up_stride + c]));
}

template <typename T>
int silu_mul_typed(const void* gate, const void* up, void* y, int64_t rows, int64_t d, int64_t gs, int64_t us,
                   hipStream_t stream) {
  constexpr int VN = VecOf<T>::N;
  const bool vec_ok = d % VN == 0 && gs % VN == 0 && us % VN == 0 && aligned_to(gate, 16) && aligned_to(up, 16) &&
                      aligned_to(y, 16);
  const int64_t work = vec_ok ? rows * (d / VN) : rows * d;
  const int64_t blocks = (work + 255) / 256;
  if (blocks > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  if (vec_ok)
    hipLaunchKernelGGL((silu_mul_kernel<T, VN>), dim3((unsigned)blocks), dim3(256), 0, stream, (const T*)gate,
                       (const T*)up, (T*)y, rows, d / VN, gs, us);
  else
    hipLaunchKernelGGL((silu_mul_scalar_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream, (const T*)gate,
                       (const T*)up, (T*)y, rows, d, gs, us);
  return status_from_hip(hipGetLastError());
}

int silu_mul_dispatch(const void* gate, const void* up, void* y, int64_t rows, int64_t d, int64_t gs, int64_t us,
                      int dtype, hipStream_t stream) {
  if (gate == nullptr || up == nullptr || y == nullptr) return XG_ERR_NULL_PTR;
  if (rows < 0 || d < 0 || gs < d || us < d) return XG_ERR_BAD_SHAPE;
  if (rows == 0 || d == 0) return XG_OK;
  switch (dtype) {
    case XG_F32:
      return silu_mul_typed<float>(gate, up, y, rows, d, gs, us, stream);
    case XG_BF16:
      return silu_mul_typed<bf16_t>(gate, up, y, rows, d, gs, us, stream);
    case XG_F16:
      return silu_mul_typed<f16_t>(gate, up, y, rows, d, gs, us, stream);
    default:
      return XG_ERR_BAD_DTYPE;
  }
}

// Backward of y = silu(gate) * up: d_gate = gy * up * s * (1 + gate * (1 - s)) with s = sigmoid(gate), d_up = gy *
// silu(gate); fp32 math on the storage-type inputs, one rounding per output.  All five tensors are contiguous.
template <typename T, int VW>
__global__ __launch_bounds__(256) void silu_mul_bwd_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                                           const T* __restrict__ gy, T* __restrict__ d_gate,
                                                           T* __restrict__ d_up, int64_t nvec) {
  typedef T VT __attribute__((ext_vector_type(VW)));
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nvec) return;
  const VT g = __builtin_nontemporal_load(reinterpret_cast<const VT*>(gate) + i);
  const VT u = __builtin_nontemporal_load(reinterpret_cast<const VT*>(up) + i);
  const VT y = __builtin_nontemporal_load(reinterpret_cast<const VT*>(gy) + i);
  VT dg, du;
#pragma unroll
  for (int j = 0; j < VW; ++j) {
    const float gf = to_f32(g[j]), uf = to_f32(u[j]), yf = to_f32(y[j]);
    const float sg = sigmoid_f32(gf);
    dg[j] = from_f32<T>(yf * uf * (sg * (1.f + gf * (1.f - sg))));
    du[j] = from_f32<T>(yf * (gf * sg));
  }
  __builtin_nontemporal_store(dg, reinterpret_cast<VT*>(d_gate) + i);
  __builtin_nontemporal_store(du, reinterpret_cast<VT*>(d_up) + i);
}

template <typename T>
int silu_mul_bwd_typed(const void* gate, const void* up, const void* gy, void* d_gate, void* d_up, int64_t n, hipStream_t stream) {
  constexpr int VN = VecOf<T>::N;
  const void* ptrs[] = {gate, up, gy, d_gate, d_up};
  bool vec_ok = n % VN == 0;
  for (const void* q : ptrs) vec_ok = vec_ok && aligned_to(q, 16);
  const int64_t work = vec_ok ? n / VN : n;
  const int64_t blocks = (work + 255) / 256;
  if (blocks > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  if (vec_ok)
    hipLaunchKernelGGL((silu_mul_bwd_kernel<T, VN>), dim3((unsigned)blocks), dim3(256), 0, stream, (const T*)gate, (const T*)up,
                       (const T*)gy, (T*)d_gate, (T*)d_up, work);
  else
    hipLaunchKernelGGL((silu_mul_bwd_kernel<T, 1>), dim3((unsigned)blocks), dim3(256), 0, stream, (const T*)gate, (const T*)up,
                       (const T*)gy, (T*)d_gate, (T*)d_up, work);
  return status_from_hip(hipGetLastError());
}

// An activation on its own, and its backward: y = act(x);  gz = gy * act'(z).  The dense layer of a differentiated graph
// keeps its pre-activation z (as eager does) and applies the activation with this kernel, so the backward is one pass
// over z and gy instead of a second product.  fp32 math, one rounding; the same formulas as the dense epilogue.
template <int ACT>
__device__ __forceinline__ float act_f32(float t) {
  if constexpr (ACT == XG_ACT_RELU) return fmaxf(t, 0.f);
  if constexpr (ACT == XG_ACT_GELU) return 0.5f * t * (1.f + erff(t * 0.70710678118654752f));
  if constexpr (ACT == XG_ACT_SILU) return silu_f32(t);
  if constexpr (ACT == XG_ACT_SIGMOID) return sigmoid_f32(t);
  return t;
}
template <int ACT>
__device__ __forceinline__ float act_grad_f32(float t) {
  if constexpr (ACT == XG_ACT_RELU) return t > 0.f ? 1.f : 0.f;
  if constexpr (ACT == XG_ACT_GELU)
    return 0.5f * (1.f + erff(t * 0.70710678118654752f)) + t * __expf(-0.5f * t * t) * 0.39894228040143268f;
  if constexpr (ACT == XG_ACT_SILU) {
    const float sg = sigmoid_f32(t);
    return sg * (1.f + t * (1.f - sg));
  }
  if constexpr (ACT == XG_ACT_SIGMOID) {
    const float sg = sigmoid_f32(t);
    return sg * (1.f - sg);
  }
  return 1.f;
}

template <typename T, int VW, int ACT, bool BWD>
__global__ __launch_bounds__(256) void act_kernel(const T* __restrict__ z, const T* __restrict__ gy, T* __restrict__ out, int64_t nvec) {
  typedef T VT __attribute__((ext_vector_type(VW)));
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nvec) return;
  const VT zv = __builtin_nontemporal_load(reinterpret_cast<const VT*>(z) + i);
  VT o;
  if constexpr (BWD) {
    const VT g = __builtin_nontemporal_load(reinterpret_cast<const VT*>(gy) + i);
#pragma unroll
    for (int j = 0; j < VW; ++j) o[j] = from_f32<T>(to_f32(g[j]) * act_grad_f32<ACT>(to_f32(zv[j])));
  } else {
#pragma unroll
    for (int j = 0; j < VW; ++j) o[j] = from_f32<T>(act_f32<ACT>(to_f32(zv[j])));
  }
  __builtin_nontemporal_store(o, reinterpret_cast<VT*>(out) + i);
}

template <typename T, int ACT, bool BWD>
int act_launch(const void* z, const void* gy, void* out, int64_t n, hipStream_t stream) {
  constexpr int VN = VecOf<T>::N;
  const bool vec_ok = n % VN == 0 && aligned_to(z, 16) && aligned_to(out, 16) && (!BWD || aligned_to(gy, 16));
  const int64_t work = vec_ok ? n / VN : n;
  const int64_t blocks = (work + 255) / 256;
  if (blocks > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  if (vec_ok)
    hipLaunchKernelGGL((act_kernel<T, VN, ACT, BWD>), dim3((unsigned)blocks), dim3(256), 0, stream, (const T*)z, (const T*)gy, (T*)out, work);
  else
    hipLaunchKernelGGL((act_kernel<T, 1, ACT, BWD>), dim3((unsigned)blocks), dim3(256), 0, stream, (const T*)z, (const T*)gy, (T*)out, work);
  return status_from_hip(hipGetLastError());
}

template <typename T, bool BWD>
int act_typed(const void* z, const void* gy, void* out, int64_t n, int act, hipStream_t stream) {
  switch (act) {
    case XG_ACT_RELU:
      return act_launch<T, XG_ACT_RELU, BWD>(z, gy, out, n, stream);
    case XG_ACT_GELU:
      return act_launch<T, XG_ACT_GELU, BWD>(z, gy, out, n, stream);
    case XG_ACT_SILU:
      return act_launch<T, XG_ACT_SILU, BWD>(z, gy, out, n, stream);
    case XG_ACT_SIGMOID:
      return act_launch<T, XG_ACT_SIGMOID, BWD>(z, gy, out, n, stream);
    default:
      return XG_ERR_BAD_ARG;  // "none" has nothing to compute
  }
}

template <bool BWD>
int act_entry(const void* z, const void* gy, void* out, int64_t n, int act, int dtype, xg_stream_t stream) {
  if (!z || !out || (BWD && !gy)) return XG_ERR_NULL_PTR;
  if (n < 0) return XG_ERR_BAD_SHAPE;
  if (n == 0) return XG_OK;
  const size_t esz = dtype == XG_F32 ? 4 : 2;
  if (!aligned_to(z, esz) || !aligned_to(out, esz) || (BWD && !aligned_to(gy, esz))) return XG_ERR_BAD_ALIGN;
  switch (dtype) {
    case XG_F32:
      return act_typed<float, BWD>(z, gy, out, n, act, (hipStream_t)stream);
    case XG_BF16:
      return act_typed<bf16_t, BWD>(z, gy, out, n, act, (hipStream_t)stream);
    case XG_F16:
      return act_typed<f16_t, BWD>(z, gy, out, n, act, (hipStream_t)stream);
    default:
      return XG_ERR_BAD_DTYPE;
  }
}

// One lane: for each of `n_windows` windows of `window_ticks` ticks of the constant-rate wall clock, the ticks of the
// shader clock and of the wall clock that went by.  Every window ends after a bounded number of polls.
__global__ void clock_probe_kernel(unsigned long long* out, int n_windows, unsigned window_ticks) {
  if (threadIdx.x != 0) return;
  for (int w = 0; w < n_windows; ++w) {
    const unsigned long long r0 = wall_clock64();
    const unsigned long long c0 = clock64();
    unsigned long long r1 = r0;
    for (int poll = 0; poll < (1 << 20) && r1 - r0 < window_ticks; ++poll) {
      __builtin_amdgcn_s_sleep(8);
      r1 = wall_clock64();
    }
    const unsigned long long c1 = clock64();
    out[2 * w] = c1 - c0;
    out[2 * w + 1] = r1 - r0;
  }
}

__global__ __launch_bounds__(256) void copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

}  // namespace
}  // namespace xg

extern "C" {

int xg_silu_mul(const void* x, void* y, int64_t rows, int64_t d, int64_t x_stride, int dtype, xg_stream_t stream) {
  if (x == nullptr) return XG_ERR_NULL_PTR;
  if (d < 0 || x_stride < 2 * d) return XG_ERR_BAD_SHAPE;
  const size_t esz = dtype == XG_F32 ? 4 : 2;
  const char* up = (const char*)x + (size_t)d * esz;
  return xg::silu_mul_dispatch(x, up, y, rows, d, x_stride, x_stride, dtype, (hipStream_t)stream);
}

int xg_silu_mul2(const void* gate, const void* up, void* y, int64_t rows, int64_t d, int64_t gate_stride,
                 int64_t up_stride, int dtype, xg_stream_t stream) {
  return xg::silu_mul_dispatch(gate, up, y, rows, d, gate_stride, up_stride, dtype, (hipStream_t)stream);
}

int xg_silu_mul2_bwd(const void* gate, const void* up, const void* gy, void* d_gate, void* d_up, int64_t n, int dtype,
                     xg_stream_t stream) {
  using namespace xg;
  if (!gate || !up || !gy || !d_gate || !d_up) return XG_ERR_NULL_PTR;
  if (n < 0) return XG_ERR_BAD_SHAPE;
  if (n == 0) return XG_OK;
  const size_t esz = dtype == XG_F32 ? 4 : 2;
  const void* ptrs[] = {gate, up, gy, d_gate, d_up};
  for (const void* q : ptrs)
    if (!aligned_to(q, esz)) return XG_ERR_BAD_ALIGN;
  switch (dtype) {
    case XG_F32:
      return silu_mul_bwd_typed<float>(gate, up, gy, d_gate, d_up, n, (hipStream_t)stream);
    case XG_BF16:
      return silu_mul_bwd_typed<bf16_t>(gate, up, gy, d_gate, d_up, n, (hipStream_t)stream);
    case XG_F16:
      return silu_mul_bwd_typed<f16_t>(gate, up, gy, d_gate, d_up, n, (hipStream_t)stream);
    default:
      return XG_ERR_BAD_DTYPE;
  }
}

int xg_activation(const void* x, void* y, int64_t n, int act, int dtype, xg_stream_t stream) {
  return xg::act_entry<false>(x, nullptr, y, n, act, dtype, stream);
}

int xg_activation_bwd(const void* z, const void* gy, void* gz, int64_t n, int act, int dtype, xg_stream_t stream) {
  return xg::act_entry<true>(z, gy, gz, n, act, dtype, stream);
}

int xg_copy_bytes(const void* src, void* dst, int64_t bytes, xg_stream_t stream) {
  using namespace xg;
  if (src == nullptr || dst == nullptr) return XG_ERR_NULL_PTR;
  if (bytes < 0 || bytes % 16 != 0) return XG_ERR_BAD_SHAPE;
  if (!aligned_to(src, 16) || !aligned_to(dst, 16)) return XG_ERR_BAD_ALIGN;
  if (bytes == 0) return XG_OK;
  const int64_t n = bytes / 16;
  const int64_t blocks = (n + 255) / 256;
  if (blocks > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const u32x4*)src,
                     (u32x4*)dst, n);
  return status_from_hip(hipGetLastError());
}

int xg_version(void) { return 100; }

const char* xg_status_string(int status) {
  switch (status) {
    case XG_OK:
      return "ok";
    case XG_ERR_BAD_DTYPE:
      return "unsupported dtype combination";
    case XG_ERR_BAD_SHAPE:
      return "inconsistent sizes or strides";
    case XG_ERR_BAD_ALIGN:
      return "pointer or stride alignment not supported";
    case XG_ERR_NULL_PTR:
      return "required pointer is NULL";
    case XG_ERR_TOO_LARGE:
      return "size beyond what the entry point supports";
    case XG_ERR_LAUNCH:
      return "kernel launch failed";
    case XG_ERR_BAD_ARG:
      return "invalid argument";
    default:
      return "unknown status";
  }
}


int xg_clock_probe(uint64_t* out, int n_windows, int64_t window_ticks, xg_stream_t stream) {
  using namespace xg;
  if (out == nullptr) return XG_ERR_NULL_PTR;
  if (n_windows < 0 || n_windows > (1 << 16) || window_ticks <= 0 || window_ticks > 1000000) return XG_ERR_BAD_ARG;
  if (!aligned_to(out, 8)) return XG_ERR_BAD_ALIGN;
  if (n_windows == 0) return XG_OK;
  hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, (unsigned long long*)out, n_windows,
                     (unsigned)window_ticks);
  return status_from_hip(hipGetLastError());
}

int64_t xg_wall_clock_khz(void) {
  int dev = 0, khz = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess) return 0;
  return khz;
}

}  // extern "C"
