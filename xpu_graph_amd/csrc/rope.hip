// Rotary position embedding for gfx950, "rotate-half" convention:
//   out[.., s, c]       = x[.., s, c]       * cos[s, c]       - x[.., s, c + D/2] * sin[s, c]
//   out[.., s, c + D/2] = x[.., s, c + D/2] * cos[s, c + D/2] + x[.., s, c]       * sin[s, c + D/2]
// i.e. x * cos + cat(-x[.., D/2:], x[.., :D/2]) * sin, evaluated in fp32 and rounded once.
//
// Memory bound: one thread owns 8 columns c..c+7 of the lower half AND their partners in the upper half of one
// row, so every element of x is read exactly once (two 16-byte loads, two 16-byte stores per thread); x and out
// are [B, H, S, D] views with element strides (the [B, S, H, D] storage a projection leaves behind is read and
// written in place); cos / sin are [S, D] tables with a row stride, a few KiB that stay in cache.
#include "xg_common.hpp"

namespace xg {
namespace {

struct RopeParams {
  const void* x;
  const void* cos;
  const void* sin;
  void* out;
  int B, H, S, D;
  int64_t xs[3], os[3];  // element strides of batch, head, sequence
  int64_t cs_stride;     // row stride of the tables
};

template <typename T, typename CT>
__global__ __launch_bounds__(256) void rope_kernel(RopeParams p) {
  typedef typename VecOf<T>::type V8;
  typedef CT C8 __attribute__((ext_vector_type(8)));
  const int half_vecs = p.D / 16;  // threads per row
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t rows = (int64_t)p.B * p.H * p.S;
  if (i >= rows * half_vecs) return;
  const int c = (int)(i % half_vecs) * 8;
  const int64_t r = i / half_vecs;
  // rows are enumerated with the head index fastest when the storage is [B, S, H, D], so that neighbouring
  // threads touch neighbouring memory either way
  int b, h, s;
  if (p.xs[1] < p.xs[2]) {
    h = (int)(r % p.H);
    s = (int)((r / p.H) % p.S);
    b = (int)(r / ((int64_t)p.H * p.S));
  } else {
    s = (int)(r % p.S);
    h = (int)((r / p.S) % p.H);
    b = (int)(r / ((int64_t)p.H * p.S));
  }
  const T* xr = reinterpret_cast<const T*>(p.x) + b * p.xs[0] + h * p.xs[1] + s * p.xs[2];
  T* orow = reinterpret_cast<T*>(p.out) + b * p.os[0] + h * p.os[1] + s * p.os[2];
  const CT* cr = reinterpret_cast<const CT*>(p.cos) + s * p.cs_stride;
  const CT* sr = reinterpret_cast<const CT*>(p.sin) + s * p.cs_stride;
  const int hd = p.D / 2;
  const V8 lo = __builtin_nontemporal_load(reinterpret_cast<const V8*>(xr + c));
  const V8 hi = __builtin_nontemporal_load(reinterpret_cast<const V8*>(xr + hd + c));
  const C8 cl = *reinterpret_cast<const C8*>(cr + c), ch = *reinterpret_cast<const C8*>(cr + hd + c);
  const C8 sl = *reinterpret_cast<const C8*>(sr + c), sh = *reinterpret_cast<const C8*>(sr + hd + c);
  V8 ol, oh;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float xl = to_f32(lo[j]), xh = to_f32(hi[j]);
    ol[j] = from_f32<T>(xl * to_f32(cl[j]) - xh * to_f32(sl[j]));
    oh[j] = from_f32<T>(xh * to_f32(ch[j]) + xl * to_f32(sh[j]));
  }
  __builtin_nontemporal_store(ol, reinterpret_cast<V8*>(orow + c));
  __builtin_nontemporal_store(oh, reinterpret_cast<V8*>(orow + hd + c));
}

template <typename T, typename CT>
int launch(const RopeParams& p, hipStream_t stream) {
  const int64_t work = (int64_t)p.B * p.H * p.S * (p.D / 16);
  const int64_t blocks = (work + 255) / 256;
  if (blocks > 0x7fffffffLL) return XG_ERR_TOO_LARGE;
  hipLaunchKernelGGL((rope_kernel<T, CT>), dim3((unsigned)blocks), dim3(256), 0, stream, p);
  return status_from_hip(hipGetLastError());
}

}  // namespace
}  // namespace xg

extern "C" int xg_rope(const void* x, const void* cos_table, const void* sin_table, void* out, int64_t B, int64_t H, int64_t S,
                       int64_t D, const int64_t x_strides[3], const int64_t o_strides[3], int64_t table_stride, int dtype,
                       int table_dtype, xg_stream_t stream) {
  using namespace xg;
  if (dtype != XG_BF16 && dtype != XG_F16) return XG_ERR_BAD_DTYPE;
  if (table_dtype != dtype && table_dtype != XG_F32) return XG_ERR_BAD_DTYPE;
  if (B < 0 || H < 0 || S < 0 || D <= 0 || D % 16 != 0 || table_stride < D) return XG_ERR_BAD_SHAPE;
  if (B == 0 || H == 0 || S == 0) return XG_OK;
  if (!x || !cos_table || !sin_table || !out || !x_strides || !o_strides) return XG_ERR_NULL_PTR;
  if (B > 0x7fffffff || H > 0x7fffffff || S > 0x7fffffff || D > 0x7fffffff) return XG_ERR_TOO_LARGE;
  const int table_vec = table_dtype == XG_F32 ? 4 : 8;  // elements per 16 bytes
  if (!aligned_to(x, 16) || !aligned_to(out, 16) || !aligned_to(cos_table, 16) || !aligned_to(sin_table, 16) ||
      table_stride % table_vec != 0)
    return XG_ERR_BAD_ALIGN;
  RopeParams p;
  for (int i = 0; i < 3; ++i) {
    if (x_strides[i] < 0 || o_strides[i] < 0) return XG_ERR_BAD_SHAPE;
    if (x_strides[i] % 8 || o_strides[i] % 8) return XG_ERR_BAD_ALIGN;
    p.xs[i] = x_strides[i];
    p.os[i] = o_strides[i];
  }
  p.x = x;
  p.cos = cos_table;
  p.sin = sin_table;
  p.out = out;
  p.B = (int)B;
  p.H = (int)H;
  p.S = (int)S;
  p.D = (int)D;
  p.cs_stride = table_stride;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (dtype == XG_BF16) return table_dtype == XG_F32 ? launch<bf16_t, float>(p, st) : launch<bf16_t, bf16_t>(p, st);
  return table_dtype == XG_F32 ? launch<f16_t, float>(p, st) : launch<f16_t, f16_t>(p, st);
}
