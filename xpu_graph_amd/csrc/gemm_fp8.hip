// fp8 (OCP e4m3) instantiation of the dense-layer kernels and the xg_dense_fp8 entry point.
#include "gemm_impl.hpp"

extern "C" {

int xg_dense_fp8(const void* a_q, const void* b_q, const float* a_scale_dev, const float* b_scale_dev, const void* bias,
                 void* out, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int b_trans, int act,
                 int out_dtype, int bias_dtype, xg_stream_t stream) {
  using namespace xg;
  using namespace xg::gemm;
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
  GemmParams p = make_params(a_q, b_q, bias, nullptr, out, M, N, K, lda, ldb, 0, act, bias && bias_dtype == XG_F32);
  p.a_scale = a_scale_dev;
  p.b_scale = b_scale_dev;
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
