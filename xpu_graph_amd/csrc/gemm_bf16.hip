// bf16 instantiation of the dense-layer kernels and the xg_dense entry point.
#include "gemm_impl.hpp"

namespace xg {
namespace gemm {
int launch_f16(const GemmParams& p, bool b_trans, hipStream_t st);  // gemm_f16.hip
int launch_at_f16(const GemmParams& p, hipStream_t st);               // gemm_f16.hip
int launch_f32(const GemmParams& p, bool b_trans, hipStream_t st);  // gemm_f32.hip
int launch_at_bf16(const GemmParams& p, hipStream_t st) { return launch_gemm_at<bf16_t, bf16_t>(p, st); }
int launch_glu_f16(const GemmParams& p, hipStream_t st);              // gemm_f16.hip
int launch_glu_bf16(const GemmParams& p, hipStream_t st) { return launch_glu<bf16_t, bf16_t>(p, st); }
int launch_bf16(const GemmParams& p, bool b_trans, hipStream_t st) {
  return b_trans ? launch_gemm<bf16_t, bf16_t, BLayout::KMajor>(p, st) : launch_gemm<bf16_t, bf16_t, BLayout::NMajor>(p, st);
}
}  // namespace gemm
}  // namespace xg

extern "C" {

int xg_dense(const void* a, const void* b, const void* bias, const void* residual, void* out, int64_t M, int64_t N,
             int64_t K, int64_t lda, int64_t ldb, int64_t ldr, int b_trans, int act, int dtype, int bias_dtype,
             xg_stream_t stream) {
  using namespace xg;
  using namespace xg::gemm;
  if (a == nullptr || b == nullptr || out == nullptr) return XG_ERR_NULL_PTR;
  if (M < 0 || N <= 0 || K <= 0 || lda < K || (b_trans ? ldb < K : ldb < N) || (residual && ldr < N)) return XG_ERR_BAD_SHAPE;
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return XG_ERR_TOO_LARGE;
  if (dtype != XG_BF16 && dtype != XG_F16 && dtype != XG_F32) return XG_ERR_BAD_DTYPE;
  if (bias && bias_dtype != dtype && bias_dtype != XG_F32) return XG_ERR_BAD_DTYPE;
  if (act < XG_ACT_NONE || act > XG_ACT_SIGMOID) return XG_ERR_BAD_ARG;
  // 16-byte operand loads (8 elements of a 16-bit type, 4 of fp32); 8 output columns per lane
  const int64_t per16 = dtype == XG_F32 ? 4 : 8;
  if (K % per16 != 0 || N % 8 != 0 || lda % per16 != 0 || ldb % per16 != 0 || (residual && ldr % per16 != 0)) return XG_ERR_BAD_ALIGN;
  if (!aligned_to(a, 16) || !aligned_to(b, 16) || !aligned_to(out, 16) || (bias && !aligned_to(bias, 16)) ||
      (residual && !aligned_to(residual, 16)))
    return XG_ERR_BAD_ALIGN;
  if (M == 0) return XG_OK;
  const GemmParams p = make_params(a, b, bias, residual, out, M, N, K, lda, ldb, ldr, act, bias && bias_dtype == XG_F32);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == XG_F32) return gemm::launch_f32(p, b_trans != 0, st);
  return dtype == XG_BF16 ? gemm::launch_bf16(p, b_trans != 0, st) : gemm::launch_f16(p, b_trans != 0, st);
}

int xg_dense_batched(const void* a, const void* b, const void* bias, const void* residual, void* out, int64_t batch,
                     int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldr, int64_t stride_a,
                     int64_t stride_b, int64_t stride_bias, int64_t stride_res, int64_t stride_out, int b_trans, int act,
                     int dtype, int bias_dtype, xg_stream_t stream) {
  using namespace xg;
  using namespace xg::gemm;
  if (a == nullptr || b == nullptr || out == nullptr) return XG_ERR_NULL_PTR;
  if (batch < 0 || M < 0 || N <= 0 || K <= 0 || lda < K || (b_trans ? ldb < K : ldb < N) || (residual && ldr < N)) return XG_ERR_BAD_SHAPE;
  if (stride_a < 0 || stride_b < 0 || stride_bias < 0 || stride_res < 0 || stride_out < M * N) return XG_ERR_BAD_SHAPE;
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff || batch > 65535) return XG_ERR_TOO_LARGE;
  if (dtype != XG_BF16 && dtype != XG_F16) return XG_ERR_BAD_DTYPE;
  if (bias && bias_dtype != dtype && bias_dtype != XG_F32) return XG_ERR_BAD_DTYPE;
  if (act < XG_ACT_NONE || act > XG_ACT_SIGMOID) return XG_ERR_BAD_ARG;
  if (K % 8 != 0 || N % 8 != 0 || lda % 8 != 0 || ldb % 8 != 0 || (residual && ldr % 8 != 0)) return XG_ERR_BAD_ALIGN;
  // every entry's operands start on a 16-byte boundary
  if (stride_a % 8 != 0 || stride_b % 8 != 0 || stride_out % 8 != 0 || (residual && stride_res % 8 != 0) ||
      (bias && stride_bias % (bias_dtype == XG_F32 ? 4 : 8) != 0))
    return XG_ERR_BAD_ALIGN;
  if (!aligned_to(a, 16) || !aligned_to(b, 16) || !aligned_to(out, 16) || (bias && !aligned_to(bias, 16)) ||
      (residual && !aligned_to(residual, 16)))
    return XG_ERR_BAD_ALIGN;
  if (M == 0 || batch == 0) return XG_OK;
  GemmParams p = make_params(a, b, bias, residual, out, M, N, K, lda, ldb, ldr, act, bias && bias_dtype == XG_F32);
  p.batch = (int)batch;
  p.a_batch = stride_a * 2;
  p.b_batch = stride_b * 2;
  p.bias_batch = stride_bias * (bias && bias_dtype == XG_F32 ? 4 : 2);
  p.res_batch = stride_res * 2;
  p.out_batch = stride_out * 2;
  hipStream_t st = (hipStream_t)stream;
  return dtype == XG_BF16 ? gemm::launch_bf16(p, b_trans != 0, st) : gemm::launch_f16(p, b_trans != 0, st);
}

int xg_dense_at(const void* a_t, const void* b, const void* residual, void* out, int64_t M, int64_t N, int64_t K,
                int64_t lda, int64_t ldb, int64_t ldr, int dtype, xg_stream_t stream) {
  using namespace xg;
  using namespace xg::gemm;
  if (a_t == nullptr || b == nullptr || out == nullptr) return XG_ERR_NULL_PTR;
  if (M <= 0 || N <= 0 || K <= 0 || lda < M || ldb < N || (residual && ldr < N)) return XG_ERR_BAD_SHAPE;
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return XG_ERR_TOO_LARGE;
  if (dtype != XG_BF16 && dtype != XG_F16) return XG_ERR_BAD_DTYPE;
  // 16-byte loads along M and N, 16-byte output stores; K is free (a partial last slab reads as zero)
  if (M % 8 != 0 || N % 8 != 0 || lda % 8 != 0 || ldb % 8 != 0 || (residual && ldr % 8 != 0)) return XG_ERR_BAD_ALIGN;
  if (!aligned_to(a_t, 16) || !aligned_to(b, 16) || !aligned_to(out, 16) || (residual && !aligned_to(residual, 16)))
    return XG_ERR_BAD_ALIGN;
  const GemmParams p = make_params(a_t, b, nullptr, residual, out, M, N, K, lda, ldb, ldr, XG_ACT_NONE, false);
  hipStream_t st = (hipStream_t)stream;
  return dtype == XG_BF16 ? gemm::launch_at_bf16(p, st) : gemm::launch_at_f16(p, st);
}

static int dense_glu_entry(const void* a, const void* w_gate, const void* w_up, void* out, void* gate_out, void* up_out, int64_t M,
                           int64_t N, int64_t K, int64_t lda, int64_t ldb, int dtype, xg_stream_t stream) {
  using namespace xg;
  using namespace xg::gemm;
  if (a == nullptr || w_gate == nullptr || w_up == nullptr || out == nullptr) return XG_ERR_NULL_PTR;
  if ((gate_out == nullptr) != (up_out == nullptr)) return XG_ERR_NULL_PTR;
  if (gate_out && (!aligned_to(gate_out, 16) || !aligned_to(up_out, 16))) return XG_ERR_BAD_ALIGN;
  if (M < 0 || N <= 0 || K <= 0 || lda < K || ldb < K) return XG_ERR_BAD_SHAPE;
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return XG_ERR_TOO_LARGE;
  if (dtype != XG_BF16 && dtype != XG_F16) return XG_ERR_BAD_DTYPE;
  if (K % 64 != 0) return XG_ERR_BAD_SHAPE;  // whole 128-byte K slabs: the gated kernel has no staged variant
  if (N % 8 != 0 || lda % 8 != 0 || ldb % 8 != 0) return XG_ERR_BAD_ALIGN;
  if (!aligned_to(a, 16) || !aligned_to(w_gate, 16) || !aligned_to(w_up, 16) || !aligned_to(out, 16)) return XG_ERR_BAD_ALIGN;
  if (M == 0) return XG_OK;
  GemmParams p = make_params(a, w_gate, nullptr, nullptr, out, M, N, K, lda, ldb, 0, XG_ACT_NONE, false);
  p.B2 = w_up;
  p.gate_out = gate_out;
  p.up_out = up_out;
  p.tiles_n = (int)((N + BN / 2 - 1) / (BN / 2));
  // the direct-to-LDS loads address each operand with a 31-bit lane offset
  const int64_t lim = 0x7fffffffLL;
  if (M * lda * 2 >= lim || N * ldb * 2 >= lim) return XG_ERR_TOO_LARGE;
  hipStream_t st = (hipStream_t)stream;
  return dtype == XG_BF16 ? gemm::launch_glu_bf16(p, st) : gemm::launch_glu_f16(p, st);
}

int xg_dense_glu(const void* a, const void* w_gate, const void* w_up, void* out, int64_t M, int64_t N, int64_t K,
                 int64_t lda, int64_t ldb, int dtype, xg_stream_t stream) {
  return dense_glu_entry(a, w_gate, w_up, out, nullptr, nullptr, M, N, K, lda, ldb, dtype, stream);
}

int xg_dense_glu_save(const void* a, const void* w_gate, const void* w_up, void* out, void* gate_out, void* up_out, int64_t M,
                      int64_t N, int64_t K, int64_t lda, int64_t ldb, int dtype, xg_stream_t stream) {
  if (gate_out == nullptr || up_out == nullptr) return XG_ERR_NULL_PTR;
  return dense_glu_entry(a, w_gate, w_up, out, gate_out, up_out, M, N, K, lda, ldb, dtype, stream);
}

}  // extern "C"
