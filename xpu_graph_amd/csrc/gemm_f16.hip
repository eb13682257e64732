// fp16 instantiation of the dense-layer kernels.
#include "gemm_impl.hpp"

namespace xg {
namespace gemm {
int launch_f16(const GemmParams& p, bool b_trans, hipStream_t st) {
  return b_trans ? launch_gemm<f16_t, f16_t, BLayout::KMajor>(p, st) : launch_gemm<f16_t, f16_t, BLayout::NMajor>(p, st);
}
int launch_at_f16(const GemmParams& p, hipStream_t st) { return launch_gemm_at<f16_t, f16_t>(p, st); }
int launch_glu_f16(const GemmParams& p, hipStream_t st) { return launch_glu<f16_t, f16_t>(p, st); }
}  // namespace gemm
}  // namespace xg
