// fp32 instantiation of the dense-layer kernels (32x32x2 fp32 MFMA, fp32 in and out).
#include "gemm_impl.hpp"

namespace xg {
namespace gemm {
int launch_f32(const GemmParams& p, bool b_trans, hipStream_t st) {
  return b_trans ? launch_gemm<float, float, BLayout::KMajor>(p, st) : launch_gemm<float, float, BLayout::NMajor>(p, st);
}
}  // namespace gemm
}  // namespace xg
