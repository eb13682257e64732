// Entry points whose kernels are not written yet: they refuse every call.
#include "xg_common.hpp"
extern "C" {
int xg_dense(const void*, const void*, const void*, const void*, void*, int64_t, int64_t, int64_t, int64_t, int64_t,
             int64_t, int, int, int, int, xg_stream_t) {
  return XG_ERR_BAD_ARG;
}
int xg_dense_fp8(const void*, const void*, const float*, const float*, const void*, void*, int64_t, int64_t, int64_t,
                 int64_t, int64_t, int, int, int, int, xg_stream_t) {
  return XG_ERR_BAD_ARG;
}
int xg_sdpa(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,
            const int64_t*, const int64_t*, const int64_t*, const int64_t*, float, int, int, xg_stream_t) {
  return XG_ERR_BAD_ARG;
}
}
