// Entry points whose kernels are not written yet: they refuse every call.
#include "xg_common.hpp"
extern "C" {
int xg_sdpa(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,
            const int64_t*, const int64_t*, const int64_t*, const int64_t*, float, int, int, xg_stream_t) {
  return XG_ERR_BAD_ARG;
}
}
