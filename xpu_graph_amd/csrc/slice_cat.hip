// Column slice + concatenate for gfx950: a pure byte mover, so any dtype is
// bit-exact.  The caller describes one output row as a list of equally sized
// chunks (<= 16 bytes each); lane t of a block owns one chunk column and walks
// down a strip of rows, so the stores of a wavefront are 64 consecutive chunks
// (up to 1 KiB contiguous) and the loads of consecutive lanes that belong to
// the same slice are contiguous too.  Source chunks only need 4-byte alignment:
// gfx950 global loads of 8/16 bytes accept dword-aligned addresses.
#include "xg_common.hpp"

#include <stdlib.h>

namespace xg {
namespace {

template <int CB>
struct Chunk;
template <>
struct Chunk<16> {
  typedef u32x4 store_t;
  typedef u32x4 load_t __attribute__((aligned(4)));
};
template <>
struct Chunk<8> {
  typedef u32x2 store_t;
  typedef u32x2 load_t __attribute__((aligned(4)));
};
template <>
struct Chunk<4> {
  typedef uint32_t store_t;
  typedef uint32_t load_t;
};
template <>
struct Chunk<2> {
  typedef uint16_t store_t;
  typedef uint16_t load_t;
};
template <>
struct Chunk<1> {
  typedef uint8_t store_t;
  typedef uint8_t load_t;
};

struct OutTable {
  char* ptr[XG_SLICE_CAT_MAX_OUTS];
  int64_t row_bytes[XG_SLICE_CAT_MAX_OUTS];
};

// RU = rows in flight per lane (unrolled loads before the matching stores); KB = lanes per block.
// Loads are ordinary (cached) loads: a slice that straddles a 128-byte line shares that line with the
// neighbouring lanes' requests and with the next row strip, and measured 3-4 % faster than streaming
// loads on the 64 x 128-byte-slice case; the stores bypass the cache (streaming stores measured 15 % faster
// than cached ones there).
template <int CB, int RU, int KB, bool MULTI>
__global__ __launch_bounds__(KB) void slice_cat_kernel(const char* __restrict__ src, int64_t src_row_bytes,
                                                           int64_t rows, OutTable outs, int n_outs,
                                                           const xg_chunk* __restrict__ table, int64_t n_chunks,
                                                           int rows_per_block) {
  typedef typename Chunk<CB>::load_t load_t;
  typedef typename Chunk<CB>::store_t store_t;
  __shared__ char* s_ptr[MULTI ? XG_SLICE_CAT_MAX_OUTS : 1];
  __shared__ int64_t s_rb[MULTI ? XG_SLICE_CAT_MAX_OUTS : 1];
  if constexpr (MULTI) {
    if ((int)threadIdx.x < n_outs) {
      s_ptr[threadIdx.x] = outs.ptr[threadIdx.x];
      s_rb[threadIdx.x] = outs.row_bytes[threadIdx.x];
    }
    __syncthreads();
  }
  const int64_t ci = (int64_t)blockIdx.x * KB + threadIdx.x;
  if (ci >= n_chunks) return;
  const xg_chunk ch = table[ci];
  char* dst;
  int64_t dst_rb;
  if constexpr (MULTI) {
    dst = s_ptr[ch.out_id];
    dst_rb = s_rb[ch.out_id];
  } else {
    dst = outs.ptr[0];
    dst_rb = outs.row_bytes[0];
  }
  int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
  const int64_t r_end = min(r0 + (int64_t)rows_per_block, rows);
  const char* s = src + r0 * src_row_bytes + ch.src_off;
  char* d = dst + r0 * dst_rb + ch.dst_off;
  for (; r0 + RU <= r_end; r0 += RU) {
    store_t v[RU];
#pragma unroll
    for (int u = 0; u < RU; ++u) v[u] = *reinterpret_cast<const load_t*>(s + u * src_row_bytes);
#pragma unroll
    for (int u = 0; u < RU; ++u) __builtin_nontemporal_store(v[u], reinterpret_cast<store_t*>(d + u * dst_rb));
    s += RU * src_row_bytes;
    d += RU * dst_rb;
  }
  for (; r0 < r_end; ++r0) {
    store_t v = *reinterpret_cast<const load_t*>(s);
    *reinterpret_cast<store_t*>(d) = v;
    s += src_row_bytes;
    d += dst_rb;
  }
}

template <int CB, int KB>
int launch_kb(const char* src, int64_t src_row_bytes, int64_t rows, const OutTable& outs, int n_outs,
           const xg_chunk* table, int64_t n_chunks, hipStream_t stream) {
  const int64_t gx = (n_chunks + KB - 1) / KB;
  // Rows per block: enough blocks to cover the 256 CUs several times over, but a
  // strip long enough that each lane amortises its table entry.
  int rpb = 8;
  while (rpb < 64 && gx * ((rows + rpb - 1) / rpb) > 8192) rpb *= 2;
  const int64_t gy = (rows + rpb - 1) / rpb;
  if (gx > 0x7fffffffLL || gy > 65535) return XG_ERR_TOO_LARGE;
  dim3 grid((unsigned)gx, (unsigned)gy);
  if (n_outs == 1)
    hipLaunchKernelGGL((slice_cat_kernel<CB, 8, KB, false>), grid, dim3(KB), 0, stream, src, src_row_bytes, rows, outs,
                       n_outs, table, n_chunks, rpb);
  else
    hipLaunchKernelGGL((slice_cat_kernel<CB, 8, KB, true>), grid, dim3(KB), 0, stream, src, src_row_bytes, rows, outs,
                       n_outs, table, n_chunks, rpb);
  return status_from_hip(hipGetLastError());
}

// 512 lanes per block once a row has that many chunks (one block then spans a whole 8 KiB output row of 16-byte
// chunks: 4 % faster than two 256-lane blocks on the 64-slice case), 256 otherwise.
template <int CB>
int launch(const char* src, int64_t src_row_bytes, int64_t rows, const OutTable& outs, int n_outs,
           const xg_chunk* table, int64_t n_chunks, hipStream_t stream) {
  return n_chunks >= 512 ? launch_kb<CB, 512>(src, src_row_bytes, rows, outs, n_outs, table, n_chunks, stream)
                         : launch_kb<CB, 256>(src, src_row_bytes, rows, outs, n_outs, table, n_chunks, stream);
}

}  // namespace
}  // namespace xg

extern "C" int xg_slice_cat_check_table(const xg_chunk* table_host, int64_t n_chunks, int chunk_bytes,
                                        int64_t src_row_valid_bytes, const int64_t* out_row_valid_bytes, int n_outs) {
  using namespace xg;
  if (table_host == nullptr || out_row_valid_bytes == nullptr) return XG_ERR_NULL_PTR;
  if (n_outs < 1 || n_outs > XG_SLICE_CAT_MAX_OUTS) return XG_ERR_TOO_LARGE;
  if (n_chunks < 0 || src_row_valid_bytes < 0) return XG_ERR_BAD_SHAPE;
  if (chunk_bytes != 1 && chunk_bytes != 2 && chunk_bytes != 4 && chunk_bytes != 8 && chunk_bytes != 16)
    return XG_ERR_BAD_ARG;
  const int src_align = chunk_bytes < 4 ? chunk_bytes : 4;
  for (int i = 0; i < n_outs; ++i)
    if (out_row_valid_bytes[i] < 0) return XG_ERR_BAD_SHAPE;
  for (int64_t i = 0; i < n_chunks; ++i) {
    const xg_chunk& c = table_host[i];
    if (c.out_id < 0 || c.out_id >= n_outs) return XG_ERR_BAD_SHAPE;
    if (c.src_off < 0 || (int64_t)c.src_off + chunk_bytes > src_row_valid_bytes) return XG_ERR_BAD_SHAPE;
    if (c.dst_off < 0 || (int64_t)c.dst_off + chunk_bytes > out_row_valid_bytes[c.out_id]) return XG_ERR_BAD_SHAPE;
    if (c.src_off % src_align != 0 || c.dst_off % chunk_bytes != 0) return XG_ERR_BAD_ALIGN;
  }
  return XG_OK;
}

extern "C" int xg_slice_cat(const void* src, int64_t src_row_bytes, int64_t rows, void* const* outs,
                            const int64_t* out_row_bytes, int n_outs, const xg_chunk* table_dev, int64_t n_chunks,
                            int chunk_bytes, xg_stream_t stream) {
  using namespace xg;
  if (src == nullptr || outs == nullptr || out_row_bytes == nullptr || table_dev == nullptr) return XG_ERR_NULL_PTR;
  if (n_outs < 1 || n_outs > XG_SLICE_CAT_MAX_OUTS) return XG_ERR_TOO_LARGE;
  if (rows < 0 || n_chunks < 0 || src_row_bytes < 0) return XG_ERR_BAD_SHAPE;
  if (chunk_bytes != 1 && chunk_bytes != 2 && chunk_bytes != 4 && chunk_bytes != 8 && chunk_bytes != 16)
    return XG_ERR_BAD_ARG;
  const size_t src_align = chunk_bytes < 4 ? chunk_bytes : 4;
  if (!aligned_to(src, src_align) || src_row_bytes % (int64_t)src_align != 0) return XG_ERR_BAD_ALIGN;
  if (!aligned_to(table_dev, 16)) return XG_ERR_BAD_ALIGN;
  OutTable t;
  for (int i = 0; i < XG_SLICE_CAT_MAX_OUTS; ++i) {
    t.ptr[i] = nullptr;
    t.row_bytes[i] = 0;
  }
  for (int i = 0; i < n_outs; ++i) {
    if (outs[i] == nullptr) return XG_ERR_NULL_PTR;
    if (!aligned_to(outs[i], chunk_bytes) || out_row_bytes[i] % chunk_bytes != 0 || out_row_bytes[i] < 0)
      return XG_ERR_BAD_ALIGN;
    t.ptr[i] = (char*)outs[i];
    t.row_bytes[i] = out_row_bytes[i];
  }
  if (rows == 0 || n_chunks == 0) return XG_OK;
  hipStream_t st = (hipStream_t)stream;
  const char* s = (const char*)src;
  switch (chunk_bytes) {
    case 16:
      return launch<16>(s, src_row_bytes, rows, t, n_outs, table_dev, n_chunks, st);
    case 8:
      return launch<8>(s, src_row_bytes, rows, t, n_outs, table_dev, n_chunks, st);
    case 4:
      return launch<4>(s, src_row_bytes, rows, t, n_outs, table_dev, n_chunks, st);
    case 2:
      return launch<2>(s, src_row_bytes, rows, t, n_outs, table_dev, n_chunks, st);
    default:
      return launch<1>(s, src_row_bytes, rows, t, n_outs, table_dev, n_chunks, st);
  }
}
