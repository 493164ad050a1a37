// Permuting row gather: out[b,h,s,:] = x[b,h,idx[b,h,s],:], rows past n_idx zero-filled.
// Stands in for indexing() (src/attn_utils.py:27-50 of the reference).  One 16-byte piece per
// lane; the lanes of a row are adjacent so every gathered row is read and written as whole
// cache lines.
#include "ha_common.h"

namespace {

__global__ __launch_bounds__(256) void gather_rows_kernel(const unsigned char* __restrict__ x,
                                                          const void* __restrict__ idx, int idx64,
                                                          unsigned char* __restrict__ out, int heads,
                                                          int64_t n_idx, int64_t n_out, int pieces,
                                                          int64_t sb_bytes, int64_t sh_bytes, int64_t sn_bytes) {
  const int bh = blockIdx.y;
  const int b = bh / heads, h = bh % heads;
  const int64_t item = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t row = item / pieces;
  const int piece = (int)(item % pieces);
  if (row >= n_out) return;
  u32x4 val = {0u, 0u, 0u, 0u};
  if (row < n_idx) {
    const int src = ha_load_idx(idx, (int64_t)bh * n_idx + row, idx64);
    val = *reinterpret_cast<const u32x4*>(x + b * sb_bytes + h * sh_bytes + (int64_t)src * sn_bytes + piece * 16);
  }
  *reinterpret_cast<u32x4*>(out + (((int64_t)bh * n_out + row) * pieces + piece) * 16) = val;
}

}  // namespace

extern "C" int ha_gather_rows(const void* x, const void* idx, int idx_type, void* out, int64_t batch,
                              int64_t heads, int64_t n_src, int64_t n_idx, int64_t n_out, int64_t d,
                              int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_n, int elem_bytes,
                              void* stream) {
  HA_REQUIRE(x && idx && out, HA_ERR_NULL, "ha_gather_rows: null pointer");
  HA_REQUIRE(idx_type == HA_IDX_I32 || idx_type == HA_IDX_I64, HA_ERR_DTYPE, "ha_gather_rows: bad idx_type");
  HA_REQUIRE(elem_bytes == 2 || elem_bytes == 4, HA_ERR_DTYPE, "ha_gather_rows: elem_bytes must be 2 or 4");
  HA_REQUIRE(batch > 0 && heads > 0 && n_src > 0 && n_idx >= 0 && n_out >= n_idx && n_out > 0 && d > 0,
             HA_ERR_SHAPE, "ha_gather_rows: bad sizes");
  HA_REQUIRE(batch * heads <= 65535, HA_ERR_SHAPE, "ha_gather_rows: batch*heads must be <= 65535");
  HA_REQUIRE((d * elem_bytes) % 16 == 0, HA_ERR_HEADDIM, "ha_gather_rows: row bytes must be a multiple of 16");
  HA_REQUIRE((x_stride_n * elem_bytes) % 16 == 0 && (x_stride_h * elem_bytes) % 16 == 0 &&
                 (x_stride_b * elem_bytes) % 16 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0,
             HA_ERR_SHAPE, "ha_gather_rows: rows must be 16-byte aligned");
  const int pieces = (int)(d * elem_bytes / 16);
  const int64_t items = n_out * pieces;
  dim3 grid((unsigned)((items + 255) / 256), (unsigned)(batch * heads));
  hipLaunchKernelGGL(gather_rows_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const unsigned char*)x, idx,
                     idx_type == HA_IDX_I64, (unsigned char*)out, (int)heads, n_idx, n_out, pieces,
                     x_stride_b * elem_bytes, x_stride_h * elem_bytes, x_stride_n * elem_bytes);
  return ha_launch_status("ha_gather_rows");
}
